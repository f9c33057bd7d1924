// Rotary position embedding for gfx950: the dense operator and the rotate-and-append
// launch.  One thread owns two 8-dim chunks of one (token, head) row -- the two halves
// of eight rotation pairs -- so every global access is a 16-byte lane access and the
// rotation needs no exchange between lanes.  Query rows and key rows ride in the same
// launch; key rows go either to a dense output or, with their value rows, into the pool.
#include "rope.h"

namespace pace_kv {

struct RopeRowsParams {
  RopeDev rope;
  const uint16_t* q;
  uint16_t* q_out;
  int64_t q_sb, q_sh, q_st;
  int32_t Hq;
  const uint16_t* k;
  uint16_t* k_out;  // dense destination (to_pool == 0)
  const uint16_t* v;
  int64_t k_sb, k_sh, k_st;
  int32_t Hk;
  pace_kv_pool_t pool;
  int32_t to_pool;
  const int32_t* table;
  int32_t table_stride;
  const int32_t* seq_lens;
  int32_t pos_offset;
  int32_t T;
  int64_t total;  // threads with work: batch * T * (Hq + Hk) * D/16
};

template <int D>
__global__ __launch_bounds__(256) void rope_rows_kernel(const RopeRowsParams p) {
  constexpr int PAIRS = D / 16;
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= p.total) return;
  const int ci = (int)(gid % PAIRS);
  const int64_t row = gid / PAIRS;
  const int heads = p.Hq + p.Hk;
  const int hh = (int)(row % heads);
  const int64_t i = row / heads;
  const int b = (int)(i / p.T), t = (int)(i % p.T);
  // position of the token in its sequence (pool destination and default table row)
  const int64_t cpos = p.seq_lens ? (int64_t)p.seq_lens[b] + p.pos_offset + t : t;
  const int tab_row = rope_row(p.rope, b, t, (int)cpos);
  int ca, cb;
  rope_chunk_pair(p.rope, ci, ca, cb);
  if (hh < p.Hq) {
    const int64_t base = (int64_t)b * p.q_sb + (int64_t)hh * p.q_sh + (int64_t)t * p.q_st;
    u32x4 xa = *reinterpret_cast<const u32x4*>(p.q + base + ca * 8);
    u32x4 xb = *reinterpret_cast<const u32x4*>(p.q + base + cb * 8);
    rope_rotate_chunks(p.rope, tab_row, ci, xa, xb);
    *reinterpret_cast<u32x4*>(p.q_out + base + ca * 8) = xa;
    *reinterpret_cast<u32x4*>(p.q_out + base + cb * 8) = xb;
    return;
  }
  const int h = hh - p.Hq;
  const int64_t base = (int64_t)b * p.k_sb + (int64_t)h * p.k_sh + (int64_t)t * p.k_st;
  if (!p.to_pool) {
    u32x4 xa = *reinterpret_cast<const u32x4*>(p.k + base + ca * 8);
    u32x4 xb = *reinterpret_cast<const u32x4*>(p.k + base + cb * 8);
    rope_rotate_chunks(p.rope, tab_row, ci, xa, xb);
    *reinterpret_cast<u32x4*>(p.k_out + base + ca * 8) = xa;
    *reinterpret_cast<u32x4*>(p.k_out + base + cb * 8) = xb;
    return;
  }
  if (cpos < 0 || cpos / PACE_KV_BLOCK_TOKENS >= p.table_stride) return;
  const int64_t blk = p.table[(int64_t)b * p.table_stride + cpos / PACE_KV_BLOCK_TOKENS];
  if (blk < 0 || blk >= p.pool.num_blocks) return;  // never write outside the pool
  const int off = (int)(cpos % PACE_KV_BLOCK_TOKENS);
  u32x4 ka = *reinterpret_cast<const u32x4*>(p.k + base + ca * 8);
  u32x4 kb = *reinterpret_cast<const u32x4*>(p.k + base + cb * 8);
  const u32x4 va = *reinterpret_cast<const u32x4*>(p.v + base + ca * 8);
  const u32x4 vb = *reinterpret_cast<const u32x4*>(p.v + base + cb * 8);
  rope_rotate_chunks(p.rope, tab_row, ci, ka, kb);
  uint16_t* kslab = reinterpret_cast<uint16_t*>(p.pool.k) + blk * p.pool.k_block_stride + h * p.pool.k_head_stride;
  uint16_t* vslab = reinterpret_cast<uint16_t*>(p.pool.v) + blk * p.pool.v_block_stride + h * p.pool.v_head_stride;
  store_kv_chunk<D>(kslab, vslab, off, ca, ka, va);
  store_kv_chunk<D>(kslab, vslab, off, cb, kb, vb);
}

// fp32 rows (the reference's operator on fp32 activations, pace/ops/rotary_embedding.py:412-443 with cos / sin
// cast to fp32): one thread per (token, head, rotation pair or pass-through pair of dims).  Every product and
// the sum are rounded separately, as the tensor operations round them -- no fused multiply-add.
struct RopeF32Params {
  const float* cos;
  const float* sin;
  int32_t rows, rot, interleaved;
  const int32_t* positions;
  int32_t pos_sb;
  const float* x[2];
  float* out[2];
  int64_t sb[2], sh[2], st[2];
  int32_t heads[2];
  int32_t T, D;
  int64_t total;  // batch * T * (heads[0] + heads[1]) * D/2
};

__global__ __launch_bounds__(256) void rope_rows_f32_kernel(const RopeF32Params p) {
#pragma clang fp contract(off)
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= p.total) return;
  const int half_d = p.D / 2;
  const int i = (int)(gid % half_d);
  const int64_t row = gid / half_d;
  const int heads = p.heads[0] + p.heads[1];
  const int hh = (int)(row % heads);
  const int64_t bt = row / heads;
  const int b = (int)(bt / p.T), t = (int)(bt % p.T);
  const int which = hh < p.heads[0] ? 0 : 1, h = which ? hh - p.heads[0] : hh;
  const int64_t base = (int64_t)b * p.sb[which] + (int64_t)h * p.sh[which] + (int64_t)t * p.st[which];
  const float* x = p.x[which] + base;
  float* o = p.out[which] + base;
  const int half_r = p.rot / 2;
  if (i >= half_r) {  // the dims past rotary_dim pass through, two per thread
    const int d = p.rot + 2 * (i - half_r);
    o[d] = x[d], o[d + 1] = x[d + 1];
    return;
  }
  int pos = p.positions[(int64_t)b * p.pos_sb + t];
  pos = pos < 0 ? 0 : (pos >= p.rows ? p.rows - 1 : pos);
  const float c = p.cos[(int64_t)pos * half_r + i], sn = p.sin[(int64_t)pos * half_r + i];
  const int d1 = p.interleaved ? 2 * i : i, d2 = p.interleaved ? 2 * i + 1 : i + half_r;
  const float x1 = x[d1], x2 = x[d2];
  const float a = x1 * c, bq = x2 * sn, cq = x2 * c, dq = x1 * sn;
  o[d1] = a - bq;
  o[d2] = cq + dq;
}

int make_rope_dev(const pace_rope_t* rope, int head_dim, bool need_positions, const char* who, RopeDev* out) {
  PACE_REQUIRE(rope != nullptr, "%s: rope is NULL", who);
  PACE_REQUIRE(rope->cos && rope->sin, "%s: NULL cos / sin table", who);
  PACE_REQUIRE(rope->table_dtype == PACE_DTYPE_BF16 || rope->table_dtype == PACE_DTYPE_F32, "%s: bad table dtype %d", who,
               rope->table_dtype);
  PACE_REQUIRE(rope->table_rows >= 1, "%s: table_rows %d", who, rope->table_rows);
  PACE_REQUIRE(rope->rotary_dim >= 16 && rope->rotary_dim % 16 == 0 && rope->rotary_dim <= head_dim,
               "%s: rotary_dim %d must be a multiple of 16 and at most head_dim %d", who, rope->rotary_dim, head_dim);
  PACE_REQUIRE(aligned16(rope->cos) && aligned16(rope->sin), "%s: cos / sin tables must be 16-byte aligned", who);
  PACE_REQUIRE(rope->interleaved == 0 || rope->interleaved == 1, "%s: interleaved must be 0 or 1", who);
  if (need_positions) PACE_REQUIRE(rope->positions != nullptr, "%s: rope positions are required here", who);
  if (rope->positions) PACE_REQUIRE(rope->pos_stride_b >= 0, "%s: negative pos_stride_b", who);
  out->cos = rope->cos, out->sin = rope->sin;
  out->is_f32 = rope->table_dtype == PACE_DTYPE_F32;
  out->rows = rope->table_rows, out->rot = rope->rotary_dim, out->interleaved = rope->interleaved;
  out->positions = rope->positions, out->pos_sb = rope->pos_stride_b;
  return PACE_KV_OK;
}

static int launch_rows(RopeRowsParams& p, int head_dim, int batch, void* stream, const char* who) {
  const int64_t total = (int64_t)batch * p.T * (p.Hq + p.Hk) * (head_dim / 16);
  if (total == 0) return PACE_KV_OK;
  PACE_REQUIRE((total + 255) / 256 < (int64_t)1 << 31, "%s: grid too large", who);
  p.total = total;
  const unsigned grid = (unsigned)((total + 255) / 256);
  hipStream_t s = static_cast<hipStream_t>(stream);
  for_head_dim(head_dim, [&](auto d) { hipLaunchKernelGGL(rope_rows_kernel<decltype(d)::value>, dim3(grid), dim3(256), 0, s, p); });
  PACE_HIP_CHECK(hipGetLastError());
  return PACE_KV_OK;
}

static int check_rows(const char* who, const char* name, const void* in, const void* out, int64_t sb, int64_t sh, int64_t st,
                      int32_t heads) {
  PACE_REQUIRE(out != nullptr, "%s: %s has no output pointer", who, name);
  PACE_REQUIRE(aligned16(in) && aligned16(out), "%s: %s must be 16-byte aligned", who, name);
  PACE_REQUIRE(sb % 8 == 0 && sh % 8 == 0 && st % 8 == 0, "%s: %s strides must be multiples of 8 elements", who, name);
  PACE_REQUIRE(heads >= 1, "%s: %s head count %d", who, name, heads);
  return PACE_KV_OK;
}

}  // namespace pace_kv

using namespace pace_kv;

extern "C" int pace_rope_apply(const pace_rope_t* rope, const void* q, void* q_out, int64_t q_stride_b, int64_t q_stride_h,
                               int64_t q_stride_t, int32_t num_q_heads, const void* k, void* k_out, int64_t k_stride_b,
                               int64_t k_stride_h, int64_t k_stride_t, int32_t num_k_heads, int32_t batch, int32_t n_tokens,
                               int32_t head_dim, void* stream) {
  const char* who = "pace_rope_apply";
  PACE_REQUIRE(head_dim_supported(head_dim), "%s: head_dim %d unsupported (64, 96, 128 or 256)", who, head_dim);
  PACE_REQUIRE(batch >= 0 && n_tokens >= 0, "%s: negative batch (%d) or n_tokens (%d)", who, batch, n_tokens);
  RopeRowsParams p = {};
  if (int rc = make_rope_dev(rope, head_dim, true, who, &p.rope)) return rc;
  if (q) {
    if (int rc = check_rows(who, "q", q, q_out, q_stride_b, q_stride_h, q_stride_t, num_q_heads)) return rc;
    p.q = static_cast<const uint16_t*>(q), p.q_out = static_cast<uint16_t*>(q_out);
    p.q_sb = q_stride_b, p.q_sh = q_stride_h, p.q_st = q_stride_t, p.Hq = num_q_heads;
  }
  if (k) {
    if (int rc = check_rows(who, "k", k, k_out, k_stride_b, k_stride_h, k_stride_t, num_k_heads)) return rc;
    p.k = static_cast<const uint16_t*>(k), p.k_out = static_cast<uint16_t*>(k_out);
    p.k_sb = k_stride_b, p.k_sh = k_stride_h, p.k_st = k_stride_t, p.Hk = num_k_heads;
  }
  p.T = n_tokens;
  if (batch == 0 || n_tokens == 0 || p.Hq + p.Hk == 0) return PACE_KV_OK;
  return launch_rows(p, head_dim, batch, stream, who);
}

extern "C" int pace_rope_append_paged(const pace_kv_pool_t* pool, const pace_rope_t* rope, const void* q, void* q_out,
                                      int64_t q_stride_b, int64_t q_stride_h, int64_t q_stride_t, int32_t num_q_heads,
                                      const void* k_new, const void* v_new, int64_t stride_b, int64_t stride_h,
                                      int64_t stride_t, int32_t batch, int32_t n_tokens, const int32_t* block_table,
                                      int32_t table_stride, const int32_t* seq_lens, int32_t pos_offset, void* stream) {
  const char* who = "pace_rope_append_paged";
  if (int rc = check_pool(pool, who)) return rc;
  PACE_REQUIRE(batch >= 0 && n_tokens >= 0, "%s: negative batch (%d) or n_tokens (%d)", who, batch, n_tokens);
  RopeRowsParams p = {};
  if (int rc = make_rope_dev(rope, pool->head_dim, false, who, &p.rope)) return rc;
  if (batch == 0 || n_tokens == 0) return PACE_KV_OK;
  PACE_REQUIRE(block_table != nullptr && seq_lens != nullptr && table_stride >= 1,
               "%s: NULL block_table / seq_lens or bad table_stride", who);
  PACE_REQUIRE(k_new && v_new, "%s: NULL input pointer", who);
  PACE_REQUIRE(aligned16(k_new) && aligned16(v_new), "%s: k_new / v_new must be 16-byte aligned", who);
  PACE_REQUIRE(stride_b % 8 == 0 && stride_h % 8 == 0 && stride_t % 8 == 0, "%s: input strides must be multiples of 8 elements",
               who);
  if (q) {
    if (int rc = check_rows(who, "q", q, q_out, q_stride_b, q_stride_h, q_stride_t, num_q_heads)) return rc;
    p.q = static_cast<const uint16_t*>(q), p.q_out = static_cast<uint16_t*>(q_out);
    p.q_sb = q_stride_b, p.q_sh = q_stride_h, p.q_st = q_stride_t, p.Hq = num_q_heads;
  }
  p.table = block_table, p.table_stride = table_stride, p.seq_lens = seq_lens, p.pos_offset = pos_offset;
  p.T = n_tokens;
  if (n_tokens >= 8) {
    // Many tokens per sequence: keys and values go through the block-wise append (slab-ordered
    // 16-byte stores, keys rotated while staged); the queries are rotated by a launch of their own.
    if (int rc = launch_block_append(who, pool, k_new, v_new, stride_b, stride_h, stride_t, batch, n_tokens, block_table,
                                     table_stride, seq_lens, pos_offset, &p.rope, static_cast<hipStream_t>(stream)))
      return rc;
    if (!q) return PACE_KV_OK;
    return launch_rows(p, pool->head_dim, batch, stream, who);  // Hk == 0: query rows only
  }
  p.k = static_cast<const uint16_t*>(k_new), p.v = static_cast<const uint16_t*>(v_new);
  p.k_sb = stride_b, p.k_sh = stride_h, p.k_st = stride_t, p.Hk = pool->num_kv_heads;
  p.pool = *pool, p.to_pool = 1;
  return launch_rows(p, pool->head_dim, batch, stream, who);
}

extern "C" int pace_rope_apply_f32(const pace_rope_t* rope, const void* q, void* q_out, int64_t q_stride_b, int64_t q_stride_h,
                                   int64_t q_stride_t, int32_t num_q_heads, const void* k, void* k_out, int64_t k_stride_b,
                                   int64_t k_stride_h, int64_t k_stride_t, int32_t num_k_heads, int32_t batch, int32_t n_tokens,
                                   int32_t head_dim, void* stream) {
  const char* who = "pace_rope_apply_f32";
  PACE_REQUIRE(rope != nullptr && rope->cos && rope->sin && rope->positions, "%s: NULL rope, table or positions", who);
  PACE_REQUIRE(rope->table_dtype == PACE_DTYPE_F32, "%s: fp32 rows take fp32 tables", who);
  PACE_REQUIRE(head_dim >= 2 && head_dim % 2 == 0, "%s: head_dim %d must be even", who, head_dim);
  PACE_REQUIRE(rope->rotary_dim >= 2 && rope->rotary_dim % 2 == 0 && rope->rotary_dim <= head_dim,
               "%s: rotary_dim %d must be even and at most head_dim %d", who, rope->rotary_dim, head_dim);
  PACE_REQUIRE(rope->table_rows >= 1 && rope->pos_stride_b >= 0, "%s: bad table_rows (%d) or pos_stride_b (%d)", who, rope->table_rows,
               rope->pos_stride_b);
  PACE_REQUIRE(rope->interleaved == 0 || rope->interleaved == 1, "%s: interleaved must be 0 or 1", who);
  PACE_REQUIRE(batch >= 0 && n_tokens >= 0, "%s: negative batch (%d) or n_tokens (%d)", who, batch, n_tokens);
  RopeF32Params p = {};
  p.cos = static_cast<const float*>(rope->cos), p.sin = static_cast<const float*>(rope->sin);
  p.rows = rope->table_rows, p.rot = rope->rotary_dim, p.interleaved = rope->interleaved;
  p.positions = rope->positions, p.pos_sb = rope->pos_stride_b;
  if (q) {
    PACE_REQUIRE(q_out != nullptr && num_q_heads >= 1, "%s: q has no output pointer or no heads", who);
    p.x[0] = static_cast<const float*>(q), p.out[0] = static_cast<float*>(q_out);
    p.sb[0] = q_stride_b, p.sh[0] = q_stride_h, p.st[0] = q_stride_t, p.heads[0] = num_q_heads;
  }
  if (k) {
    PACE_REQUIRE(k_out != nullptr && num_k_heads >= 1, "%s: k has no output pointer or no heads", who);
    p.x[1] = static_cast<const float*>(k), p.out[1] = static_cast<float*>(k_out);
    p.sb[1] = k_stride_b, p.sh[1] = k_stride_h, p.st[1] = k_stride_t, p.heads[1] = num_k_heads;
  }
  p.T = n_tokens, p.D = head_dim;
  p.total = (int64_t)batch * n_tokens * (p.heads[0] + p.heads[1]) * (head_dim / 2);
  if (p.total == 0) return PACE_KV_OK;
  PACE_REQUIRE((p.total + 255) / 256 < (int64_t)1 << 31, "%s: grid too large", who);
  hipLaunchKernelGGL(rope_rows_f32_kernel, dim3((unsigned)((p.total + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream), p);
  PACE_HIP_CHECK(hipGetLastError());
  return PACE_KV_OK;
}
