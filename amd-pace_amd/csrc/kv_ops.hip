// Pool data movement for gfx950: append by slot, block-table gather, block copy.
// All three are pure byte movers bounded by HBM bandwidth; every global access
// is a 16-byte lane access, coalesced over rows of the token-major side.
#include "common.h"
#include "rope.h"

namespace pace_kv {

// ---------------------------------------------------------------------------------
// Append.  One thread moves eight dims (16 bytes) of one (token, head) row of K and
// of V.  The K chunk stays one 16-byte store; the V chunk is written token-minor, so
// its eight values land 16 bytes apart (one per dim) at the token's column.
// ---------------------------------------------------------------------------------
// Where the tokens go: either an explicit slot id per token, or "position
// seq_lens[b] + pos_offset + t of sequence b" resolved through the block table.
struct AppendDest {
  const int64_t* slots;
  const int32_t* table;
  const int32_t* seq_lens;
  int32_t table_stride;
  int32_t pos_offset;
  const int32_t* offset_dev;  // optional: one more offset, read on the device (a counter a captured graph advances)
};

template <int D, bool PAGED>
__global__ __launch_bounds__(256) void kv_append_kernel(pace_kv_pool_t pool, const uint16_t* __restrict__ k_new,
                                                        const uint16_t* __restrict__ v_new, int64_t sb, int64_t sh,
                                                        int64_t st, int32_t n_tokens, int32_t total_rows,
                                                        const AppendDest dest) {
  constexpr int CHUNKS = D / 8;
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int chunk = (int)(gid % CHUNKS);
  const int64_t row = gid / CHUNKS;  // (token i, head h), head fastest
  if (row >= total_rows) return;
  const int H = pool.num_kv_heads;
  const int h = (int)(row % H);
  const int64_t i = row / H;  // b * n_tokens + t
  const int64_t b = i / n_tokens, t = i % n_tokens;
  int64_t blk;
  int off;
  if (PAGED) {
    const int64_t pos = (int64_t)dest.seq_lens[b] + dest.pos_offset + (dest.offset_dev ? *dest.offset_dev : 0) + t;
    if (pos < 0 || pos / PACE_KV_BLOCK_TOKENS >= dest.table_stride) return;
    blk = dest.table[b * dest.table_stride + pos / PACE_KV_BLOCK_TOKENS];
    off = (int)(pos % PACE_KV_BLOCK_TOKENS);
  } else {
    const int64_t slot = dest.slots[i];
    if (slot < 0) return;
    blk = slot / PACE_KV_BLOCK_TOKENS;
    off = (int)(slot % PACE_KV_BLOCK_TOKENS);
  }
  if (blk < 0 || blk >= pool.num_blocks) return;  // never write outside the pool
  const int64_t src = b * sb + h * sh + t * st + chunk * 8;
  const u32x4 kv = *reinterpret_cast<const u32x4*>(k_new + src);
  const u32x4 vv = *reinterpret_cast<const u32x4*>(v_new + src);
  store_kv_chunk<D>(reinterpret_cast<uint16_t*>(pool.k) + blk * pool.k_block_stride + h * pool.k_head_stride,
                    reinterpret_cast<uint16_t*>(pool.v) + blk * pool.v_block_stride + h * pool.v_head_stride, off, chunk, kv,
                    vv);
}

// The same scatter into a pool of fp32 rows ([16 tokens][head_dim] floats per (block, head)): one thread moves
// four dims (16 bytes) of one (token, head) row of K and of V, row to row.
template <bool PAGED>
__global__ __launch_bounds__(256) void kv_append_f32_kernel(pace_kv_pool_t pool, const float* __restrict__ k_new,
                                                            const float* __restrict__ v_new, int64_t sb, int64_t sh,
                                                            int64_t st, int32_t n_tokens, int32_t total_rows,
                                                            const AppendDest dest) {
  const int D = pool.head_dim, chunks = D / 4;
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int chunk = (int)(gid % chunks);
  const int64_t row = gid / chunks;  // (token i, head h), head fastest
  if (row >= total_rows) return;
  const int H = pool.num_kv_heads;
  const int h = (int)(row % H);
  const int64_t i = row / H;  // b * n_tokens + t
  const int64_t b = i / n_tokens, t = i % n_tokens;
  int64_t blk;
  int off;
  if (PAGED) {
    const int64_t pos = (int64_t)dest.seq_lens[b] + dest.pos_offset + (dest.offset_dev ? *dest.offset_dev : 0) + t;
    if (pos < 0 || pos / PACE_KV_BLOCK_TOKENS >= dest.table_stride) return;
    blk = dest.table[b * dest.table_stride + pos / PACE_KV_BLOCK_TOKENS];
    off = (int)(pos % PACE_KV_BLOCK_TOKENS);
  } else {
    const int64_t slot = dest.slots[i];
    if (slot < 0) return;
    blk = slot / PACE_KV_BLOCK_TOKENS;
    off = (int)(slot % PACE_KV_BLOCK_TOKENS);
  }
  if (blk < 0 || blk >= pool.num_blocks) return;  // never write outside the pool
  const int64_t src = b * sb + h * sh + t * st + chunk * 4;
  const int64_t in_slab = (int64_t)off * D + chunk * 4;
  const u32x4 kv = *reinterpret_cast<const u32x4*>(k_new + src);
  const u32x4 vv = *reinterpret_cast<const u32x4*>(v_new + src);
  *reinterpret_cast<u32x4*>(static_cast<float*>(pool.k) + blk * pool.k_block_stride + h * pool.k_head_stride + in_slab) = kv;
  *reinterpret_cast<u32x4*>(static_cast<float*>(pool.v) + blk * pool.v_block_stride + h * pool.v_head_stride + in_slab) = vv;
}

// ---------------------------------------------------------------------------------
// Block append (many tokens per sequence: prefill chunks).  One 256-thread workgroup
// fills one destination block of one (sequence, head): the token rows that land in the
// block are staged row-major in LDS, then written out in slab order, 16 bytes per lane
// -- K chunks straight from the rows, V chunks transposed (eight tokens of one dim).
// Slabs of blocks the append only partly covers are written element-wise for V so that
// earlier tokens of the block stay untouched.
// ---------------------------------------------------------------------------------
template <int D, bool ROPE>
__global__ __launch_bounds__(256) void kv_append_block_kernel(pace_kv_pool_t pool, const uint16_t* __restrict__ k_new,
                                                              const uint16_t* __restrict__ v_new, int64_t sb, int64_t sh,
                                                              int64_t st, int32_t n_tokens, const AppendDest dest,
                                                              const RopeDev rope) {
  constexpr int CHUNKS = D / 8;
  constexpr int BT = PACE_KV_BLOCK_TOKENS;
  __shared__ uint16_t ks[ROPE ? BT * D : 8];  // keys pass through LDS only where they are rotated on the way
  __shared__ uint16_t vs[BT * (D + 8)];       // padded rows: column reads hit different banks
  const int h = blockIdx.y, b = blockIdx.z;
  const int64_t pos0 = (int64_t)dest.seq_lens[b] + dest.pos_offset;  // position of new token 0
  if (pos0 < 0) return;
  // Destination blocks touched by this sequence: pos0/16 .. (pos0+n_tokens-1)/16.
  const int jb = (int)(pos0 / BT) + blockIdx.x;
  const int64_t blk_pos0 = (int64_t)jb * BT;
  const int t_lo = (int)max((int64_t)0, blk_pos0 - pos0);                 // first new token in this block
  const int t_hi = (int)min((int64_t)n_tokens, blk_pos0 + BT - pos0);     // one past the last
  if (t_lo >= t_hi || jb >= dest.table_stride) return;  // uniform over the workgroup
  const int64_t blk = dest.table[(int64_t)b * dest.table_stride + jb];
  if (blk < 0 || blk >= pool.num_blocks) return;  // never write outside the pool
  const int off_lo = (int)(pos0 + t_lo - blk_pos0), n_here = t_hi - t_lo;  // slots off_lo .. off_lo+n_here-1
  const uint16_t* kin = k_new + (int64_t)b * sb + (int64_t)h * sh;
  const uint16_t* vin = v_new + (int64_t)b * sb + (int64_t)h * sh;
  if (ROPE) {
    // keys are rotated on their way into LDS: a thread takes the two chunks of eight rotation pairs
    for (int c = threadIdx.x; c < n_here * (CHUNKS / 2); c += 256) {
      const int r = c / (CHUNKS / 2), ci = c % (CHUNKS / 2);
      const int t = t_lo + r;
      int ca, cb;
      rope_chunk_pair(rope, ci, ca, cb);
      const int64_t src = (int64_t)t * st;
      u32x4 ka = load16_stream(kin + src + ca * 8);
      u32x4 kb = load16_stream(kin + src + cb * 8);
      rope_rotate_chunks(rope, rope_row(rope, b, t, (int)(pos0 + t)), ci, ka, kb);
      *reinterpret_cast<u32x4*>(&ks[(off_lo + r) * D + ca * 8]) = ka;
      *reinterpret_cast<u32x4*>(&ks[(off_lo + r) * D + cb * 8]) = kb;
      *reinterpret_cast<u32x4*>(&vs[(off_lo + r) * (D + 8) + ca * 8]) = load16_stream(vin + src + ca * 8);
      *reinterpret_cast<u32x4*>(&vs[(off_lo + r) * (D + 8) + cb * 8]) = load16_stream(vin + src + cb * 8);
    }
  } else {
    for (int c = threadIdx.x; c < n_here * CHUNKS; c += 256) {
      const int r = c / CHUNKS, ch = c % CHUNKS;
      const int64_t src = (int64_t)(t_lo + r) * st + ch * 8;
      *reinterpret_cast<u32x4*>(&vs[(off_lo + r) * (D + 8) + ch * 8]) = load16_stream(vin + src);
    }
  }
  uint16_t* kslab = reinterpret_cast<uint16_t*>(pool.k) + blk * pool.k_block_stride + h * pool.k_head_stride;
  uint16_t* vslab = reinterpret_cast<uint16_t*>(pool.v) + blk * pool.v_block_stride + h * pool.v_head_stride;
  const bool whole = (n_here == BT);
  // K: slab chunk c = (tile, dim chunk, slot) holds dims 8*chunk.. of token tok(tile, slot).  Keys that are not
  // rotated need no staging: the chunk goes from its row to its slab place through a register (a wave reads eight
  // 128-byte runs and writes 1 KiB in one piece), before the barrier, so that it travels along with the V loads.
  if (!ROPE) {
    for (int c = threadIdx.x; c < BT * CHUNKS; c += 256) {
      const int tile = c / (CHUNKS * 8), chunk = (c / 8) % CHUNKS, slot = c % 8;
      const int tok = ((slot >> 2) << 3) | (tile << 2) | (slot & 3);
      if (tok >= off_lo && tok < off_lo + n_here)
        store16_stream(kslab + c * 8, load16_stream(kin + (int64_t)(t_lo + tok - off_lo) * st + chunk * 8));
    }
  }
  __syncthreads();
  if (ROPE) {
    for (int c = threadIdx.x; c < BT * CHUNKS; c += 256) {
      const int tile = c / (CHUNKS * 8), chunk = (c / 8) % CHUNKS, slot = c % 8;
      const int tok = ((slot >> 2) << 3) | (tile << 2) | (slot & 3);
      if (tok >= off_lo && tok < off_lo + n_here)
        store16_stream(kslab + c * 8, *reinterpret_cast<const u32x4*>(&ks[tok * D + chunk * 8]));
    }
  }
  // V: slab chunk c = (dim tile, token half, dim) holds tokens 8*half..+7 of one dim.
  for (int c = threadIdx.x; c < BT * CHUNKS; c += 256) {
    const int jt = c / 32, half = (c / 16) % 2, dn = c % 16;
    const int dim = jt * 16 + dn;
    if (whole) {
      u32x4 w;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        w[e] = (uint32_t)vs[(8 * half + 2 * e) * (D + 8) + dim] | ((uint32_t)vs[(8 * half + 2 * e + 1) * (D + 8) + dim] << 16);
      store16_stream(vslab + c * 8, w);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int tok = 8 * half + e;
        if (tok >= off_lo && tok < off_lo + n_here) vslab[c * 8 + e] = vs[tok * (D + 8) + dim];
      }
    }
  }
}

// ---------------------------------------------------------------------------------
// Gather.  One 256-thread workgroup rebuilds one logical block (16 tokens) of one KV
// head of one sequence as token rows.  K chunks are read from their slab position; V
// slabs are staged in LDS and read back transposed.  Two output forms:
//   dense   [B][H*n_rep][out_len][D]   (the reference's layout; rows >= len zero-filled on request)
//   packed  [sum len][H*n_rep][D]      (sequence b starts at row cu_seqlens[b]; no padding at all)
// A workgroup past the end of its sequence leaves at once; the packed form launches none (its grid is
// built from cu_seqlens).
// ---------------------------------------------------------------------------------
struct GatherOut {
  uint16_t* k;
  uint16_t* v;
  const int32_t* cu_seqlens;  // packed form only
  int64_t stride_b;           // dense: elements between sequences
  int64_t stride_h;           // elements between output heads
  int64_t stride_t;           // elements between token rows
  int32_t out_len;            // dense: rows per sequence; packed: unused
  int32_t zero_fill;          // dense: write zeros to rows in [len, out_len)
  int32_t batch;              // packed: sequences (cu_seqlens has batch + 1 entries)
  int32_t total_rows;         // packed: rows of the outputs
  int32_t dense_rows;         // packed grid (one workgroup per block that exists), rows written in the dense layout
};

// Packed grid: which (sequence, head, logical block) workgroup `entry` stands for.
// One grid entry per (logical block that can exist, KV head): sequence b owns the block entries
// [cu[b] / 16 + b, cu[b+1] / 16 + b + 1) -- at least ceil(len_b / 16) of them, disjoint, in order -- so a
// ragged batch launches (almost) no workgroup without rows.  Entries run sequence by sequence, head by
// head, block by block (the order of the dense grid: with the heads of a block side by side instead the
// launch measured 6 % slower).  The owner is found by bisection, uniform over the workgroup: scalar loads
// from a table that stays in the scalar cache.
__device__ __forceinline__ void packed_entry(const int32_t* __restrict__ cu, int batch, int H, unsigned entry, int& b, int& h, int& j) {
  int lo = 0, hi = batch;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if ((int64_t)(cu[mid] / PACE_KV_BLOCK_TOKENS + mid) * H <= (int64_t)entry) lo = mid; else hi = mid;
  }
  b = lo;
  const int first = cu[b] / PACE_KV_BLOCK_TOKENS + b;
  const int n = cu[b + 1] / PACE_KV_BLOCK_TOKENS + b + 1 - first;  // >= 1
  const int r = (int)((int64_t)entry - (int64_t)first * H);
  h = min(r / n, H - 1), j = r % n;
}

template <int D, bool PACKED>
__global__ __launch_bounds__(256) void kv_gather_kernel(pace_kv_pool_t pool, const int32_t* __restrict__ table,
                                                        int32_t table_stride, const int32_t* __restrict__ seq_lens,
                                                        int32_t len_bias, int32_t n_rep, const GatherOut out) {
  constexpr int CHUNKS = D / 8;                             // 16-byte chunks per row
  constexpr int SLAB_CHUNKS = PACE_KV_BLOCK_TOKENS * CHUNKS;  // per (block, head)
  __shared__ uint16_t vt[D * PACE_KV_BLOCK_TOKENS + 8];
  int j = blockIdx.x, b = blockIdx.z, h = blockIdx.y;
  if (PACKED) packed_entry(out.cu_seqlens, out.batch, pool.num_kv_heads, blockIdx.x, b, h, j);
  // The length and the block id are fetched side by side (the table row exists whatever the length is; an
  // entry past the live blocks is clamped into the pool and never used): one round trip, not two, before
  // the slab loads can start.
  const int len = seq_lens[b] + len_bias;
  int64_t blk = table[(int64_t)b * table_stride + min(j, table_stride - 1)];
  const int t0 = j * PACE_KV_BLOCK_TOKENS;
  const bool live = t0 < len;  // uniform per workgroup
  const bool dense_rows = PACKED && out.dense_rows != 0;  // the dense layout from the packed grid
  const int row_end = PACKED ? (dense_rows ? min(len, out.out_len) : len) : out.out_len;
  if (!live && (PACKED || !out.zero_fill || t0 >= row_end)) return;  // nothing to write
  blk = blk < 0 ? 0 : (blk >= pool.num_blocks ? pool.num_blocks - 1 : blk);  // never read outside the pool
  const uint16_t* ksrc = reinterpret_cast<const uint16_t*>(pool.k) + blk * pool.k_block_stride + h * pool.k_head_stride;
  const uint16_t* vsrc = reinterpret_cast<const uint16_t*>(pool.v) + blk * pool.v_block_stride + h * pool.v_head_stride;
  // Every load of the workgroup goes out before the barrier: the V slab (to LDS, to be read back transposed)
  // and the K chunks of this lane's rows (kept in registers).
  constexpr int PER = (SLAB_CHUNKS + 255) / 256;
  u32x4 kreg[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int c = threadIdx.x + i * 256;
    kreg[i] = u32x4{0u, 0u, 0u, 0u};
    if (live && c < SLAB_CHUNKS) {
      const u32x4 vraw = load16_stream(vsrc + c * 8);
      const int tok = c / CHUNKS, chunk = c % CHUNKS;
      if (t0 + tok < len) kreg[i] = load16_stream(ksrc + k_slab_offset<D>(tok, chunk * 8));
      *reinterpret_cast<u32x4*>(&vt[c * 8]) = vraw;
    }
  }
  __syncthreads();
  const int64_t base = (PACKED && !dense_rows) ? (int64_t)out.cu_seqlens[b] * out.stride_t : (int64_t)b * out.stride_b;
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int c = threadIdx.x + i * 256;
    if (c >= SLAB_CHUNKS) continue;
    const int tok = c / CHUNKS, chunk = c % CHUNKS;
    const int t = t0 + tok;
    if (t >= row_end) continue;
    if (PACKED && !dense_rows && out.cu_seqlens[b] + t >= out.total_rows) continue;  // never write past the outputs
    u32x4 vv = {0u, 0u, 0u, 0u};
    if (t < len) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const uint32_t lo = vt[v_slab_offset<D>(tok, chunk * 8 + 2 * e)];
        const uint32_t hi = vt[v_slab_offset<D>(tok, chunk * 8 + 2 * e + 1)];
        vv[e] = lo | (hi << 16);
      }
    } else if (!out.zero_fill) {
      continue;
    }
    for (int r = 0; r < n_rep; ++r) {
      const int64_t o = base + (int64_t)(h * n_rep + r) * out.stride_h + (int64_t)t * out.stride_t + chunk * 8;
      store16_stream(out.k + o, kreg[i]);
      store16_stream(out.v + o, vv);
    }
  }
}

// The gather out of a pool of fp32 rows: the same grid, rows copied as they are (16 bytes per lane access).
template <bool PACKED>
__global__ __launch_bounds__(256) void kv_gather_f32_kernel(pace_kv_pool_t pool, const int32_t* __restrict__ table,
                                                            int32_t table_stride, const int32_t* __restrict__ seq_lens,
                                                            int32_t len_bias, int32_t n_rep, const GatherOut out) {
  int j = blockIdx.x, b = blockIdx.z, h = blockIdx.y;
  if (PACKED) packed_entry(out.cu_seqlens, out.batch, pool.num_kv_heads, blockIdx.x, b, h, j);
  const int len = seq_lens[b] + len_bias;
  int64_t blk = table[(int64_t)b * table_stride + min(j, table_stride - 1)];
  const int t0 = j * PACE_KV_BLOCK_TOKENS;
  const bool live = t0 < len;  // uniform per workgroup
  const bool dense_rows = PACKED && out.dense_rows != 0;  // the dense layout from the packed grid
  const int row_end = PACKED ? (dense_rows ? min(len, out.out_len) : len) : out.out_len;
  if (!live && (PACKED || !out.zero_fill || t0 >= row_end)) return;  // nothing to write
  blk = blk < 0 ? 0 : (blk >= pool.num_blocks ? pool.num_blocks - 1 : blk);  // never read outside the pool
  const int D = pool.head_dim, chunks = D / 4;
  const float* ksrc = static_cast<const float*>(pool.k) + blk * pool.k_block_stride + h * pool.k_head_stride;
  const float* vsrc = static_cast<const float*>(pool.v) + blk * pool.v_block_stride + h * pool.v_head_stride;
  float* ko = reinterpret_cast<float*>(out.k);
  float* vo = reinterpret_cast<float*>(out.v);
  const int64_t base = (PACKED && !dense_rows) ? (int64_t)out.cu_seqlens[b] * out.stride_t : (int64_t)b * out.stride_b;
  for (int c = threadIdx.x; c < PACE_KV_BLOCK_TOKENS * chunks; c += 256) {
    const int tok = c / chunks, chunk = c % chunks;
    const int t = t0 + tok;
    if (t >= row_end) continue;
    if (PACKED && !dense_rows && out.cu_seqlens[b] + t >= out.total_rows) continue;  // never write past the outputs
    u32x4 kk = {0u, 0u, 0u, 0u}, vv = {0u, 0u, 0u, 0u};
    if (t < len) {
      kk = load16_stream(ksrc + c * 4), vv = load16_stream(vsrc + c * 4);
    } else if (!out.zero_fill) {
      continue;
    }
    for (int r = 0; r < n_rep; ++r) {
      const int64_t o = base + (int64_t)(h * n_rep + r) * out.stride_h + (int64_t)t * out.stride_t + chunk * 4;
      store16_stream(ko + o, kk);
      store16_stream(vo + o, vv);
    }
  }
}

// ---------------------------------------------------------------------------------
// Block copy.  Layout-agnostic (a slab is copied verbatim), 16 bytes per lane access.
// kv_copy_blocks_kernel: one workgroup per (pair, head), both slabs of that head.
// kv_copy_whole_blocks_kernel: pools whose blocks are one contiguous run each (all heads, K and V):
// one workgroup per pair moves the whole run, every lane with several loads in flight.
// ---------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void kv_copy_blocks_kernel(pace_kv_pool_t src, pace_kv_pool_t dst,
                                                             const int32_t* __restrict__ pairs) {
  const int pair = blockIdx.y, h = blockIdx.x;  // heads fastest: the slabs of one block move together
  const int64_t s = pairs[2 * pair], d = pairs[2 * pair + 1];
  if (s < 0 || s >= src.num_blocks || d < 0 || d >= dst.num_blocks) return;  // uniform per workgroup
  const int slab_chunks = PACE_KV_BLOCK_TOKENS * src.head_dim / 8;
  const u32x4* ks = reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(src.k) + s * src.k_block_stride +
                                                   h * src.k_head_stride);
  const u32x4* vs = reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(src.v) + s * src.v_block_stride +
                                                   h * src.v_head_stride);
  u32x4* kd = reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(dst.k) + d * dst.k_block_stride + h * dst.k_head_stride);
  u32x4* vd = reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(dst.v) + d * dst.v_block_stride + h * dst.v_head_stride);
  for (int c = threadIdx.x; c < slab_chunks; c += blockDim.x) {
    const u32x4 a = load16_stream(ks + c);
    const u32x4 bq = load16_stream(vs + c);
    store16_stream(kd + c, a);
    store16_stream(vd + c, bq);
  }
}

__global__ __launch_bounds__(256) void kv_copy_whole_blocks_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                                   int64_t src_block_chunks, int64_t dst_block_chunks,
                                                                   int32_t run_chunks, int32_t src_blocks, int32_t dst_blocks,
                                                                   const int32_t* __restrict__ pairs) {
  // blockIdx.x: 4 KiB piece of the run (fastest, so that the pieces of one block are in flight together and
  // both streams stay inside a few DRAM pages); blockIdx.y: pair.  One 16-byte access per lane: workgroups this
  // small measured 14 % faster than one workgroup per 64 KiB block with eight loads in flight per lane.
  const int pair = blockIdx.y;
  const int64_t s = pairs[2 * pair], d = pairs[2 * pair + 1];
  if (s < 0 || s >= src_blocks || d < 0 || d >= dst_blocks) return;  // uniform per workgroup
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c < run_chunks) store16_stream(dst + d * dst_block_chunks + c, load16_stream(src + s * src_block_chunks + c));
}

}  // namespace pace_kv

using namespace pace_kv;

namespace pace_kv {
// Launches the block-wise append (n_tokens >= 8 per sequence, destination through the block table),
// rotating the keys on the way when rope is given.  Arguments are already checked.
int launch_block_append(const char* who, const pace_kv_pool_t* pool, const void* k_new, const void* v_new, int64_t stride_b,
                        int64_t stride_h, int64_t stride_t, int32_t batch, int32_t n_tokens, const int32_t* block_table,
                        int32_t table_stride, const int32_t* seq_lens, int32_t pos_offset, const RopeDev* rope,
                        hipStream_t stream) {
  PACE_REQUIRE(batch <= 65535 && pool->num_kv_heads <= 65535, "%s: batch / heads exceed grid limits", who);
  const AppendDest dest = {nullptr, block_table, seq_lens, table_stride, pos_offset, nullptr};
  const unsigned blocks_x = (unsigned)((n_tokens + PACE_KV_BLOCK_TOKENS - 1) / PACE_KV_BLOCK_TOKENS + 1);
  dim3 grid(blocks_x, pool->num_kv_heads, batch);
  const uint16_t* kq = static_cast<const uint16_t*>(k_new);
  const uint16_t* vq = static_cast<const uint16_t*>(v_new);
  const RopeDev none = {};
#define PACE_BLOCK_APPEND(DIM, R_)                                                                                        \
  hipLaunchKernelGGL((kv_append_block_kernel<DIM, R_>), grid, dim3(256), 0, stream, *pool, kq, vq, stride_b, stride_h, stride_t, \
                     n_tokens, dest, rope ? *rope : none)
  for_head_dim(pool->head_dim, [&](auto d) {
    constexpr int DIM = decltype(d)::value;
    if (rope) PACE_BLOCK_APPEND(DIM, true); else PACE_BLOCK_APPEND(DIM, false);
  });
#undef PACE_BLOCK_APPEND
  PACE_HIP_CHECK(hipGetLastError());
  return PACE_KV_OK;
}
}  // namespace pace_kv

static int run_append(const char* who, const pace_kv_pool_t* pool, const void* k_new, const void* v_new,
                      int64_t stride_b, int64_t stride_h, int64_t stride_t, int32_t batch, int32_t n_tokens,
                      const AppendDest& dest, bool paged, void* stream) {
  if (int rc = check_pool(pool, who, true)) return rc;
  PACE_REQUIRE(batch >= 0 && n_tokens >= 0, "%s: negative batch (%d) or n_tokens (%d)", who, batch, n_tokens);
  if (batch == 0 || n_tokens == 0) return PACE_KV_OK;
  PACE_REQUIRE(k_new && v_new, "%s: NULL input pointer", who);
  PACE_REQUIRE(aligned16(k_new) && aligned16(v_new), "%s: k_new / v_new must be 16-byte aligned", who);
  const int per16 = pool_is_f32(pool) ? 4 : 8;
  PACE_REQUIRE(stride_b % per16 == 0 && stride_h % per16 == 0 && stride_t % per16 == 0,
               "%s: input strides must be multiples of %d elements", who, per16);
  hipStream_t s_early = static_cast<hipStream_t>(stream);
  if (pool_is_f32(pool)) {
    const int64_t rows = (int64_t)batch * n_tokens * pool->num_kv_heads;
    PACE_REQUIRE(rows < (int64_t)1 << 31, "%s: too many rows (%lld)", who, (long long)rows);
    const int64_t threads = rows * (pool->head_dim / 4);
    PACE_REQUIRE((threads + 255) / 256 < (int64_t)1 << 31, "%s: grid too large", who);
    const dim3 grid((unsigned)((threads + 255) / 256));
    const float* k = static_cast<const float*>(k_new);
    const float* v = static_cast<const float*>(v_new);
    if (paged)
      hipLaunchKernelGGL(kv_append_f32_kernel<true>, grid, dim3(256), 0, s_early, *pool, k, v, stride_b, stride_h, stride_t, n_tokens,
                         (int32_t)rows, dest);
    else
      hipLaunchKernelGGL(kv_append_f32_kernel<false>, grid, dim3(256), 0, s_early, *pool, k, v, stride_b, stride_h, stride_t, n_tokens,
                         (int32_t)rows, dest);
    PACE_HIP_CHECK(hipGetLastError());
    return PACE_KV_OK;
  }
  if (paged && n_tokens >= 8 && !dest.offset_dev)  // enough tokens per sequence to fill slabs: one workgroup per destination block
    return launch_block_append(who, pool, k_new, v_new, stride_b, stride_h, stride_t, batch, n_tokens, dest.table,
                               dest.table_stride, dest.seq_lens, dest.pos_offset, nullptr, s_early);
  const int64_t rows = (int64_t)batch * n_tokens * pool->num_kv_heads;
  PACE_REQUIRE(rows < (int64_t)1 << 31, "%s: too many rows (%lld)", who, (long long)rows);
  const int chunks = pool->head_dim / 8;
  const int64_t threads = rows * chunks;
  PACE_REQUIRE((threads + 255) / 256 < (int64_t)1 << 31, "%s: grid too large", who);
  const unsigned grid = (unsigned)((threads + 255) / 256);
  const uint16_t* k = static_cast<const uint16_t*>(k_new);
  const uint16_t* v = static_cast<const uint16_t*>(v_new);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define PACE_LAUNCH_APPEND(DIM, PG)                                                                                  \
  hipLaunchKernelGGL((kv_append_kernel<DIM, PG>), dim3(grid), dim3(256), 0, s, *pool, k, v, stride_b, stride_h, stride_t, \
                     n_tokens, (int32_t)rows, dest)
  for_head_dim(pool->head_dim, [&](auto d) {
    constexpr int DIM = decltype(d)::value;
    if (paged) PACE_LAUNCH_APPEND(DIM, true); else PACE_LAUNCH_APPEND(DIM, false);
  });
#undef PACE_LAUNCH_APPEND
  PACE_HIP_CHECK(hipGetLastError());
  return PACE_KV_OK;
}

extern "C" int pace_kv_append(const pace_kv_pool_t* pool, const void* k_new, const void* v_new, int64_t stride_b,
                              int64_t stride_h, int64_t stride_t, int32_t batch, int32_t n_tokens,
                              const int64_t* slot_mapping, void* stream) {
  if (batch > 0 && n_tokens > 0) PACE_REQUIRE(slot_mapping != nullptr, "pace_kv_append: slot_mapping is NULL");
  AppendDest dest = {slot_mapping, nullptr, nullptr, 0, 0, nullptr};
  return run_append("pace_kv_append", pool, k_new, v_new, stride_b, stride_h, stride_t, batch, n_tokens, dest, false,
                    stream);
}

extern "C" int pace_kv_append_paged(const pace_kv_pool_t* pool, const void* k_new, const void* v_new, int64_t stride_b,
                                    int64_t stride_h, int64_t stride_t, int32_t batch, int32_t n_tokens,
                                    const int32_t* block_table, int32_t table_stride, const int32_t* seq_lens,
                                    int32_t pos_offset, void* stream) {
  if (batch > 0 && n_tokens > 0)
    PACE_REQUIRE(block_table != nullptr && seq_lens != nullptr && table_stride >= 1,
                 "pace_kv_append_paged: NULL block_table / seq_lens or bad table_stride");
  AppendDest dest = {nullptr, block_table, seq_lens, table_stride, pos_offset, nullptr};
  return run_append("pace_kv_append_paged", pool, k_new, v_new, stride_b, stride_h, stride_t, batch, n_tokens, dest, true,
                    stream);
}

extern "C" int pace_kv_append_paged_at(const pace_kv_pool_t* pool, const void* k_new, const void* v_new, int64_t stride_b,
                                       int64_t stride_h, int64_t stride_t, int32_t batch, int32_t n_tokens,
                                       const int32_t* block_table, int32_t table_stride, const int32_t* seq_lens,
                                       int32_t pos_offset, const int32_t* pos_offset_dev, void* stream) {
  if (batch > 0 && n_tokens > 0)
    PACE_REQUIRE(block_table != nullptr && seq_lens != nullptr && table_stride >= 1,
                 "pace_kv_append_paged_at: NULL block_table / seq_lens or bad table_stride");
  AppendDest dest = {nullptr, block_table, seq_lens, table_stride, pos_offset, pos_offset_dev};
  return run_append("pace_kv_append_paged_at", pool, k_new, v_new, stride_b, stride_h, stride_t, batch, n_tokens, dest, true,
                    stream);
}

static int run_gather(const char* who, const pace_kv_pool_t* pool, const int32_t* block_table, int32_t table_stride,
                      const int32_t* seq_lens, int32_t seq_len_bias, int32_t batch, int32_t n_rep, int32_t rows,
                      const GatherOut& out_in, bool packed, void* stream) {
  const GatherOut& out = out_in;
  if (int rc = check_pool(pool, who, true)) return rc;
  PACE_REQUIRE(batch >= 0 && rows >= 0 && n_rep >= 1, "%s: bad batch (%d), row count (%d) or n_rep (%d)", who, batch, rows, n_rep);
  if (batch == 0 || rows == 0) return PACE_KV_OK;
  PACE_REQUIRE(block_table && seq_lens && out.k && out.v, "%s: NULL pointer", who);
  PACE_REQUIRE(aligned16(out.k) && aligned16(out.v), "%s: outputs must be 16-byte aligned", who);
  const int per16 = pool_is_f32(pool) ? 4 : 8;
  PACE_REQUIRE(out.stride_b % per16 == 0 && out.stride_h % per16 == 0 && out.stride_t % per16 == 0 && out.stride_t >= pool->head_dim &&
                   out.stride_h >= pool->head_dim,
               "%s: output strides must be multiples of %d elements and hold a row of head_dim", who, per16);
  const int n_blocks = (rows + PACE_KV_BLOCK_TOKENS - 1) / PACE_KV_BLOCK_TOKENS;
  PACE_REQUIRE(table_stride >= 1, "%s: table_stride %d", who, table_stride);
  // the dense form puts heads and sequences on the grid's y and z axes; the packed form's grid is one-dimensional
  if (!packed) PACE_REQUIRE(batch <= 65535 && pool->num_kv_heads <= 65535, "%s: batch/heads exceed grid limits", who);
  dim3 grid(n_blocks, packed ? 1 : pool->num_kv_heads, packed ? 1 : batch);
  if (packed) {
    const int64_t entries = ((int64_t)out.total_rows / PACE_KV_BLOCK_TOKENS + batch) * pool->num_kv_heads;
    PACE_REQUIRE(entries < ((int64_t)1 << 31), "%s: grid too large", who);
    grid = dim3((unsigned)entries, 1, 1);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (pool_is_f32(pool)) {
    if (packed)
      hipLaunchKernelGGL(kv_gather_f32_kernel<true>, grid, dim3(256), 0, s, *pool, block_table, table_stride, seq_lens, seq_len_bias, n_rep,
                         out);
    else
      hipLaunchKernelGGL(kv_gather_f32_kernel<false>, grid, dim3(256), 0, s, *pool, block_table, table_stride, seq_lens, seq_len_bias, n_rep,
                         out);
    PACE_HIP_CHECK(hipGetLastError());
    return PACE_KV_OK;
  }
  for_head_dim(pool->head_dim, [&](auto d) {
    constexpr int DIM = decltype(d)::value;
    if (packed)
      hipLaunchKernelGGL((kv_gather_kernel<DIM, true>), grid, dim3(256), 0, s, *pool, block_table, table_stride, seq_lens,
                         seq_len_bias, n_rep, out);
    else
      hipLaunchKernelGGL((kv_gather_kernel<DIM, false>), grid, dim3(256), 0, s, *pool, block_table, table_stride, seq_lens,
                         seq_len_bias, n_rep, out);
  });
  PACE_HIP_CHECK(hipGetLastError());
  return PACE_KV_OK;
}

extern "C" int pace_kv_gather(const pace_kv_pool_t* pool, const int32_t* block_table, int32_t table_stride,
                              const int32_t* seq_lens, int32_t seq_len_bias, int32_t batch, int32_t n_rep, void* k_out, void* v_out,
                              int64_t out_stride_b, int64_t out_stride_h, int32_t out_len, int32_t zero_fill, void* stream) {
  PACE_REQUIRE(pool != nullptr, "pace_kv_gather: pool is NULL");
  GatherOut out = {static_cast<uint16_t*>(k_out), static_cast<uint16_t*>(v_out), nullptr, out_stride_b, out_stride_h,
                   pool->head_dim, out_len, zero_fill ? 1 : 0, batch, 0, 0};
  return run_gather("pace_kv_gather", pool, block_table, table_stride, seq_lens, seq_len_bias, batch, n_rep, out_len, out, false,
                    stream);
}

extern "C" int pace_kv_gather_live(const pace_kv_pool_t* pool, const int32_t* block_table, int32_t table_stride,
                                   const int32_t* seq_lens, int32_t seq_len_bias, const int32_t* cu_seqlens, int32_t batch,
                                   int32_t n_rep, void* k_out, void* v_out, int64_t out_stride_b, int64_t out_stride_h,
                                   int32_t out_len, int32_t total_tokens, void* stream) {
  PACE_REQUIRE(pool != nullptr, "pace_kv_gather_live: pool is NULL");
  if (batch > 0 && total_tokens > 0) PACE_REQUIRE(cu_seqlens != nullptr, "pace_kv_gather_live: cu_seqlens is NULL");
  PACE_REQUIRE(out_len >= 0 && total_tokens >= 0, "pace_kv_gather_live: negative out_len (%d) or total_tokens (%d)", out_len, total_tokens);
  if (out_len == 0) return PACE_KV_OK;
  GatherOut out = {static_cast<uint16_t*>(k_out), static_cast<uint16_t*>(v_out), cu_seqlens, out_stride_b, out_stride_h,
                   pool->head_dim, out_len, 0, batch, total_tokens, 1};
  return run_gather("pace_kv_gather_live", pool, block_table, table_stride, seq_lens, seq_len_bias, batch, n_rep, total_tokens, out, true,
                    stream);
}

extern "C" int pace_kv_gather_packed(const pace_kv_pool_t* pool, const int32_t* block_table, int32_t table_stride,
                                     const int32_t* seq_lens, int32_t seq_len_bias, const int32_t* cu_seqlens, int32_t batch,
                                     int32_t n_rep, void* k_out, void* v_out, int32_t total_tokens, void* stream) {
  PACE_REQUIRE(pool != nullptr, "pace_kv_gather_packed: pool is NULL");
  if (batch > 0 && total_tokens > 0) PACE_REQUIRE(cu_seqlens != nullptr, "pace_kv_gather_packed: cu_seqlens is NULL");
  PACE_REQUIRE(n_rep >= 1, "pace_kv_gather_packed: bad n_rep (%d)", n_rep);
  const int64_t row = (int64_t)pool->num_kv_heads * n_rep * pool->head_dim;  // one token, every output head
  GatherOut out = {static_cast<uint16_t*>(k_out), static_cast<uint16_t*>(v_out), cu_seqlens, 0, pool->head_dim, row, 0, 0, batch, total_tokens, 0};
  return run_gather("pace_kv_gather_packed", pool, block_table, table_stride, seq_lens, seq_len_bias, batch, n_rep, total_tokens,
                    out, true, stream);
}

// A slab is copied verbatim, so a pool of fp32 rows is described to the copy kernels in their 2-byte units.
static pace_kv_pool_t in_halfwords(const pace_kv_pool_t* p) {
  pace_kv_pool_t q = *p;
  if (pool_is_f32(p)) {
    q.k_block_stride *= 2, q.k_head_stride *= 2, q.v_block_stride *= 2, q.v_head_stride *= 2, q.head_dim *= 2;
    q.elem_bytes = 2;
  }
  return q;
}

extern "C" int pace_kv_copy_blocks(const pace_kv_pool_t* src_in, const pace_kv_pool_t* dst_in, const int32_t* pairs,
                                   int32_t n_pairs, void* stream) {
  if (int rc = check_pool(src_in, "pace_kv_copy_blocks(src)", true)) return rc;
  if (int rc = check_pool(dst_in, "pace_kv_copy_blocks(dst)", true)) return rc;
  PACE_REQUIRE(pool_is_f32(src_in) == pool_is_f32(dst_in), "pace_kv_copy_blocks: src and dst pools differ in element type");
  const pace_kv_pool_t src_h = in_halfwords(src_in), dst_h = in_halfwords(dst_in);
  const pace_kv_pool_t* src = &src_h;
  const pace_kv_pool_t* dst = &dst_h;
  PACE_REQUIRE(src->head_dim == dst->head_dim && src->num_kv_heads == dst->num_kv_heads,
               "pace_kv_copy_blocks: src and dst pools differ in head_dim or num_kv_heads");
  PACE_REQUIRE(n_pairs >= 0, "pace_kv_copy_blocks: negative n_pairs");
  if (n_pairs == 0) return PACE_KV_OK;
  PACE_REQUIRE(pairs != nullptr, "pace_kv_copy_blocks: pairs is NULL");
  hipStream_t s = static_cast<hipStream_t>(stream);
  // A pool laid out [block][head][K|V][16 * head_dim] holds a block as one contiguous run: move it whole.
  const int64_t slab = (int64_t)PACE_KV_BLOCK_TOKENS * src->head_dim;
  auto one_run = [&](const pace_kv_pool_t* p) {
    return static_cast<const uint16_t*>(p->v) == static_cast<const uint16_t*>(p->k) + slab && p->k_head_stride == 2 * slab &&
           p->v_head_stride == 2 * slab && p->k_block_stride == p->v_block_stride &&
           p->k_block_stride >= (int64_t)p->num_kv_heads * 2 * slab;
  };
  if (one_run(src) && one_run(dst)) {
    const int64_t run_chunks = (int64_t)src->num_kv_heads * 2 * slab / 8;
    PACE_REQUIRE(n_pairs <= 65535 * 32, "pace_kv_copy_blocks: too many pairs (%d)", n_pairs);
    // grid.y holds at most 65535 pairs per launch
    for (int32_t p0 = 0; p0 < n_pairs; p0 += 65535) {
      const int32_t n = n_pairs - p0 < 65535 ? n_pairs - p0 : 65535;
      hipLaunchKernelGGL(kv_copy_whole_blocks_kernel, dim3((unsigned)((run_chunks + 255) / 256), n), dim3(256), 0, s,
                         static_cast<const u32x4*>(src->k), static_cast<u32x4*>(dst->k), src->k_block_stride / 8,
                         dst->k_block_stride / 8, (int32_t)run_chunks, src->num_blocks, dst->num_blocks, pairs + 2 * (int64_t)p0);
    }
  } else {
    PACE_REQUIRE(n_pairs <= 65535 * 32, "pace_kv_copy_blocks: too many pairs (%d)", n_pairs);
    for (int32_t p0 = 0; p0 < n_pairs; p0 += 65535) {
      const int32_t n = n_pairs - p0 < 65535 ? n_pairs - p0 : 65535;
      hipLaunchKernelGGL(kv_copy_blocks_kernel, dim3(src->num_kv_heads, n), dim3(256), 0, s, *src, *dst, pairs + 2 * (int64_t)p0);
    }
  }
  PACE_HIP_CHECK(hipGetLastError());
  return PACE_KV_OK;
}

extern "C" int32_t pace_kv_compact_blocks(const pace_kv_pool_t* const* pools, int32_t n_pools, const int32_t* block_table,
                                          int32_t table_stride, const int64_t* n_blocks, int32_t batch, const uint8_t* is_free,
                                          int32_t* moves_host, int32_t capacity, int32_t* moves_dev, void* stream) {
  const char* who = "pace_kv_compact_blocks";
  if (!pools || n_pools < 1 || !moves_host || !moves_dev) {
    set_error("%s: NULL pools / moves_host / moves_dev or no pool", who);
    return PACE_KV_EINVAL;
  }
  for (int i = 0; i < n_pools; ++i) {
    if (int rc = check_pool(pools[i], who, true)) return rc;
    if (pools[i]->num_blocks != pools[0]->num_blocks) {
      set_error("%s: pools of one table must have the same number of blocks", who);
      return PACE_KV_EINVAL;
    }
  }
  // the plan reads the table only (apply = 0): the caller rewrites it with pace_kv_apply_moves while the copies run
  // (from the allocator's free flags when the caller has them: a pass over one byte per block instead of the table)
  const int32_t n = is_free ? pace_kv_plan_compaction_flags(is_free, pools[0]->num_blocks, moves_host, capacity)
                            : pace_kv_plan_compaction(const_cast<int32_t*>(block_table), table_stride, n_blocks, batch,
                                                      pools[0]->num_blocks, moves_host, capacity, 0, nullptr);
  if (n <= 0) return n;
  if (hipMemcpyAsync(moves_dev, moves_host, (size_t)n * 2 * sizeof(int32_t), hipMemcpyHostToDevice, static_cast<hipStream_t>(stream)) !=
      hipSuccess) {
    set_error("%s: upload of the moves failed: %s", who, hipGetErrorString(hipGetLastError()));
    return PACE_KV_EHIP;
  }
  for (int i = 0; i < n_pools; ++i)
    if (int rc = pace_kv_copy_blocks(pools[i], pools[i], moves_dev, n, stream)) return rc;
  return n;
}
