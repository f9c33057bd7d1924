// Paged scaled-dot-product attention for gfx950 (decode and multi-token verify).
//
// Work decomposition: one 64-lane wavefront per (sequence, KV head, context
// partition, group of query rows).  The query rows of one KV head are the
// q_len * n_rep (token, GQA replica) pairs; up to 16*NQT of them ride along in
// registers, so K and V are read from HBM once per KV head, not once per query
// head.  A second small kernel merges the partitions of a sequence.
//
// The inner step (one 32-token unit on the matrix cores) is in attn_core.h.
#include <algorithm>
#include <mutex>
#include <type_traits>
#include <vector>

#include "attn_core.h"

namespace pace_kv {

// 16 bytes of the cache.  ONCE (a kernel template argument: with both forms behind a run-time branch
// the compiler merges the two arms and the hint is lost): nothing will read them again in this launch
// (one group of query rows per sequence and KV head), so they are fetched non-temporally and leave the caches to what is
// re-used; the decode step runs 10 % faster for it (186 -> 169 us).  With several row groups
// (prefill) the later ones find K / V in L2 and the plain load is the faster one (778 vs 623 TFLOP/s).
template <bool ONCE>
__device__ __forceinline__ u32x4 load_kv16(const uint16_t* p) {
  if (ONCE) return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return *reinterpret_cast<const u32x4*>(p);
}

// Issue the 16-byte loads of one 32-token unit.  ids: pool block ids of the
// unit's two blocks (wave-uniform).
template <int D, bool ONCE>
__device__ __forceinline__ void load_unit_k(UnitRegs<D>& r, const PagedAttnParams& p, int kvh, int idA, int idB, int n, int g) {
  // K: lane (n, g) supplies token 8*(n/4) + 4*tile + n%4 of the unit, i.e. token slot
  // n % 8 of slab tile `tile` in block A (n < 8) or B; dims 32*kk + 8g .. +8 are dim
  // chunk 4*kk + g.  A 16-lane quarter (fixed g) reads 128 contiguous bytes per block.
  const int64_t offA = (int64_t)idA * p.k_bs, offB = (int64_t)idB * p.k_bs;  // wave-uniform products
  const uint16_t* kp = p.kpool + ((n >= 8) ? offB : offA) + (int64_t)kvh * p.k_hs + g * 64 + (n & 7) * 8;
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int kk = 0; kk < D / 32; ++kk) r.k[t][kk] = load_kv16<ONCE>(kp + t * (D * 8) + kk * 256);
}
template <int D, bool ONCE>
__device__ __forceinline__ void load_unit_v(UnitRegs<D>& r, const PagedAttnParams& p, int kvh, int idA, int idB, int n, int g) {
  // V: lane (n, g) supplies dim 16j + n, tokens 8g..8g+7 of the unit: token half g & 1
  // of block A (g < 2) or B.  A 16-lane quarter reads 256 contiguous bytes.
  const int64_t voffA = (int64_t)idA * p.v_bs, voffB = (int64_t)idB * p.v_bs;
  const uint16_t* vp = p.vpool + ((g >= 2) ? voffB : voffA) + (int64_t)kvh * p.v_hs + ((g & 1) * 16 + n) * 8;
#pragma unroll
  for (int j = 0; j < D / 16; ++j) r.v[j] = load_kv16<ONCE>(vp + j * 256);
}
template <int D, bool ONCE>
__device__ __forceinline__ void load_unit(UnitRegs<D>& r, const PagedAttnParams& p, int kvh, int idA, int idB, int n, int g) {
  load_unit_k<D, ONCE>(r, p, kvh, idA, idB, n, g);
  load_unit_v<D, ONCE>(r, p, kvh, idA, idB, n, g);
}

// The "unit" made of the step's new tokens, read straight from the caller's [T][D] rows
// (token idx of the unit = new token idx; tokens >= n_new are zero and get masked).
template <int D, bool ROPE>
__device__ __forceinline__ void load_new_unit(UnitRegs<D>& r, const PagedAttnParams& p, int b, int kvh, int pos0, int n_new, int n,
                                              int g) {
  const uint16_t* kb = p.k_new + (int64_t)b * p.n_sb + (int64_t)kvh * p.n_sh;
  const uint16_t* vb = p.v_new + (int64_t)b * p.n_sb + (int64_t)kvh * p.n_sh;
  const u32x4 zero = {0u, 0u, 0u, 0u};
  // Every load is issued unconditionally from a clamped (valid) token row and masked afterwards:
  // without branches around them the loads all go out before the first wait.
  u32x4 tab[ROPE ? 2 : 1][kRopeTabRegs<D>];
  bool live[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int idx = 8 * (n >> 2) + 4 * t + (n & 3);
    live[t] = idx < n_new;
    const int tok = live[t] ? idx : 0;
    if (ROPE) rope_fetch_row<D>(p.rope, rope_row(p.rope, b, tok, pos0 + tok), g, tab[t]);
    const uint16_t* row = kb + (int64_t)tok * p.n_st + 8 * g;
#pragma unroll
    for (int kk = 0; kk < D / 32; ++kk) r.k[t][kk] = *reinterpret_cast<const u32x4*>(row + kk * 32);
  }
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    if (ROPE) rope_apply_row<D>(p.rope, tab[t], r.k[t]);
#pragma unroll
    for (int kk = 0; kk < D / 32; ++kk) r.k[t][kk] = live[t] ? r.k[t][kk] : zero;
  }
  // V: 2-byte gathers (dim 16j + n of tokens 8g..8g+7), four dim tiles (32 loads) per round.
  constexpr int JR = 4;
#pragma unroll
  for (int j0 = 0; j0 < D / 16; j0 += JR) {
    uint32_t vals[JR][8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int tok = 8 * g + e;
      const uint16_t* row = vb + (int64_t)(tok < n_new ? tok : 0) * p.n_st + n;
#pragma unroll
      for (int j = 0; j < JR; ++j) vals[j][e] = row[16 * (j0 + j)];
    }
#pragma unroll
    for (int j = 0; j < JR; ++j) {
      u32x4 w = zero;
#pragma unroll
      for (int e = 0; e < 8; ++e) w[e >> 1] |= (8 * g + e < n_new ? vals[j][e] : 0u) << (16 * (e & 1));
      r.v[j0 + j] = w;
    }
  }
}

// Write the step's new tokens of (b, kvh) into their pool slots (positions pool_end ..).
// With ROPE a lane moves two 8-dim chunks of a token (the two halves of eight rotation
// pairs) and rotates the key chunks on the way; without, one chunk.
template <int D, bool ROPE>
__device__ __forceinline__ void write_new_tokens(const PagedAttnParams& p, int b, int kvh, int pool_end, int n_new, int lane) {
  constexpr int PER_ROW = ROPE ? D / 16 : D / 8;
  for (int item = lane; item < n_new * PER_ROW; item += 64) {
    const int idx = item / PER_ROW, ci = item % PER_ROW;
    const int pos = pool_end + idx;
    const int jb = pos / PACE_KV_BLOCK_TOKENS;
    if (jb >= p.table_stride) continue;
    const int64_t blk = p.table[(int64_t)b * p.table_stride + jb];
    if (blk < 0 || blk >= p.num_blocks) continue;  // never write outside the pool
    const int64_t src = (int64_t)b * p.n_sb + (int64_t)kvh * p.n_sh + (int64_t)idx * p.n_st;
    uint16_t* kslab = const_cast<uint16_t*>(p.kpool) + blk * p.k_bs + (int64_t)kvh * p.k_hs;
    uint16_t* vslab = const_cast<uint16_t*>(p.vpool) + blk * p.v_bs + (int64_t)kvh * p.v_hs;
    if (ROPE) {
      int ca, cb;
      rope_chunk_pair(p.rope, ci, ca, cb);
      u32x4 ka = *reinterpret_cast<const u32x4*>(p.k_new + src + ca * 8);
      u32x4 kb = *reinterpret_cast<const u32x4*>(p.k_new + src + cb * 8);
      const u32x4 va = *reinterpret_cast<const u32x4*>(p.v_new + src + ca * 8);
      const u32x4 vb = *reinterpret_cast<const u32x4*>(p.v_new + src + cb * 8);
      rope_rotate_chunks(p.rope, rope_row(p.rope, b, idx, pos), ci, ka, kb);
      store_kv_chunk<D>(kslab, vslab, pos % PACE_KV_BLOCK_TOKENS, ca, ka, va);
      store_kv_chunk<D>(kslab, vslab, pos % PACE_KV_BLOCK_TOKENS, cb, kb, vb);
    } else {
      const u32x4 kv = *reinterpret_cast<const u32x4*>(p.k_new + src + ci * 8);
      const u32x4 vv = *reinterpret_cast<const u32x4*>(p.v_new + src + ci * 8);
      store_kv_chunk<D>(kslab, vslab, pos % PACE_KV_BLOCK_TOKENS, ci, kv, vv);
    }
  }
}


// Pool block ids of 64 consecutive units of one wave (128 blocks), one id per lane in each of two
// registers, fetched with one load each and read back with v_readlane (no memory access inside the
// unit loop; a wave that walks more than 64 units fetches the next 128 ids when it gets there).
struct WaveBlockIds {
  int lo, hi;
  __device__ __forceinline__ int get(int idx) const {  // idx is wave-uniform, 0..127
    return idx < 64 ? __builtin_amdgcn_readlane(lo, idx) : __builtin_amdgcn_readlane(hi, idx - 64);
  }
};

// The waves of a workgroup take the partition's 32-token units in turn: wave w walks units w, w + NW,
// w + 2 NW, ...  Ids of this wave's units first .. first + 63: lane l holds block (l & 1) of unit
// first + l / 2 in `lo`, of unit first + 32 + l / 2 in `hi`.  The loads depend on nothing but the
// partition's first token, not on the sequence's length: a table row exists in full, entries past the
// live blocks are clamped into the pool and belong to units that are never walked.
template <int NW>
__device__ __forceinline__ WaveBlockIds load_block_ids(const PagedAttnParams& p, int b, int part_begin, int wave, int first,
                                                       int lane) {
  const int32_t* row = p.table + (int64_t)b * p.table_stride;
  const int at = part_begin / PACE_KV_BLOCK_TOKENS + 2 * (wave + NW * (first + (lane >> 1))) + (lane & 1);
  const int at2 = at + 2 * NW * 32;
  const int lo = at < p.table_stride ? row[at] : 0;
  const int hi = at2 < p.table_stride ? row[at2] : 0;
  WaveBlockIds ids;
  // never read outside the pool, whatever the table holds
  ids.lo = lo < 0 ? 0 : (lo >= p.num_blocks ? p.num_blocks - 1 : lo);
  ids.hi = hi < 0 ? 0 : (hi >= p.num_blocks ? p.num_blocks - 1 : hi);
  return ids;
}

// NW waves per workgroup split the partition's units among themselves and merge their
// softmax states through LDS.  OCC is the least number of waves that must fit on one SIMD
// (caps the register budget) and OCC_MAX the most that may share it; latency is hidden by
// the other resident waves, each wave keeps one unit (16 KiB) in flight.  With FUSED, the last
// wave of a sequence's last partition also takes the step's new tokens as one more unit (attends
// to them from the caller's buffers and stores them into the pool); a workgroup of its own shape
// for that (a fifth wave) measured 4 % slower on the decode step than this.  With ROPE, query rows
// and the new keys are rotated on their way in.
template <int D, int NQT, bool HAS_MASK, int NW, int OCC, int OCC_MAX, bool FUSED, bool ROPE, bool ONCE>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(OCC, OCC_MAX))) void paged_attn_kernel(
    const PagedAttnParams p) {
  constexpr int KK = D / 32;
  constexpr int MT = D / 16;
  constexpr int NWT = NW;  // waves per work item
  // One slot of 16*NQT query rows per sender of the first merge round.  Kept as small as the
  // shape allows: LDS is one of the limits on how many workgroups share a compute unit.
  constexpr int MERGE_SLOTS = NWT / 2 > 0 ? NWT / 2 : 1;
  static_assert(MERGE_SLOTS * 16 * NQT <= 128, "LDS merge buffer holds at most 128 query rows");
  __shared__ float merge_buf[MERGE_SLOTS * 16 * NQT * (D + 2)];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 15, g = lane >> 4;
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);  // the same number, known to be uniform
  // Linear work index -> (KV head, row group, sequence, partition); KV head fastest.
  // (32-bit arithmetic: the host keeps total_items below 2^31.)
  const uint32_t L = blockIdx.x;
  const bool active_item = L < (uint32_t)p.total_items;
  const bool listed = p.items != nullptr;
  int kvh = 0, part = 0, b = 0, qg = 0;
  int d_parts = 1, d_begin = 0, d_end = -1, d_first = 0, pre_a = 0, pre_b = 0;
  if (active_item) {
    kvh = (int)(L % (uint32_t)p.num_kv_heads);
    const uint32_t rest = L / (uint32_t)p.num_kv_heads;
    if (listed) {
      // Work list: one 64-byte descriptor per (sequence, partition), in scheduling order.  It carries
      // everything the first loads need -- the partition's token range and the pool blocks of its first
      // units -- so a wave's first K / V loads wait for this one read only; the sequence's length, the
      // rest of its block ids and the query rows are fetched while those loads travel.
      qg = (int)(rest % (uint32_t)p.n_qgroups);
      const int32_t* d = p.items + (int64_t)(rest / (uint32_t)p.n_qgroups) * PACE_ATTN_WORK_INTS;
      b = min(max(d[0], 0), p.batch - 1), part = min(max(d[1], 0), p.max_parts - 1);
      d_parts = d[2], d_begin = max(d[3], 0) & ~31, d_end = d[4], d_first = d[5];
      pre_a = d[8 + 2 * wave_s], pre_b = d[9 + 2 * wave_s];
    } else {
      part = (int)(rest % (uint32_t)p.max_parts);
      const uint32_t bz = rest / (uint32_t)p.max_parts;
      b = (int)(bz / (uint32_t)p.n_qgroups), qg = (int)(bz % (uint32_t)p.n_qgroups);
    }
  }
  UnitRegs<D> buf;
  bool pre = false;  // buf already holds (or is being sent) this wave's first unit
  if (listed && wave_s < d_first) {
    pre_a = pre_a < 0 ? 0 : (pre_a >= p.num_blocks ? p.num_blocks - 1 : pre_a);  // never read outside the pool
    pre_b = pre_b < 0 ? 0 : (pre_b >= p.num_blocks ? p.num_blocks - 1 : pre_b);
    load_unit<D, ONCE>(buf, p, kvh, pre_a, pre_b, n, g);
    pre = true;
  }
  const int len_b = p.seq_lens[b] + p.len_bias + (p.len_bias_dev ? *p.len_bias_dev : 0);
  // An idle slot (past the end of the work, or a partition this sequence does not have) runs
  // as an empty sequence without query rows: it loads and stores nothing but keeps the barriers.
  const int n_parts_b = listed ? max(1, d_parts) : partition_count(len_b, p.part_tokens);
  const bool active = active_item && part < n_parts_b;
  const int len = active ? len_b : 0;
  const int n_parts = active ? n_parts_b : 1;
  if (!active) part = 0;
  const int start = p.kv_start ? p.kv_start[b] : 0;
  // Token range of the partition.  Listed: as the host cut it (the last partition of a sequence is open
  // ended: it grows with the sequence).  Otherwise: equal shares of the current length.
  int part_begin, part_end;
  if (listed) {
    part_begin = d_begin, part_end = d_end < 0 ? 0x7fffffff : d_end;
  } else {
    const int P = partition_size(len, n_parts);
    part_begin = part * P, part_end = part_begin + P;
  }
  // Tokens [pool_end, len) are this step's new tokens when the append is fused in.
  const int n_new = FUSED ? min(p.n_new, len) : 0;
  const int pool_end = len - n_new;
  const int S = p.q_len, R = active ? S * p.n_rep : 0;
  // Causal rows read tokens <= len - S + s: nothing past the limit of the group's last row is
  // needed, which halves the work of a prefill chunk (whole units are skipped, not masked).
  const int last_row = min(R, (qg + 1) * NQT * 16) - 1;
  const int group_end = (p.causal && last_row >= 0) ? len - S + last_row / p.n_rep + 1 : len;

  // Query rows of this wave (B operand of the first product) and per-row limits.
  u32x4 qreg[NQT][KK];
  u32x4 qtab[ROPE ? NQT : 1][kRopeTabRegs<D>];  // cos / sin of the rows: fetched here, applied once the first unit is on its way
  RowState<D, NQT> st;
  int row_s[NQT], row_h[NQT];
  int min_limit = 0x7fffffff;
  // Table rows first: a position id that has to be loaded is waited for before any other load
  // of the wave is in flight.
  int tab_row[ROPE ? NQT : 1];
  if (ROPE) {
#pragma unroll
    for (int qt = 0; qt < NQT; ++qt) {
      const int r = (qg * NQT + qt) * 16 + n;
      const int s = r < R ? r / p.n_rep : 0;
      tab_row[qt] = rope_row(p.rope, b, s, len - S + s);
    }
  }
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    const int r = (qg * NQT + qt) * 16 + n;
    const bool valid = r < R;
    const int s = valid ? r / p.n_rep : 0;
    const int hq = kvh * p.n_rep + (valid ? r % p.n_rep : 0);
    row_s[qt] = s;
    row_h[qt] = hq;
    st.limit[qt] = valid ? (p.causal ? len - S + s : len - 1) : -1;
    if (valid) min_limit = min(min_limit, st.limit[qt]);
    st.mask_off[qt] = HAS_MASK ? (int64_t)b * p.m_sb + (int64_t)s * p.m_ss : 0;
    st.m[qt] = kNegInf, st.m_top[qt] = kNegInf, st.m_neg[qt] = 0.f;
    st.l[qt] = 0.f;
    const uint16_t* qp = p.q + (int64_t)b * p.q_sb + (int64_t)hq * p.q_sh + (int64_t)s * p.q_ss + 8 * g;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      u32x4 z = {0u, 0u, 0u, 0u};
      qreg[qt][kk] = valid ? *reinterpret_cast<const u32x4*>(qp + kk * 32) : z;
    }
    if (ROPE) {
      if (valid) {
        rope_fetch_row<D>(p.rope, tab_row[qt], g, qtab[qt]);
      } else {
#pragma unroll
        for (int kk = 0; kk < kRopeTabRegs<D>; ++kk) qtab[qt][kk] = u32x4{0u, 0u, 0u, 0u};
      }
    }
#pragma unroll
    for (int j = 0; j < MT; ++j) st.o[qt][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  // Rows of padding lanes must not relax the "whole unit readable" test.
  min_limit = min(min_limit, __shfl_xor(min_limit, 1, 64));
  min_limit = min(min_limit, __shfl_xor(min_limit, 2, 64));
  min_limit = min(min_limit, __shfl_xor(min_limit, 4, 64));
  min_limit = min(min_limit, __shfl_xor(min_limit, 8, 64));
  // the same in every lane (rows do not depend on the lane quarter): make that known, so that the
  // full / partial decision per unit is a scalar branch
  min_limit = __builtin_amdgcn_readfirstlane(min_limit);

  int tok_end = min(min(pool_end, part_end), group_end);
  if (HAS_MASK && p.row_last) {
    // Explicit mask on a prefill-sized launch: nothing past the last column any row of the group can
    // use is needed (the diagonal of a causal mask) -- provided every row has a real score somewhere,
    // so that the columns left out weigh exactly 0; a row masked everywhere must end as the average of
    // V and keeps every column.  All waves of the workgroup hold the same rows and decide alike.
    int last = -1;
    bool real = true;
#pragma unroll
    for (int qt = 0; qt < NQT; ++qt) {
      if (st.limit[qt] >= 0) {
        const int v = p.row_last[(int64_t)b * S + row_s[qt]];
        last = max(last, v);
        real = real && v >= 0;
      }
    }
#pragma unroll
    for (int o = 1; o < 64; o *= 2) last = max(last, __shfl_xor(last, o, 64));
    if (__all(real)) tok_end = min(tok_end, __builtin_amdgcn_readfirstlane(last) + 1);
  }
  // This wave's share of the partition's 32-token units: units wave, wave + NW, wave + 2 NW, ...
  const int part_units = max(0, (tok_end - part_begin + 31) / 32);
  const int n_units = part_units > wave ? (part_units - wave + NW - 1) / NW : 0;

  WaveBlockIds ids = load_block_ids<NW>(p, b, part_begin, wave, 0, lane);
  // a first unit the descriptor did not name (or no descriptor): its blocks come from the table like all others
  if (!pre && n_units > 0) load_unit<D, ONCE>(buf, p, kvh, ids.get(0), ids.get(1), n, g);
  if (ROPE) {
    // rotate the query rows while the first unit travels (padding rows stay zero)
#pragma unroll
    for (int qt = 0; qt < NQT; ++qt) rope_apply_row<D>(p.rope, qtab[qt], qreg[qt]);
  }
  MaskRegs<NQT> mregs;
  for (int uu = 0; uu < n_units; ++uu) {
    if (uu != 0 && (uu & 63) == 0) ids = load_block_ids<NW>(p, b, part_begin, wave, uu, lane);
    const int t0 = part_begin + 32 * (wave + NW * uu);  // a multiple of 32: partitions begin on whole units
    // The mask values go first, so that they are back before the unit's K / V: the wait for those
    // is then the only one, as without a mask.
    if (HAS_MASK) load_mask_regs<NQT>(mregs, p, st.mask_off, t0, g);
    if (uu > 0) load_unit<D, ONCE>(buf, p, kvh, ids.get(2 * (uu & 63)), ids.get(2 * (uu & 63) + 1), n, g);  // the first one is on its way
    const bool full = (t0 + 32 <= tok_end) && (t0 + 31 <= min_limit) && (t0 >= start);
    compute_unit<D, NQT, HAS_MASK>(buf, qreg, st, p, t0, tok_end, start, full, g, mregs);
  }
  if (FUSED) {
    // The step's new tokens: the last wave of the sequence's last partition takes them after its
    // share of the pool (attends to them from the caller's buffers and stores them into the pool).
    if (wave == NW - 1 && n_new > 0 && part == n_parts - 1) {
      load_new_unit<D, ROPE>(buf, p, b, kvh, pool_end, n_new, n, g);
      MaskRegs<NQT> mnew;
      if (HAS_MASK) load_mask_regs<NQT>(mnew, p, st.mask_off, pool_end, g);  // pool_end is any position
      if (qg == 0) write_new_tokens<D, ROPE>(p, b, kvh, pool_end, n_new, lane);
      compute_unit<D, NQT, HAS_MASK>(buf, qreg, st, p, pool_end, len, start, false, g, mnew);
    }
  }

  finish_rows<D, NQT, HAS_MASK>(st, p);  // row sums over the lanes of a row, running max in log2 units

  // Pairwise merge of the waves' states through LDS (fixed order: deterministic).
  if (NWT > 1) {
    constexpr int ROW_F = D + 2;
    constexpr int SLOT_F = 16 * NQT * ROW_F;
#pragma unroll
    for (int stride = 1; stride < NWT; stride *= 2) {
      const int slot = wave / (2 * stride);
      const bool sender = (wave & (2 * stride - 1)) == stride;
      const bool receiver = (wave & (2 * stride - 1)) == 0 && wave + stride < NWT;
      if (sender) {
#pragma unroll
        for (int qt = 0; qt < NQT; ++qt) {
          float* rowp = merge_buf + slot * SLOT_F + (qt * 16 + n) * ROW_F;
#pragma unroll
          for (int j = 0; j < MT; ++j) {
            rowp[16 * j + 4 * g + 0] = st.o[qt][j][0];
            rowp[16 * j + 4 * g + 1] = st.o[qt][j][1];
            rowp[16 * j + 4 * g + 2] = st.o[qt][j][2];
            rowp[16 * j + 4 * g + 3] = st.o[qt][j][3];
          }
          if (g == 0) {
            rowp[D] = st.m[qt];
            rowp[D + 1] = st.l[qt];
          }
        }
      }
      __syncthreads();
      if (receiver) {
#pragma unroll
        for (int qt = 0; qt < NQT; ++qt) {
          const float* rowp = merge_buf + slot * SLOT_F + (qt * 16 + n) * ROW_F;
          const float m_b = rowp[D], l_b = rowp[D + 1];
          const float m_new = fmaxf(st.m[qt], m_b);
          const float m_use = (m_new == kNegInf) ? 0.f : m_new;
          const float wa = __builtin_amdgcn_exp2f(st.m[qt] - m_use);
          const float wb = __builtin_amdgcn_exp2f(m_b - m_use);
#pragma unroll
          for (int j = 0; j < MT; ++j) {
#pragma unroll
            for (int i = 0; i < 4; ++i) st.o[qt][j][i] = st.o[qt][j][i] * wa + rowp[16 * j + 4 * g + i] * wb;
          }
          st.l[qt] = st.l[qt] * wa + l_b * wb;
          st.m[qt] = m_new;
        }
      }
      __syncthreads();
    }
    if (wave != 0) return;
  }

#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    const int r = (qg * NQT + qt) * 16 + n;
    const float l = st.l[qt];
    if (r >= R) continue;
    if (p.max_parts == 1) {
      const float inv = l > 0.f ? 1.0f / l : 0.f;
      uint16_t* op = p.out + (int64_t)b * p.o_sb + (int64_t)row_h[qt] * p.o_sh + (int64_t)row_s[qt] * p.o_ss + 4 * g;
#pragma unroll
      for (int j = 0; j < MT; ++j) {
        u32x2 w;
        w[0] = pack_bf16x2(st.o[qt][j][0] * inv, st.o[qt][j][1] * inv);
        w[1] = pack_bf16x2(st.o[qt][j][2] * inv, st.o[qt][j][3] * inv);
        *reinterpret_cast<u32x2*>(op + 16 * j) = w;
      }
    } else {
      const int64_t row = ((int64_t)b * p.num_q_heads + row_h[qt]) * S + row_s[qt];
      float* po = p.part_o + (row * p.max_parts + part) * D + 4 * g;
#pragma unroll
      for (int j = 0; j < MT; ++j) *reinterpret_cast<f32x4*>(po + 16 * j) = st.o[qt][j];
      if (g == 0) {
        float* ml = p.part_ml + (row * p.max_parts + part) * 2;
        ml[0] = st.m[qt];
        ml[1] = l;
      }
    }
  }
}

// ---------------------------------------------------------------------------------
// Prefill-sized launches without a mask tensor: many groups of query rows read the same K / V.  Here the four
// waves of a workgroup own 16*NQT query rows each and walk the context together.  Every 32-token unit is fetched
// once per workgroup, straight from the pool into LDS (global_load_lds_dwordx4: no registers in between), one
// unit ahead of its use, and each wave reads its operands back lane for lane: the pool's slab order is the
// operand order, so lane l takes the 16 bytes lane l would have loaded from the pool.  Against one load of the
// whole unit per wave (paged_attn_kernel) this moves a quarter of the bytes through the vector memory path and
// takes the K / V latency out of the wave's cycle.  No merge: a row's softmax state never leaves its wave.
// With HAS_MASK the additive mask tensor decides what a row reads; its values for the next unit are fetched a unit
// ahead, like K / V, and where the per-row summary of the mask is at hand (row_last) the wave and the workgroup stop
// at the last column their rows can use -- the diagonal of a causal mask.
// Not fused with the append, one partition per sequence; the host falls back to paged_attn_kernel otherwise.
// ---------------------------------------------------------------------------------
template <int D, int NQT, bool ROPE, bool HAS_MASK>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 8))) void paged_prefill_kernel(const PagedAttnParams p) {
  constexpr int KK = D / 32, MT = D / 16, NW = 4;
  constexpr int UNIT_CHUNKS = 2 * MT * 64;  // 16-byte pieces of a unit: MT loads of K, then MT loads of V, 64 lanes each
  constexpr int PER = MT / NW;              // K loads and V loads each wave sends per unit
  static_assert(MT % NW == 0, "a unit's loads must divide over the four waves");
  typedef const __attribute__((address_space(1))) void* gptr;
  typedef __attribute__((address_space(3))) void* lptr;
  __shared__ __attribute__((aligned(16))) u32x4 stage[2][UNIT_CHUNKS];
  const int lane = threadIdx.x & 63, n = lane & 15, g = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // Linear index -> (KV head, row group, sequence); KV head fastest: workgroups are dealt to the eight XCDs in
  // turn, so that one head's K / V stay in one L2.  Row groups from the last to the first: under the causal
  // limit the later rows read more, and the longest workgroups should not be the last to start.
  const uint32_t item = blockIdx.x;
  const int kvh = (int)(item % (uint32_t)p.num_kv_heads);
  const uint32_t rest = item / (uint32_t)p.num_kv_heads;
  const int rg = p.n_qgroups - 1 - (int)(rest % (uint32_t)p.n_qgroups);
  const int b = min((int)(rest / (uint32_t)p.n_qgroups), p.batch - 1);
  const int len = max(p.seq_lens[b] + p.len_bias + (p.len_bias_dev ? *p.len_bias_dev : 0), 0);
  int lo_tok = p.kv_start ? min(max(p.kv_start[b], 0), len) : 0;
  bool plain = false;  // HAS_MASK: the mask lines of the workgroup's rows are known to be plain (see row_first)
  const int S = p.q_len, R = S * p.n_rep;
  const int tile0 = (rg * NW + wave) * NQT;  // first query tile of this wave

  u32x4 qreg[NQT][KK];
  u32x4 qtab[ROPE ? NQT : 1][kRopeTabRegs<D>];
  RowState<D, NQT> st;
  int row_s[NQT], row_h[NQT];
  int min_limit = 0x7fffffff;
  int tab_row[ROPE ? NQT : 1];
  if (ROPE) {
#pragma unroll
    for (int qt = 0; qt < NQT; ++qt) {
      const int r = (tile0 + qt) * 16 + n;
      const int s = r < R ? r / p.n_rep : 0;
      tab_row[qt] = rope_row(p.rope, b, s, len - S + s);
    }
  }
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    const int r = (tile0 + qt) * 16 + n;
    const bool valid = r < R;
    const int s = valid ? r / p.n_rep : 0;
    const int hq = kvh * p.n_rep + (valid ? r % p.n_rep : 0);
    row_s[qt] = s;
    row_h[qt] = hq;
    st.limit[qt] = valid ? (p.causal ? len - S + s : len - 1) : -1;
    if (valid) min_limit = min(min_limit, st.limit[qt]);
    st.mask_off[qt] = HAS_MASK ? (int64_t)b * p.m_sb + (int64_t)s * p.m_ss : 0;
    st.m[qt] = kNegInf, st.m_top[qt] = kNegInf, st.m_neg[qt] = 0.f;
    st.l[qt] = 0.f;
    const uint16_t* qp = p.q + (int64_t)b * p.q_sb + (int64_t)hq * p.q_sh + (int64_t)s * p.q_ss + 8 * g;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      const u32x4 z = {0u, 0u, 0u, 0u};
      qreg[qt][kk] = valid ? *reinterpret_cast<const u32x4*>(qp + kk * 32) : z;
    }
    if (ROPE) {
      if (valid) {
        rope_fetch_row<D>(p.rope, tab_row[qt], g, qtab[qt]);
      } else {
#pragma unroll
        for (int kk = 0; kk < kRopeTabRegs<D>; ++kk) qtab[qt][kk] = u32x4{0u, 0u, 0u, 0u};
      }
    }
#pragma unroll
    for (int j = 0; j < MT; ++j) st.o[qt][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  min_limit = min(min_limit, __shfl_xor(min_limit, 1, 64));
  min_limit = min(min_limit, __shfl_xor(min_limit, 2, 64));
  min_limit = min(min_limit, __shfl_xor(min_limit, 4, 64));
  min_limit = min(min_limit, __shfl_xor(min_limit, 8, 64));
  min_limit = __builtin_amdgcn_readfirstlane(min_limit);

  // Where the workgroup stops (the causal limit of its last row) and where this wave does (of its own last row).
  const int wg_last = min(R, (rg + 1) * NW * NQT * 16) - 1;  // >= 0: the grid has no empty row group
  const int wave_last = min(R, (tile0 + NQT) * 16) - 1;      // < tile0 * 16: this wave has no rows
  const bool wave_rows = tile0 * 16 < R;
  int wg_end = p.causal ? min(len, len - S + wg_last / p.n_rep + 1) : len;
  int wave_end = !wave_rows ? 0 : (p.causal ? min(len, len - S + wave_last / p.n_rep + 1) : len);
  if (HAS_MASK && p.row_last) {
    // Nothing past the last column any row can use is needed -- provided every row has a real score somewhere, so
    // that the columns left out weigh exactly 0; a row masked everywhere ends as the average of V and keeps every
    // column.  Once over this wave's rows, once over the workgroup's (each lane looks up NQT of its 64 * NQT rows).
    const int32_t* last_of = p.row_last + (int64_t)b * S;
    int mine = -1, ours = -1;
    bool mine_real = true, ours_real = true;
#pragma unroll
    for (int qt = 0; qt < NQT; ++qt) {
      if (st.limit[qt] >= 0) {
        const int v = last_of[row_s[qt]];
        mine = max(mine, v), mine_real = mine_real && v >= 0;
      }
      const int r = rg * (NW * NQT * 16) + qt * 64 + lane;
      if (r < R) {
        const int v = last_of[r / p.n_rep];
        ours = max(ours, v), ours_real = ours_real && v >= 0;
      }
    }
#pragma unroll
    for (int o = 1; o < 64; o *= 2) mine = max(mine, __shfl_xor(mine, o, 64)), ours = max(ours, __shfl_xor(ours, o, 64));
    if (__all(mine_real)) wave_end = min(wave_end, __builtin_amdgcn_readfirstlane(mine) + 1);
    if (__all(ours_real)) wg_end = min(wg_end, __builtin_amdgcn_readfirstlane(ours) + 1);
    wave_end = min(wave_end, wg_end);
    if (p.row_first) {
      // Every row of the workgroup plain, and from the same first column (a causal mask, padded or not): the rows
      // are then walked as rows without a mask tensor -- first column, own last column -- and the mask is not read.
      const int32_t* first_of = p.row_first + (int64_t)b * S;
      int f_min = 0x7fffffff, f_max = -1;
#pragma unroll
      for (int qt = 0; qt < NQT; ++qt) {
        const int r = rg * (NW * NQT * 16) + qt * 64 + lane;
        if (r < R) {
          const int f = first_of[r / p.n_rep];
          f_min = min(f_min, f), f_max = max(f_max, f);
        }
      }
#pragma unroll
      for (int o = 1; o < 64; o *= 2) f_min = min(f_min, __shfl_xor(f_min, o, 64)), f_max = max(f_max, __shfl_xor(f_max, o, 64));
      f_min = __builtin_amdgcn_readfirstlane(f_min), f_max = __builtin_amdgcn_readfirstlane(f_max);
      plain = f_min >= 0 && f_min == f_max;  // (-1 marks a row that is not plain)
      if (plain) {
        lo_tok = max(lo_tok, f_min);
        min_limit = 0x7fffffff;
#pragma unroll
        for (int qt = 0; qt < NQT; ++qt) {
          if (st.limit[qt] >= 0) {
            st.limit[qt] = min(st.limit[qt], last_of[row_s[qt]]);
            min_limit = min(min_limit, st.limit[qt]);
          }
        }
#pragma unroll
        for (int o = 1; o < 64; o *= 2) min_limit = min(min_limit, __shfl_xor(min_limit, o, 64));
        min_limit = __builtin_amdgcn_readfirstlane(min_limit);
      }
    }
  }
  const int start = lo_tok;                      // first token any row of the workgroup reads
  const int u0 = start / 32;                     // units before the first readable token are not walked
  const int u_end = max((wg_end + 31) / 32, u0);  // workgroup-uniform: every wave makes the same trips

  WaveBlockIds ids = load_block_ids<1>(p, b, 0, 0, u0, lane);
  int ids_first = u0;
  // This wave's share of a unit's loads, sent into stage `s`: K loads wave*PER .. and V loads wave*PER .. of the
  // unit's MT each.  A wave's K loads lie 512 bytes apart inside one token tile (PER divides KK), and so do its
  // V loads: one address per operand and unit, the rest are immediate offsets.  What does not depend on the unit
  // is added up here, once; the unit adds its blocks' offsets, which are wave-uniform products.
  static_assert(KK % PER == 0, "a wave's K loads must stay inside one token tile");
  const int k_first = wave * PER;
  const uint16_t* const k_lane = p.kpool + (int64_t)kvh * p.k_hs + g * 64 + (n & 7) * 8 + (k_first / KK) * (D * 8) + (k_first % KK) * 256;
  const uint16_t* const v_lane = p.vpool + (int64_t)kvh * p.v_hs + ((g & 1) * 16 + n) * 8 + k_first * 256;
  auto send = [&](int u, int s) {
    const int rel = u - ids_first;
    const int ia = ids.get(2 * rel), ib = ids.get(2 * rel + 1);
    const int64_t ka = (int64_t)ia * p.k_bs, kb = (int64_t)ib * p.k_bs, va = (int64_t)ia * p.v_bs, vb = (int64_t)ib * p.v_bs;
    const uint16_t* kp = k_lane + (n >= 8 ? kb : ka);
    const uint16_t* vp = v_lane + (g >= 2 ? vb : va);
    // The instruction's immediate offset (a literal for the builtin) moves the address in the pool and the
    // address in LDS alike: the second load of an operand is 512 bytes on in the pool but 1024 in the stage, so
    // its LDS base makes up the difference.
    static_assert(PER == 1 || PER == 2, "one or two loads per operand and wave");
    u32x4* const ks = &stage[s][k_first * 64];
    u32x4* const vs = &stage[s][(MT + k_first) * 64];
    __builtin_amdgcn_global_load_lds((gptr)kp, (lptr)ks, 16, 0, 0);
    if (PER == 2) __builtin_amdgcn_global_load_lds((gptr)kp, (lptr)(ks + 32), 16, 512, 0);
    __builtin_amdgcn_global_load_lds((gptr)vp, (lptr)vs, 16, 0, 0);
    if (PER == 2) __builtin_amdgcn_global_load_lds((gptr)vp, (lptr)(vs + 32), 16, 512, 0);
  };
  if (u0 < u_end) send(u0, 0);
  if (ROPE) {
#pragma unroll
    for (int qt = 0; qt < NQT; ++qt) rope_apply_row<D>(p.rope, qtab[qt], qreg[qt]);
  }
  // Unit u is complete in its stage once every wave's loads are back (each waits for its own, then the barrier);
  // the same barrier says that every wave has taken unit u - 1 out of the other stage, which the next loads reuse.
  auto turn = [&](int u) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (u + 1 < u_end) {
      if (u + 1 - ids_first == 64) {
        ids = load_block_ids<1>(p, b, 0, 0, u + 1, lane);
        ids_first = u + 1;
      }
      send(u + 1, ((u - u0) & 1) ^ 1);
    }
  };
  // The units every row of the wave reads in full lie in one stretch: from the first readable token to the
  // causal limit of the wave's first row.  Before and after it, masked units; past the wave's own last row,
  // only the loads and the barriers.  One loop per kind: with the masked and the whole form of the inner step in
  // one loop body the accumulators have two paths through it, and the register allocator spills them.
  const int u_mine = min(max((wave_end + 31) / 32, u0), u_end);
  const int u_whole_end = min(max((min(wave_end - 1, min_limit) + 1) / 32, u0), u_mine);
  const int u_whole_begin = min((start + 31) / 32, u_whole_end);
  // Mask values travel a unit ahead of their use, as K / V do: `coming` holds those of the next unit this wave walks.
  MaskRegs<NQT> coming;
  auto walk = [&](int from, int to, auto whole, auto masked) {
    constexpr bool MASKED = decltype(masked)::value;
    for (int u = from; u < to; ++u) {
      turn(u);
      const int s = (u - u0) & 1, t0 = 32 * u;
      MaskRegs<NQT> mregs;
      if (MASKED) {
        mregs = coming;
        if (u + 1 < u_mine) load_mask_regs<NQT>(coming, p, st.mask_off, t0 + 32, g);
      }
      UnitRegs<D> buf;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int kk = 0; kk < KK; ++kk) buf.k[t][kk] = stage[s][(t * KK + kk) * 64 + lane];
#pragma unroll
      for (int j = 0; j < MT; ++j) buf.v[j] = stage[s][(MT + j) * 64 + lane];
      compute_unit_impl<D, NQT, MASKED, decltype(whole)::value>(buf, qreg, st, p, t0, wave_end, start, g, mregs);
    }
  };
  bool by_mask = false;
  if constexpr (HAS_MASK) by_mask = !plain;
  if (by_mask) {
    if constexpr (HAS_MASK) {
      if (u0 < u_mine) load_mask_regs<NQT>(coming, p, st.mask_off, 32 * u0, g);
      walk(u0, u_whole_begin, std::false_type{}, std::true_type{});
      walk(u_whole_begin, u_whole_end, std::true_type{}, std::true_type{});
      walk(u_whole_end, u_mine, std::false_type{}, std::true_type{});
    }
  } else {
    walk(u0, u_whole_begin, std::false_type{}, std::false_type{});
    walk(u_whole_begin, u_whole_end, std::true_type{}, std::false_type{});
    walk(u_whole_end, u_mine, std::false_type{}, std::false_type{});
  }
  for (int u = u_mine; u < u_end; ++u) turn(u);
  // (the running maximum is in units of the scores the walk used: scaled with a mask, raw without)
  if (by_mask) finish_rows<D, NQT, true>(st, p);
  else finish_rows<D, NQT, false>(st, p);
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    const int r = (tile0 + qt) * 16 + n;
    if (r >= R) continue;
    const float l = st.l[qt];
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    uint16_t* op = p.out + (int64_t)b * p.o_sb + (int64_t)row_h[qt] * p.o_sh + (int64_t)row_s[qt] * p.o_ss + 4 * g;
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      u32x2 w;
      w[0] = pack_bf16x2(st.o[qt][j][0] * inv, st.o[qt][j][1] * inv);
      w[1] = pack_bf16x2(st.o[qt][j][2] * inv, st.o[qt][j][3] * inv);
      *reinterpret_cast<u32x2*>(op + 16 * j) = w;
    }
  }
}

// One wave per (sequence, query token): the last column of the row's mask line, among those the
// row can read ([kv_start, len) and inside the mask), that holds a value above the floor; -1 if none.
// With it a workgroup knows where its rows stop needing the context -- the diagonal of a causal mask
// -- and whether every row has a real score at all, without walking the mask itself.
// first_out (optional): the first such column if the line is plain -- exactly 0 on every column from there to the
// last one, which then are all above the floor -- else -1.
__global__ __launch_bounds__(64) void mask_row_last_kernel(const PagedAttnParams p, int32_t* out, int32_t* first_out) {
  const int row = blockIdx.x, S = p.q_len, b = row / S, s = row % S, lane = threadIdx.x;
  const int len = p.seq_lens[b] + p.len_bias + (p.len_bias_dev ? *p.len_bias_dev : 0);
  const int start = p.kv_start ? p.kv_start[b] : 0;
  int last, first;
  mask_line_summary(p.mask, p.mask_is_f32 != 0, (int64_t)b * p.m_sb + (int64_t)s * p.m_ss, start, min(len, p.mask_len), lane, last, first);
  if (lane == 0) {
    out[row] = last;
    if (first_out) first_out[row] = first;
  }
}

// Merge the partitions of one query row: out = sum_p 2^(m_p - M) o_p / sum_p 2^(m_p - M) l_p.
template <int D>
__global__ __launch_bounds__(64) void paged_attn_merge_kernel(const PagedAttnParams p) {
  const int64_t row = blockIdx.x;  // (b, hq, s)
  const int S = p.q_len;
  const int s = (int)(row % S);
  const int hq = (int)((row / S) % p.num_q_heads);
  const int b = (int)(row / ((int64_t)S * p.num_q_heads));
  int n_parts;
  if (p.seq_parts) {
    n_parts = p.seq_parts[b];
  } else {
    const int len = p.seq_lens[b] + p.len_bias + (p.len_bias_dev ? *p.len_bias_dev : 0);
    n_parts = partition_count(len, p.part_tokens);
  }
  n_parts = min(max(n_parts, 1), p.max_parts);  // the workspace holds max_parts partials per row
  const float* ml = p.part_ml + row * p.max_parts * 2;
  const float* po = p.part_o + row * p.max_parts * D;
  float M = kNegInf;
  for (int i = 0; i < n_parts; ++i) M = fmaxf(M, ml[2 * i]);
  const float m_use = (M == kNegInf) ? 0.f : M;
  constexpr int PASSES = (D + 127) / 128;  // a lane owns the dim pairs 2 * lane + 128 * pass that exist
  float acc[PASSES][2];
#pragma unroll
  for (int e = 0; e < PASSES; ++e) acc[e][0] = acc[e][1] = 0.f;
  float L = 0.f;
  const int d0 = 2 * threadIdx.x;
  for (int i = 0; i < n_parts; ++i) {
    const float w = __builtin_amdgcn_exp2f(ml[2 * i] - m_use);
    L += w * ml[2 * i + 1];
#pragma unroll
    for (int e = 0; e < PASSES; ++e) {
      if (d0 + 128 * e < D) {
        const u32x2 v = *reinterpret_cast<const u32x2*>(po + (int64_t)i * D + d0 + 128 * e);
        acc[e][0] += w * __uint_as_float(v[0]);
        acc[e][1] += w * __uint_as_float(v[1]);
      }
    }
  }
  const float inv = L > 0.f ? 1.0f / L : 0.f;
  uint16_t* op = p.out + (int64_t)b * p.o_sb + (int64_t)hq * p.o_sh + (int64_t)s * p.o_ss + d0;
#pragma unroll
  for (int e = 0; e < PASSES; ++e)
    if (d0 + 128 * e < D) *reinterpret_cast<uint32_t*>(op + 128 * e) = pack_bf16x2(acc[e][0] * inv, acc[e][1] * inv);
}

// Launch shape per query-tile count: waves per workgroup and unit buffers per wave.
struct Shape {
  int nqt, nw, occ;
  int occ_max;  // most waves per SIMD (8: no limit)
};

// A launch with the append fused in has the shape of one without.
static Shape shape_for(int head_dim, int tiles, bool masked = false) {
  if (head_dim == 256) {
    // One unit is 32 KiB in 128 registers and a query tile's output 64 more: one wave per SIMD (it may
    // then use all 512 registers), and two tiles at most.  Two tiles' merge slots leave room in LDS for two
    // waves per workgroup only.
    return tiles <= 1 ? Shape{1, 2, 1, 8} : Shape{2, 2, 1, 8};
  }
  if (tiles <= 1) return Shape{1, 4, 2, 8};
  // An explicit mask costs eight more registers per tile (its values travel with the unit): no more
  // than two tiles per wave then (four tiles with a mask spilled and ran at half the speed).
  if (masked) return Shape{2, 4, 2, 8};
  // Two query tiles need about 230 registers: two waves per SIMD, eight per compute unit, that is
  // two workgroups of four waves.
  // Four tiles (64 query rows, one wave per SIMD) read K/V once for up to 64 rows, which pays
  // while the launch is bound by HBM (a verify step of a wide GQA group).  Beyond 64 rows K/V
  // are re-read per row group anyway and the launch is bound by the matrix cores and by the rate
  // at which operands reach them: three tiles per wave are the most that still leave two waves
  // per SIMD (one hides the other's softmax and load latency).  Measured on a 512-token prefill
  // chunk: 768 TFLOP/s with three tiles, 708 with two, 468 with four, 450 with one.
  if (tiles > 4) return Shape{3, 4, 2, 8};
  if (tiles == 2) return Shape{2, 4, 2, 8};
  return Shape{4, 2, 1, 8};
}

// Tokens one work item may cover: each wave holds at most 128 block ids.
static int max_partition(int nw) { return nw * 2048; }

// Largest partition any shape of this tile count can take (with a mask or without), so that one
// resolved value is valid for every launch of the same problem size.
static int partition_cap(int head_dim, int tiles) {
  const Shape a = shape_for(head_dim, tiles, false), b = shape_for(head_dim, tiles, true);
  return max_partition(a.nw < b.nw ? a.nw : b.nw);
}

static int resolve_partition(int32_t requested, int32_t max_seq_len, int32_t batch, int32_t num_kv_heads, int32_t rows,
                             int32_t head_dim) {
  const int tiles = (rows + 15) / 16;
  const Shape sh = shape_for(head_dim, tiles);
  const int granule = 128;
  if (requested > 0) return requested;
  // Enough workgroups to fill every compute unit with as many as fit (4 * occ waves each); a batch
  // that already does so is not split at all.
  const int64_t groups = (int64_t)batch * num_kv_heads * ((tiles + sh.nqt - 1) / sh.nqt);
  const int64_t slots = (int64_t)compute_units() * 4 * sh.occ / sh.nw;
  int64_t parts = (slots + groups - 1) / groups;
  if (parts < 1) parts = 1;
  int64_t per = ((int64_t)max_seq_len + parts - 1) / parts;
  per = (per + granule - 1) / granule * granule;
  if (per < granule) per = granule;
  if (per > partition_cap(head_dim, tiles)) per = partition_cap(head_dim, tiles);
  return (int)per;
}

// pace_paged_attn_kernel_name(): while this points at a buffer, launch() writes the name of the kernel
// instantiation it would start there instead of starting it.
static thread_local char* g_name_out = nullptr;
static thread_local size_t g_name_cap = 0;

template <int D, int NQT, int NW, int OCC, int OCC_MAX>
static void launch(const PagedAttnParams& p, bool has_mask, hipStream_t s) {
  const bool fused = p.n_new > 0;
  const unsigned blocks = (unsigned)p.total_items;
  // K / V are read once per launch when one group of query rows covers a sequence's rows: always with one
  // or four tiles per wave, never with three, either way with two.
#define PACE_GO1(M_, F_, R_, O_)                                                                                          \
  do {                                                                                                                    \
    if (g_name_out)                                                                                                       \
      snprintf(g_name_out, g_name_cap, "pace_kv::paged_attn_kernel<%d, %d, %s, %d, %d, %d, %s, %s, %s>", D, NQT, #M_, NW, OCC, \
               OCC_MAX, #F_, #R_, (O_) ? "true" : "false");                                                               \
    else                                                                                                                  \
      hipLaunchKernelGGL((paged_attn_kernel<D, NQT, M_, NW, OCC, OCC_MAX, F_, R_, O_>), dim3(blocks), dim3(64 * NW), 0, s, p); \
  } while (0)
#define PACE_GO(M_, F_, R_)                                                              \
  do {                                                                                   \
    if constexpr (NQT == 2) {                                                            \
      if (p.n_qgroups == 1) PACE_GO1(M_, F_, R_, true); else PACE_GO1(M_, F_, R_, false); \
    } else {                                                                             \
      PACE_GO1(M_, F_, R_, NQT != 3);                                                    \
    }                                                                                    \
  } while (0)
  if (p.rope.cos) {  // never together with an explicit mask (checked by the caller)
    if (fused) PACE_GO(false, true, true); else PACE_GO(false, false, true);
  } else if (has_mask) {
    if constexpr (NQT <= 2) {  // shape_for() never asks for more tiles with a mask
      if (fused) PACE_GO(true, true, false); else PACE_GO(true, false, false);
    }
  } else {
    if (fused) PACE_GO(false, true, false); else PACE_GO(false, false, false);
  }
#undef PACE_GO1
#undef PACE_GO
}

// The same merge for rows cut into many partitions (a few long sequences spread over the whole GPU): the loop above
// waits out a memory round trip per partition, twice.  Here a lane fetches the (max, sum) pair of partition
// base + lane, so 64 pairs arrive together, the partial outputs are fetched eight partitions at a time, and the
// four waves of the workgroup take those groups of eight in turn; wave 0 adds the four partial results in wave
// order.  (The sum is therefore taken in another order than above: same result to rounding, the same bits from
// call to call.)
template <int D>
__global__ __launch_bounds__(256) void paged_attn_merge_wide_kernel(const PagedAttnParams p) {
  constexpr int PASSES = (D + 127) / 128;  // a lane owns the dim pairs 2 * lane + 128 * pass that exist
  __shared__ float part_sum[3][64][2 * PASSES + 1];
  const int64_t row = blockIdx.x;  // (b, hq, s)
  const int S = p.q_len;
  const int s = (int)(row % S);
  const int hq = (int)((row / S) % p.num_q_heads);
  const int b = (int)(row / ((int64_t)S * p.num_q_heads));
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  int n_parts;
  if (p.seq_parts) {
    n_parts = p.seq_parts[b];
  } else {
    const int len = p.seq_lens[b] + p.len_bias + (p.len_bias_dev ? *p.len_bias_dev : 0);
    n_parts = partition_count(len, p.part_tokens);
  }
  n_parts = min(max(n_parts, 1), p.max_parts);  // the workspace holds max_parts partials per row
  const float* ml = p.part_ml + row * p.max_parts * 2;
  const float* po = p.part_o + row * p.max_parts * D;
  float M = kNegInf;
  for (int base = 0; base < n_parts; base += 64) {
    const float m_i = base + lane < n_parts ? ml[2 * (base + lane)] : kNegInf;
    M = fmaxf(M, m_i);
  }
#pragma unroll
  for (int o = 1; o < 64; o *= 2) M = fmaxf(M, __shfl_xor(M, o, 64));
  const float m_use = (M == kNegInf) ? 0.f : M;
  float acc[PASSES][2];
#pragma unroll
  for (int e = 0; e < PASSES; ++e) acc[e][0] = acc[e][1] = 0.f;
  float L = 0.f;
  const int d0 = 2 * lane;
  for (int base = 0; base < n_parts; base += 64) {
    const bool mine = base + lane < n_parts;
    const u32x2 pair = mine ? *reinterpret_cast<const u32x2*>(ml + 2 * (base + lane)) : u32x2{0xff800000u, 0u};
    const float w_mine = __builtin_amdgcn_exp2f(__uint_as_float(pair[0]) - m_use), l_mine = __uint_as_float(pair[1]);
    const int here = min(64, n_parts - base);
    for (int j0 = 8 * wave; j0 < here; j0 += 32) {
      u32x2 v[8][PASSES];
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int e = 0; e < PASSES; ++e) {
          v[j][e] = u32x2{0u, 0u};
          if (j0 + j < here && d0 + 128 * e < D) v[j][e] = *reinterpret_cast<const u32x2*>(po + (int64_t)(base + j0 + j) * D + d0 + 128 * e);
        }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (j0 + j < here) {  // uniform
          const float w = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(w_mine), j0 + j));
          const float l = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(l_mine), j0 + j));
          L += w * l;
#pragma unroll
          for (int e = 0; e < PASSES; ++e) {
            acc[e][0] += w * __uint_as_float(v[j][e][0]);
            acc[e][1] += w * __uint_as_float(v[j][e][1]);
          }
        }
      }
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int e = 0; e < PASSES; ++e) part_sum[wave - 1][lane][2 * e] = acc[e][0], part_sum[wave - 1][lane][2 * e + 1] = acc[e][1];
    part_sum[wave - 1][lane][2 * PASSES] = L;
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int w = 0; w < 3; ++w) {
#pragma unroll
    for (int e = 0; e < PASSES; ++e) acc[e][0] += part_sum[w][lane][2 * e], acc[e][1] += part_sum[w][lane][2 * e + 1];
    L += part_sum[w][lane][2 * PASSES];
  }
  const float inv = L > 0.f ? 1.0f / L : 0.f;
  uint16_t* op = p.out + (int64_t)b * p.o_sb + (int64_t)hq * p.o_sh + (int64_t)s * p.o_ss + d0;
#pragma unroll
  for (int e = 0; e < PASSES; ++e)
    if (d0 + 128 * e < D) *reinterpret_cast<uint32_t*>(op + 128 * e) = pack_bf16x2(acc[e][0] * inv, acc[e][1] * inv);
}
template <int D>
static bool launch_shape(const Shape& sh, const PagedAttnParams& p, bool has_mask, hipStream_t s) {
#define PACE_TRY(NQT_, NW_, OCC_, MAX_)                                          \
  if (sh.nqt == NQT_ && sh.nw == NW_ && sh.occ == OCC_ && sh.occ_max == MAX_) {     \
    launch<D, NQT_, NW_, OCC_, MAX_>(p, has_mask, s);                               \
    return true;                                                                    \
  }
  if constexpr (D == 256) {
    PACE_TRY(1, 2, 1, 8)
    PACE_TRY(2, 2, 1, 8)
  } else {
    PACE_TRY(1, 4, 2, 8)
    PACE_TRY(2, 4, 2, 8)
    PACE_TRY(3, 4, 2, 8)
    PACE_TRY(4, 2, 1, 8)
  }
#undef PACE_TRY
  return false;
}

// Query tiles per wave for paged_prefill_kernel (four waves per workgroup, two workgroups per compute unit), or 0
// when the launch should keep paged_attn_kernel: with few row groups the compute units are better filled by
// splitting the context over more workgroups, which only paged_attn_kernel does.  Measured with 512-token chunks of
// 32 Q / 8 KV heads: one sequence (a quarter of the GPU's workgroup slots) is 23 % faster here on 512 cached tokens
// and 23 % slower on 3584; from two sequences on this kernel wins at either length.
// Between two and three tiles the number of rounds the workgroups need decides: a row group of three tiles per
// wave takes 1.5 times as long as one of two, and a last round that is nearly empty costs as much as a full one.
static int prefill_tiles_per_wave(int head_dim, int tiles, int64_t pairs, int max_seq_len, bool masked) {
  if (head_dim != 64 && head_dim != 128) return 0;
  if (tiles < 8) return 0;
  const int64_t slots = (int64_t)compute_units() * 2;
  const int64_t least = max_seq_len <= 2048 ? slots / 4 : slots / 2;
  int best = 0;
  double best_cost = 0.;
  for (int nqt = masked ? 2 : 3; nqt >= 2; --nqt) {  // a mask's values take eight more registers per tile: two tiles then
    const int64_t groups = pairs * ((tiles + 4 * nqt - 1) / (4 * nqt));
    if (groups < least) continue;
    const double cost = (double)((groups + slots - 1) / slots) * nqt * (nqt == 2 ? 1.05 : 1.0);
    if (best == 0 || cost < best_cost) best = nqt, best_cost = cost;
  }
  return best;
}

template <int D>
static bool launch_prefill(int nqt, const PagedAttnParams& p, hipStream_t s) {
  if constexpr (D == 64 || D == 128) {
    const bool rope = p.rope.cos != nullptr, masked = p.mask != nullptr;  // never both (checked by the caller)
    if (g_name_out) {
      snprintf(g_name_out, g_name_cap, "pace_kv::paged_prefill_kernel<%d, %d, %s, %s>", D, nqt, rope ? "true" : "false",
               masked ? "true" : "false");
      return true;
    }
    const dim3 grid((unsigned)p.total_items), block(256);
    if (nqt == 3 && !masked) {
      if (rope) hipLaunchKernelGGL((paged_prefill_kernel<D, 3, true, false>), grid, block, 0, s, p);
      else hipLaunchKernelGGL((paged_prefill_kernel<D, 3, false, false>), grid, block, 0, s, p);
      return true;
    }
    if (nqt == 2) {
      if (masked) hipLaunchKernelGGL((paged_prefill_kernel<D, 2, false, true>), grid, block, 0, s, p);
      else if (rope) hipLaunchKernelGGL((paged_prefill_kernel<D, 2, true, false>), grid, block, 0, s, p);
      else hipLaunchKernelGGL((paged_prefill_kernel<D, 2, false, false>), grid, block, 0, s, p);
      return true;
    }
  }
  return false;
}

// Scratch of the entry point that allocates nothing: one array per GPU, in the library's own device image.
// In host code the array's name is only a stand-in; the address each device holds it at comes from
// hipGetSymbolAddress, once per device, and that address is what kernels and checks are given.
constexpr size_t kStaticScratchBytes = (size_t)PACE_PAGED_ATTN_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device (resolved on the first call there).
static int static_scratch(const char* who, void** out) {
  int dev = 0;
  PACE_HIP_CHECK(hipGetDevice(&dev));
  PACE_REQUIRE(dev >= 0 && dev < kMaxDevices, "%s: device ordinal %d out of range", who, dev);
  if (void* known = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE)) {  // every call after the first
    *out = known;
    return PACE_KV_OK;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    PACE_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    PACE_REQUIRE(ptr != nullptr, "%s: the scratch array has no device address", who);
    __atomic_store_n(&g_scratch_ptr[dev], ptr, __ATOMIC_RELEASE);
  }
  *out = g_scratch_ptr[dev];
  return PACE_KV_OK;
}

static int run_paged_attn(const pace_kv_pool_t* pool, const pace_paged_attn_args_t* a_in, void* stream, const char* who,
                          bool use_static_scratch = false) {
  PACE_REQUIRE(a_in != nullptr, "%s: args is NULL", who);
  pace_paged_attn_args_t a_copy = *a_in;
  // The array's address is looked up on the first attention call of any entry point on a device, not on the first
  // call of the entry point that uses it: a caller that captures pace_paged_attn_verify_static into a graph has run
  // a step eagerly before (any entry point will do), so the look-up never falls inside a capture.
  if (use_static_scratch) {
    void* static_ptr = nullptr;
    if (int rc = static_scratch(who, &static_ptr)) return rc;
    a_copy.workspace = static_ptr;
    a_copy.workspace_bytes = kStaticScratchBytes;
  }
  const pace_paged_attn_args_t* a = &a_copy;
  if (int rc = check_pool(pool, who, true)) return rc;
  PACE_REQUIRE(a->batch >= 0 && a->q_len >= 1 && a->num_q_heads >= 1, "%s: bad batch (%d), q_len (%d) or num_q_heads (%d)",
               who, a->batch, a->q_len, a->num_q_heads);
  if (a->batch == 0) return PACE_KV_OK;
  PACE_REQUIRE(a->q && a->out && a->block_table && a->seq_lens, "%s: NULL q / out / block_table / seq_lens", who);
  PACE_REQUIRE(a->num_q_heads % pool->num_kv_heads == 0, "%s: num_q_heads %d not a multiple of num_kv_heads %d", who,
               a->num_q_heads, pool->num_kv_heads);
  if (pool_is_f32(pool)) {
    // rows of fp32: the general kernel of the dense operator walks the block table (dense_attn.hip)
    PACE_REQUIRE(!a->rope, "%s: an fp32 pool takes no rotary embedding inside the attention launch", who);
    if (a->k_new || a->v_new) {
      PACE_REQUIRE(a->k_new && a->v_new, "%s: k_new and v_new must be given together", who);
      PACE_REQUIRE(a->n_new >= 1 && a->n_new <= 32, "%s: fused append takes 1..32 new tokens (got %d)", who, a->n_new);
      PACE_REQUIRE(aligned16(a->k_new) && aligned16(a->v_new) && (a->new_stride_b % 4) == 0 && (a->new_stride_h % 4) == 0 &&
                       (a->new_stride_t % 4) == 0,
                   "%s: k_new / v_new must be 16-byte aligned with strides that are multiples of 4 elements", who);
    }
    PACE_REQUIRE(aligned16(a->q) && aligned16(a->out) && (a->q_stride_b % 4) == 0 && (a->q_stride_h % 4) == 0 &&
                     (a->q_stride_s % 4) == 0 && (a->o_stride_b % 4) == 0 && (a->o_stride_h % 4) == 0 && (a->o_stride_s % 4) == 0,
                 "%s: q and out must be 16-byte aligned with strides that are multiples of 4 elements", who);
    PACE_REQUIRE(a->max_seq_len >= 0 && a->table_stride >= 1 && (int64_t)a->table_stride * PACE_KV_BLOCK_TOKENS >= a->max_seq_len,
                 "%s: block table row (%d blocks) cannot hold max_seq_len %d", who, a->table_stride, a->max_seq_len);
    PACE_REQUIRE(a->scale > 0.f && a->scale < __builtin_inff(), "%s: softmax scale must be positive and finite (got %g)", who,
                 (double)a->scale);
    if (a->mask)
      PACE_REQUIRE((a->mask_dtype == PACE_DTYPE_F32 || a->mask_dtype == PACE_DTYPE_BF16) && a->mask_len >= 0,
                   "%s: bad mask dtype %d or mask_len %d", who, a->mask_dtype, a->mask_len);
    if (g_name_out) {  // (pace_paged_attn_kernel_name: nothing is launched)
      const int H = pool->head_dim, hp = H <= 32 ? 32 : (H <= 64 ? 64 : (H <= 96 ? 96 : (H <= 128 ? 128 : 256)));
      snprintf(g_name_out, g_name_cap, "pace_kv::attn_paged_f32_kernel<%s, %d, %s, %s>",
               a->mask_dtype == PACE_DTYPE_F32 ? "float" : "unsigned short", hp, H == hp ? "true" : "false", a->k_new ? "true" : "false");
      return PACE_KV_OK;
    }
    return launch_paged_f32(pool, a, who, static_cast<hipStream_t>(stream));
  }
  PACE_REQUIRE(aligned16(a->q) && (a->q_stride_b % 8) == 0 && (a->q_stride_h % 8) == 0 && (a->q_stride_s % 8) == 0,
               "%s: q must be 16-byte aligned with strides that are multiples of 8 elements", who);
  PACE_REQUIRE((reinterpret_cast<uintptr_t>(a->out) & 7u) == 0 && (a->o_stride_b % 4) == 0 && (a->o_stride_h % 4) == 0 &&
                   (a->o_stride_s % 4) == 0,
               "%s: out must be 8-byte aligned with strides that are multiples of 4 elements", who);
  PACE_REQUIRE(a->max_seq_len >= 0 && a->table_stride >= 1, "%s: bad max_seq_len (%d) or table_stride (%d)", who,
               a->max_seq_len, a->table_stride);
  PACE_REQUIRE((int64_t)a->table_stride * PACE_KV_BLOCK_TOKENS >= a->max_seq_len,
               "%s: block table row (%d blocks) cannot hold max_seq_len %d", who, a->table_stride, a->max_seq_len);
  PACE_REQUIRE(a->scale > 0.f && a->scale < __builtin_inff(), "%s: softmax scale must be positive and finite (got %g)", who,
               (double)a->scale);
  if (a->mask) {
    PACE_REQUIRE(a->mask_dtype == PACE_DTYPE_F32 || a->mask_dtype == PACE_DTYPE_BF16, "%s: bad mask dtype %d", who,
                 a->mask_dtype);
    PACE_REQUIRE(a->mask_len >= 0, "%s: negative mask_len", who);
  }
  if (a->k_new || a->v_new) {
    PACE_REQUIRE(a->k_new && a->v_new, "%s: k_new and v_new must be given together", who);
    PACE_REQUIRE(a->n_new >= 1 && a->n_new <= 32, "%s: fused append takes 1..32 new tokens (got %d)", who, a->n_new);
    PACE_REQUIRE(aligned16(a->k_new) && aligned16(a->v_new) && (a->new_stride_b % 8) == 0 && (a->new_stride_h % 8) == 0 &&
                     (a->new_stride_t % 8) == 0,
                 "%s: k_new / v_new must be 16-byte aligned with strides that are multiples of 8 elements", who);
  }
  RopeDev rope_dev = {};
  if (a->rope) {
    if (int rc = make_rope_dev(a->rope, pool->head_dim, false, who, &rope_dev)) return rc;
    PACE_REQUIRE(rope_dev.rot == pool->head_dim, "%s: rotary_dim %d must equal head_dim %d when rope rides in the attention launch",
                 who, rope_dev.rot, pool->head_dim);
    PACE_REQUIRE(a->mask == nullptr, "%s: rope in the attention launch cannot be combined with an explicit mask", who);
    PACE_REQUIRE(!a->k_new || a->n_new == a->q_len, "%s: with rope, the fused append takes n_new == q_len (got %d, %d)", who,
                 a->n_new, a->q_len);
  }
  if (!g_name_out && !use_static_scratch) {  // (the arguments are in order: this call will launch)
    void* unused = nullptr;
    (void)static_scratch(who, &unused);  // a failure here only matters to the entry point that uses the array
  }
  const int n_rep = a->num_q_heads / pool->num_kv_heads;
  const int rows = a->q_len * n_rep;
  const int tiles = (rows + 15) / 16;
  const Shape sh = shape_for(pool->head_dim, tiles, a->mask != nullptr);
  const int part = resolve_partition(a->partition_tokens, a->max_seq_len, a->batch, pool->num_kv_heads, rows, pool->head_dim);
  PACE_REQUIRE(part % 32 == 0 && part >= 32, "%s: partition_tokens %d must be a positive multiple of 32", who, part);
  int max_parts = a->max_seq_len > 0 ? (a->max_seq_len + part - 1) / part : 1;
  if (a->work_items || a->seq_parts) {
    PACE_REQUIRE(a->work_items != nullptr && a->seq_parts != nullptr && a->max_parts >= 1 && a->n_work_items >= 1,
                 "%s: a work list comes with seq_parts, max_parts (the largest entry of seq_parts) and n_work_items; see "
                 "pace_paged_attn_plan",
                 who);
    max_parts = a->max_parts;
  }

  // Many row groups per KV head, no fused append: the cooperative kernel, which takes every sequence
  // in one piece -- unless the caller asked for a split (an explicit partition_tokens, or a work list that has one).
  int prefill_nqt = !a->k_new ? prefill_tiles_per_wave(pool->head_dim, tiles, (int64_t)a->batch * pool->num_kv_heads, a->max_seq_len, a->mask != nullptr) : 0;
  if (prefill_nqt) {
    if (a->work_items ? max_parts != 1 : (a->partition_tokens > 0 && max_parts != 1)) prefill_nqt = 0;
    else max_parts = 1;
  }

  PagedAttnParams p;
  p.q = static_cast<const uint16_t*>(a->q);
  p.q_sb = a->q_stride_b, p.q_sh = a->q_stride_h, p.q_ss = a->q_stride_s;
  p.out = static_cast<uint16_t*>(a->out);
  p.o_sb = a->o_stride_b, p.o_sh = a->o_stride_h, p.o_ss = a->o_stride_s;
  p.kpool = static_cast<const uint16_t*>(pool->k);
  p.vpool = static_cast<const uint16_t*>(pool->v);
  p.k_bs = pool->k_block_stride, p.k_hs = pool->k_head_stride;
  p.v_bs = pool->v_block_stride, p.v_hs = pool->v_head_stride;
  p.num_blocks = pool->num_blocks;
  p.table = a->block_table, p.table_stride = a->table_stride;
  p.seq_lens = a->seq_lens, p.len_bias = a->seq_len_bias, p.len_bias_dev = a->seq_len_bias_ptr, p.kv_start = a->kv_start;
  p.mask = a->mask, p.mask_is_f32 = a->mask_dtype == PACE_DTYPE_F32, p.mask_len = a->mask_len;
  p.m_sb = a->mask_stride_b, p.m_ss = a->mask_stride_s;
  p.n_rep = n_rep, p.q_len = a->q_len, p.num_q_heads = a->num_q_heads, p.batch = a->batch;
  p.causal = a->causal;
  p.part_tokens = part, p.max_parts = max_parts;
  p.scale_log2 = a->scale * kLog2e;
  p.scale = a->scale;
  p.part_o = nullptr, p.part_ml = nullptr;
  p.k_new = static_cast<const uint16_t*>(a->k_new), p.v_new = static_cast<const uint16_t*>(a->v_new);
  p.n_sb = a->new_stride_b, p.n_sh = a->new_stride_h, p.n_st = a->new_stride_t;
  p.n_new = a->k_new ? a->n_new : 0;
  p.n_qgroups = (tiles + sh.nqt - 1) / sh.nqt;
  p.rope = rope_dev;

  if (max_parts > 1) {
    const size_t rows_total = (size_t)a->batch * a->num_q_heads * a->q_len;
    const size_t need = rows_total * max_parts * (pool->head_dim + 2) * sizeof(float);
    if (use_static_scratch)
      PACE_REQUIRE(need <= kStaticScratchBytes,
                   "%s: this launch needs %zu bytes of scratch, the static buffer holds %zu; use pace_paged_attn_verify with a "
                   "workspace of that size",
                   who, need, kStaticScratchBytes);
    PACE_REQUIRE(a->workspace != nullptr && a->workspace_bytes >= need,
                 "%s: workspace too small (%zu bytes given, %zu needed)", who, a->workspace_bytes, need);
    PACE_REQUIRE(aligned16(a->workspace), "%s: workspace must be 16-byte aligned", who);
    p.part_o = static_cast<float*>(a->workspace);
    p.part_ml = p.part_o + rows_total * max_parts * pool->head_dim;
  }
  p.row_last = nullptr, p.row_first = nullptr;
  int32_t* row_last = nullptr;
  int32_t* row_first = nullptr;
  if (a->mask && rows > 64) {
    // room behind the partials for the per-row summary, one int per (sequence, query token)?  (pace_paged_attn_workspace_bytes*
    // asks for it; a caller that sized its workspace otherwise simply goes without)
    const size_t part_bytes = max_parts > 1 ? (size_t)a->batch * a->num_q_heads * a->q_len * max_parts * (pool->head_dim + 2) * sizeof(float) : 0;
    const size_t at = (part_bytes + 15) & ~(size_t)15;
    const size_t per_array = (size_t)a->batch * a->q_len * sizeof(int32_t);
    if (a->workspace && aligned16(a->workspace) && a->workspace_bytes >= at + per_array)
      row_last = reinterpret_cast<int32_t*>(static_cast<char*>(a->workspace) + at);
    p.row_last = row_last;
    // and for a second one: the first column of the rows whose mask line is plain (the cooperative kernel's fast walk)
    if (row_last && prefill_nqt && a->workspace_bytes >= at + 2 * per_array) row_first = row_last + (size_t)a->batch * a->q_len;
    p.row_first = row_first;
  }
  p.num_kv_heads = pool->num_kv_heads;
  p.items = nullptr;
  p.seq_parts = a->seq_parts;
  long long pairs = (long long)a->batch * max_parts;  // (sequence, partition) pairs of the dense grid
  if (a->work_items) {
    p.items = a->work_items;
    pairs = a->n_work_items;
  }
  p.total_items = pairs * pool->num_kv_heads * p.n_qgroups;
  PACE_REQUIRE(p.total_items < (1ll << 31), "%s: grid too large", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool has_mask = a->mask != nullptr;
  if (row_last && !g_name_out) {
    PACE_REQUIRE((long long)a->batch * a->q_len < (1ll << 31), "%s: too many query rows", who);
    hipLaunchKernelGGL(mask_row_last_kernel, dim3((unsigned)(a->batch * a->q_len)), dim3(64), 0, s, p, row_last, row_first);
    PACE_HIP_CHECK(hipGetLastError());
  }
  bool ok = false;
  if (prefill_nqt) {
    p.items = nullptr;  // one partition per sequence: a work list only orders the sequences, and this kernel has its own order
    p.n_qgroups = (tiles + 4 * prefill_nqt - 1) / (4 * prefill_nqt);
    p.total_items = (long long)a->batch * pool->num_kv_heads * p.n_qgroups;
    for_head_dim(pool->head_dim, [&](auto d) { ok = launch_prefill<decltype(d)::value>(prefill_nqt, p, s); });
    PACE_REQUIRE(ok, "%s: no prefill kernel built for head_dim %d with %d tiles per wave", who, pool->head_dim, prefill_nqt);
    if (g_name_out) return PACE_KV_OK;
    PACE_HIP_CHECK(hipGetLastError());
    return PACE_KV_OK;
  }
  for_head_dim(pool->head_dim, [&](auto d) { ok = launch_shape<decltype(d)::value>(sh, p, has_mask, s); });
  PACE_REQUIRE(ok, "%s: no kernel built for shape nqt=%d nw=%d occ=%d..%d", who, sh.nqt, sh.nw, sh.occ, sh.occ_max);
  if (g_name_out) return PACE_KV_OK;
  PACE_HIP_CHECK(hipGetLastError());
  if (max_parts > 1) {
    const size_t rows_total = (size_t)a->batch * a->num_q_heads * a->q_len;
    PACE_REQUIRE(rows_total < ((size_t)1 << 31), "%s: too many query rows", who);
    for_head_dim(pool->head_dim, [&](auto d) {
      if (p.max_parts > 8) hipLaunchKernelGGL(paged_attn_merge_wide_kernel<decltype(d)::value>, dim3((unsigned)rows_total), dim3(256), 0, s, p);
      else hipLaunchKernelGGL(paged_attn_merge_kernel<decltype(d)::value>, dim3((unsigned)rows_total), dim3(64), 0, s, p);
    });
    PACE_HIP_CHECK(hipGetLastError());
  }
  return PACE_KV_OK;
}

}  // namespace pace_kv

using namespace pace_kv;


extern "C" int32_t pace_paged_attn_partition_tokens(int32_t batch, int32_t num_q_heads, int32_t q_len, int32_t head_dim,
                                                    int32_t max_seq_len, int32_t partition_tokens, int32_t num_kv_heads) {
  if (batch <= 0 || num_q_heads <= 0 || q_len <= 0 || head_dim <= 0 || max_seq_len <= 0 || num_kv_heads <= 0) return 0;
  return resolve_partition(partition_tokens, max_seq_len, batch, num_kv_heads, q_len * (num_q_heads / num_kv_heads),
                           head_dim);
}

// Partials of every (row, partition) when a sequence is cut into several partitions, then (16-byte
// aligned) two ints per (sequence, query token) for launches of more than 64 query rows per KV head:
// the per-row summary of an explicit mask (mask_row_last_kernel: last column, first column of a plain line).
static size_t workspace_need(int batch, int num_q_heads, int q_len, int head_dim, int max_parts, int rows) {
  size_t need = max_parts > 1 ? (size_t)batch * num_q_heads * q_len * max_parts * (head_dim + 2) * sizeof(float) : 0;
  if (rows > 64) need = ((need + 15) & ~(size_t)15) + 2 * (size_t)batch * q_len * sizeof(int32_t);
  return need;
}

extern "C" size_t pace_paged_attn_workspace_bytes(int32_t batch, int32_t num_q_heads, int32_t q_len, int32_t head_dim,
                                                  int32_t max_seq_len, int32_t partition_tokens, int32_t num_kv_heads) {
  if (batch <= 0 || num_q_heads <= 0 || q_len <= 0 || head_dim <= 0 || max_seq_len <= 0 || num_kv_heads <= 0) return 0;
  const int rows = q_len * (num_q_heads / num_kv_heads);
  const int part = resolve_partition(partition_tokens, max_seq_len, batch, num_kv_heads, rows, head_dim);
  const int max_parts = (max_seq_len + part - 1) / part;
  return workspace_need(batch, num_q_heads, q_len, head_dim, max_parts, rows);
}

extern "C" size_t pace_paged_attn_workspace_bytes_for_parts(int32_t batch, int32_t num_q_heads, int32_t q_len, int32_t head_dim,
                                                            int32_t max_parts) {
  if (batch <= 0 || num_q_heads <= 0 || q_len <= 0 || head_dim <= 0 || max_parts < 1) return 0;
  // rows per KV head are not known here: room for the per-row mask summary whenever the launch could be prefill-sized
  return workspace_need(batch, num_q_heads, q_len, head_dim, max_parts, q_len * num_q_heads);
}

extern "C" int pace_paged_attn_kernel_name(const pace_kv_pool_t* pool, const pace_paged_attn_args_t* args, char* out,
                                           size_t out_bytes) {
  PACE_REQUIRE(out != nullptr && out_bytes > 0, "pace_paged_attn_kernel_name: no output buffer");
  out[0] = 0;
  g_name_out = out, g_name_cap = out_bytes;
  const int rc = run_paged_attn(pool, args, nullptr, "pace_paged_attn_kernel_name");
  g_name_out = nullptr, g_name_cap = 0;
  return rc;
}

// Host-side planner: how the sequences of a batch are cut into (sequence, partition) work items, in which
// order they are scheduled, and the descriptors the kernel reads.  Pure host arithmetic on host arrays.
extern "C" int pace_paged_attn_plan(const int32_t* seq_lens, const int32_t* block_table, int32_t table_stride, int32_t batch,
                                    int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim, int32_t q_len, int32_t masked,
                                    int32_t partition_tokens, int32_t* work_items, int32_t work_capacity, int32_t* seq_parts,
                                    pace_attn_plan_t* plan) {
  const char* who = "pace_paged_attn_plan";
  PACE_REQUIRE(plan != nullptr, "%s: plan is NULL", who);
  *plan = pace_attn_plan_t{};
  PACE_REQUIRE(batch >= 0 && num_q_heads >= 1 && num_kv_heads >= 1 && q_len >= 1 && table_stride >= 1,
               "%s: bad batch (%d), heads (%d / %d), q_len (%d) or table_stride (%d)", who, batch, num_q_heads, num_kv_heads, q_len,
               table_stride);
  PACE_REQUIRE(num_q_heads % num_kv_heads == 0, "%s: num_q_heads %d not a multiple of num_kv_heads %d", who, num_q_heads,
               num_kv_heads);
  PACE_REQUIRE(head_dim_supported(head_dim), "%s: head_dim %d unsupported (64, 96, 128 or 256)", who, head_dim);
  PACE_REQUIRE(partition_tokens >= 0 && partition_tokens % 32 == 0, "%s: partition_tokens %d must be 0 or a multiple of 32", who,
               partition_tokens);
  if (batch == 0) return PACE_KV_OK;
  PACE_REQUIRE(seq_lens && block_table && seq_parts && (work_items || work_capacity == 0), "%s: NULL pointer", who);
  const int rows = q_len * (num_q_heads / num_kv_heads), tiles = (rows + 15) / 16;
  const Shape sh = shape_for(head_dim, tiles, masked != 0);
  const int n_qgroups = (tiles + sh.nqt - 1) / sh.nqt;
  int64_t total = 0;
  int max_len = 0;
  bool uniform = true;
  for (int b = 0; b < batch; ++b) {
    PACE_REQUIRE(seq_lens[b] >= 0 && (int64_t)seq_lens[b] <= (int64_t)table_stride * PACE_KV_BLOCK_TOKENS,
                 "%s: length %d of sequence %d does not fit a table row of %d blocks", who, seq_lens[b], b, table_stride);
    total += seq_lens[b];
    max_len = seq_lens[b] > max_len ? seq_lens[b] : max_len;
    uniform = uniform && seq_lens[b] == seq_lens[0];
  }
  // A ragged batch is cut at about its mean length: the long sequences then spread over several workgroups
  // (scheduled longest first) instead of forming the tail of the launch.
  int want = partition_tokens;
  const double mean = (double)total / batch;
  if (want == 0 && batch > 1 && !uniform && max_len > 1.5 * mean) {
    want = ((int)mean + 127) / 128 * 128;
    if (want < 1024) want = 1024;
  }
  const int part = max_len > 0 ? resolve_partition(want, max_len, batch, num_kv_heads, rows, head_dim) : 128;
  const int cap = partition_cap(head_dim, tiles);
  // A launch the cooperative prefill kernel takes (many row groups) walks every sequence in one piece.
  const bool one_each = partition_tokens == 0 && prefill_tiles_per_wave(head_dim, tiles, (int64_t)batch * num_kv_heads, max_len, masked != 0) > 0;
  // Workgroups resident at a time, per (KV head, row group): the launch's slots for (sequence, partition) pairs.
  const int64_t slots = std::max<int64_t>(1, (int64_t)compute_units() * 4 * sh.occ / sh.nw / ((int64_t)num_kv_heads * n_qgroups));
  std::vector<int> n(batch);
  int64_t sum_base = 0, sum_cap = 0;
  for (int b = 0; b < batch; ++b) {
    n[b] = one_each ? 1 : std::max(1, (seq_lens[b] + part - 1) / part);
    sum_base += n[b];
    sum_cap += std::max(1, (seq_lens[b] + cap - 1) / cap);
  }
  if (!one_each && !uniform && sum_cap < slots && sum_base <= slots) {
    // The whole launch fits the GPU in one round: choose the partition counts so that the partitions are as
    // equal as possible and fill the slots (the longest share is cut next, while a cut leaves 256 tokens or more).
    int64_t used = 0;
    for (int b = 0; b < batch; ++b) used += n[b] = std::max(1, (seq_lens[b] + cap - 1) / cap);
    while (used < slots) {
      int best = -1;
      double best_size = 0.0;
      for (int b = 0; b < batch; ++b) {
        const double size = (double)seq_lens[b] / n[b];
        if (size > best_size) best_size = size, best = b;
      }
      if (best < 0 || (double)seq_lens[best] / (n[best] + 1) < 256.0) break;
      ++n[best], ++used;
    }
  }
  // Equal partitions of whole 32-token units; none may be empty.
  std::vector<int> psize(batch);
  int64_t n_items = 0;
  int max_parts = 1;
  for (int b = 0; b < batch; ++b) {
    psize[b] = std::max(32, partition_size(seq_lens[b], n[b]));
    n[b] = std::max(1, (seq_lens[b] + psize[b] - 1) / psize[b]);
    seq_parts[b] = n[b];
    n_items += n[b];
    max_parts = std::max(max_parts, n[b]);
  }
  plan->n_work_items = (int32_t)std::min<int64_t>(n_items, 0x7fffffff);
  plan->max_parts = max_parts;
  plan->partition_tokens = part;
  plan->workspace_bytes = workspace_need(batch, num_q_heads, q_len, head_dim, max_parts, rows);
  PACE_REQUIRE(n_items <= work_capacity, "%s: %lld work items do not fit the capacity of %d", who, (long long)n_items, work_capacity);
  // Scheduling order: longest partitions first in a ragged batch (short tail), as they come otherwise.
  struct Item { int b, part; double size; };
  std::vector<Item> items;
  items.reserve((size_t)n_items);
  for (int b = 0; b < batch; ++b)
    for (int i = 0; i < n[b]; ++i) items.push_back({b, i, (double)seq_lens[b] / n[b]});
  if (!uniform) std::stable_sort(items.begin(), items.end(), [](const Item& x, const Item& y) { return x.size > y.size; });
  for (size_t k = 0; k < items.size(); ++k) {
    const Item& it = items[k];
    int32_t* d = work_items + k * PACE_ATTN_WORK_INTS;
    const int len = seq_lens[it.b];
    const int begin = it.part * psize[it.b];
    const bool last = it.part == n[it.b] - 1;
    const int end = last ? len : begin + psize[it.b];
    d[0] = it.b, d[1] = it.part, d[2] = n[it.b], d[3] = begin, d[4] = last ? -1 : end;
    int first = 0;
    for (int u = 0; u < PACE_ATTN_WORK_FIRST_UNITS; ++u) {
      const int j = begin / PACE_KV_BLOCK_TOKENS + 2 * u;
      const bool whole = begin + 32 * (u + 1) <= end && j + 1 < table_stride && first == u;
      d[8 + 2 * u] = whole ? block_table[(int64_t)it.b * table_stride + j] : 0;
      d[9 + 2 * u] = whole ? block_table[(int64_t)it.b * table_stride + j + 1] : 0;
      if (whole) first = u + 1;
    }
    d[5] = first, d[6] = 0, d[7] = 0;
  }
  return PACE_KV_OK;
}

extern "C" int pace_paged_attn_decode(const pace_kv_pool_t* pool, const pace_paged_attn_args_t* args, void* stream) {
  if (args && args->q_len != 1) {
    set_error("pace_paged_attn_decode: q_len must be 1 (got %d); use pace_paged_attn_verify", args->q_len);
    return PACE_KV_EINVAL;
  }
  return run_paged_attn(pool, args, stream, "pace_paged_attn_decode");
}

extern "C" int pace_paged_attn_verify(const pace_kv_pool_t* pool, const pace_paged_attn_args_t* args, void* stream) {
  return run_paged_attn(pool, args, stream, "pace_paged_attn_verify");
}

extern "C" int pace_paged_attn_verify_static(const pace_kv_pool_t* pool, const pace_paged_attn_args_t* args, void* stream) {
  return run_paged_attn(pool, args, stream, "pace_paged_attn_verify_static", true);
}
