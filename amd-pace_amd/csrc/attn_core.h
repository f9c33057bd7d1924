// Inner step shared by the paged and the dense attention kernels (gfx950 matrix cores).
//
// Inner step ("unit") = 32 tokens = two pool blocks.  With lane = (n, g),
// n = lane % 16, g = lane / 16:
//   S^T tile  = K[16 tokens x 32 dims] * Q^T[32 dims x 16 rows]   (v_mfma_f32_16x16x32_bf16)
//       A operand: lane (n, g) holds 16 bytes of K row tok(n): dims 32*kk + 8g .. +8
//       C layout : lane (n, g) holds rows 4g..4g+3 of the tile, column n = query row
//   Token rows of the two tiles are interleaved so that lane (n, g) ends up with
//   the scores of tokens 8g..8g+7 of the unit for query row n -- exactly the B
//   operand slot of the second product:
//   O^T tile  = V^T[16 dims x 32 tokens] * P^T[32 tokens x 16 rows]
//       A operand: lane (n, g) holds 16 bytes of the token-minor V slab: dim 16j+n,
//                  tokens 8g..8g+7 of the unit  (one coalesced 16-byte load)
//   so probabilities never leave their lane between the two products, and the
//   softmax state (running max, sum, output accumulators) of query row n lives
//   in the four lanes (n, 0..3).
#pragma once
#include "common.h"
#include "rope.h"

namespace pace_kv {

struct PagedAttnParams {
  const uint16_t* q;
  int64_t q_sb, q_sh, q_ss;
  uint16_t* out;
  int64_t o_sb, o_sh, o_ss;
  const uint16_t* kpool;
  const uint16_t* vpool;
  int64_t k_bs, k_hs, v_bs, v_hs;
  int32_t num_blocks;
  const int32_t* table;
  int32_t table_stride;
  const int32_t* seq_lens;
  int32_t len_bias;
  const int32_t* len_bias_dev;  // optional device-side addend (advanced between graph replays)
  const int32_t* kv_start;
  const void* mask;
  int32_t mask_is_f32;
  int32_t mask_len;
  int64_t m_sb, m_ss;
  int32_t n_rep, q_len, num_q_heads;
  int32_t causal;
  int32_t n_qgroups;
  int32_t num_kv_heads;
  long long total_items;  // work items of the launch: KV heads x row groups x (sequence, partition) pairs
  const int32_t* items;      // optional work list: one descriptor of PACE_ATTN_WORK_INTS ints per (sequence, partition)
  const int32_t* seq_parts;  // with a work list: partitions per sequence (else derived from part_tokens)
  int32_t batch;
  int32_t part_tokens;
  int32_t max_parts;  // 1: write bf16 output directly; >1: write partials
  float scale_log2;   // softmax scale * log2(e)
  float scale;        // softmax scale
  // Fused append: the last n_new tokens of every sequence are taken from k_new / v_new
  // (and written to the pool by this launch) instead of being read from the pool.
  const uint16_t* k_new;
  const uint16_t* v_new;
  int64_t n_sb, n_sh, n_st;
  int32_t n_new;
  float* part_o;      // [B][Hq][S][max_parts][D]
  float* part_ml;     // [B][Hq][S][max_parts][2]  (running max in log2 units, sum)
  // Optional, prefill-sized launches with an explicit mask: per (sequence, query token) the last
  // column the row can read whose mask value is above the floor, -1 if there is none (written by
  // mask_row_last_kernel just before the attention launch).
  const int32_t* row_last;
  // Optional, with row_last: per (sequence, query token) the first column above the floor if the row's mask line is
  // "plain" -- exactly 0 from there to row_last, at or below the floor everywhere else it can read (a causal or
  // padding mask) -- and -1 if it is anything else.  A plain row needs its two columns, not its mask line.
  const int32_t* row_first;
  // Optional rotary embedding (rope.cos == NULL: off): q rows are rotated as they are loaded,
  // the fused append's new keys before they are used and stored.  rotary_dim == D here.
  RopeDev rope;
};

constexpr float kNegInf = -__builtin_inff();
constexpr float kLog2e = 1.4426950408889634f;
// Additive mask values are held at -2^100: far below any score, so such a column weighs nothing
// next to an unmasked one, yet finite, so that a row masked everywhere (finfo.min in every column)
// still ends as the reference's uniform average instead of 0 / 0; and a power of two, so that
// (value * log2(e)) is exact and equal values cancel exactly in the exponent.
constexpr float kMaskFloor = -0x1p100f;
constexpr uint32_t kMaskFloorBf16x2 = 0xf180f180u;  // the same value as a pair of bf16
// How far (in powers of two of the weight) a row's scores may rise above the softmax reference before the reference
// is moved and the accumulators rescaled.
constexpr float kLazyLog2 = 8.0f;

__device__ __forceinline__ float xor_lanes(float v, int mask) { return __shfl_xor(v, mask, 64); }

// Maximum over the four lanes (n, 0..3) that share query row n, left in all four.  The lane swaps
// hand every lane the value 16 resp. 32 lanes away without a trip through LDS.
__device__ __forceinline__ float row_max4(float v) {
  typedef unsigned v2u __attribute__((ext_vector_type(2)));
  const unsigned x = __float_as_uint(v);
  const v2u a = __builtin_amdgcn_permlane16_swap(x, x, false, false);
  const float m1 = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  const unsigned y = __float_as_uint(m1);
  const v2u b = __builtin_amdgcn_permlane32_swap(y, y, false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

template <int D>
struct UnitRegs {
  u32x4 k[2][D / 32];  // [tile][contraction step]
  u32x4 v[D / 16];     // [dim tile]
};

template <int D, int NQT>
struct RowState {
  f32x4 o[NQT][D / 16];  // O^T accumulators: dims 16j + 4g + i, query row n
  float m[NQT];          // running max while units are consumed: of the raw score products (no mask) or
                         // of scale * product + mask (with a mask); in log2 units after finish_rows()
  float m_top[NQT];      // m + the slack a score may have over the reference before the reference moves
  float m_neg[NQT];      // -(m * c), the addend of the exponent (0 while m is -inf); c: see softmax_and_output
  float l[NQT];          // this lane's share of the running sum
  int limit[NQT];        // last readable token of the row (-1: row is padding)
  int64_t mask_off[NQT]; // element offset of the row's mask line
};

// Unsigned minimum of two pairs of 16-bit values.  On bf16 bit patterns it holds negative values
// at the negative value `b` (a larger pattern is a more negative number) and leaves positive
// ones alone.
__device__ __forceinline__ uint32_t min_u16x2(uint32_t a, uint32_t b) {
  typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b)));
}

// Additive mask values of one unit, fetched by the caller while the unit's K / V travel:
// a[qt][c] belongs to token t0 + 8g + c of query tile qt's row n, held at kMaskFloor, and is -inf
// where the mask has no such column.
template <int NQT>
struct MaskRegs {
  float a[NQT][8];
};

// Eight packed bf16 mask values -> MaskRegs line (held at the floor).
__device__ __forceinline__ void mask_line_from_bf16x8(const u32x4 raw, float (&a)[8]) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const uint32_t w = min_u16x2(raw[e], kMaskFloorBf16x2);
    a[2 * e] = bf16_bits_to_f32(w & 0xffffu);
    a[2 * e + 1] = __uint_as_float(w & 0xffff0000u);
  }
}

// 16 bytes from an address that is only element-aligned (mask lines start wherever the caller's
// row length puts them; the hardware takes unaligned multi-dword loads).
__device__ __forceinline__ u32x4 load16_unaligned(const void* p) {
  u32x4 r;
  __builtin_memcpy(&r, p, 16);
  return r;
}

// Mask values of the unit at t0 for every query tile, read from p.mask (lines at mask_off[qt]).
// A lane whose eight columns all exist takes them in one 16-byte load (two for fp32); the lanes at
// the end of a line whose length is no multiple of 8 go element by element.
template <int NQT>
__device__ __forceinline__ void load_mask_regs(MaskRegs<NQT>& mr, const PagedAttnParams& p, const int64_t (&mask_off)[NQT],
                                               int t0, int g) {
  const int base = t0 + 8 * g;
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    if (base + 8 <= p.mask_len) {
      if (p.mask_is_f32) {
        const float* line = static_cast<const float*>(p.mask) + mask_off[qt] + base;
        const u32x4 lo = load16_unaligned(line), hi = load16_unaligned(line + 4);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          mr.a[qt][c] = fmaxf(__uint_as_float(lo[c]), kMaskFloor);
          mr.a[qt][4 + c] = fmaxf(__uint_as_float(hi[c]), kMaskFloor);
        }
      } else {
        mask_line_from_bf16x8(load16_unaligned(static_cast<const uint16_t*>(p.mask) + mask_off[qt] + base), mr.a[qt]);
      }
    } else {
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        float v = kNegInf;
        if (base + c < p.mask_len) {
          const float x = p.mask_is_f32 ? static_cast<const float*>(p.mask)[mask_off[qt] + base + c]
                                        : bf16_bits_to_f32(static_cast<const uint16_t*>(p.mask)[mask_off[qt] + base + c]);
          v = fmaxf(x, kMaskFloor);
        }
        mr.a[qt][c] = v;
      }
    }
  }
}

// The same values as fetched, for a caller that fetches a unit ahead: converting them where they are loaded would
// make the wave wait for the load there.  bf16: eight values in w[qt][0]; fp32: in w[qt][0], w[qt][1].  Columns the mask
// does not have come as -inf.
template <int NQT>
struct MaskRaw {
  u32x4 w[NQT][2];
};
template <int NQT>
__device__ __forceinline__ void load_mask_raw(MaskRaw<NQT>& raw, const PagedAttnParams& p, const int64_t (&mask_off)[NQT], int t0, int g) {
  const int base = t0 + 8 * g;
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    if (p.mask_is_f32) {
      const float* line = static_cast<const float*>(p.mask) + mask_off[qt] + base;
      if (base + 8 <= p.mask_len) {
        raw.w[qt][0] = load16_unaligned(line), raw.w[qt][1] = load16_unaligned(line + 4);
      } else {
#pragma unroll
        for (int c = 0; c < 8; ++c) raw.w[qt][c >> 2][c & 3] = base + c < p.mask_len ? __float_as_uint(line[c]) : 0xff800000u;
      }
    } else {
      const uint16_t* line = static_cast<const uint16_t*>(p.mask) + mask_off[qt] + base;
      if (base + 8 <= p.mask_len) {
        raw.w[qt][0] = load16_unaligned(line);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t lo = base + 2 * e < p.mask_len ? line[2 * e] : 0xff80u, hi = base + 2 * e + 1 < p.mask_len ? line[2 * e + 1] : 0xff80u;
          raw.w[qt][0][e] = lo | (hi << 16);
        }
      }
    }
  }
}
template <int NQT>
__device__ __forceinline__ void mask_regs_from_raw(MaskRegs<NQT>& mr, const MaskRaw<NQT>& raw, const PagedAttnParams& p) {
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    if (p.mask_is_f32) {
#pragma unroll
      for (int c = 0; c < 8; ++c) mr.a[qt][c] = fmaxf(__uint_as_float(raw.w[qt][c >> 2][c & 3]), kMaskFloor);
    } else {
      mask_line_from_bf16x8(raw.w[qt][0], mr.a[qt]);
    }
  }
}

// One wave looks over the columns [start, end) of a mask line (element offset `off` in `mask`): `last` = the last
// column whose value is above the floor (-1: none; NaN counts as masked), `first_if_plain` = the first such column
// if the line is plain -- exactly 0 on every column from there to `last`, which then are all above the floor -- and
// -1 if it is anything else.  Both are the same in every lane on return.
__device__ __forceinline__ void mask_line_summary(const void* mask, bool is_f32, int64_t off, int start, int end, int lane,
                                                  int& last_out, int& first_if_plain) {
  int last = -1, first = 0x7fffffff, above = 0;
  bool zero = true;  // every value above the floor is 0
  for (int c0 = start + 8 * lane; c0 < end; c0 += 8 * 64) {
    float a[8];
    if (c0 + 8 <= end) {
      if (is_f32) {
        const float* line = static_cast<const float*>(mask) + off + c0;
        const u32x4 lo = load16_unaligned(line), hi = load16_unaligned(line + 4);
#pragma unroll
        for (int c = 0; c < 4; ++c) a[c] = __uint_as_float(lo[c]), a[4 + c] = __uint_as_float(hi[c]);
      } else {
        const u32x4 raw = load16_unaligned(static_cast<const uint16_t*>(mask) + off + c0);
#pragma unroll
        for (int e = 0; e < 4; ++e) a[2 * e] = bf16_bits_to_f32(raw[e] & 0xffffu), a[2 * e + 1] = __uint_as_float(raw[e] & 0xffff0000u);
      }
    } else {
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        a[c] = kNegInf;
        if (c0 + c < end)
          a[c] = is_f32 ? static_cast<const float*>(mask)[off + c0 + c] : bf16_bits_to_f32(static_cast<const uint16_t*>(mask)[off + c0 + c]);
      }
    }
#pragma unroll
    for (int c = 0; c < 8; ++c)
      if (a[c] > kMaskFloor) {  // ascending: the largest column wins
        last = c0 + c;
        first = min(first, c0 + c);
        above += 1;
        zero = zero && a[c] == 0.f;
      }
  }
#pragma unroll
  for (int o = 1; o < 64; o *= 2) {
    last = max(last, __shfl_xor(last, o, 64));
    first = min(first, __shfl_xor(first, o, 64));
    above += __shfl_xor(above, o, 64);
  }
  const bool plain = __all(zero) && last >= 0 && above == last - first + 1;
  last_out = last;
  first_if_plain = plain ? first : -1;
}

// A unit can be left out altogether when it cannot change any row of the wave: every mask value
// in it is at the floor (weight exactly 0 next to any real score) and every row has already met a
// real score -- the upper triangle of a causal mask, which is half of a prefill.  Rows that have
// met nothing but floor values so far still need the unit (they may end as a uniform average).
// Wave-uniform.
template <int D, int NQT>
__device__ __forceinline__ bool unit_is_masked_out(const MaskRegs<NQT>& mr, const RowState<D, NQT>& st) {
  bool out = true;
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    float top = mr.a[qt][0];
#pragma unroll
    for (int c = 1; c < 8; ++c) top = fmaxf(top, mr.a[qt][c]);
    // rows that are padding are never written: whatever their mask line holds does not matter
    out = out && (st.limit[qt] < 0 || (top <= kMaskFloor && st.m[qt] > 0.5f * kMaskFloor));
  }
  return __all(out);
}

// First product of a unit: the scores of its 32 tokens against every query tile.  All of them are
// issued before any softmax, so that the matrix cores work through them (and later through the
// previous tile's second product) while the vector unit does a tile's softmax.
template <int D, int NQT>
__device__ __forceinline__ void score_products(const u32x4 (&k)[2][D / 32], const u32x4 (&qreg)[NQT][D / 32],
                                               f32x4 (&sc)[NQT][2]) {
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt)
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < D / 32; ++kk)
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, k[t][kk]),
                                                      __builtin_bit_cast(bf16x8, qreg[qt][kk]), acc, 0, 0, 0);
      sc[qt][t] = acc;
    }
}

// Second half of a unit: masking, online softmax and the product with V.
// FULL: every token of the unit exists and is readable by every query row (no masking code at all;
// the caller decides once per unit, wave-uniformly).  With HAS_MASK the unit's mask values come in
// `mregs`.
template <int D, int NQT, bool HAS_MASK, bool FULL>
__device__ __forceinline__ void softmax_and_output(const f32x4 (&sc)[NQT][2], const u32x4 (&v)[D / 16], RowState<D, NQT>& st,
                                                   const PagedAttnParams& p, int t0, int tok_end, int start, int g,
                                                   const MaskRegs<NQT>& mregs = MaskRegs<NQT>{}) {
  // No fused multiply-add contraction in here: which operations the compiler would fuse depends on
  // the instantiation, and the variants of one kernel are meant to give the same bits.
#pragma clang fp contract(off)
  constexpr bool full = FULL;
  constexpr int MT = D / 16;
  // Zero V columns past the end of the sequence so that stale pool contents
  // (possibly non-finite bit patterns) cannot reach the accumulators.
  u32x4 vreg[MT];
#pragma unroll
  for (int j = 0; j < MT; ++j) vreg[j] = v[j];
  if (!full) {
    const int nvalid = tok_end - (t0 + 8 * g);  // tokens of this lane's 8 that exist
    if (nvalid < 8) {
      u32x4 keep;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int c = nvalid - 2 * e;  // tokens 2e, 2e+1 live in dword e
        keep[e] = c >= 2 ? 0xffffffffu : (c == 1 ? 0x0000ffffu : 0u);
      }
#pragma unroll
      for (int j = 0; j < MT; ++j) vreg[j] &= keep;
    }
  }
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    // Without a mask, scores stay in units of the raw products and the softmax scale enters once, in
    // the exponent.  With one they are scale * product + mask in fp32, the reference's sum, with the
    // mask value held at kMaskFloor.
    f32x4 s[2] = {sc[qt][0], sc[qt][1]};
    // lane (n, g): s[t][i] is the score of token t0 + 8g + 4t + i for query row n.
    if (HAS_MASK) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) s[t][i] = __builtin_fmaf(s[t][i], p.scale, mregs.a[qt][4 * t + i]);
    }
    // A whole unit needs no range check, masked or not: mask values are -inf where the mask has no
    // column, and rows that are padding are never written.
    if (!full) {
      // token t0 + 8g + c (c = 4t + i) is readable iff lo <= c <= hi, both relative to the lane's first token
      const int base = t0 + 8 * g;
      const int hi = min(st.limit[qt], tok_end - 1) - base, lo = start - base;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (4 * t + i > hi || 4 * t + i < lo) s[t][i] = kNegInf;
          // a NaN score can only come from a stale K row; it is replaced above
          // when out of range, and propagates (like the reference) when in range.
        }
    }
    const float top = st.m_top[qt];
    bool above = false;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) above = above || s[t][i] > top;
    // exponent = (score - reference) * c with c = log2(e) (masked: natural units) or scale * log2(e).
    // The reference st.m follows the row's maximum lazily: it moves (and the accumulators are rescaled) only when
    // a score exceeds it by more than 2^kLazyLog2 in weight, for any row of the wave; until then weights may
    // exceed 1, which fp32 sums and bf16 weights (fp32's exponent range) take without loss.  A launch bound by the
    // SIMD's issue saves the rescaling -- one multiply per accumulator register -- in most of its units: with the
    // reference at the exact maximum, some row of a tile sees a new maximum in most units of a short walk.
    const float c = HAS_MASK ? kLog2e : p.scale_log2;
    // (a row's four lanes hold the same threshold: some lane's own maximum exceeds it exactly when the row's does,
    // so the maximum over the row's lanes is only formed when the reference moves)
    if (__any(above)) {  // m_top = -inf at first: the first real score always moves the reference
      const float mx = row_max4(fmaxf(fmaxf(fmaxf(s[0][0], s[0][1]), fmaxf(s[0][2], s[0][3])),
                                      fmaxf(fmaxf(s[1][0], s[1][1]), fmaxf(s[1][2], s[1][3]))));
      const float m_old = st.m[qt];
      const float m_new = fmaxf(m_old, mx);
      const float m_use = (m_new == kNegInf) ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f((m_old - m_use) * c);  // m_old = -inf -> 0
      st.m[qt] = m_new;
      st.m_top[qt] = m_new + kLazyLog2 / c;
      st.m_neg[qt] = -(m_use * c);
      st.l[qt] *= alpha;
#pragma unroll
      for (int j = 0; j < MT; ++j) st.o[qt][j] *= alpha;
    }
    const float m_neg = st.m_neg[qt];
    float psum = 0.f;
    f32x4 pr[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        pr[t][i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][i], c, m_neg));
        psum += pr[t][i];
      }
    st.l[qt] += psum;
    u32x4 pb;
    pb[0] = pack_bf16x2(pr[0][0], pr[0][1]);
    pb[1] = pack_bf16x2(pr[0][2], pr[0][3]);
    pb[2] = pack_bf16x2(pr[1][0], pr[1][1]);
    pb[3] = pack_bf16x2(pr[1][2], pr[1][3]);
#pragma unroll
    for (int j = 0; j < MT; ++j)
      st.o[qt][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, vreg[j]),
                                                           __builtin_bit_cast(bf16x8, pb), st.o[qt][j], 0, 0, 0);
  }
}

// After the last unit: complete the row sums over the four lanes of a row and express the running
// max in log2 units, as the merges between waves and partitions expect it.
template <int D, int NQT, bool HAS_MASK>
__device__ __forceinline__ void finish_rows(RowState<D, NQT>& st, const PagedAttnParams& p) {
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    float l = st.l[qt];
    l += xor_lanes(l, 16);
    l += xor_lanes(l, 32);
    st.l[qt] = l;
    st.m[qt] *= HAS_MASK ? kLog2e : p.scale_log2;  // -inf stays -inf: the factor is positive
  }
}

// One whole unit from registers.
template <int D, int NQT, bool HAS_MASK, bool FULL>
__device__ __forceinline__ void compute_unit_impl(const UnitRegs<D>& r, const u32x4 (&qreg)[NQT][D / 32],
                                                  RowState<D, NQT>& st, const PagedAttnParams& p, int t0, int tok_end,
                                                  int start, int g, const MaskRegs<NQT>& mregs = MaskRegs<NQT>{}) {
  f32x4 sc[NQT][2];
  score_products<D, NQT>(r.k, qreg, sc);
  softmax_and_output<D, NQT, HAS_MASK, FULL>(sc, r.v, st, p, t0, tok_end, start, g, mregs);
}

template <int D, int NQT, bool HAS_MASK>
__device__ __forceinline__ void compute_unit(const UnitRegs<D>& r, const u32x4 (&qreg)[NQT][D / 32],
                                             RowState<D, NQT>& st, const PagedAttnParams& p, int t0, int tok_end,
                                             int start, bool full, int g, const MaskRegs<NQT>& mregs = MaskRegs<NQT>{}) {
  if (full)
    compute_unit_impl<D, NQT, HAS_MASK, true>(r, qreg, st, p, t0, tok_end, start, g, mregs);
  else
    compute_unit_impl<D, NQT, HAS_MASK, false>(r, qreg, st, p, t0, tok_end, start, g, mregs);
}

// A sequence of `len` tokens is cut into ceil(len / part_tokens) partitions of equal size
// (rounded up to whole 32-token units), so no partition is a short remainder.
__host__ __device__ __forceinline__ int partition_count(int len, int part_tokens) {
  return len > 0 ? (len + part_tokens - 1) / part_tokens : 1;
}
__host__ __device__ __forceinline__ int partition_size(int len, int n_parts) {
  return (((len + n_parts - 1) / n_parts) + 31) & ~31;
}

}  // namespace pace_kv
