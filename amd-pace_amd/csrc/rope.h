// Rotary position embedding on bf16 rows, in registers (gfx950).
//
// Arithmetic follows the reference operator step by step
// (pace/ops/rotary_embedding.py:412-443 on bf16 tensors): cos / sin are bf16, every
// product and the final sum are rounded to bf16 separately,
//   o1 = rnd(rnd(x1*cos) - rnd(x2*sin)),   o2 = rnd(rnd(x2*cos) + rnd(x1*sin)),
// so the rotated keys stored in the pool are bit-identical to the reference's.
// A product of two bf16 values is exact in fp32, hence computing in fp32 and rounding
// reproduces the bf16 tensor operations.
#pragma once
#include "common.h"

namespace pace_kv {

// Device-side view of pace_rope_t.
struct RopeDev {
  const void* cos;  // NULL = no rotation
  const void* sin;
  int32_t is_f32;
  int32_t rows;
  int32_t rot;          // rotated leading dims of a head row
  int32_t interleaved;  // 0: dim i pairs with i + rot/2;  1: dim 2i pairs with 2i + 1
  const int32_t* positions;  // optional [batch][tokens] table rows
  int32_t pos_sb;
};

// Two pairs at once -- the low and the high bf16 of the packed words x1, x2 rotated by the low
// and high bf16 of c, s -- so that every rounding is one packed conversion.
__device__ __forceinline__ void rope_pair2(uint32_t x1, uint32_t x2, uint32_t c, uint32_t s, uint32_t& o1, uint32_t& o2) {
  const float a0 = bf16_bits_to_f32(x1 & 0xffffu), a1 = __uint_as_float(x1 & 0xffff0000u);
  const float b0 = bf16_bits_to_f32(x2 & 0xffffu), b1 = __uint_as_float(x2 & 0xffff0000u);
  const float c0 = bf16_bits_to_f32(c & 0xffffu), c1 = __uint_as_float(c & 0xffff0000u);
  const float s0 = bf16_bits_to_f32(s & 0xffffu), s1 = __uint_as_float(s & 0xffff0000u);
  const uint32_t ac = pack_bf16x2(a0 * c0, a1 * c1), bs = pack_bf16x2(b0 * s0, b1 * s1);
  const uint32_t bc = pack_bf16x2(b0 * c0, b1 * c1), as = pack_bf16x2(a0 * s0, a1 * s1);
  o1 = pack_bf16x2(bf16_bits_to_f32(ac & 0xffffu) - bf16_bits_to_f32(bs & 0xffffu),
                   __uint_as_float(ac & 0xffff0000u) - __uint_as_float(bs & 0xffff0000u));
  o2 = pack_bf16x2(bf16_bits_to_f32(bc & 0xffffu) + bf16_bits_to_f32(as & 0xffffu),
                   __uint_as_float(bc & 0xffff0000u) + __uint_as_float(as & 0xffff0000u));
}

// Eight consecutive table values starting at element `off` (a multiple of 8), as packed bf16.
__device__ __forceinline__ u32x4 rope_load8(const void* tab, int is_f32, int64_t off) {
  if (is_f32) {
    const float* p = static_cast<const float*>(tab) + off;
    const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
    return u32x4{pack_bf16x2(a[0], a[1]), pack_bf16x2(a[2], a[3]), pack_bf16x2(b[0], b[1]), pack_bf16x2(b[2], b[3])};
  }
  return *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(tab) + off);
}

// Four consecutive table values starting at element `off` (a multiple of 4).
__device__ __forceinline__ u32x2 rope_load4(const void* tab, int is_f32, int64_t off) {
  if (is_f32) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(static_cast<const float*>(tab) + off);
    return u32x2{pack_bf16x2(a[0], a[1]), pack_bf16x2(a[2], a[3])};
  }
  return *reinterpret_cast<const u32x2*>(static_cast<const uint16_t*>(tab) + off);
}

// Halves pairing: `lo` holds dims d..d+7 (d < rot/2), `hi` dims d+rot/2..; c8 / s8 the table
// columns d..d+7.
__device__ __forceinline__ void rope_rotate_halves(u32x4& lo, u32x4& hi, const u32x4 c8, const u32x4 s8) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    uint32_t a, b;
    rope_pair2(lo[e], hi[e], c8[e], s8[e], a, b);
    lo[e] = a, hi[e] = b;
  }
}

// Adjacent pairing: x holds dims d..d+7 = four pairs (2i, 2i+1); c4 / s4 the table columns d/2..d/2+3.
__device__ __forceinline__ void rope_rotate_adjacent(u32x4& x, const u32x2 c4, const u32x2 s4) {
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    // words 2e, 2e+1 hold the pairs (x1 | x2 << 16); regroup into x1s and x2s of both pairs
    const uint32_t w0 = x[2 * e], w1 = x[2 * e + 1];
    const uint32_t x1 = (w0 & 0xffffu) | (w1 << 16), x2 = (w0 >> 16) | (w1 & 0xffff0000u);
    uint32_t a, b;
    rope_pair2(x1, x2, c4[e], s4[e], a, b);
    x[2 * e] = (a & 0xffffu) | (b << 16);
    x[2 * e + 1] = (a >> 16) | (b & 0xffff0000u);
  }
}

// Table row of token `t` of sequence `b`; `fallback` is the token's position in its sequence.
// Clamped so that a bad id never reads outside the table.
__device__ __forceinline__ int rope_row(const RopeDev& r, int b, int t, int fallback) {
  const int pos = r.positions ? r.positions[(int64_t)b * r.pos_sb + t] : fallback;
  return pos < 0 ? 0 : (pos >= r.rows ? r.rows - 1 : pos);
}

// Rotate the two 8-dim chunks a thread owns.  The chunk pair of index ci (0 .. D/16-1) is
//   halves:   (ci, ci + rot/16) for ci < rot/16, else the pass-through pair rot/8 + 2*(ci - rot/16), +1
//   adjacent: (2*ci, 2*ci + 1), rotated while inside the first rot dims
// rope_chunk_pair tells which chunks those are, rope_rotate_chunks applies the rotation.
__device__ __forceinline__ void rope_chunk_pair(const RopeDev& r, int ci, int& ca, int& cb) {
  const int rp = r.rot >> 4;
  if (r.cos && !r.interleaved && ci < rp) {
    ca = ci, cb = ci + rp;
  } else if (r.cos && !r.interleaved) {
    ca = 2 * rp + 2 * (ci - rp), cb = ca + 1;
  } else {
    ca = 2 * ci, cb = ca + 1;
  }
}

__device__ __forceinline__ void rope_rotate_chunks(const RopeDev& r, int row, int ci, u32x4& xa, u32x4& xb) {
  if (!r.cos) return;
  const int rp = r.rot >> 4;
  if (ci >= rp) return;  // pass-through dims
  const int64_t base = (int64_t)row * (r.rot >> 1);
  if (!r.interleaved) {
    rope_rotate_halves(xa, xb, rope_load8(r.cos, r.is_f32, base + 8 * ci), rope_load8(r.sin, r.is_f32, base + 8 * ci));
  } else {
    const u32x4 c8 = rope_load8(r.cos, r.is_f32, base + 8 * ci), s8 = rope_load8(r.sin, r.is_f32, base + 8 * ci);
    rope_rotate_adjacent(xa, u32x2{c8[0], c8[1]}, u32x2{s8[0], s8[1]});
    rope_rotate_adjacent(xb, u32x2{c8[2], c8[3]}, u32x2{s8[2], s8[3]});
  }
}

// Rotate one head row held in operand order: x[kk] = dims 32*kk + 8g .. +8 of the row (lane
// quarter g).  Both members of every rotation pair sit in the same lane: dim d pairs with
// d + D/2 (register kk + KK/2) or, interleaved, with its neighbour inside the 16 bytes.
// Split in two so that the table loads can be issued early and consumed late.
// A head size that is no multiple of 64 (96) paired by halves: the partner of dim d, d + D/2, falls into another
// lane quarter -- dims 8g .. of quarter g pair with dims 32 + 8 (g + 2) .. of quarter g + 2, and so on round the
// three registers -- so the quarters g and g ^ 2 (the lanes 32 apart, which hold the same row) exchange their
// registers; every lane then rotates the three chunks it owns.  The table registers number 2 KK there (a cos and a
// sin chunk per register of the row).
template <int D>
constexpr int kRopeTabRegs = (D % 64 == 0) ? D / 32 : 2 * (D / 32);

// Odd KK: the table column of register k of the row, and whether the register holds the lower member of its pairs.
template <int D>
__device__ __forceinline__ void rope_odd_chunk(int k, int g, int& col, bool& is_lo) {
  const int dim = 32 * k + 8 * g;
  is_lo = dim < D / 2;
  col = is_lo ? dim : dim - D / 2;
}

template <int D>
__device__ __forceinline__ void rope_fetch_row(const RopeDev& rope, int row, int g, u32x4 (&tab)[kRopeTabRegs<D>]) {
  constexpr int KK = D / 32;
  const int64_t base = (int64_t)row * (D / 2);
  if constexpr (KK % 2 != 0) {
    if (!rope.interleaved) {
#pragma unroll
      for (int k = 0; k < KK; ++k) {
        int col;
        bool is_lo;
        rope_odd_chunk<D>(k, g, col, is_lo);
        tab[2 * k] = rope_load8(rope.cos, rope.is_f32, base + col);
        tab[2 * k + 1] = rope_load8(rope.sin, rope.is_f32, base + col);
      }
      return;
    }
  }
  if (!rope.interleaved) {
#pragma unroll
    for (int kk = 0; kk < KK / 2; ++kk) {
      const int64_t col = base + 32 * kk + 8 * g;
      tab[2 * kk] = rope_load8(rope.cos, rope.is_f32, col);
      tab[2 * kk + 1] = rope_load8(rope.sin, rope.is_f32, col);
    }
  } else {
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      const int64_t col = base + 16 * kk + 4 * g;
      const u32x2 c4 = rope_load4(rope.cos, rope.is_f32, col), s4 = rope_load4(rope.sin, rope.is_f32, col);
      tab[kk] = u32x4{c4[0], c4[1], s4[0], s4[1]};
    }
  }
}

template <int D>
__device__ __forceinline__ void rope_apply_row(const RopeDev& rope, const u32x4 (&tab)[kRopeTabRegs<D>], u32x4 (&x)[D / 32]) {
  constexpr int KK = D / 32;
  if constexpr (KK % 2 != 0) {
    // every lane of the wave comes through here together (the exchange below reads the lane 32 away)
    static_assert(KK == 3, "head size 96");
    const int g = (threadIdx.x & 63) >> 4;
    u32x4 y[KK];  // the registers of the lane 32 away: the same row, quarter g ^ 2
#pragma unroll
    for (int k = 0; k < KK; ++k)
#pragma unroll
      for (int e = 0; e < 4; ++e) y[k][e] = (uint32_t)__shfl_xor((int)x[k][e], 32, 64);
    if (!rope.interleaved) {
      // partner of register k: k + 1 (mod 3) in the lower quarters, k + 2 (mod 3) in the upper ones
      const bool upper = g >= 2;
#pragma unroll
      for (int k = 0; k < KK; ++k) {
        int col;
        bool is_lo;
        rope_odd_chunk<D>(k, g, col, is_lo);
        u32x4 out;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const uint32_t other = upper ? y[(k + 2) % KK][e] : y[(k + 1) % KK][e];
          const uint32_t lo = is_lo ? x[k][e] : other, hi = is_lo ? other : x[k][e];
          uint32_t a, b;
          rope_pair2(lo, hi, tab[2 * k][e], tab[2 * k + 1][e], a, b);
          out[e] = is_lo ? a : b;
        }
        x[k] = out;  // (the partners were read from y: nothing rotated is read again)
      }
      return;
    }
  }
  if (!rope.interleaved) {
#pragma unroll
    for (int kk = 0; kk < KK / 2; ++kk) rope_rotate_halves(x[kk], x[kk + KK / 2], tab[2 * kk], tab[2 * kk + 1]);
  } else {
#pragma unroll
    for (int kk = 0; kk < KK; ++kk)
      rope_rotate_adjacent(x[kk], u32x2{tab[kk][0], tab[kk][1]}, u32x2{tab[kk][2], tab[kk][3]});
  }
}

template <int D>
__device__ __forceinline__ void rotate_row_regs(const RopeDev& rope, int row, int g, u32x4 (&x)[D / 32]) {
  u32x4 tab[kRopeTabRegs<D>];
  rope_fetch_row<D>(rope, row, g, tab);
  rope_apply_row<D>(rope, tab, x);
}

// Block-wise append with optional key rotation (kv_ops.hip).
int launch_block_append(const char* who, const pace_kv_pool_t* pool, const void* k_new, const void* v_new, int64_t stride_b,
                        int64_t stride_h, int64_t stride_t, int32_t batch, int32_t n_tokens, const int32_t* block_table,
                        int32_t table_stride, const int32_t* seq_lens, int32_t pos_offset, const RopeDev* rope,
                        hipStream_t stream);

// Host: checks a pace_rope_t and fills the device view.  Returns 0 or PACE_KV_EINVAL.
int make_rope_dev(const pace_rope_t* rope, int head_dim, bool need_positions, const char* who, RopeDev* out);

}  // namespace pace_kv
