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

__device__ __forceinline__ float rope_rnd(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

// One pair (x1, x2) of bf16 bit patterns rotated by (c, s), all bf16 bit patterns.
__device__ __forceinline__ void rope_pair(uint32_t x1, uint32_t x2, uint32_t c, uint32_t s, uint32_t& o1, uint32_t& o2) {
  const float a = bf16_bits_to_f32(x1), b = bf16_bits_to_f32(x2);
  const float cf = bf16_bits_to_f32(c), sf = bf16_bits_to_f32(s);
  const float t1 = rope_rnd(a * cf), t2 = rope_rnd(b * sf);
  const float t3 = rope_rnd(b * cf), t4 = rope_rnd(a * sf);
  o1 = f32_to_bf16_bits(t1 - t2);
  o2 = f32_to_bf16_bits(t3 + t4);
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
    uint32_t a0, b0, a1, b1;
    rope_pair(lo[e] & 0xffffu, hi[e] & 0xffffu, c8[e] & 0xffffu, s8[e] & 0xffffu, a0, b0);
    rope_pair(lo[e] >> 16, hi[e] >> 16, c8[e] >> 16, s8[e] >> 16, a1, b1);
    lo[e] = a0 | (a1 << 16);
    hi[e] = b0 | (b1 << 16);
  }
}

// Adjacent pairing: x holds dims d..d+7 = four pairs (2i, 2i+1); c4 / s4 the table columns d/2..d/2+3.
__device__ __forceinline__ void rope_rotate_adjacent(u32x4& x, const u32x2 c4, const u32x2 s4) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const uint32_t c = (e & 1) ? (c4[e >> 1] >> 16) : (c4[e >> 1] & 0xffffu);
    const uint32_t s = (e & 1) ? (s4[e >> 1] >> 16) : (s4[e >> 1] & 0xffffu);
    uint32_t a, b;
    rope_pair(x[e] & 0xffffu, x[e] >> 16, c, s, a, b);
    x[e] = a | (b << 16);
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

// Host: checks a pace_rope_t and fills the device view.  Returns 0 or PACE_KV_EINVAL.
int make_rope_dev(const pace_rope_t* rope, int head_dim, bool need_positions, const char* who, RopeDev* out);

}  // namespace pace_kv
