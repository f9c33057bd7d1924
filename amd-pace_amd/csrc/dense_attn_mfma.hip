// Dense bf16 attention on the matrix cores for head_dim 64 / 128: the fast path of the torch op
// pace::attention (dense_attn.hip holds the general kernel and the entry point).
#include "attn_core.h"

namespace pace_kv {

// ---------------------------------------------------------------------------------
// Dense bf16 attention with the same inner step: K and V are the reference's row-major
// [B][N][L][D] tensors.  K rows feed the first product directly (16 bytes of a row per
// lane); V rows are staged per wave in LDS and read back token-minor for the second.
// One workgroup of 4 waves per (batch, head, group of 16*NQT query rows); the waves split
// the L axis and merge through LDS like the paged kernel.
// ---------------------------------------------------------------------------------
struct DenseMfmaParams {
  PagedAttnParams base;  // q / out / mask fields and scale are shared with the paged kernel
  const uint16_t* k;
  const uint16_t* v;
  int32_t B, N, S, L;
  int32_t mB, mN, mS;
  int32_t n_qgroups;
};

template <int D, int NQT, bool HAS_MASK>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1))) void dense_attn_mfma_kernel(const DenseMfmaParams dp) {
  constexpr int KK = D / 32;
  constexpr int MT = D / 16;
  constexpr int NW = 4;
  constexpr int VROW = D + 24;                    // padded LDS row (elements): keeps the transposed reads off each other's banks
  constexpr int STAGE = 32 * VROW;                // one wave's V unit
  constexpr int MERGE_FLOATS = 2 * 16 * NQT * (D + 2);
  constexpr int LDS_BYTES = (NW * STAGE * 2 > MERGE_FLOATS * 4) ? NW * STAGE * 2 : MERGE_FLOATS * 4;
  __shared__ __attribute__((aligned(16))) unsigned char lds_raw[LDS_BYTES];
  const PagedAttnParams& p = dp.base;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n = lane & 15, g = lane >> 4;
  const int qg = blockIdx.x % dp.n_qgroups;
  const int head = (blockIdx.x / dp.n_qgroups) % dp.N;
  const int b = blockIdx.x / (dp.n_qgroups * dp.N);
  const int L = dp.L, S = dp.S;
  const uint16_t* kbase = dp.k + ((int64_t)b * dp.N + head) * (int64_t)L * D;
  const uint16_t* vbase = dp.v + ((int64_t)b * dp.N + head) * (int64_t)L * D;
  uint16_t* stage = reinterpret_cast<uint16_t*>(lds_raw) + wave * STAGE;

  u32x4 qreg[NQT][KK];
  RowState<D, NQT> st;
  int row_s[NQT];
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    const int s = (qg * NQT + qt) * 16 + n;
    const bool valid = s < S;
    row_s[qt] = s;
    st.limit[qt] = valid ? L - 1 : -1;
    if (HAS_MASK) {
      const int64_t mb = dp.mB == 1 ? 0 : b, mn = dp.mN == 1 ? 0 : head, ms = dp.mS == 1 ? 0 : (valid ? s : 0);
      st.mask_off[qt] = ((mb * dp.mN + mn) * dp.mS + ms) * (int64_t)L;
    } else {
      st.mask_off[qt] = 0;
    }
    st.m[qt] = kNegInf;
    st.l[qt] = 0.f;
    const uint16_t* qp = p.q + (((int64_t)b * dp.N + head) * S + (valid ? s : 0)) * D + 8 * g;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      u32x4 z = {0u, 0u, 0u, 0u};
      qreg[qt][kk] = valid ? *reinterpret_cast<const u32x4*>(qp + kk * 32) : z;
    }
#pragma unroll
    for (int j = 0; j < MT; ++j) st.o[qt][j] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  const int units = (L + 31) / 32;
  const int per_wave = (units + NW - 1) / NW;
  const int u_begin = min(units, wave * per_wave);
  const int n_units = min(units, u_begin + per_wave) - u_begin;
  UnitRegs<D> buf;
  for (int uu = 0; uu < n_units; ++uu) {
    const int t0 = 32 * (u_begin + uu);
    // K: token 8*(n/4) + 4*tile + n%4 of the unit, dims 32*kk + 8g.. (clamped rows are masked later).
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int tok = min(L - 1, t0 + 8 * (n >> 2) + 4 * t + (n & 3));
      const uint16_t* kp = kbase + (int64_t)tok * D + 8 * g;
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) buf.k[t][kk] = *reinterpret_cast<const u32x4*>(kp + kk * 32);
    }
    // V: the unit's 32 rows go to this wave's LDS stage (coalesced 16-byte chunks) ...
    constexpr int CH = D / 8;  // chunks per row
#pragma unroll
    for (int i = 0; i < 32 * CH / 64; ++i) {
      const int c = i * 64 + lane, r = c / CH, ch = c % CH;
      const int tok = min(L - 1, t0 + r);
      *reinterpret_cast<u32x4*>(stage + r * VROW + ch * 8) = *reinterpret_cast<const u32x4*>(vbase + (int64_t)tok * D + ch * 8);
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's LDS writes have landed
    __builtin_amdgcn_wave_barrier();
    // ... and come back token-minor: lane (n, g) takes dim 16j + n of tokens 8g..8g+7.  The LDS
    // transpose read hands lane i of a 16-lane group element i % 4 of the 8-byte pieces that
    // lanes 4j + i / 4 (j = 0..3) point at; with lane s of the group pointing at token
    // 8g + s / 4, dims 16j + 4 (s % 4) .. +3, lane n receives tokens 8g .. 8g+3 of dim 16j + n,
    // and a second read four token rows further down completes the operand.
    typedef short tr_v4 __attribute__((ext_vector_type(4)));
    typedef tr_v4 __attribute__((address_space(3))) * tr_ptr;
    const uint16_t* tr_base = stage + (8 * g + (n >> 2)) * VROW + 4 * (n & 3);
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      const tr_v4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr)(tr_base + 16 * j));
      const tr_v4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_ptr)(tr_base + 4 * VROW + 16 * j));
      const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
      buf.v[j] = u32x4{l2[0], l2[1], h2[0], h2[1]};
    }
    __builtin_amdgcn_wave_barrier();
    const bool full = t0 + 32 <= L;
    compute_unit<D, NQT, HAS_MASK>(buf, qreg, st, p, t0, L, 0, full, g);
  }
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    float l = st.l[qt];
    l += xor_lanes(l, 16);
    l += xor_lanes(l, 32);
    st.l[qt] = l;
  }
  __syncthreads();  // every wave is done with its V stage; the space becomes the merge buffer
  float* merge_buf = reinterpret_cast<float*>(lds_raw);
  constexpr int ROW_F = D + 2;
  constexpr int SLOT_F = 16 * NQT * ROW_F;
#pragma unroll
  for (int stride = 1; stride < NW; stride *= 2) {
    const int slot = wave / (2 * stride);
    const bool sender = (wave & (2 * stride - 1)) == stride;
    const bool receiver = (wave & (2 * stride - 1)) == 0;
    if (sender) {
#pragma unroll
      for (int qt = 0; qt < NQT; ++qt) {
        float* rowp = merge_buf + slot * SLOT_F + (qt * 16 + n) * ROW_F;
#pragma unroll
        for (int j = 0; j < MT; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) rowp[16 * j + 4 * g + i] = st.o[qt][j][i];
        if (g == 0) rowp[D] = st.m[qt], rowp[D + 1] = st.l[qt];
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
        const float wa = __builtin_amdgcn_exp2f(st.m[qt] - m_use), wb = __builtin_amdgcn_exp2f(m_b - m_use);
#pragma unroll
        for (int j = 0; j < MT; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) st.o[qt][j][i] = st.o[qt][j][i] * wa + rowp[16 * j + 4 * g + i] * wb;
        st.l[qt] = st.l[qt] * wa + l_b * wb;
        st.m[qt] = m_new;
      }
    }
    __syncthreads();
  }
  if (wave != 0) return;
#pragma unroll
  for (int qt = 0; qt < NQT; ++qt) {
    if (row_s[qt] >= S) continue;
    const float l = st.l[qt];
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    uint16_t* op = p.out + (((int64_t)b * dp.N + head) * S + row_s[qt]) * D + 4 * g;
#pragma unroll
    for (int j = 0; j < MT; ++j) {
      u32x2 w;
      w[0] = pack_bf16x2(st.o[qt][j][0] * inv, st.o[qt][j][1] * inv);
      w[1] = pack_bf16x2(st.o[qt][j][2] * inv, st.o[qt][j][3] * inv);
      *reinterpret_cast<u32x2*>(op + 16 * j) = w;
    }
  }
}

// Launches the dense bf16 kernel; returns false when the shape is not one it handles.
bool launch_dense_mfma(const void* q, const void* k, const void* v, void* out, int B, int N, int S, int L, int H,
                       const void* mask, bool mask_is_f32, int mB, int mN, int mS, float scale, hipStream_t stream) {
  if ((H != 64 && H != 128) || L < 1) return false;
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || (reinterpret_cast<uintptr_t>(out) & 7u)) return false;
  DenseMfmaParams dp = {};
  dp.base.q = static_cast<const uint16_t*>(q);
  dp.base.out = static_cast<uint16_t*>(out);
  dp.base.mask = mask, dp.base.mask_is_f32 = mask_is_f32, dp.base.mask_len = L;
  dp.base.scale_log2 = scale * kLog2e;
  dp.k = static_cast<const uint16_t*>(k), dp.v = static_cast<const uint16_t*>(v);
  dp.B = B, dp.N = N, dp.S = S, dp.L = L, dp.mB = mB, dp.mN = mN, dp.mS = mS;
  const int tiles = (S + 15) / 16;
  const int nqt = tiles >= 2 ? 2 : 1;
  dp.n_qgroups = (tiles + nqt - 1) / nqt;
  const long long blocks = (long long)B * N * dp.n_qgroups;
  if (blocks >= (1ll << 31)) return false;
  const dim3 grid((unsigned)blocks), block(256);
  const bool m = mask != nullptr;
#define PACE_DENSE(D_, Q_, M_) hipLaunchKernelGGL((dense_attn_mfma_kernel<D_, Q_, M_>), grid, block, 0, stream, dp)
  if (H == 128) {
    if (nqt == 2) { if (m) PACE_DENSE(128, 2, true); else PACE_DENSE(128, 2, false); }
    else { if (m) PACE_DENSE(128, 1, true); else PACE_DENSE(128, 1, false); }
  } else {
    if (nqt == 2) { if (m) PACE_DENSE(64, 2, true); else PACE_DENSE(64, 2, false); }
    else { if (m) PACE_DENSE(64, 1, true); else PACE_DENSE(64, 1, false); }
  }
#undef PACE_DENSE
  return true;
}

}  // namespace pace_kv
