// Dense scaled-dot-product attention for gfx950: the body of the torch op
// pace::attention for arbitrary head_dim, fp32 or bf16 tensors and an arbitrary
// additive mask broadcast from [mB][mN][mS][L].
//
// One 256-thread workgroup owns 16 query rows of one (batch, head) and streams
// the keys / values in chunks through LDS with an online softmax, so the
// [S][L] score matrix is never materialised.  fp32 arithmetic throughout.
#include "common.h"

namespace pace_kv {

constexpr int kRows = 16;

template <typename T>
__device__ __forceinline__ float load_f32(const T* p);
template <>
__device__ __forceinline__ float load_f32<float>(const float* p) {
  return *p;
}
template <>
__device__ __forceinline__ float load_f32<uint16_t>(const uint16_t* p) {
  return bf16_bits_to_f32(*p);
}
__device__ __forceinline__ void store_out(float* p, float v) { *p = v; }
__device__ __forceinline__ void store_out(uint16_t* p, float v) { *p = (uint16_t)f32_to_bf16_bits(v); }

struct DenseParams {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  const void* mask;
  int32_t B, N, S, L, H;
  int32_t mB, mN, mS;
  int32_t TL;  // tokens per chunk
  float scale;
};

template <typename T, typename MT>
__global__ __launch_bounds__(256) void attn_dense_kernel(const DenseParams p) {
  extern __shared__ float smem[];
  const int H = p.H, L = p.L, TL = p.TL;
  float* qs = smem;                        // [kRows][H]
  float* kv = qs + kRows * H;              // [TL][H + 1]
  float* sc = kv + TL * (H + 1);           // [kRows][TL + 1]
  float* row_m = sc + kRows * (TL + 1);    // [kRows]
  float* row_l = row_m + kRows;            // [kRows]
  float* row_a = row_l + kRows;            // [kRows]
  const int tid = threadIdx.x;
  const int s0 = blockIdx.x * kRows, n = blockIdx.y, b = blockIdx.z;
  const int rows = min(kRows, p.S - s0);
  const T* q = static_cast<const T*>(p.q) + (((int64_t)b * p.N + n) * p.S + s0) * H;
  const T* k = static_cast<const T*>(p.k) + ((int64_t)b * p.N + n) * (int64_t)L * H;
  const T* v = static_cast<const T*>(p.v) + ((int64_t)b * p.N + n) * (int64_t)L * H;
  T* out = static_cast<T*>(p.out) + (((int64_t)b * p.N + n) * p.S + s0) * H;
  const MT* mask = static_cast<const MT*>(p.mask);
  const int64_t m_b = p.mB == 1 ? 0 : b, m_n = p.mN == 1 ? 0 : n;

  for (int i = tid; i < kRows * H; i += 256) qs[i] = (i / H) < rows ? load_f32<T>(q + i) : 0.f;
  if (tid < kRows) {
    row_m[tid] = -__builtin_inff();
    row_l[tid] = 0.f;
  }
  // Output ownership: thread (r, c) = (tid / 16, tid % 16) accumulates dims c, c+16, ...
  const int r_own = tid >> 4, c_own = tid & 15;
  constexpr int kMaxOwn = 16;  // H <= 256
  float acc[kMaxOwn];
#pragma unroll
  for (int i = 0; i < kMaxOwn; ++i) acc[i] = 0.f;
  __syncthreads();

  for (int l0 = 0; l0 < L; l0 += TL) {
    const int nt = min(TL, L - l0);
    for (int i = tid; i < nt * H; i += 256) kv[(i / H) * (H + 1) + (i % H)] = load_f32<T>(k + (int64_t)l0 * H + i);
    __syncthreads();
    for (int idx = tid; idx < kRows * TL; idx += 256) {
      const int r = idx / TL, t = idx % TL;
      float val = -__builtin_inff();
      if (r < rows && t < nt) {
        float dot = 0.f;
        const float* qr = qs + r * H;
        const float* kr = kv + t * (H + 1);
        for (int h = 0; h < H; ++h) dot += qr[h] * kr[h];
        val = dot * p.scale;
        if (mask) {
          const int64_t m_s = p.mS == 1 ? 0 : (s0 + r);
          val += load_f32<MT>(mask + ((m_b * p.mN + m_n) * p.mS + m_s) * (int64_t)L + l0 + t);
        }
      }
      sc[r * (TL + 1) + t] = val;
    }
    __syncthreads();
    for (int i = tid; i < nt * H; i += 256) kv[(i / H) * (H + 1) + (i % H)] = load_f32<T>(v + (int64_t)l0 * H + i);
    if (tid < kRows) {
      float* sr = sc + tid * (TL + 1);
      float mx = row_m[tid];
      for (int t = 0; t < nt; ++t) mx = fmaxf(mx, sr[t]);
      const float m_use = (mx == -__builtin_inff()) ? 0.f : mx;
      const float alpha = expf(row_m[tid] - m_use);
      float sum = 0.f;
      for (int t = 0; t < nt; ++t) {
        const float e = expf(sr[t] - m_use);
        sr[t] = e;
        sum += e;
      }
      row_m[tid] = mx;
      row_l[tid] = row_l[tid] * alpha + sum;
      row_a[tid] = alpha;
    }
    __syncthreads();
    {
      const float alpha = row_a[r_own];
      const float* pr = sc + r_own * (TL + 1);
#pragma unroll
      for (int i = 0; i < kMaxOwn; ++i) {
        const int d = c_own + 16 * i;
        if (d < H) {
          float a = acc[i] * alpha;
          for (int t = 0; t < nt; ++t) a += pr[t] * kv[t * (H + 1) + d];
          acc[i] = a;
        }
      }
    }
    __syncthreads();
  }
  if (r_own < rows) {
    const float l = row_l[r_own];
    const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
    for (int i = 0; i < kMaxOwn; ++i) {
      const int d = c_own + 16 * i;
      if (d < H) store_out(out + (int64_t)r_own * H + d, acc[i] * inv);
    }
  }
}

}  // namespace pace_kv

using namespace pace_kv;

extern "C" int pace_attn_dense(const void* q, const void* k, const void* v, void* out, int32_t qkv_dtype, int32_t B,
                               int32_t N, int32_t S, int32_t L, int32_t H, const void* mask, int32_t mask_dtype,
                               int32_t mB, int32_t mN, int32_t mS, void* stream) {
  PACE_REQUIRE(qkv_dtype == PACE_DTYPE_F32 || qkv_dtype == PACE_DTYPE_BF16, "pace_attn_dense: bad qkv dtype %d", qkv_dtype);
  PACE_REQUIRE(B >= 0 && N >= 0 && S >= 0 && L >= 0 && H >= 1, "pace_attn_dense: negative extent");
  if (B == 0 || N == 0 || S == 0) return PACE_KV_OK;
  PACE_REQUIRE(L >= 1, "pace_attn_dense: empty key/value length");
  PACE_REQUIRE(H <= 256, "pace_attn_dense: head_dim %d unsupported (max 256)", H);
  PACE_REQUIRE(q && k && v && out, "pace_attn_dense: NULL tensor pointer");
  if (mask) {
    PACE_REQUIRE(mask_dtype == PACE_DTYPE_F32 || mask_dtype == PACE_DTYPE_BF16, "pace_attn_dense: bad mask dtype %d",
                 mask_dtype);
    PACE_REQUIRE((mB == 1 || mB == B) && (mN == 1 || mN == N) && (mS == 1 || mS == S),
                 "pace_attn_dense: mask dims [%d][%d][%d] not broadcastable to [%d][%d][%d]", mB, mN, mS, B, N, S);
  }
  PACE_REQUIRE(B <= 65535 && N <= 65535, "pace_attn_dense: batch / heads exceed grid limits");
  hipStream_t s = static_cast<hipStream_t>(stream);
  // bf16 with head_dim 64 / 128 runs on the matrix cores; everything else (fp32, other head
  // sizes) takes the general kernel below.
  if (qkv_dtype == PACE_DTYPE_BF16 &&
      launch_dense_mfma(q, k, v, out, B, N, S, L, H, mask, mask_dtype == PACE_DTYPE_F32, mB, mN, mS,
                        1.0f / sqrtf((float)H), s)) {
    PACE_HIP_CHECK(hipGetLastError());
    return PACE_KV_OK;
  }
  DenseParams p;
  p.q = q, p.k = k, p.v = v, p.out = out, p.mask = mask;
  p.B = B, p.N = N, p.S = S, p.L = L, p.H = H;
  p.mB = mB, p.mN = mN, p.mS = mS;
  p.TL = H > 128 ? 32 : 64;
  p.scale = 1.0f / sqrtf((float)H);
  const size_t smem = ((size_t)kRows * H + (size_t)p.TL * (H + 1) + (size_t)kRows * (p.TL + 1) + 3 * kRows) * sizeof(float);
  dim3 grid((S + kRows - 1) / kRows, N, B);
  const bool f32 = qkv_dtype == PACE_DTYPE_F32;
  const bool mf32 = mask_dtype == PACE_DTYPE_F32;
  if (f32 && mf32)
    hipLaunchKernelGGL((attn_dense_kernel<float, float>), grid, dim3(256), smem, s, p);
  else if (f32)
    hipLaunchKernelGGL((attn_dense_kernel<float, uint16_t>), grid, dim3(256), smem, s, p);
  else if (mf32)
    hipLaunchKernelGGL((attn_dense_kernel<uint16_t, float>), grid, dim3(256), smem, s, p);
  else
    hipLaunchKernelGGL((attn_dense_kernel<uint16_t, uint16_t>), grid, dim3(256), smem, s, p);
  PACE_HIP_CHECK(hipGetLastError());
  return PACE_KV_OK;
}
