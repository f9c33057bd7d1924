// Micro-benchmarks of what one SIMD of a gfx950 compute unit issues per cycle: the figures the attention kernels'
// design notes quote (how far matrix and vector instructions overlap, what a dependent instruction waits, how fast
// LDS hands operands back).  Stand-alone: no library code is used.
//   hipcc -O3 --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops -o simd_issue simd_issue.hip
// One workgroup per compute unit (96 KiB of LDS each), 256 workgroups, WAVES waves each; every line reports the time
// of one launch and the time per instruction and wave.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

#define CHECK(x)                                                                  \
  do {                                                                            \
    hipError_t e_ = (x);                                                          \
    if (e_ != hipSuccess) {                                                       \
      fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                    \
      exit(1);                                                                    \
    }                                                                             \
  } while (0)
#define MFMA(acc) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0)

enum Mode {
  kMfmaChain,     // 8 matrix instructions on one accumulator
  kFma,           // 32 independent fused multiply-adds
  kFmaChain,      // 32 dependent ones
  kExp,           // 16 independent exp2
  kMfmaThenFma,   // 8 x (matrix instruction, multiply-add that reads its result)
  kSplit,         // first half of the waves: kMfmaChain; second half: kFma
  kInterleaved,   // every wave: 8 x (matrix instruction, 3 multiply-adds that do not depend on it)
  kExpFma,        // 16 x (exp2, multiply-add that does not depend on it)
  kSplitExp,      // first half of the waves: kMfmaChain; second half: kExp
  kMfmaExp,       // every wave: 8 x (matrix instruction, 2 exp2 that do not depend on it)
  kMfmaF32,       // 8 fp32 matrix instructions (16x16x4) on eight accumulators
  kMfmaF32Chain,  // 8 fp32 matrix instructions on one accumulator
};

template <int MODE, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void issue_kernel(float* out, int iters) {
  __shared__ float pad[24 * 1024];
  const int wave = threadIdx.x >> 6;
  f32x4 acc[8];
  float x[16];
  const u32x4 a = {threadIdx.x, 2u, 3u, 4u}, b = {5u, 6u, 7u, threadIdx.x};
  for (int i = 0; i < 8; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int i = 0; i < 16; ++i) x[i] = threadIdx.x * 0.001f + i * 0.01f;
  const bool first_half = wave < WAVES / 2;
  for (int it = 0; it < iters; ++it) {
    if (MODE == kMfmaChain) {
#pragma unroll
      for (int i = 0; i < 8; ++i) MFMA(acc[0]);
    } else if (MODE == kFma) {
#pragma unroll
      for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int i = 0; i < 16; ++i) x[i] = __builtin_fmaf(x[i], 1.0001f, 0.5f);
    } else if (MODE == kFmaChain) {
#pragma unroll
      for (int r = 0; r < 32; ++r) x[0] = __builtin_fmaf(x[0], 1.0001f, 0.5f);
    } else if (MODE == kExp) {
#pragma unroll
      for (int i = 0; i < 16; ++i) x[i] = __builtin_amdgcn_exp2f(x[i]);
    } else if (MODE == kMfmaThenFma) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        MFMA(acc[i]);
        x[i] = __builtin_fmaf(acc[i][0], 1.0001f, x[i]);
      }
    } else if (MODE == kSplit) {
      if (first_half) {
#pragma unroll
        for (int i = 0; i < 8; ++i) MFMA(acc[0]);
      } else {
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
          for (int i = 0; i < 16; ++i) x[i] = __builtin_fmaf(x[i], 1.0001f, 0.5f);
      }
    } else if (MODE == kExpFma) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        x[i] = __builtin_amdgcn_exp2f(x[i]);
        acc[i & 7][i >> 3] = __builtin_fmaf(acc[i & 7][i >> 3], 1.0001f, 0.5f);
      }
    } else if (MODE == kSplitExp) {
      if (first_half) {
#pragma unroll
        for (int i = 0; i < 8; ++i) MFMA(acc[0]);
      } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) x[i] = __builtin_amdgcn_exp2f(x[i]);
      }
    } else if (MODE == kMfmaExp) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        MFMA(acc[0]);
        x[2 * i] = __builtin_amdgcn_exp2f(x[2 * i]);
        x[2 * i + 1] = __builtin_amdgcn_exp2f(x[2 * i + 1]);
      }
    } else if (MODE == kMfmaF32) {
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(x[i], x[i + 8], acc[i], 0, 0, 0);
    } else if (MODE == kMfmaF32Chain) {
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(x[i], x[i + 8], acc[0], 0, 0, 0);
    } else if (MODE == kInterleaved) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        MFMA(acc[0]);
#pragma unroll
        for (int j = 0; j < 3; ++j) x[(3 * i + j) & 15] = __builtin_fmaf(x[(3 * i + j) & 15], 1.0001f, 0.5f);
      }
    }
  }
  float s = pad[threadIdx.x & 1023] * 0.f;
  for (int i = 0; i < 8; ++i) s += acc[i][0] + acc[i][3];
  for (int i = 0; i < 16; ++i) s += x[i];
  out[blockIdx.x * 64 * WAVES + threadIdx.x] = s;
}

// 8 waves per compute unit, each reading 16 KiB per iteration, lane l taking the l-th piece of every KiB.
template <int BYTES>
__global__ __launch_bounds__(512) void lds_read_kernel(float* out, int iters) {
  __shared__ __attribute__((aligned(16))) u32x4 buf[4096];
  for (int i = threadIdx.x; i < 4096; i += 512) buf[i] = u32x4{(unsigned)i, 1u, 2u, 3u};
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  unsigned acc = 0;
  const u32x4* base = buf + (wave & 3) * 1024;
  for (int it = 0; it < iters; ++it) {
    if (BYTES == 16) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const u32x4 v = base[i * 64 + lane];
        acc += v[0] ^ v[1] ^ v[2] ^ v[3];
      }
    } else if (BYTES == 8) {
#pragma unroll
      for (int i = 0; i < 32; ++i) {
        const u32x2 v = reinterpret_cast<const u32x2*>(base)[i * 64 + lane];
        acc += v[0] ^ v[1];
      }
    } else {
#pragma unroll
      for (int i = 0; i < 64; ++i) acc += reinterpret_cast<const unsigned*>(base)[i * 64 + lane];
    }
    asm volatile("" ::: "memory");
  }
  out[blockIdx.x * 512 + threadIdx.x] = (float)acc;
}

template <typename Launch>
static float timed(Launch launch) {
  hipEvent_t e0, e1;
  CHECK(hipEventCreate(&e0));
  CHECK(hipEventCreate(&e1));
  launch();  // warm-up
  CHECK(hipEventRecord(e0));
  launch();
  CHECK(hipEventRecord(e1));
  CHECK(hipEventSynchronize(e1));
  CHECK(hipGetLastError());
  float ms = 0.f;
  CHECK(hipEventElapsedTime(&ms, e0, e1));
  return ms;
}

template <int MODE, int WAVES>
static void issue(float* out, int iters, const char* what, int per_iter) {
  const float ms = timed([&] { hipLaunchKernelGGL((issue_kernel<MODE, WAVES>), dim3(256), dim3(64 * WAVES), 0, 0, out, iters); });
  printf("%-62s %d wave(s)/SIMD  %7.3f ms", what, WAVES / 4, ms);
  if (per_iter) printf("  %6.2f ns per instruction and wave", ms * 1e6 / ((double)iters * per_iter));
  printf("\n");
}

template <int BYTES>
static void lds(float* out, int iters) {
  const float ms = timed([&] { hipLaunchKernelGGL(lds_read_kernel<BYTES>, dim3(256), dim3(512), 0, 0, out, iters); });
  printf("LDS reads of %2d bytes per lane, lane-contiguous                  2 wave(s)/SIMD  %7.3f ms  %6.1f bytes per ns and compute unit\n", BYTES, ms,
         8.0 * 16384 * iters / (ms * 1e6));
}

int main() {
  float* out = nullptr;
  CHECK(hipMalloc(&out, 256 * 512 * sizeof(float)));
  const int it = 20000;
  issue<kMfmaChain, 4>(out, it, "8 MFMA 16x16x32 bf16 on one accumulator", 8);
  issue<kMfmaChain, 8>(out, it, "8 MFMA 16x16x32 bf16 on one accumulator", 8);
  issue<kFma, 4>(out, it, "32 independent FMA", 32);
  issue<kFma, 8>(out, it, "32 independent FMA", 32);
  issue<kFmaChain, 4>(out, it, "32 dependent FMA", 32);
  issue<kExp, 4>(out, it, "16 independent exp2", 16);
  issue<kExp, 8>(out, it, "16 independent exp2", 16);
  issue<kMfmaThenFma, 4>(out, it, "8 x (MFMA, FMA on its result)", 8);
  issue<kMfmaThenFma, 8>(out, it, "8 x (MFMA, FMA on its result)", 8);
  issue<kSplit, 8>(out, it, "one wave: 8 MFMA per turn, the other: 32 FMA per turn", 0);
  issue<kInterleaved, 8>(out, it, "each wave: 8 x (MFMA, 3 independent FMA) per turn", 0);
  issue<kExpFma, 4>(out, it, "16 x (exp2, independent FMA)", 16);
  issue<kExpFma, 8>(out, it, "16 x (exp2, independent FMA)", 16);
  issue<kSplitExp, 8>(out, it, "one wave: 8 MFMA per turn, the other: 16 exp2 per turn", 0);
  issue<kMfmaExp, 4>(out, it, "each wave: 8 x (MFMA, 2 independent exp2) per turn", 0);
  issue<kMfmaExp, 8>(out, it, "each wave: 8 x (MFMA, 2 independent exp2) per turn", 0);
  issue<kMfmaF32, 4>(out, it, "8 MFMA 16x16x4 f32 on eight accumulators", 8);
  issue<kMfmaF32, 8>(out, it, "8 MFMA 16x16x4 f32 on eight accumulators", 8);
  issue<kMfmaF32Chain, 4>(out, it, "8 MFMA 16x16x4 f32 on one accumulator", 8);
  issue<kMfmaF32Chain, 8>(out, it, "8 MFMA 16x16x4 f32 on one accumulator", 8);
  lds<16>(out, 5000);
  lds<8>(out, 5000);
  lds<4>(out, 5000);
  CHECK(hipFree(out));
  return 0;
}
