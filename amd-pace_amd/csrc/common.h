// Shared helpers for the gfx950 KV-cache kernels: error reporting, bf16 bit
// helpers and the vector types the matrix-core builtins take.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <type_traits>

#include "pace_kv_hip.h"

namespace pace_kv {

void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

// Returns PACE_KV_EINVAL from the enclosing entry point with a message.
#define PACE_REQUIRE(cond, ...)           \
  do {                                    \
    if (!(cond)) {                        \
      ::pace_kv::set_error(__VA_ARGS__);  \
      return PACE_KV_EINVAL;              \
    }                                     \
  } while (0)

#define PACE_HIP_CHECK(expr)                                                      \
  do {                                                                            \
    hipError_t e_ = (expr);                                                       \
    if (e_ != hipSuccess) {                                                       \
      ::pace_kv::set_error("%s failed: %s", #expr, hipGetErrorString(e_));        \
      return PACE_KV_EHIP;                                                        \
    }                                                                             \
  } while (0)

// f32_ok: the entry point also takes pools of fp32 rows (elem_bytes 4); otherwise such a pool is refused.
int check_pool(const pace_kv_pool_t* pool, const char* who, bool f32_ok = false);
inline bool pool_is_f32(const pace_kv_pool_t* pool) { return pool->elem_bytes == 4; }
int compute_units();  // of the current device

// Dense bf16 attention on the matrix cores (dense_attn_mfma.hip); false = shape not handled, nothing launched.
// workspace (optional): room for the summary of an explicit mask (dense_mfma_workspace_bytes).
bool launch_dense_mfma(const void* q, const void* k, const void* v, void* out, int B, int N, int S, int L, int H,
                       const void* mask, bool mask_is_f32, int mB, int mN, int mS, float scale, void* workspace,
                       size_t workspace_bytes, hipStream_t stream);
size_t dense_mfma_workspace_bytes(int S, int H, int mB, int mN, int mS, bool has_mask);
// Attention over a pool of fp32 rows (dense_attn.hip); pool and args are already checked.
int launch_paged_f32(const pace_kv_pool_t* pool, const pace_paged_attn_args_t* args, const char* who, hipStream_t stream);

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

// Streaming accesses: 16 bytes that this launch touches once.  Fetched / stored non-temporally they
// do not displace what the caches hold for re-use; on this GPU a pure stream runs about 10 % faster.
__device__ __forceinline__ u32x4 load16_stream(const void* p) { return __builtin_nontemporal_load(static_cast<const u32x4*>(p)); }
__device__ __forceinline__ void store16_stream(void* p, u32x4 v) { __builtin_nontemporal_store(v, static_cast<u32x4*>(p)); }

// Element offsets inside one (block, head) slab of 16 tokens x D dims.
// K slab  [tile 2][dim chunk D/8][token slot 8][dim 8]   with token -> (tile, slot):
//         tile = (tok >> 2) & 1,  slot = ((tok >> 3) << 2) | (tok & 3)
// V slab  [dim tile D/16][token half 2][dim 16][token 8]
// Both make every 16-lane quarter of a wavefront-wide 16-byte load read one
// contiguous run (128 B per block for K, 256 B for V) in the operand order of
// the 16x16x32 matrix-core instruction.
template <int D>
__host__ __device__ __forceinline__ int k_slab_offset(int tok, int dim) {
  const int tile = (tok >> 2) & 1, slot = ((tok >> 3) << 2) | (tok & 3);
  return tile * (D * 8) + (dim >> 3) * 64 + slot * 8 + (dim & 7);
}
template <int D>
__host__ __device__ __forceinline__ int v_slab_offset(int tok, int dim) {
  return (((dim >> 4) * 2 + (tok >> 3)) * 16 + (dim & 15)) * 8 + (tok & 7);
}

// Store eight dims (chunk) of one token's K and V into the slabs of its (block, head).
// K is one 16-byte store; the V values sit 8 elements apart (token-minor slab).
template <int D>
__device__ __forceinline__ void store_kv_chunk(uint16_t* kslab, uint16_t* vslab, int tok, int chunk, u32x4 kv, u32x4 vv) {
  *reinterpret_cast<u32x4*>(kslab + k_slab_offset<D>(tok, chunk * 8)) = kv;
  uint16_t* vdst = vslab + v_slab_offset<D>(tok, chunk * 8);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    vdst[(2 * j) * 8] = (uint16_t)(vv[j] & 0xffffu);
    vdst[(2 * j + 1) * 8] = (uint16_t)(vv[j] >> 16);
  }
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// Round-to-nearest-even fp32 -> bf16 bits (NaN stays NaN): the hardware conversion
// (v_cvt_pk_bf16_f32), two values per instruction.
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const f32x2 f = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}

__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) { return pack_bf16x2(f, 0.f) & 0xffffu; }

// Head sizes the pool kernels are built for.  Calls f(std::integral_constant<int, D>) for the one that
// matches; false if none does (check_pool() has then already refused the pool).
template <class F>
inline bool for_head_dim(int head_dim, F&& f) {
  switch (head_dim) {
    case 64: f(std::integral_constant<int, 64>{}); return true;
    case 96: f(std::integral_constant<int, 96>{}); return true;
    case 128: f(std::integral_constant<int, 128>{}); return true;
    case 256: f(std::integral_constant<int, 256>{}); return true;
    default: return false;
  }
}
inline bool head_dim_supported(int head_dim) { return head_dim == 64 || head_dim == 96 || head_dim == 128 || head_dim == 256; }

}  // namespace pace_kv
