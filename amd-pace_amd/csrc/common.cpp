// Error text storage and checks shared by every entry point.
#include "common.h"

#include <stdarg.h>

namespace pace_kv {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

// Compute units of the current device (cached per process; 256 if the query fails).
int compute_units() {
  static int n = 0;
  if (n == 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
      n = v;
    else
      n = 256;
  }
  return n;
}

int check_pool(const pace_kv_pool_t* pool, const char* who, bool f32_ok) {
  PACE_REQUIRE(pool != nullptr, "%s: pool is NULL", who);
  PACE_REQUIRE(pool->k != nullptr && pool->v != nullptr, "%s: pool has a NULL K or V pointer", who);
  PACE_REQUIRE(pool->block_size == PACE_KV_BLOCK_TOKENS, "%s: block_size %d unsupported (must be %d)", who,
               pool->block_size, PACE_KV_BLOCK_TOKENS);
  PACE_REQUIRE(pool->elem_bytes == 0 || pool->elem_bytes == 2 || pool->elem_bytes == 4, "%s: elem_bytes %d (0 / 2: bf16, 4: fp32)", who,
               pool->elem_bytes);
  const bool f32 = pool_is_f32(pool);
  PACE_REQUIRE(!f32 || f32_ok, "%s: this entry point takes bf16 pools only (the pool holds fp32)", who);
  if (f32)
    PACE_REQUIRE(pool->head_dim >= 4 && pool->head_dim <= 256 && pool->head_dim % 4 == 0,
                 "%s: head_dim %d unsupported for an fp32 pool (a multiple of 4, at most 256)", who, pool->head_dim);
  else
    PACE_REQUIRE(head_dim_supported(pool->head_dim), "%s: head_dim %d unsupported (64, 96, 128 or 256)", who, pool->head_dim);
  PACE_REQUIRE(pool->num_blocks > 0 && pool->num_kv_heads > 0, "%s: empty pool (%d blocks, %d heads)", who,
               pool->num_blocks, pool->num_kv_heads);
  const int64_t slab = (int64_t)pool->block_size * pool->head_dim;
  PACE_REQUIRE(pool->k_head_stride >= slab && pool->v_head_stride >= slab, "%s: head stride smaller than a slab", who);
  PACE_REQUIRE(pool->k_block_stride >= pool->k_head_stride && pool->v_block_stride >= pool->v_head_stride,
               "%s: block stride smaller than head stride", who);
  const int per16 = f32 ? 4 : 8;  // elements in 16 bytes
  PACE_REQUIRE((pool->k_head_stride % per16) == 0 && (pool->v_head_stride % per16) == 0 && (pool->k_block_stride % per16) == 0 &&
                   (pool->v_block_stride % per16) == 0,
               "%s: pool strides must be multiples of %d elements (16 bytes)", who, per16);
  PACE_REQUIRE(aligned16(pool->k) && aligned16(pool->v), "%s: pool pointers must be 16-byte aligned", who);
  return PACE_KV_OK;
}

}  // namespace pace_kv

extern "C" const char* pace_kv_last_error(void) { return pace_kv::g_error; }

extern "C" int32_t pace_kv_abi_version(void) { return 14; }
