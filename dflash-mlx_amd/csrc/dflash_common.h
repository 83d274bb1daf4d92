// Shared helpers of libdflash_mi355.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "dflash_mi355.h"

namespace dflash {

// printf-style message kept per host thread; returned by dflash_last_error().
void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

#define DFLASH_REQUIRE(cond, code, ...)  \
  do {                                   \
    if (!(cond)) {                       \
      ::dflash::set_error(__VA_ARGS__);  \
      return (code);                     \
    }                                    \
  } while (0)

#define DFLASH_HIP_OK(expr)                                                              \
  do {                                                                                   \
    hipError_t e_ = (expr);                                                              \
    if (e_ != hipSuccess) {                                                              \
      ::dflash::set_error("%s failed: %s", #expr, hipGetErrorString(e_));                \
      return DFLASH_ERR_HIP;                                                             \
    }                                                                                    \
  } while (0)

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// Round-to-nearest-even fp32 -> bf16 bit pattern (NaN kept quiet).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
  union { uint16_t u; _Float16 f; } v;
  v.u = (uint16_t)h;
  return (float)v.f;
}

__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  union { uint16_t u; _Float16 f; } v;
  v.f = (_Float16)f;  // RNE
  return v.u;
}

// Load element i of an array whose element type is one of the DFLASH_* dtypes.
__device__ __forceinline__ float load_as_f32(const void* p, size_t i, int dt) {
  if (dt == DFLASH_BF16) return bf16_bits_to_f32(((const uint16_t*)p)[i]);
  if (dt == DFLASH_FP16) return f16_bits_to_f32(((const uint16_t*)p)[i]);
  return ((const float*)p)[i];
}

// Store v as element i of an array whose element type is one of the DFLASH_* dtypes (RNE).
__device__ __forceinline__ void store_from_f32(void* p, size_t i, float v, int dt) {
  if (dt == DFLASH_BF16) {
    ((uint16_t*)p)[i] = (uint16_t)f32_to_bf16_bits(v);
  } else if (dt == DFLASH_FP16) {
    ((uint16_t*)p)[i] = (uint16_t)f32_to_f16_bits(v);
  } else {
    ((float*)p)[i] = v;
  }
}

__device__ __forceinline__ float round_through(float v, int dt) {
  if (dt == DFLASH_BF16) return bf16_bits_to_f32(f32_to_bf16_bits(v));
  if (dt == DFLASH_FP16) return f16_bits_to_f32(f32_to_f16_bits(v));
  return v;
}

}  // namespace dflash
