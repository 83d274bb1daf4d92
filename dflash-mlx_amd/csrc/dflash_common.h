// Shared helpers of libdflash_mi355.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "dflash_mi355.h"

namespace dflash {

// printf-style message kept per host thread; returned by dflash_last_error().
void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
int option(int which);  // dflash_set_option's value for DFLASH_OPT_*

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

// Index of the current device for per-device caches (function attributes, CU counts); devices
// beyond the table share its last entry, which is then refreshed on every call.
constexpr int kMaxDevices = 16;
inline int current_device_slot() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0) dev = 0;
  return dev < kMaxDevices ? dev : kMaxDevices - 1;
}

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

// Eight consecutive elements of a tensor as loaded: 16 bytes for the 16-bit types (WIDE = false),
// 32 bytes for fp32.
template <bool WIDE>
struct Raw8 {
  uint4 w[WIDE ? 2 : 1];
};
// Eight consecutive elements from element i (a multiple of 8) of a 16-byte aligned array.
template <bool WIDE>
__device__ __forceinline__ Raw8<WIDE> load8_raw(const void* p, size_t i) {
  Raw8<WIDE> r;
  if (WIDE) {
    const uint4* src = reinterpret_cast<const uint4*>((const float*)p + i);
    r.w[0] = src[0];
    r.w[WIDE ? 1 : 0] = src[1];
  } else {
    r.w[0] = *reinterpret_cast<const uint4*>((const uint16_t*)p + i);
  }
  return r;
}
template <bool WIDE>
__device__ __forceinline__ void raw8_to_lds(const Raw8<WIDE>& r, int dt, float* dst) {
  const uint4 hi = r.w[WIDE ? 1 : 0];
  const uint32_t w[8] = {r.w[0].x, r.w[0].y, r.w[0].z, r.w[0].w, hi.x, hi.y, hi.z, hi.w};
  float o[8];
  if (WIDE) {
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = __uint_as_float(w[j]);
  } else if (dt == DFLASH_BF16) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      o[2 * j] = __uint_as_float(w[j] << 16);
      o[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      o[2 * j] = f16_bits_to_f32(w[j] & 0xffffu);
      o[2 * j + 1] = f16_bits_to_f32(w[j] >> 16);
    }
  }
  reinterpret_cast<float4*>(dst)[0] = float4{o[0], o[1], o[2], o[3]};
  reinterpret_cast<float4*>(dst)[1] = float4{o[4], o[5], o[6], o[7]};
}
__device__ __forceinline__ f32x4_t mfma4(float x, float y, f32x4_t acc) {
  return __builtin_amdgcn_mfma_f32_16x16x4f32(x, y, acc, 0, 0, 0);
}

// A 128 x 128 fp32 state S[dv][dk] (dk contiguous) held by four waves in matrix-core accumulator
// layout: wave w owns rows 32 w .. 32 w + 31; register (t2, c) of lane (li = lane % 16, kq = lane / 16)
// holds S[32 w + 16 t2 + li][16 c + 4 kq .. + 3], i.e. tile (t2, c) is C[i = dk][j = dv] of a
// 16 x 16 x 4 fp32 MFMA.  That layout puts 4 lanes (kq) on a row of S per 16-byte access: 64 contiguous
// bytes per row, which the memory system moves at about half the rate of full 128-byte lines
// (stores above all).  Memory is therefore accessed with 8 lanes per row - register (t2, c) of
// lane (li, kq) is row 16 t2 + 8 (c & 1) + li % 8, 16-byte column 8 (c / 2) + 4 (li / 8) + kq -
// and swap_row_bit() exchanges lane bit 3 with the low bit of c between the two layouts:
// the odd register of lanes li < 8 trades places with the even register of lanes li >= 8
// (DPP row_ror:8 reads lane li ^ 8; the bank mask picks the half row that is written).
__device__ __forceinline__ int memory_index(int wave, int li, int kq, int t2, int c) {
  return (32 * wave + 16 * t2 + 8 * (c & 1) + (li & 7)) * 32 + 8 * (c >> 1) + 4 * (li >> 3) + kq;
}
__device__ __forceinline__ void swap_row_bit(f32x4_t& even, f32x4_t& odd) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int x = __float_as_int(even[e]), y = __float_as_int(odd[e]);
    even[e] = __int_as_float(__builtin_amdgcn_update_dpp(x, y, 0x128, 0xF, 0xC, false));
    odd[e] = __int_as_float(__builtin_amdgcn_update_dpp(y, x, 0x128, 0xF, 0x3, false));
  }
}

// One output row of the conv-window rebuild (dflash_mlx/recurrent_rollback_cache.py:129-146):
// row j of `slot` is row steps + j of concat([prev or zeros, qkv]), copied by a workgroup in
// pieces of type V.  Shared by the kernel of its own and by the replay launches that carry the
// conv window along.
template <typename V>
__device__ __forceinline__ void conv_rebuild_row(const char* __restrict__ prev, const char* __restrict__ qkv,
                                                 char* __restrict__ out, int steps, int T, int keep,
                                                 size_t row_bytes, int slot, int j) {
  steps = steps < 0 ? 0 : (steps > T ? T : steps);
  const int src = steps + j;  // row of concat([prev, qkv]); always < keep + T
  const V* from = nullptr;
  if (src >= keep) {
    from = reinterpret_cast<const V*>(qkv + ((size_t)slot * T + (src - keep)) * row_bytes);
  } else if (prev != nullptr) {
    from = reinterpret_cast<const V*>(prev + ((size_t)slot * keep + src) * row_bytes);
  }
  V* to = reinterpret_cast<V*>(out + ((size_t)slot * keep + j) * row_bytes);
  const size_t n = row_bytes / sizeof(V);
  if (from != nullptr) {
    for (size_t i = threadIdx.x; i < n; i += blockDim.x) to[i] = from[i];
  } else {
    V zero;
    __builtin_memset(&zero, 0, sizeof(V));
    for (size_t i = threadIdx.x; i < n; i += blockDim.x) to[i] = zero;
  }
}

}  // namespace dflash
