// Conv-state rebuild after a partial acceptance (gfx950).
//
// The reference rebuilds the depthwise-conv window of a GatedDeltaNet layer with
// array ops (dflash_mlx/recurrent_rollback_cache.py:129-146):
//     conv_input = concat([snapshot_conv_state or zeros, qkv_tape], axis=1)
//     new_state  = conv_input[:, steps : steps + keep]          (keep = kernel - 1)
// Pure row gathering: output row j of a slot is source row steps + j, taken from
// the snapshot while steps + j < keep and from the recorded qkv rows afterwards.
// One workgroup per output row; rows are copied with 16-byte accesses when the
// row size and all bases allow it, byte-wise otherwise.  The accepted length can
// come from device memory so it matches the replay launch.
#include "dflash_common.h"

namespace dflash {
namespace {

template <typename V>
__global__ __launch_bounds__(256) void conv_rebuild_kernel(
    const char* __restrict__ prev, const char* __restrict__ qkv, char* __restrict__ out,
    const int32_t* __restrict__ steps_dev, int steps_host, int T, int keep, size_t row_bytes) {
  const int slot = blockIdx.x / keep, j = blockIdx.x % keep;
  int steps = steps_dev ? steps_dev[slot] : steps_host;
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

}  // namespace
}  // namespace dflash

extern "C" int dflash_conv_state_rebuild(const void* conv_prev, const void* qkv, void* conv_out,
                                         const int32_t* steps_dev, int steps_host, int slots,
                                         int T, int keep, int C, int elem_bytes, void* stream) {
  using namespace dflash;
  DFLASH_REQUIRE(qkv && conv_out, DFLASH_ERR_ARG, "dflash_conv_state_rebuild: null operand");
  DFLASH_REQUIRE(conv_out != conv_prev, DFLASH_ERR_ARG,
                 "dflash_conv_state_rebuild: conv_out must not alias conv_prev");
  DFLASH_REQUIRE(slots >= 0 && T > 0 && keep > 0 && C > 0 && elem_bytes > 0, DFLASH_ERR_SHAPE,
                 "dflash_conv_state_rebuild: non-positive dimension");
  if (slots == 0) return DFLASH_OK;
  const size_t row_bytes = (size_t)C * elem_bytes;
  const dim3 grid((unsigned)(slots * keep)), block(256);
  hipStream_t s = (hipStream_t)stream;
  const bool vec = row_bytes % 16 == 0 && (uintptr_t)qkv % 16 == 0 && (uintptr_t)conv_out % 16 == 0 &&
                   (uintptr_t)conv_prev % 16 == 0;
  if (vec) {
    hipLaunchKernelGGL(conv_rebuild_kernel<uint4>, grid, block, 0, s, (const char*)conv_prev,
                       (const char*)qkv, (char*)conv_out, steps_dev, steps_host, T, keep, row_bytes);
  } else {
    hipLaunchKernelGGL(conv_rebuild_kernel<unsigned char>, grid, block, 0, s, (const char*)conv_prev,
                       (const char*)qkv, (char*)conv_out, steps_dev, steps_host, T, keep, row_bytes);
  }
  DFLASH_HIP_OK(hipGetLastError());
  return DFLASH_OK;
}

extern "C" int dflash_rollback_layer(const void* tape, const void* k, const void* g, const void* state_in,
                                     void* state_out, const void* conv_prev, const void* qkv, void* conv_out,
                                     const int32_t* steps_dev, int steps_host, int slots, int T, int Hk,
                                     int Hv, int Dk, int Dv, int state_dtype, int tape_dtype, int k_dtype,
                                     int g_dtype, int g_per_dk, int exact_order, int keep, int C,
                                     int qkv_elem_bytes, void* stream) {
  const int rc = dflash_tape_replay(tape, k, g, state_in, state_out, steps_dev, steps_host, nullptr, slots, T, Hk,
                                    Hv, Dk, Dv, state_dtype, tape_dtype, k_dtype, g_dtype, g_per_dk, exact_order,
                                    stream);
  if (rc != DFLASH_OK || qkv == nullptr || keep <= 0) return rc;
  return dflash_conv_state_rebuild(conv_prev, qkv, conv_out, steps_dev, steps_host, slots, T, keep, C,
                                   qkv_elem_bytes, stream);
}
