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
  conv_rebuild_row<V>(prev, qkv, out, steps_dev ? steps_dev[slot] : steps_host, T, keep, row_bytes, slot, j);
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
