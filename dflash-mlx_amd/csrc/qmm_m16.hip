// M=16 int4 affine quantized matmul for gfx950 (MI355X), y[16,N] = x[16,K] . (s*q + b)^T.
//
// Functional counterpart of the reference's two Metal kernels
// (dflash_mlx/verify_qmm.py:28-127 `mma2big`, :130-243 `mma2big_pipe` + host
// reduction :314), designed around the CDNA4 matrix instruction instead of 8x8
// simdgroup tiles:
//
//  * One v_mfma_f32_16x16x32 covers all 16 rows of x.  Lane l supplies, for
//    output column n = l%16, the 8 consecutive-k values of k-block l/16 - which is
//    exactly one packed uint32 of the MLX layout.  The B operand is therefore
//    built in registers straight from the packed word, no LDS weight tile.
//  * The 4-bit codes are turned into bf16/fp16 *integers* with one and-or per
//    pair of codes (0x4300|q is bf16(128+q), 0x6400|q is fp16(1024+q)); the MFMA
//    runs on raw codes per quantisation group and scale/bias are applied once
//    per (column, group) to the fp32 accumulators:
//        acc += s * (sum_k x*(OFF+q)) + (b - OFF*s) * (sum_k x)
//    where the per-group row sums of x come from an MFMA against a ones operand
//    (same accumulator layout).  This costs ~1 VALU op per weight instead of ~3
//    for a per-weight dequantisation and skips the reference's per-weight
//    rounding to T (verify_qmm.py:75), i.e. it is closer to the exact affine
//    product.
//  * The and-or unpack leaves the 8 codes of a word in slot order
//    k0,k4,k1,k5,k2,k6,k3,k7; x is loaded in natural order and permuted to the
//    same slot order with four v_perm_b32 (the contraction is order-free).
//
// Work split: one workgroup (4 waves) owns 16*NT output columns and one of
// k_parts K-ranges; its waves take quantisation groups round-robin and are
// reduced through LDS.  With k_parts > 1 each workgroup stores its fp32 partial
// tile; the last workgroup to arrive for a column block (agent-scope counter)
// sums the partials in slice order and rounds once, so the result does not
// depend on arrival order.
#include <mutex>

#include "dflash_common.h"

namespace dflash {
namespace {

template <bool FP16>
struct Act;

template <>
struct Act<false> {  // bf16 activations
  static constexpr uint32_t kMagic = 0x43004300u;  // bf16 128.0 twice
  static constexpr float kOffset = 128.0f;
  static constexpr uint32_t kOnes = 0x3F803F80u;
  static __device__ __forceinline__ f32x4_t mfma(uint4 a, uint4 b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t from_f32(float v) { return f32_to_bf16_bits(v); }
};

template <>
struct Act<true> {  // fp16 activations
  static constexpr uint32_t kMagic = 0x64006400u;  // fp16 1024.0 twice
  static constexpr float kOffset = 1024.0f;
  static constexpr uint32_t kOnes = 0x3C003C00u;
  static __device__ __forceinline__ f32x4_t mfma(uint4 a, uint4 b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a),
                                                  __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t from_f32(float v) { return f32_to_f16_bits(v); }
};

template <bool FP16>
__device__ __forceinline__ float sb_to_f32(uint16_t h) {
  return FP16 ? f16_bits_to_f32(h) : bf16_bits_to_f32(h);
}

// 8 codes of one packed word -> MFMA operand, slot order k0,k4,k1,k5,k2,k6,k3,k7.
template <bool FP16>
__device__ __forceinline__ uint4 unpack_codes(uint32_t w) {
  constexpr uint32_t M = Act<FP16>::kMagic;
  uint4 r;
  r.x = (w & 0x000F000Fu) | M;
  r.y = ((w >> 4) & 0x000F000Fu) | M;
  r.z = ((w >> 8) & 0x000F000Fu) | M;
  r.w = ((w >> 12) & 0x000F000Fu) | M;
  return r;
}

// 8 consecutive 16-bit activations (natural order) -> the same slot order.
__device__ __forceinline__ uint4 permute_x(uint4 v) {
  uint4 r;
  r.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);  // (x0, x4)
  r.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);  // (x1, x5)
  r.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);  // (x2, x6)
  r.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);  // (x3, x7)
  return r;
}

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * 64;

template <int GS, bool ACT_FP16, bool SB_FP16, int NT>
__global__ __launch_bounds__(kThreads) void qmm_m16_kernel(
    const uint16_t* __restrict__ x, const uint32_t* __restrict__ w,
    const uint16_t* __restrict__ scales, const uint16_t* __restrict__ biases,
    uint16_t* __restrict__ y, float* __restrict__ partials, uint32_t* __restrict__ counters, int K,
    int N, int k_parts) {
  using A = Act<ACT_FP16>;
  constexpr int WPL = GS / 32;  // packed words (= MFMA k-steps) per lane per group

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int col = lane & 15;   // MFMA row of x (A operand) / column of W (B operand)
  const int kblk = lane >> 4;  // which quarter of the group this lane feeds
  const int n0 = blockIdx.x * (16 * NT);
  const int part = blockIdx.y;

  const int G = K / GS;
  const int g_begin = (int)(((long long)part * G) / k_parts);
  const int g_end = (int)(((long long)(part + 1) * G) / k_parts);
  const int words_per_row = K >> 3;

  f32x4_t acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  const uint4 ones = make_uint4(A::kOnes, A::kOnes, A::kOnes, A::kOnes);
  const uint16_t* xrow = x + (size_t)col * K + kblk * (GS / 4);

  for (int g = g_begin + wave; g < g_end; g += kWaves) {
    // x operands of this group: lane (m=col, kblk) holds k = g*GS + kblk*GS/4 + [0, GS/4).
    uint4 a[WPL];
#pragma unroll
    for (int j = 0; j < WPL; ++j) {
      a[j] = permute_x(*reinterpret_cast<const uint4*>(xrow + (size_t)g * GS + 8 * j));
    }
    f32x4_t xs = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < WPL; ++j) xs = A::mfma(a[j], ones, xs);

#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int n = n0 + 16 * t + col;
      const uint32_t* wp = w + (size_t)n * words_per_row + (size_t)g * (GS / 8) + kblk * WPL;
      uint32_t wd[WPL];
      if constexpr (WPL == 1) {
        wd[0] = wp[0];
      } else if constexpr (WPL == 2) {
        const uint2 v = *reinterpret_cast<const uint2*>(wp);
        wd[0] = v.x;
        wd[1] = v.y;
      } else {
        const uint4 v = *reinterpret_cast<const uint4*>(wp);
        wd[0] = v.x;
        wd[1] = v.y;
        wd[2] = v.z;
        wd[3] = v.w;
      }
      f32x4_t c = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < WPL; ++j) c = A::mfma(a[j], unpack_codes<ACT_FP16>(wd[j]), c);
      const float s = sb_to_f32<SB_FP16>(scales[(size_t)n * G + g]);
      const float b = sb_to_f32<SB_FP16>(biases[(size_t)n * G + g]);
      const float bb = b - A::kOffset * s;
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[t][r] += s * c[r] + bb * xs[r];
    }
  }

  // Cross-wave reduction.  Accumulator element (t, r) of lane l is output
  // (m = 4*(l/16) + r, n = n0 + 16*t + l%16).
  __shared__ float red[kWaves][NT][4][64];
  __shared__ int is_last;
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][t][r][lane] = acc[t][r];
  __syncthreads();

  const int r = wave;  // thread (wave, lane) now owns accumulator register r of every tile
  const int m = 4 * (lane >> 4) + r;
  float v[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    v[t] = (red[0][t][r][lane] + red[1][t][r][lane]) + (red[2][t][r][lane] + red[3][t][r][lane]);
  }

  if (k_parts == 1) {
#pragma unroll
    for (int t = 0; t < NT; ++t) y[(size_t)m * N + n0 + 16 * t + col] = (uint16_t)A::from_f32(v[t]);
    return;
  }

  // Partial tiles travel as agent-scope relaxed atomics (written through to / read from
  // the level all XCDs share).  Every wave waits until its stores are acknowledged before
  // it joins the barrier behind which the counter is bumped: the barrier alone does not -
  // a workgroup-scope fence leaves global stores in flight on this target, and the arrival
  // could overtake them, so that the last workgroup would add what an earlier call left in
  // the slot.  A release fence instead would write back the whole L2 per workgroup, which
  // costs tens of microseconds.
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    __hip_atomic_store(&partials[((size_t)part * 16 + m) * N + n0 + 16 * t + col], v[t],
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (threadIdx.x == 0) {
    // wrapping increment: the k_parts-th arrival sees k_parts-1 and puts the counter
    // back to 0 in the same atomic, which leaves the workspace ready for the next call
    const uint32_t prev = atomicInc(&counters[blockIdx.x], (uint32_t)(k_parts - 1));
    is_last = (prev == (uint32_t)(k_parts - 1));
  }
  __syncthreads();
  if (!is_last) return;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    float sum = 0.f;
    for (int p = 0; p < k_parts; ++p) {
      float* slot = &partials[((size_t)p * 16 + m) * N + n0 + 16 * t + col];
      sum += __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      // the workspace is left zero-filled: the streaming kernel, which may share it, takes a
      // non-zero word in a slot of its own for a partial tile that has arrived
      __hip_atomic_store(slot, 0.f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    y[(size_t)m * N + n0 + 16 * t + col] = (uint16_t)A::from_f32(sum);
  }
}

template <int GS, bool ACT_FP16, bool SB_FP16>
int launch(const void* x, const uint32_t* w, const void* scales, const void* biases, void* y,
           float* partials, uint32_t* counters, int K, int N, int k_parts, hipStream_t stream) {
  const dim3 block(kThreads);
  if (N % 32 == 0) {
    const dim3 grid(N / 32, k_parts);
    hipLaunchKernelGGL((qmm_m16_kernel<GS, ACT_FP16, SB_FP16, 2>), grid, block, 0, stream,
                       (const uint16_t*)x, w, (const uint16_t*)scales, (const uint16_t*)biases,
                       (uint16_t*)y, partials, counters, K, N, k_parts);
  } else {
    const dim3 grid(N / 16, k_parts);
    hipLaunchKernelGGL((qmm_m16_kernel<GS, ACT_FP16, SB_FP16, 1>), grid, block, 0, stream,
                       (const uint16_t*)x, w, (const uint16_t*)scales, (const uint16_t*)biases,
                       (uint16_t*)y, partials, counters, K, N, k_parts);
  }
  DFLASH_HIP_OK(hipGetLastError());
  return DFLASH_OK;
}

template <int GS>
int launch_gs(int act_dtype, int sb_dtype, const void* x, const uint32_t* w, const void* scales,
              const void* biases, void* y, float* partials, uint32_t* counters, int K, int N,
              int k_parts, hipStream_t stream) {
  const bool a16 = act_dtype == DFLASH_FP16, s16 = sb_dtype == DFLASH_FP16;
  if (!a16 && !s16) return launch<GS, false, false>(x, w, scales, biases, y, partials, counters, K, N, k_parts, stream);
  if (!a16 && s16) return launch<GS, false, true>(x, w, scales, biases, y, partials, counters, K, N, k_parts, stream);
  if (a16 && !s16) return launch<GS, true, false>(x, w, scales, biases, y, partials, counters, K, N, k_parts, stream);
  return launch<GS, true, true>(x, w, scales, biases, y, partials, counters, K, N, k_parts, stream);
}

// ---------------------------------------------------------------------------
// Gathered per-expert form: row p of x is multiplied by the weights of expert
// expert_ids[p].  One workgroup per (column block, expert); a workgroup whose
// expert owns no row exits at once.  Rows of one expert are collected in ascending
// row order (so results do not depend on scheduling), processed 16 at a time as the
// M dimension of the same MFMA tile, rows beyond the expert's count are zero.
// ---------------------------------------------------------------------------
constexpr int kMaxGatherRows = 2048;

template <int GS, bool ACT_FP16, bool SB_FP16, int NT>
__global__ __launch_bounds__(kThreads) void qmm_m16_gather_kernel(
    const uint16_t* __restrict__ x, const int32_t* __restrict__ expert_ids,
    const uint32_t* __restrict__ w, const uint16_t* __restrict__ scales,
    const uint16_t* __restrict__ biases, uint16_t* __restrict__ y, int P, int K, int N) {
  using A = Act<ACT_FP16>;
  constexpr int WPL = GS / 32;
  __shared__ int rows[kMaxGatherRows];
  __shared__ int n_rows;
  __shared__ float red[kWaves][NT][4][64];

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int col = lane & 15;
  const int kblk = lane >> 4;
  const int n0 = blockIdx.x * (16 * NT);
  const int e = blockIdx.y;

  // wave 0 lists the rows of expert e in ascending order
  if (wave == 0) {
    int count = 0;
    for (int base = 0; base < P; base += 64) {
      const int pidx = base + lane;
      const bool mine = pidx < P && expert_ids[pidx] == e;
      const unsigned long long m = __ballot(mine);
      if (mine) rows[count + __popcll(m & ((1ull << lane) - 1ull))] = pidx;
      count += __popcll(m);
    }
    if (lane == 0) n_rows = count;
  } else if (e == 0) {
    // A row whose expert id is outside [0, E) belongs to no expert: its output is zero (the
    // workgroups of expert 0 write it, each for its columns, so that no row of y is left as
    // it was found).
    for (int pidx = (int)threadIdx.x - 64; pidx < P; pidx += kThreads - 64) {
      const int id = expert_ids[pidx];
      if (id < 0 || id >= (int)gridDim.y) {
        for (int n = n0; n < n0 + 16 * NT && n < N; ++n) y[(size_t)pidx * N + n] = 0;
      }
    }
  }
  __syncthreads();
  const int count = n_rows;
  if (count == 0) return;

  const int G = K / GS;
  const int words_per_row = K >> 3;
  const uint32_t* we = w + (size_t)e * N * words_per_row;
  const uint16_t* se = scales + (size_t)e * N * G;
  const uint16_t* be = biases + (size_t)e * N * G;
  const uint4 ones = make_uint4(A::kOnes, A::kOnes, A::kOnes, A::kOnes);
  const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);

  for (int base = 0; base < count; base += 16) {
    const int my_row = base + col < count ? rows[base + col] : -1;
    const uint16_t* xrow = x + (size_t)(my_row < 0 ? 0 : my_row) * K + kblk * (GS / 4);
    f32x4_t acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    for (int g = wave; g < G; g += kWaves) {
      uint4 a[WPL];
#pragma unroll
      for (int j = 0; j < WPL; ++j) {
        const uint4 v = *reinterpret_cast<const uint4*>(xrow + (size_t)g * GS + 8 * j);
        a[j] = permute_x(my_row < 0 ? zero4 : v);
      }
      f32x4_t xs = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int j = 0; j < WPL; ++j) xs = A::mfma(a[j], ones, xs);
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const int n = n0 + 16 * t + col;
        const uint32_t* wp = we + (size_t)n * words_per_row + (size_t)g * (GS / 8) + kblk * WPL;
        uint32_t wd[WPL];
        if constexpr (WPL == 1) {
          wd[0] = wp[0];
        } else if constexpr (WPL == 2) {
          const uint2 v = *reinterpret_cast<const uint2*>(wp);
          wd[0] = v.x;
          wd[1] = v.y;
        } else {
          const uint4 v = *reinterpret_cast<const uint4*>(wp);
          wd[0] = v.x;
          wd[1] = v.y;
          wd[2] = v.z;
          wd[3] = v.w;
        }
        f32x4_t c = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < WPL; ++j) c = A::mfma(a[j], unpack_codes<ACT_FP16>(wd[j]), c);
        const float s = sb_to_f32<SB_FP16>(se[(size_t)n * G + g]);
        const float b = sb_to_f32<SB_FP16>(be[(size_t)n * G + g]);
        const float bb = b - A::kOffset * s;
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[t][r] += s * c[r] + bb * xs[r];
      }
    }
    __syncthreads();  // red[] of the previous 16 rows has been read
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][t][r][lane] = acc[t][r];
    __syncthreads();
    const int r = wave;
    const int m = base + 4 * (lane >> 4) + r;
    if (m < count) {
      const int out_row = rows[m];
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const float v = (red[0][t][r][lane] + red[1][t][r][lane]) + (red[2][t][r][lane] + red[3][t][r][lane]);
        y[(size_t)out_row * N + n0 + 16 * t + col] = (uint16_t)A::from_f32(v);
      }
    }
  }
}

template <int GS>
int launch_gather_gs(int act_dtype, int sb_dtype, const void* x, const int32_t* ids, const uint32_t* w,
                     const void* scales, const void* biases, void* y, int P, int K, int N, int E,
                     hipStream_t stream) {
  const bool a16 = act_dtype == DFLASH_FP16, s16 = sb_dtype == DFLASH_FP16;
  const dim3 block(kThreads);
#define DFLASH_GATHER_LAUNCH(A16, S16)                                                             \
  do {                                                                                             \
    if (N % 32 == 0) {                                                                             \
      hipLaunchKernelGGL((qmm_m16_gather_kernel<GS, A16, S16, 2>), dim3(N / 32, E), block, 0,      \
                         stream, (const uint16_t*)x, ids, w, (const uint16_t*)scales,              \
                         (const uint16_t*)biases, (uint16_t*)y, P, K, N);                          \
    } else {                                                                                       \
      hipLaunchKernelGGL((qmm_m16_gather_kernel<GS, A16, S16, 1>), dim3(N / 16, E), block, 0,      \
                         stream, (const uint16_t*)x, ids, w, (const uint16_t*)scales,              \
                         (const uint16_t*)biases, (uint16_t*)y, P, K, N);                          \
    }                                                                                              \
  } while (0)
  if (!a16 && !s16) DFLASH_GATHER_LAUNCH(false, false);
  if (!a16 && s16) DFLASH_GATHER_LAUNCH(false, true);
  if (a16 && !s16) DFLASH_GATHER_LAUNCH(true, false);
  if (a16 && s16) DFLASH_GATHER_LAUNCH(true, true);
#undef DFLASH_GATHER_LAUNCH
  DFLASH_HIP_OK(hipGetLastError());
  return DFLASH_OK;
}

// Layout of the workspace: [arrival counters, fixed 64 KiB][partials: k_parts*16*N fp32].
// The counter block has the same size for every shape so that calls of different
// shapes sharing one workspace never put partial sums where another call keeps its
// counters (counters must read zero when a call starts; so must the partials, for the sake
// of the streaming kernel, and every kernel leaves them so).
constexpr size_t kCounterBytes = 64 * 1024;
constexpr int kMaxCounterTiles = (int)(kCounterBytes / sizeof(uint32_t));

}  // namespace
}  // namespace dflash

namespace dflash {
// qmm_m16_stream.hip
bool qmm_stream_eligible(int K, int N, int group_size);
size_t qmm_stream_workspace_bytes(int N, int grid);
int qmm_stream_grid();
int qmm_stream_launch(const void* x, const uint32_t* w, const void* scales, const void* biases,
                      void* y, void* workspace, size_t workspace_bytes, int K, int N,
                      int act_dtype, int sb_dtype, hipStream_t stream);
bool qmm_stream_gather_eligible(int P, int K, int N, int E, int group_size);
int qmm_stream_gather_launch(const void* x, const int32_t* expert_ids, const uint32_t* w,
                             const void* scales, const void* biases, void* y, void* workspace,
                             size_t workspace_bytes, int P, int K, int N, int E, int act_dtype,
                             int sb_dtype, hipStream_t stream);
bool qmm_stream_packed_eligible(int K, int N, int group_size);
void qmm_stream_packed_bytes(int K, int N, size_t* w_bytes, size_t* sb_bytes);
int qmm_stream_pack(const uint32_t* w, const void* scales, const void* biases, void* w_out,
                    void* s_out, void* b_out, int K, int N, hipStream_t stream);
int qmm_stream_packed_launch(const void* x, const void* w_img, const void* s_img, const void* b_img,
                             void* y, void* workspace, size_t workspace_bytes, int K, int N,
                             int act_dtype, int sb_dtype, hipStream_t stream);
}  // namespace dflash

extern "C" size_t dflash_qmm_m16_workspace_bytes(int K, int N, int group_size, int variant,
                                                 int k_parts, int kernel) {
  size_t need = 0;
  if (N <= 0) return 0;
  if (kernel != DFLASH_QMM_KERNEL_STREAM && variant == DFLASH_QMM_MMA2BIG_PIPE && k_parts > 1) {
    need = dflash::kCounterBytes + (size_t)k_parts * 16 * (size_t)N * sizeof(float);
  }
  if (kernel != DFLASH_QMM_KERNEL_TILE && dflash::qmm_stream_eligible(K, N, group_size)) {
    const size_t s = dflash::qmm_stream_workspace_bytes(N, dflash::qmm_stream_grid());
    need = s > need ? s : need;
  }
  return need;
}

extern "C" int dflash_qmm_m16(const void* x, const uint32_t* w_q, const void* scales,
                              const void* biases, void* y, void* workspace, size_t workspace_bytes,
                              int K, int N, int group_size, int act_dtype, int sb_dtype,
                              int variant, int k_parts, int kernel, void* stream) {
  using namespace dflash;
  DFLASH_REQUIRE(x && w_q && scales && biases && y, DFLASH_ERR_ARG, "dflash_qmm_m16: null operand");
  DFLASH_REQUIRE(act_dtype == DFLASH_BF16 || act_dtype == DFLASH_FP16, DFLASH_ERR_ARG,
                 "dflash_qmm_m16: act_dtype %d is not bf16/fp16", act_dtype);
  DFLASH_REQUIRE(sb_dtype == DFLASH_BF16 || sb_dtype == DFLASH_FP16, DFLASH_ERR_ARG,
                 "dflash_qmm_m16: sb_dtype %d is not bf16/fp16", sb_dtype);
  DFLASH_REQUIRE(variant == DFLASH_QMM_MMA2BIG || variant == DFLASH_QMM_MMA2BIG_PIPE,
                 DFLASH_ERR_ARG, "dflash_qmm_m16: unknown variant %d", variant);
  DFLASH_REQUIRE(group_size == 32 || group_size == 64 || group_size == 128, DFLASH_ERR_SHAPE,
                 "dflash_qmm_m16: group_size %d not in {32,64,128}", group_size);
  DFLASH_REQUIRE(K > 0 && N > 0 && N % 16 == 0 && K % group_size == 0, DFLASH_ERR_SHAPE,
                 "dflash_qmm_m16: need N %% 16 == 0 and K %% group_size == 0 (K=%d N=%d gs=%d)", K,
                 N, group_size);
  DFLASH_REQUIRE(kernel == DFLASH_QMM_KERNEL_AUTO || kernel == DFLASH_QMM_KERNEL_TILE ||
                     kernel == DFLASH_QMM_KERNEL_STREAM,
                 DFLASH_ERR_ARG, "dflash_qmm_m16: unknown kernel selector %d", kernel);
  if (variant == DFLASH_QMM_MMA2BIG) k_parts = 1;
  DFLASH_REQUIRE(k_parts >= 1 && K % (32 * k_parts) == 0, DFLASH_ERR_SHAPE,
                 "dflash_qmm_m16: K=%d is not a multiple of 32*k_parts (k_parts=%d)", K, k_parts);
  DFLASH_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)w_q % 16) == 0, DFLASH_ERR_ARG,
                 "dflash_qmm_m16: x and w_q must be 16-byte aligned");
  if (kernel != DFLASH_QMM_KERNEL_TILE && qmm_stream_eligible(K, N, group_size)) {
    return qmm_stream_launch(x, w_q, scales, biases, y, workspace, workspace_bytes, K, N, act_dtype,
                             sb_dtype, (hipStream_t)stream);
  }
  DFLASH_REQUIRE(kernel != DFLASH_QMM_KERNEL_STREAM, DFLASH_ERR_SHAPE,
                 "dflash_qmm_m16: the streaming kernel needs group_size 64 and K %% 1024 == 0 "
                 "(K=%d gs=%d)", K, group_size);
  float* partials = nullptr;
  uint32_t* counters = nullptr;
  if (k_parts > 1) {
    const size_t need = dflash_qmm_m16_workspace_bytes(K, N, group_size, variant, k_parts,
                                                       DFLASH_QMM_KERNEL_TILE);
    DFLASH_REQUIRE(workspace && workspace_bytes >= need, DFLASH_ERR_WORKSPACE,
                   "dflash_qmm_m16: workspace of %zu bytes needed, %zu given", need,
                   workspace ? workspace_bytes : (size_t)0);
    DFLASH_REQUIRE(N / 16 <= kMaxCounterTiles, DFLASH_ERR_SHAPE,
                   "dflash_qmm_m16: N=%d exceeds the %d column tiles of the split-K path", N,
                   kMaxCounterTiles);
    counters = (uint32_t*)workspace;
    partials = (float*)((char*)workspace + kCounterBytes);
  }
  hipStream_t s = (hipStream_t)stream;
  switch (group_size) {
    case 32:
      return launch_gs<32>(act_dtype, sb_dtype, x, w_q, scales, biases, y, partials, counters, K, N, k_parts, s);
    case 64:
      return launch_gs<64>(act_dtype, sb_dtype, x, w_q, scales, biases, y, partials, counters, K, N, k_parts, s);
    default:
      return launch_gs<128>(act_dtype, sb_dtype, x, w_q, scales, biases, y, partials, counters, K, N, k_parts, s);
  }
}

// ---------------------------------------------------------------------------------
// dflash_qmm_m16_static: the same product for callers that cannot allocate.
// ---------------------------------------------------------------------------------
// The workspace of dflash_qmm_m16 (arrival counters, then fp32 partial tiles) lives in a
// device array that is part of the library's image: every GPU the library runs on holds
// its own copy from the first use to the end of the process.
constexpr size_t kStaticScratchBytes = DFLASH_QMM_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace dflash {
namespace {
// Device address of `scratch` on the current device.  In host code the array's name is only
// a handle for the runtime, never an address a kernel could use: the address is asked for
// once per device (each device has its own copy at its own address) and kept.  Nothing is
// enqueued: the array reads zero when the image is loaded, which is the state a workspace
// starts from, and every call leaves it zero-filled where the next one needs it.
int static_scratch(void** out) {
  static std::mutex mu;
  static void* ptrs[kMaxDevices] = {};
  const int slot = current_device_slot();
  std::lock_guard<std::mutex> lock(mu);
  // devices beyond the table share its last entry: looked up on every call
  if (ptrs[slot] == nullptr || slot == kMaxDevices - 1) {
    void* ptr = nullptr;
    DFLASH_HIP_OK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    DFLASH_REQUIRE(ptr != nullptr, DFLASH_ERR_HIP, "dflash_qmm_m16_static: no device address for the scratch array");
    ptrs[slot] = ptr;
  }
  *out = ptrs[slot];
  return DFLASH_OK;
}
}  // namespace
}  // namespace dflash

extern "C" int dflash_qmm_m16_static(const void* x, const uint32_t* w_q, const void* scales,
                                     const void* biases, void* y, int K, int N, int group_size,
                                     int act_dtype, int sb_dtype, int variant, int k_parts,
                                     int kernel, void* stream) {
  using namespace dflash;
  const size_t need = dflash_qmm_m16_workspace_bytes(K, N, group_size, variant,
                                                     variant == DFLASH_QMM_MMA2BIG ? 1 : k_parts, kernel);
  DFLASH_REQUIRE(need <= kStaticScratchBytes, DFLASH_ERR_WORKSPACE,
                 "dflash_qmm_m16_static: this call needs %zu bytes of scratch memory, the built-in "
                 "array holds %zu; use dflash_qmm_m16 with a workspace of the caller's",
                 need, kStaticScratchBytes);
  void* ptr = nullptr;
  const int rc = static_scratch(&ptr);
  if (rc != DFLASH_OK) return rc;
  return dflash_qmm_m16(x, w_q, scales, biases, y, ptr, kStaticScratchBytes, K, N, group_size,
                        act_dtype, sb_dtype, variant, k_parts, kernel, stream);
}

extern "C" int dflash_qmm_m16_packed_bytes(int K, int N, int group_size, size_t* codes_bytes,
                                           size_t* scales_bytes) {
  using namespace dflash;
  DFLASH_REQUIRE(codes_bytes && scales_bytes, DFLASH_ERR_ARG, "dflash_qmm_m16_packed_bytes: null result");
  DFLASH_REQUIRE(qmm_stream_packed_eligible(K, N, group_size), DFLASH_ERR_SHAPE,
                 "dflash_qmm_m16_packed_bytes: the packed form needs group_size 64, K %% 1024 == 0 and "
                 "N %% 16 == 0 (K=%d N=%d gs=%d)", K, N, group_size);
  qmm_stream_packed_bytes(K, N, codes_bytes, scales_bytes);
  return DFLASH_OK;
}

extern "C" int dflash_qmm_m16_pack(const uint32_t* w_q, const void* scales, const void* biases,
                                   void* codes_out, void* scales_out, void* biases_out, int K, int N,
                                   int group_size, void* stream) {
  using namespace dflash;
  DFLASH_REQUIRE(w_q && scales && biases && codes_out && scales_out && biases_out, DFLASH_ERR_ARG,
                 "dflash_qmm_m16_pack: null operand");
  DFLASH_REQUIRE(qmm_stream_packed_eligible(K, N, group_size), DFLASH_ERR_SHAPE,
                 "dflash_qmm_m16_pack: the packed form needs group_size 64, K %% 1024 == 0 and "
                 "N %% 16 == 0 (K=%d N=%d gs=%d)", K, N, group_size);
  DFLASH_REQUIRE(((uintptr_t)w_q % 16) == 0 && ((uintptr_t)scales % 16) == 0 && ((uintptr_t)biases % 16) == 0 &&
                     ((uintptr_t)codes_out % 16) == 0 && ((uintptr_t)scales_out % 16) == 0 &&
                     ((uintptr_t)biases_out % 16) == 0,
                 DFLASH_ERR_ARG, "dflash_qmm_m16_pack: operands must be 16-byte aligned");
  return qmm_stream_pack(w_q, scales, biases, codes_out, scales_out, biases_out, K, N, (hipStream_t)stream);
}

extern "C" int dflash_qmm_m16_packed(const void* x, const void* codes, const void* scales,
                                     const void* biases, void* y, void* workspace,
                                     size_t workspace_bytes, int K, int N, int group_size,
                                     int act_dtype, int sb_dtype, void* stream) {
  using namespace dflash;
  DFLASH_REQUIRE(x && codes && scales && biases && y, DFLASH_ERR_ARG, "dflash_qmm_m16_packed: null operand");
  DFLASH_REQUIRE(act_dtype == DFLASH_BF16 || act_dtype == DFLASH_FP16, DFLASH_ERR_ARG,
                 "dflash_qmm_m16_packed: act_dtype %d is not bf16/fp16", act_dtype);
  DFLASH_REQUIRE(sb_dtype == DFLASH_BF16 || sb_dtype == DFLASH_FP16, DFLASH_ERR_ARG,
                 "dflash_qmm_m16_packed: sb_dtype %d is not bf16/fp16", sb_dtype);
  DFLASH_REQUIRE(qmm_stream_packed_eligible(K, N, group_size), DFLASH_ERR_SHAPE,
                 "dflash_qmm_m16_packed: the packed form needs group_size 64, K %% 1024 == 0 and "
                 "N %% 16 == 0 (K=%d N=%d gs=%d)", K, N, group_size);
  DFLASH_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)codes % 16) == 0 && ((uintptr_t)scales % 16) == 0 &&
                     ((uintptr_t)biases % 16) == 0,
                 DFLASH_ERR_ARG, "dflash_qmm_m16_packed: operands must be 16-byte aligned");
  return qmm_stream_packed_launch(x, codes, scales, biases, y, workspace, workspace_bytes, K, N,
                                  act_dtype, sb_dtype, (hipStream_t)stream);
}

extern "C" size_t dflash_qmm_m16_gather_workspace_bytes(int P, int K, int N, int E,
                                                        int group_size) {
  if (!dflash::qmm_stream_gather_eligible(P, K, N, E, group_size)) return 0;
  return dflash::qmm_stream_workspace_bytes(N, dflash::qmm_stream_grid());
}

extern "C" int dflash_qmm_m16_gather(const void* x, const int32_t* expert_ids, const uint32_t* w_q,
                                     const void* scales, const void* biases, void* y,
                                     void* workspace, size_t workspace_bytes, int P, int K, int N,
                                     int E, int group_size, int act_dtype, int sb_dtype,
                                     void* stream) {
  using namespace dflash;
  DFLASH_REQUIRE(x && expert_ids && w_q && scales && biases && y, DFLASH_ERR_ARG,
                 "dflash_qmm_m16_gather: null operand");
  DFLASH_REQUIRE(act_dtype == DFLASH_BF16 || act_dtype == DFLASH_FP16, DFLASH_ERR_ARG,
                 "dflash_qmm_m16_gather: act_dtype %d is not bf16/fp16", act_dtype);
  DFLASH_REQUIRE(sb_dtype == DFLASH_BF16 || sb_dtype == DFLASH_FP16, DFLASH_ERR_ARG,
                 "dflash_qmm_m16_gather: sb_dtype %d is not bf16/fp16", sb_dtype);
  DFLASH_REQUIRE(group_size == 32 || group_size == 64 || group_size == 128, DFLASH_ERR_SHAPE,
                 "dflash_qmm_m16_gather: group_size %d not in {32,64,128}", group_size);
  DFLASH_REQUIRE(K > 0 && N > 0 && E > 0 && P >= 0 && N % 16 == 0 && K % group_size == 0,
                 DFLASH_ERR_SHAPE,
                 "dflash_qmm_m16_gather: need N %% 16 == 0 and K %% group_size == 0 (K=%d N=%d gs=%d)",
                 K, N, group_size);
  DFLASH_REQUIRE(P <= kMaxGatherRows, DFLASH_ERR_SHAPE,
                 "dflash_qmm_m16_gather: at most %d rows per call, got %d", kMaxGatherRows, P);
  DFLASH_REQUIRE(E <= 65535, DFLASH_ERR_SHAPE, "dflash_qmm_m16_gather: too many experts (%d)", E);
  DFLASH_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)w_q % 16) == 0 && (K * 2) % 16 == 0,
                 DFLASH_ERR_ARG, "dflash_qmm_m16_gather: x and w_q must be 16-byte aligned");
  if (P == 0) return DFLASH_OK;
  hipStream_t s = (hipStream_t)stream;
  // With a workspace, shapes the streaming kernel covers go through it; everything else,
  // and callers without a workspace, through the one-workgroup-per-(columns, expert) kernel.
  if (workspace != nullptr && qmm_stream_gather_eligible(P, K, N, E, group_size)) {
    return qmm_stream_gather_launch(x, expert_ids, w_q, scales, biases, y, workspace, workspace_bytes,
                                    P, K, N, E, act_dtype, sb_dtype, s);
  }
  switch (group_size) {
    case 32:
      return launch_gather_gs<32>(act_dtype, sb_dtype, x, expert_ids, w_q, scales, biases, y, P, K, N, E, s);
    case 64:
      return launch_gather_gs<64>(act_dtype, sb_dtype, x, expert_ids, w_q, scales, biases, y, P, K, N, E, s);
    default:
      return launch_gather_gs<128>(act_dtype, sb_dtype, x, expert_ids, w_q, scales, biases, y, P, K, N, E, s);
  }
}
