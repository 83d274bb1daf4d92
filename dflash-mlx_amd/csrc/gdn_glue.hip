// GatedDeltaNet layer glue for gfx950: everything between the input projections and the
// recurrence in one launch, and the gated output norm in another.
//
// Mirrors the array operators of the reference's speculative GDN call
// (dflash_mlx/runtime.py:381-407 and :448): mask, depthwise causal conv over
// [conv_state | qkv], silu, split into q / k / v heads, rms_norm and scaling of q and k,
// g = exp(-exp(A_log) * softplus(a + dt_bias)), beta = sigmoid(b), the next conv state;
// then rms_norm(out, weight) * silu(z).  Every array-level operator of that sequence rounds
// to the array dtype once; the arithmetic inside an operator is fp32.
//
// These operators are a few hundred KB of data per layer: the point of fusing them is the
// launch count (two launches instead of about twenty elementwise kernels per layer and
// verify step), not bandwidth.
#include "dflash_common.h"

#include <cmath>

namespace dflash {
namespace {

constexpr int kWavesPerGroup = 4;
constexpr int kMaxPerLane = 4;  // head dims up to 256

struct PrepareArgs {
  const void* qkv;         // [B, S, C]
  const void* conv_state;  // [B, K-1, C] or null (zeros)
  const void* conv_w;      // [C, K]
  const void* a;           // [B, S, Hv]
  const void* b;           // [B, S, Hv]
  const void* A_log;       // [Hv]
  const void* dt_bias;     // [Hv]
  const uint8_t* mask;     // [B, S] or null
  void* conv_next;         // [B, K-1, C]
  void* q;                 // [B, S, Hk, Dk]
  void* k;                 // [B, S, Hk, Dk]
  void* v;                 // [B, S, Hv, Dv]
  float* g;                // [B, S, Hv]
  void* beta;              // [B, S, Hv]
  int B, S, Hk, Hv, Dk, Dv, K, dt, param_dt;
  float eps, scale_q, scale_k;  // scales already rounded to the array dtype
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-x)); }

// x * sigmoid(x) with the sigmoid and the product each rounded to the array dtype
__device__ __forceinline__ float silu_rounded(float x, int dt) {
  return round_through(x * round_through(sigmoid_f32(x), dt), dt);
}

// PER adjacent elements of an array of dtype dt, starting at element i (a multiple of PER):
// 2-byte types in 64-bit accesses when PER is a multiple of 4, one 32-bit access for a pair.
template <int PER>
__device__ __forceinline__ void load_adjacent(const void* p, size_t i, int dt, float (&out)[PER]) {
  if (dt == DFLASH_FP32) {
    const float* src = (const float*)p + i;
#pragma unroll
    for (int e = 0; e < PER; ++e) out[e] = src[e];
    return;
  }
  uint16_t h[PER];
  if (PER % 4 == 0) {
#pragma unroll
    for (int e = 0; e < PER; e += 4) {
      const uint2 w = *reinterpret_cast<const uint2*>((const uint16_t*)p + i + e);
      h[e] = (uint16_t)w.x, h[e + 1 < PER ? e + 1 : 0] = (uint16_t)(w.x >> 16);
      h[e + 2 < PER ? e + 2 : 0] = (uint16_t)w.y, h[e + 3 < PER ? e + 3 : 0] = (uint16_t)(w.y >> 16);
    }
  } else if (PER == 2) {
    const uint32_t w = *reinterpret_cast<const uint32_t*>((const uint16_t*)p + i);
    h[0] = (uint16_t)w, h[PER > 1 ? 1 : 0] = (uint16_t)(w >> 16);
  } else {
#pragma unroll
    for (int e = 0; e < PER; ++e) h[e] = ((const uint16_t*)p)[i + e];
  }
#pragma unroll
  for (int e = 0; e < PER; ++e) out[e] = dt == DFLASH_BF16 ? bf16_bits_to_f32(h[e]) : f16_bits_to_f32(h[e]);
}

// One wave per (batch, step, head); heads 0..Hk-1 are q, Hk..2Hk-1 are k, the rest v.  A lane
// holds PER = D / 64 adjacent channels of its head, so a row of the head is one access per lane
// and the K taps of those channels are PER * K adjacent weights.  All loads of a wave are issued
// before anything is computed: the kernel moves a few hundred KB and lives on latency.
template <int PER, int K>
__device__ __forceinline__ void prepare_head(const PrepareArgs& p, int b, int s, int h, int lane) {
  const int key_dim = p.Hk * p.Dk;
  const int C = 2 * key_dim + p.Hv * p.Dv;
  constexpr int keep = K - 1;
  const bool is_v = h >= 2 * p.Hk;
  const int D = PER * 64;
  const int cb = is_v ? 2 * key_dim + (h - 2 * p.Hk) * p.Dv : h * p.Dk;  // q and k heads are contiguous
  const int c = cb + PER * lane;

  float x[K][PER], w[PER * K];
#pragma unroll
  for (int j = 0; j < K; ++j) {
    const int r = s + j;  // row of [conv_state | qkv]
#pragma unroll
    for (int e = 0; e < PER; ++e) x[j][e] = 0.f;
    if (r < keep) {
      if (p.conv_state) load_adjacent<PER>(p.conv_state, ((size_t)b * keep + r) * C + c, p.dt, x[j]);
    } else if (p.mask == nullptr || p.mask[(size_t)b * p.S + (r - keep)]) {
      load_adjacent<PER>(p.qkv, ((size_t)b * p.S + (r - keep)) * C + c, p.dt, x[j]);
    }
  }
  load_adjacent<PER * K>(p.conv_w, (size_t)c * K, p.dt, w);
  float gate_a = 0.f, gate_b = 0.f, a_log = 0.f, bias = 0.f;
  const int hv = h - 2 * p.Hk;
  const size_t vrow = ((size_t)b * p.S + s) * p.Hv + (is_v ? hv : 0);
  if (is_v && lane == 0) {
    gate_a = load_as_f32(p.a, vrow, p.dt);
    gate_b = load_as_f32(p.b, vrow, p.dt);
    a_log = load_as_f32(p.A_log, hv, p.param_dt);
    bias = load_as_f32(p.dt_bias, hv, p.param_dt);
  }

  // the last `keep` rows of [conv_state | qkv] are the next conv state
  if (s + keep >= p.S) {
#pragma unroll
    for (int e = 0; e < PER; ++e)
      store_from_f32(p.conv_next, ((size_t)b * keep + (s + keep - p.S)) * C + c + e, x[K - 1][e], p.dt);
  }
  if (s == 0) {
    for (int r = p.S; r < keep; ++r) {  // blocks shorter than the state: old rows move up
      float old[PER];
#pragma unroll
      for (int e = 0; e < PER; ++e) old[e] = 0.f;
      if (p.conv_state) load_adjacent<PER>(p.conv_state, ((size_t)b * keep + r) * C + c, p.dt, old);
#pragma unroll
      for (int e = 0; e < PER; ++e) store_from_f32(p.conv_next, ((size_t)b * keep + (r - p.S)) * C + c + e, old[e], p.dt);
    }
  }

  float act[PER];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < K; ++j) acc += x[j][e] * w[e * K + j];
    act[e] = silu_rounded(round_through(acc, p.dt), p.dt);
    ss += act[e] * act[e];
  }

  if (is_v) {
#pragma unroll
    for (int e = 0; e < PER; ++e) store_from_f32(p.v, vrow * p.Dv + PER * lane + e, act[e], p.dt);
    if (lane == 0) {
      // a + dt_bias and the softplus live in the promoted dtype of the two operands
      const int sum_dt = p.param_dt == DFLASH_FP32 ? DFLASH_FP32 : p.dt;
      const float apb = round_through(gate_a + bias, sum_dt);
      const float sp = round_through(fmaxf(apb, 0.f) + log1pf(expf(-fabsf(apb))), sum_dt);
      p.g[vrow] = expf(-expf(a_log) * sp);
      store_from_f32(p.beta, vrow, sigmoid_f32(gate_b), p.dt);
    }
    return;
  }

  const float inv_rms = 1.0f / sqrtf(wave_sum(ss) / (float)D + p.eps);
  const bool is_q = h < p.Hk;
  const float scale = is_q ? p.scale_q : p.scale_k;
  void* out = is_q ? p.q : p.k;
  const size_t row = ((size_t)b * p.S + s) * p.Hk + (is_q ? h : h - p.Hk);
#pragma unroll
  for (int e = 0; e < PER; ++e)
    store_from_f32(out, row * p.Dk + PER * lane + e, scale * round_through(act[e] * inv_rms, p.dt), p.dt);
}

template <int K>
__global__ __launch_bounds__(kWavesPerGroup * 64) void gdn_prepare_kernel(PrepareArgs p) {
  const int lane = threadIdx.x & 63;
  const int heads = 2 * p.Hk + p.Hv;
  const long long w = (long long)blockIdx.x * kWavesPerGroup + (threadIdx.x >> 6);
  if (w >= (long long)p.B * p.S * heads) return;
  const int h = (int)(w % heads);
  const int s = (int)((w / heads) % p.S);
  const int b = (int)(w / ((long long)heads * p.S));
  switch ((h >= 2 * p.Hk ? p.Dv : p.Dk) / 64) {
    case 1: prepare_head<1, K>(p, b, s, h, lane); break;
    case 2: prepare_head<2, K>(p, b, s, h, lane); break;
    case 3: prepare_head<3, K>(p, b, s, h, lane); break;
    default: prepare_head<4, K>(p, b, s, h, lane); break;
  }
}

struct NormArgs {
  const void* x;       // [rows, D]
  const void* z;       // [rows, D]
  const void* weight;  // [D]
  void* y;             // [rows, D]
  long long rows;
  int D, dt, weight_dt;
  float eps;
};

// One wave per row: rms_norm(x, weight) * silu(z).
__global__ __launch_bounds__(kWavesPerGroup * 64) void gdn_gated_norm_kernel(NormArgs p) {
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * kWavesPerGroup + (threadIdx.x >> 6);
  if (row >= p.rows) return;
  const int per_lane = p.D / 64;
  float x[kMaxPerLane];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    x[i] = i < per_lane ? load_as_f32(p.x, (size_t)row * p.D + lane + 64 * i, p.dt) : 0.f;
    ss += x[i] * x[i];
  }
  const float inv_rms = 1.0f / sqrtf(wave_sum(ss) / (float)p.D + p.eps);
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    if (i >= per_lane) continue;
    const int c = lane + 64 * i;
    const float normed = round_through(x[i] * inv_rms * load_as_f32(p.weight, c, p.weight_dt), p.dt);
    const float gate = silu_rounded(load_as_f32(p.z, (size_t)row * p.D + c, p.dt), p.dt);
    store_from_f32(p.y, (size_t)row * p.D + c, gate * normed, p.dt);
  }
}

bool known_dtype(int dt) { return dt == DFLASH_BF16 || dt == DFLASH_FP16 || dt == DFLASH_FP32; }
bool head_dim_ok(int d) { return d > 0 && d % 64 == 0 && d <= 64 * kMaxPerLane; }

// the value a Python float takes when it meets an array of dtype dt
float as_array_scalar(double v, int dt) {
  const float f = (float)v;
  if (dt == DFLASH_FP32) return f;
  uint32_t u;
  __builtin_memcpy(&u, &f, 4);
  if (dt == DFLASH_BF16) {
    u += 0x7fffu + ((u >> 16) & 1u);
    u &= 0xffff0000u;
    float r;
    __builtin_memcpy(&r, &u, 4);
    return r;
  }
  return (float)(_Float16)f;
}

}  // namespace
}  // namespace dflash

extern "C" int dflash_gdn_prepare(const void* qkv, const void* conv_state, const void* conv_w, const void* a,
                                  const void* b, const void* A_log, const void* dt_bias, const uint8_t* mask,
                                  void* conv_next, void* q, void* k, void* v, float* g, void* beta, int B,
                                  int S, int Hk, int Hv, int Dk, int Dv, int conv_kernel, int dtype,
                                  int param_dtype, float eps, void* stream) {
  using namespace dflash;
  DFLASH_REQUIRE(qkv && conv_w && a && b && A_log && dt_bias && conv_next && q && k && v && g && beta,
                 DFLASH_ERR_ARG, "dflash_gdn_prepare: null operand");
  DFLASH_REQUIRE(known_dtype(dtype) && known_dtype(param_dtype), DFLASH_ERR_ARG,
                 "dflash_gdn_prepare: unknown dtype code");
  DFLASH_REQUIRE(B >= 0 && S >= 0 && Hk > 0 && Hv > 0 && conv_kernel >= 2 && conv_kernel <= 4, DFLASH_ERR_SHAPE,
                 "dflash_gdn_prepare: bad dimension (conv kernels of 2 to 4 taps)");
  DFLASH_REQUIRE(head_dim_ok(Dk) && head_dim_ok(Dv), DFLASH_ERR_SHAPE,
                 "dflash_gdn_prepare: head dims must be multiples of 64 up to 256, got %d and %d", Dk, Dv);
  const long long waves = (long long)B * S * (2 * Hk + Hv);
  DFLASH_REQUIRE(waves < (1ll << 31), DFLASH_ERR_SHAPE, "dflash_gdn_prepare: too many rows");
  if (B == 0) return DFLASH_OK;
  DFLASH_REQUIRE(S > 0, DFLASH_ERR_SHAPE, "dflash_gdn_prepare: empty block");
  PrepareArgs p;
  p.qkv = qkv; p.conv_state = conv_state; p.conv_w = conv_w; p.a = a; p.b = b; p.A_log = A_log;
  p.dt_bias = dt_bias; p.mask = mask; p.conv_next = conv_next; p.q = q; p.k = k; p.v = v; p.g = g;
  p.beta = beta; p.B = B; p.S = S; p.Hk = Hk; p.Hv = Hv; p.Dk = Dk; p.Dv = Dv; p.K = conv_kernel;
  p.dt = dtype; p.param_dt = param_dtype; p.eps = eps;
  const double inv_scale = 1.0 / sqrt((double)Dk);
  p.scale_q = as_array_scalar(inv_scale * inv_scale, dtype);
  p.scale_k = as_array_scalar(inv_scale, dtype);
  const unsigned groups = (unsigned)((waves + kWavesPerGroup - 1) / kWavesPerGroup);
  const dim3 grid(groups), block(kWavesPerGroup * 64);
  if (conv_kernel == 4) {
    hipLaunchKernelGGL(gdn_prepare_kernel<4>, grid, block, 0, (hipStream_t)stream, p);
  } else if (conv_kernel == 3) {
    hipLaunchKernelGGL(gdn_prepare_kernel<3>, grid, block, 0, (hipStream_t)stream, p);
  } else {
    hipLaunchKernelGGL(gdn_prepare_kernel<2>, grid, block, 0, (hipStream_t)stream, p);
  }
  DFLASH_HIP_OK(hipGetLastError());
  return DFLASH_OK;
}

extern "C" int dflash_gdn_gated_norm(const void* x, const void* z, const void* weight, void* y, long long rows,
                                     int D, int dtype, int weight_dtype, float eps, void* stream) {
  using namespace dflash;
  DFLASH_REQUIRE(x && z && weight && y, DFLASH_ERR_ARG, "dflash_gdn_gated_norm: null operand");
  DFLASH_REQUIRE(known_dtype(dtype) && known_dtype(weight_dtype), DFLASH_ERR_ARG,
                 "dflash_gdn_gated_norm: unknown dtype code");
  DFLASH_REQUIRE(rows >= 0 && rows < (1ll << 31), DFLASH_ERR_SHAPE, "dflash_gdn_gated_norm: bad row count");
  DFLASH_REQUIRE(head_dim_ok(D), DFLASH_ERR_SHAPE,
                 "dflash_gdn_gated_norm: row length must be a multiple of 64 up to 256, got %d", D);
  if (rows == 0) return DFLASH_OK;
  NormArgs p;
  p.x = x; p.z = z; p.weight = weight; p.y = y; p.rows = rows; p.D = D; p.dt = dtype;
  p.weight_dt = weight_dtype; p.eps = eps;
  const unsigned groups = (unsigned)((rows + kWavesPerGroup - 1) / kWavesPerGroup);
  hipLaunchKernelGGL(gdn_gated_norm_kernel, dim3(groups), dim3(kWavesPerGroup * 64), 0, (hipStream_t)stream, p);
  DFLASH_HIP_OK(hipGetLastError());
  return DFLASH_OK;
}
