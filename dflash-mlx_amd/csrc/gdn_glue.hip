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

// PER adjacent elements of an array, starting at element i (a multiple of PER), as raw bits
// (16-bit types zero-extended): 2-byte types in 64-bit accesses when PER is a multiple of 4, one
// 32-bit access for a pair.  Loading and interpreting are separate steps so that a wave can have
// all of its requests out before it waits for the first answer: with the dtype switch inside, every
// load sits in a branch of its own together with its conversion and is awaited there.
template <int PER>
__device__ __forceinline__ void load_adjacent_raw(const void* p, size_t i, bool wide, uint32_t (&raw)[PER]) {
  // no arithmetic on what comes back: the words stay as loaded (two elements per word for an even
  // number of 16-bit elements) until unpack_adjacent()
  if (wide) {
    const uint32_t* src = (const uint32_t*)p + i;
#pragma unroll
    for (int e = 0; e < PER; ++e) raw[e] = src[e];
  } else if (PER % 4 == 0) {
#pragma unroll
    for (int e = 0; e < PER; e += 4) {
      const uint2 w = *reinterpret_cast<const uint2*>((const uint16_t*)p + i + e);
      raw[e / 2] = w.x, raw[e / 2 + 1 < PER ? e / 2 + 1 : 0] = w.y;
    }
  } else if (PER == 2) {
    raw[0] = *reinterpret_cast<const uint32_t*>((const uint16_t*)p + i);
  } else {
#pragma unroll
    for (int e = 0; e < PER; ++e) raw[e] = ((const uint16_t*)p)[i + e];
  }
}
__device__ __forceinline__ float bits_as_f32(uint32_t bits, int dt) {
  return dt == DFLASH_BF16 ? bf16_bits_to_f32(bits) : dt == DFLASH_FP16 ? f16_bits_to_f32(bits) : __uint_as_float(bits);
}
template <int PER>
__device__ __forceinline__ void unpack_adjacent(const uint32_t (&raw)[PER], int dt, float (&out)[PER]) {
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    constexpr bool kPacked = PER % 4 == 0 || PER == 2;  // as load_adjacent_raw() packs 16-bit elements
    if (dt == DFLASH_FP32 || !kPacked) {
      out[e] = bits_as_f32(raw[e], dt);
    } else {
      out[e] = bits_as_f32((e & 1) ? raw[e / 2] >> 16 : raw[e / 2] & 0xFFFFu, dt);
    }
  }
}
__device__ __forceinline__ uint32_t load_bits(const void* p, size_t i, bool wide) {
  if (wide) return ((const uint32_t*)p)[i];
  return ((const uint16_t*)p)[i];
}
template <int PER>
__device__ __forceinline__ void load_adjacent(const void* p, size_t i, int dt, float (&out)[PER]) {
  uint32_t raw[PER];
  load_adjacent_raw<PER>(p, i, dt == DFLASH_FP32, raw);
  unpack_adjacent<PER>(raw, dt, out);
}
// PER adjacent elements stored from fp32 (round to nearest even), packed like the loads.
template <int PER>
__device__ __forceinline__ void store_adjacent(void* p, size_t i, int dt, const float (&v)[PER]) {
  if (dt == DFLASH_FP32) {
    float* dst = (float*)p + i;
#pragma unroll
    for (int e = 0; e < PER; ++e) dst[e] = v[e];
    return;
  }
  uint32_t h[PER];
#pragma unroll
  for (int e = 0; e < PER; ++e) h[e] = dt == DFLASH_BF16 ? f32_to_bf16_bits(v[e]) : f32_to_f16_bits(v[e]);
  if (PER % 4 == 0) {
#pragma unroll
    for (int e = 0; e < PER; e += 4)
      *reinterpret_cast<uint2*>((uint16_t*)p + i + e) =
          uint2{h[e] | (h[e + 1 < PER ? e + 1 : 0] << 16), h[e + 2 < PER ? e + 2 : 0] | (h[e + 3 < PER ? e + 3 : 0] << 16)};
  } else if (PER == 2) {
    *reinterpret_cast<uint32_t*>((uint16_t*)p + i) = h[0] | (h[PER > 1 ? 1 : 0] << 16);
  } else {
#pragma unroll
    for (int e = 0; e < PER; ++e) ((uint16_t*)p)[i + e] = (uint16_t)h[e];
  }
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

  const bool wide = p.dt == DFLASH_FP32, pwide = p.param_dt == DFLASH_FP32;
  // Every load below is unconditional: which row of which array a tap comes from, and whether it
  // counts at all, is decided by selecting the address (a tap that does not count reads some
  // readable row and is zeroed afterwards).  Loads inside branches, with the registers they
  // write preset to zero, make the compiler wait for earlier loads that used the same registers.
  uint32_t xr[K][PER], wr[PER * K], mask_byte[K];
  bool counts[K];
#pragma unroll
  for (int j = 0; j < K; ++j) {
    const int r = s + j;  // row of [conv_state | qkv]
    const bool from_state = r < keep;
    counts[j] = !from_state || p.conv_state != nullptr;
    const void* base = (from_state && p.conv_state != nullptr) ? p.conv_state : p.qkv;
    const size_t row = !counts[j] ? (size_t)b * p.S
                                  : from_state ? (size_t)b * keep + r : (size_t)b * p.S + (r - keep);
    load_adjacent_raw<PER>(base, row * C + c, wide, xr[j]);
    // the mask byte of a qkv row; without a mask (or for a state row) some byte that is not looked at
    const uint8_t* mp = (p.mask != nullptr && !from_state) ? p.mask + (size_t)b * p.S + (r - keep)
                                                           : (const uint8_t*)p.qkv;
    mask_byte[j] = *mp;
  }
  load_adjacent_raw<PER * K>(p.conv_w, (size_t)c * K, wide, wr);
  const int hv = h - 2 * p.Hk;
  const size_t vrow = ((size_t)b * p.S + s) * p.Hv + (is_v ? hv : 0);
  // gates of the value head (key heads read head 0's and do not use them)
  const uint32_t a_bits = load_bits(p.a, vrow, wide);
  const uint32_t b_bits = load_bits(p.b, vrow, wide);
  const uint32_t a_log_bits = load_bits(p.A_log, is_v ? hv : 0, pwide);
  const uint32_t bias_bits = load_bits(p.dt_bias, is_v ? hv : 0, pwide);
  asm volatile("" ::: "memory");  // every request above is out before the first value is interpreted
  float x[K][PER], w[PER * K];
#pragma unroll
  for (int j = 0; j < K; ++j) {
    unpack_adjacent<PER>(xr[j], p.dt, x[j]);
    {
      const bool from_state = s + j < keep;
      const bool on = counts[j] && (p.mask == nullptr || from_state || mask_byte[j] != 0);
#pragma unroll
      for (int e = 0; e < PER; ++e) x[j][e] = on ? x[j][e] : 0.f;
    }
  }
  unpack_adjacent<PER * K>(wr, p.dt, w);
  const float gate_a = bits_as_f32(a_bits, p.dt), gate_b = bits_as_f32(b_bits, p.dt);
  const float a_log = bits_as_f32(a_log_bits, p.param_dt), bias = bits_as_f32(bias_bits, p.param_dt);

  // the last `keep` rows of [conv_state | qkv] are the next conv state
  if (s + keep >= p.S) store_adjacent<PER>(p.conv_next, ((size_t)b * keep + (s + keep - p.S)) * C + c, p.dt, x[K - 1]);
  if (s == 0) {
    for (int r = p.S; r < keep; ++r) {  // blocks shorter than the state: old rows move up
      float old[PER];
#pragma unroll
      for (int e = 0; e < PER; ++e) old[e] = 0.f;
      if (p.conv_state) load_adjacent<PER>(p.conv_state, ((size_t)b * keep + r) * C + c, p.dt, old);
      store_adjacent<PER>(p.conv_next, ((size_t)b * keep + (r - p.S)) * C + c, p.dt, old);
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
    store_adjacent<PER>(p.v, vrow * p.Dv + PER * lane, p.dt, act);
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
  float scaled[PER];
#pragma unroll
  for (int e = 0; e < PER; ++e) scaled[e] = scale * round_through(act[e] * inv_rms, p.dt);
  store_adjacent<PER>(out, row * p.Dk + PER * lane, p.dt, scaled);
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

// One wave per row: rms_norm(x, weight) * silu(z); a lane holds PER = D / 64 adjacent elements.
template <int PER>
__device__ __forceinline__ void gated_norm_row(const NormArgs& p, long long row, int lane) {
  const bool wide = p.dt == DFLASH_FP32;
  const size_t at = (size_t)row * p.D + PER * lane;
  uint32_t xr[PER], zr[PER], wr[PER];
  load_adjacent_raw<PER>(p.x, at, wide, xr);
  load_adjacent_raw<PER>(p.z, at, wide, zr);
  load_adjacent_raw<PER>(p.weight, PER * lane, p.weight_dt == DFLASH_FP32, wr);
  asm volatile("" ::: "memory");  // all three requests are out before the first value is interpreted
  float x[PER], z[PER], wt[PER];
  unpack_adjacent<PER>(xr, p.dt, x);
  unpack_adjacent<PER>(zr, p.dt, z);
  unpack_adjacent<PER>(wr, p.weight_dt, wt);
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < PER; ++e) ss += x[e] * x[e];
  const float inv_rms = 1.0f / sqrtf(wave_sum(ss) / (float)p.D + p.eps);
  float y[PER];
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    const float normed = round_through(x[e] * inv_rms * wt[e], p.dt);
    y[e] = silu_rounded(z[e], p.dt) * normed;
  }
  store_adjacent<PER>(p.y, at, p.dt, y);
}

__global__ __launch_bounds__(kWavesPerGroup * 64) void gdn_gated_norm_kernel(NormArgs p) {
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * kWavesPerGroup + (threadIdx.x >> 6);
  if (row >= p.rows) return;
  switch (p.D / 64) {
    case 1: gated_norm_row<1>(p, row, lane); break;
    case 2: gated_norm_row<2>(p, row, lane); break;
    case 3: gated_norm_row<3>(p, row, lane); break;
    default: gated_norm_row<4>(p, row, lane); break;
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
