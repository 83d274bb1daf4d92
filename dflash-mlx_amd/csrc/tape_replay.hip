// GatedDeltaNet tape replay for gfx950 (MI355X).
//
// Counterpart of the reference's `tape_replay{,_vec}{,_mask}` Metal kernels
// (dflash_mlx/kernels.py:227-325, dispatcher :361-407; array-op form :328-358):
// re-apply the first `steps` recorded (k_t, delta_t, g_t) updates to a recurrent
// state S[Dv][Dk] (Dk contiguous),
//     S[dv][dk] <- g_t * S[dv][dk] + k_t[dk] * delta_t[dv].
//
// The operation moves 2*Dv*Dk*4 bytes of state per head and almost nothing
// else, so it is laid out for HBM streaming, not for the matrix cores:
//  * one workgroup per (slot, value head); a thread owns one float4 column of
//    Dk and walks the rows, so every wave load/store is 512 contiguous bytes
//    and the whole 64 KiB tile of a 128x128 head is in flight at once;
//  * the tape (k, delta, g of <= T steps) is staged once into LDS as fp32;
//  * for an fp32 state the T sequential sweeps are folded into a single sweep
//    using  S_a = (prod g) S0 + sum_t delta_t (x) (c_t k_t),  c_t = prod_{u>t} g_u
//    (c_t folded into the staged k rows, per-Dk gates included), which halves
//    the VALU work - at 16 steps the step-by-step form would be VALU-bound
//    before it is HBM-bound on this part.  bf16/fp16 states, which the
//    reference rounds after every step (kernels.py:281-283), and callers that
//    ask for it keep the step-by-step order;
//  * the accepted length is read per slot from device memory, so a rollback
//    does not need the host to know it, and one launch covers all layers.
#include "dflash_common.h"

namespace dflash {
namespace {

constexpr int kThreads = 256;

struct ReplayArgs {
  const void* tape;
  const void* k;
  const void* g;
  const void* state_in;
  void* state_out;
  const int32_t* steps_dev;
  const uint8_t* mask;
  int steps_host;
  int T, Hk, Hv, Dk, Dv;
  int state_dtype, tape_dtype, k_dtype, g_dtype, g_per_dk;
};

// LDS layout (floats): sA[Dv][T] (delta, t contiguous) | sK[T][Dk] | sG[T][Dk or 1] | sGt[Dk]
struct Smem {
  float* sA;
  float* sK;
  float* sG;
  float* sGt;
};

// `Tl` is the number of step slots the LDS tables hold (>= the steps staged).
__device__ __forceinline__ Smem carve(float* base, const ReplayArgs& a, int Tl) {
  Smem s;
  s.sA = base;
  s.sK = s.sA + (size_t)a.Dv * Tl;
  s.sG = s.sK + (size_t)Tl * a.Dk;
  s.sGt = s.sG + (size_t)Tl * (a.g_per_dk ? a.Dk : 1);
  return s;
}

// Stage the first `n` steps of this (slot, head) into LDS tables of `Tl` step
// slots.  Masked steps become delta = 0, k = 0, g = 1 (a no-op step) so later code
// need not look at the mask; step slots n..fill-1 are zero-filled (g = 1) as well.
__device__ __forceinline__ void stage_tape(const ReplayArgs& a, const Smem& s, int slot, int hv,
                                           int n, int Tl, int fill) {
  const int hk = hv / (a.Hv / a.Hk);
  const int tid = threadIdx.x;
  const size_t slotT = (size_t)slot * a.T;
  for (int i = tid; i < fill * a.Dv; i += kThreads) {
    const int t = i / a.Dv, dv = i - t * a.Dv;
    float d = 0.f;
    if (t < n && (a.mask == nullptr || a.mask[slotT + t] != 0)) {
      d = load_as_f32(a.tape, ((slotT + t) * a.Hv + hv) * a.Dv + dv, a.tape_dtype);
    }
    s.sA[(size_t)dv * Tl + t] = d;
  }
  for (int i = tid; i < fill * a.Dk; i += kThreads) {
    const int t = i / a.Dk, dk = i - t * a.Dk;
    const bool on = t < n && (a.mask == nullptr || a.mask[slotT + t] != 0);
    float kv = 0.f;
    if (on) kv = load_as_f32(a.k, ((slotT + t) * a.Hk + hk) * a.Dk + dk, a.k_dtype);
    s.sK[i] = kv;
    if (a.g_per_dk) {
      float gv = 1.f;
      if (on) gv = load_as_f32(a.g, ((slotT + t) * a.Hv + hv) * a.Dk + dk, a.g_dtype);
      s.sG[i] = gv;
    }
  }
  if (!a.g_per_dk) {
    for (int t = tid; t < fill; t += kThreads) {
      float gv = 1.f;
      if (t < n && (a.mask == nullptr || a.mask[slotT + t] != 0)) {
        gv = load_as_f32(a.g, (slotT + t) * a.Hv + hv, a.g_dtype);
      }
      s.sG[t] = gv;
    }
  }
}

// Fold the suffix products of g into the staged k rows; leave prod(g) in sGt.
__device__ __forceinline__ void fold_gates(const ReplayArgs& a, const Smem& s, int n) {
  for (int dk = threadIdx.x; dk < a.Dk; dk += kThreads) {
    float c = 1.f;
    for (int t = n - 1; t >= 0; --t) {
      s.sK[(size_t)t * a.Dk + dk] *= c;
      c *= a.g_per_dk ? s.sG[(size_t)t * a.Dk + dk] : s.sG[t];
    }
    s.sGt[dk] = c;
  }
}

__device__ __forceinline__ int slot_steps(const ReplayArgs& a, int slot) {
  int n = a.steps_dev ? a.steps_dev[slot] : a.steps_host;
  n = n < 0 ? 0 : n;
  return n > a.T ? a.T : n;
}

// ---------------------------------------------------------------------------
// fp32 state, Dk = Dv = 128, T <= 16: register-resident single sweep.
// Thread (row0 = tid/32, c4 = tid%32) owns float4 column c4 of rows row0 + 8*i.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void replay_f32_128(ReplayArgs a) {
  extern __shared__ float smem[];
  constexpr int Tl = 16;
  const Smem s = carve(smem, a, Tl);
  const int slot = blockIdx.x / a.Hv, hv = blockIdx.x % a.Hv;
  const int n = slot_steps(a, slot);
  const int tid = threadIdx.x, c4 = tid & 31, row0 = tid >> 5;

  const f32x4_t* in = reinterpret_cast<const f32x4_t*>(a.state_in) + (size_t)blockIdx.x * (128 * 32);
  f32x4_t* out = reinterpret_cast<f32x4_t*>(a.state_out) + (size_t)blockIdx.x * (128 * 32);

  // The tape is asked for first and the state right behind it: loads return in issue order,
  // so the tape is in LDS and the gates are folded while the 64 KiB of state are still on
  // their way, instead of the state waiting in registers for the tape.
  float td[8], tk[8], tg[8];
  float tg1 = 1.f;
  {
    const int hk = hv / (a.Hv / a.Hk);
    const size_t slotT = (size_t)slot * a.T;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = tid + kThreads * j, t = i >> 7, d = i & 127;  // step, element
      const bool on = t < n && (a.mask == nullptr || a.mask[slotT + t] != 0);
      td[j] = 0.f, tk[j] = 0.f, tg[j] = 1.f;
      if (on) {
        td[j] = load_as_f32(a.tape, ((slotT + t) * a.Hv + hv) * 128 + d, a.tape_dtype);
        tk[j] = load_as_f32(a.k, ((slotT + t) * a.Hk + hk) * 128 + d, a.k_dtype);
        if (a.g_per_dk) tg[j] = load_as_f32(a.g, ((slotT + t) * a.Hv + hv) * 128 + d, a.g_dtype);
      }
    }
    if (!a.g_per_dk && tid < Tl) {
      if (tid < n && (a.mask == nullptr || a.mask[slotT + tid] != 0))
        tg1 = load_as_f32(a.g, (slotT + tid) * a.Hv + hv, a.g_dtype);
    }
  }

  f32x4_t st[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) st[i] = __builtin_nontemporal_load(&in[(row0 + 8 * i) * 32 + c4]);

  // same tables as stage_tape(): masked and missing steps are (delta = 0, k = 0, g = 1)
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int i = tid + kThreads * j, t = i >> 7, d = i & 127;
    s.sA[(size_t)d * Tl + t] = td[j];
    s.sK[i] = tk[j];
    if (a.g_per_dk) s.sG[i] = tg[j];
  }
  if (!a.g_per_dk && tid < Tl) s.sG[tid] = tg1;
  __syncthreads();
  fold_gates(a, s, n);
  __syncthreads();

  float4 bk[16];
#pragma unroll
  for (int t = 0; t < 16; ++t) bk[t] = reinterpret_cast<const float4*>(s.sK + (size_t)t * 128)[c4];
  const float4 gt = reinterpret_cast<const float4*>(s.sGt)[c4];

#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int row = row0 + 8 * i;
    f32x4_t v = st[i];
    v.x *= gt.x;
    v.y *= gt.y;
    v.z *= gt.z;
    v.w *= gt.w;
    const float4* dl = reinterpret_cast<const float4*>(s.sA + (size_t)row * Tl);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float4 d4 = dl[q];
      const float d[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float4 b = bk[4 * q + u];
        v.x += d[u] * b.x;
        v.y += d[u] * b.y;
        v.z += d[u] * b.z;
        v.w += d[u] * b.w;
      }
    }
    __builtin_nontemporal_store(v, &out[row * 32 + c4]);
  }
}

// ---------------------------------------------------------------------------
// Generic shapes / dtypes.  EXACT = step-by-step order with a round-trip through
// the state dtype after every step; otherwise the folded single sweep (fp32 state).
// ---------------------------------------------------------------------------
template <bool EXACT>
__global__ __launch_bounds__(kThreads) void replay_generic(ReplayArgs a) {
  extern __shared__ float smem[];
  const Smem s = carve(smem, a, a.T);
  const int slot = blockIdx.x / a.Hv, hv = blockIdx.x % a.Hv;
  const int n = slot_steps(a, slot);
  const int dk4n = a.Dk >> 2;
  const size_t base = (size_t)blockIdx.x * a.Dv * a.Dk;

  stage_tape(a, s, slot, hv, n, a.T, n);
  __syncthreads();
  if (!EXACT) {
    fold_gates(a, s, n);
    __syncthreads();
  }

  for (int e = threadIdx.x; e < a.Dv * dk4n; e += kThreads) {
    const int dv = e / dk4n, c4 = e - dv * dk4n;
    const size_t off = base + (size_t)dv * a.Dk + 4 * c4;
    float v[4];
    if (a.state_dtype == DFLASH_FP32) {
      const float4 q = *reinterpret_cast<const float4*>((const float*)a.state_in + off);
      v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = load_as_f32(a.state_in, off + j, a.state_dtype);
    }
    const float* dl = s.sA + (size_t)dv * a.T;
    if (EXACT) {
      // masked steps were staged as (delta=0, k=0, g=1): s*1 + 0*0 keeps s bit-for-bit
      for (int t = 0; t < n; ++t) {
        const float d = dl[t];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float gv = a.g_per_dk ? s.sG[(size_t)t * a.Dk + 4 * c4 + j] : s.sG[t];
          float sv = v[j] * gv;
          sv = sv + s.sK[(size_t)t * a.Dk + 4 * c4 + j] * d;
          v[j] = round_through(sv, a.state_dtype);
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] *= s.sGt[4 * c4 + j];
      for (int t = 0; t < n; ++t) {
        const float d = dl[t];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] += d * s.sK[(size_t)t * a.Dk + 4 * c4 + j];
      }
    }
    if (a.state_dtype == DFLASH_FP32) {
      *reinterpret_cast<float4*>((float*)a.state_out + off) = make_float4(v[0], v[1], v[2], v[3]);
    } else if (a.state_dtype == DFLASH_BF16) {
#pragma unroll
      for (int j = 0; j < 4; ++j) ((uint16_t*)a.state_out)[off + j] = (uint16_t)f32_to_bf16_bits(v[j]);
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) ((uint16_t*)a.state_out)[off + j] = (uint16_t)f32_to_f16_bits(v[j]);
    }
  }
}

bool valid_dtype(int dt) { return dt == DFLASH_BF16 || dt == DFLASH_FP16 || dt == DFLASH_FP32; }

}  // namespace
}  // namespace dflash

extern "C" int dflash_tape_replay(const void* tape, const void* k, const void* g,
                                  const void* state_in, void* state_out, const int32_t* steps_dev,
                                  int steps_host, const uint8_t* mask, int slots, int T, int Hk,
                                  int Hv, int Dk, int Dv, int state_dtype, int tape_dtype,
                                  int k_dtype, int g_dtype, int g_per_dk, int exact_order,
                                  void* stream) {
  using namespace dflash;
  DFLASH_REQUIRE(state_in && state_out, DFLASH_ERR_ARG, "dflash_tape_replay: null state");
  DFLASH_REQUIRE(state_in != state_out, DFLASH_ERR_ARG,
                 "dflash_tape_replay: state_out must not alias state_in");
  DFLASH_REQUIRE(valid_dtype(state_dtype) && valid_dtype(tape_dtype) && valid_dtype(k_dtype) &&
                     valid_dtype(g_dtype),
                 DFLASH_ERR_ARG, "dflash_tape_replay: unknown dtype code");
  DFLASH_REQUIRE(slots >= 0 && T >= 0 && Hk > 0 && Hv > 0 && Dk > 0 && Dv > 0, DFLASH_ERR_SHAPE,
                 "dflash_tape_replay: non-positive dimension");
  DFLASH_REQUIRE(Hv % Hk == 0, DFLASH_ERR_SHAPE,
                 "dflash_tape_replay: cannot align K heads %d to tape heads %d", Hk, Hv);
  DFLASH_REQUIRE(Dk % 4 == 0 && Dk <= 1024, DFLASH_ERR_SHAPE,
                 "dflash_tape_replay: Dk=%d must be a multiple of 4 and <= 1024", Dk);
  DFLASH_REQUIRE(T == 0 || (tape && k && g), DFLASH_ERR_ARG, "dflash_tape_replay: null tape");
  if (slots == 0) return DFLASH_OK;
  const bool exact = exact_order != 0 || state_dtype != DFLASH_FP32;
  const bool fast = !exact && Dk == 128 && Dv == 128 && T <= 16;
  const size_t Tl = fast ? 16 : (size_t)T;
  const size_t smem_floats = (size_t)Dv * Tl + Tl * Dk + Tl * (g_per_dk ? Dk : 1) + (size_t)Dk;
  const size_t smem = smem_floats * sizeof(float);
  DFLASH_REQUIRE(state_dtype != DFLASH_FP32 ||
                     (((uintptr_t)state_in % 16) == 0 && ((uintptr_t)state_out % 16) == 0),
                 DFLASH_ERR_ARG, "dflash_tape_replay: fp32 state must be 16-byte aligned");
  DFLASH_REQUIRE(smem <= 64 * 1024, DFLASH_ERR_SHAPE,
                 "dflash_tape_replay: tape of T=%d steps needs %zu bytes of LDS (> 64 KiB)", T,
                 smem);
  DFLASH_REQUIRE((long long)slots * Hv < (1ll << 31), DFLASH_ERR_SHAPE,
                 "dflash_tape_replay: too many (slot, head) pairs");

  ReplayArgs a;
  a.tape = tape; a.k = k; a.g = g; a.state_in = state_in; a.state_out = state_out;
  a.steps_dev = steps_dev; a.mask = mask; a.steps_host = steps_host;
  a.T = T; a.Hk = Hk; a.Hv = Hv; a.Dk = Dk; a.Dv = Dv;
  a.state_dtype = state_dtype; a.tape_dtype = tape_dtype; a.k_dtype = k_dtype;
  a.g_dtype = g_dtype; a.g_per_dk = g_per_dk ? 1 : 0;

  const dim3 grid((unsigned)(slots * Hv)), block(kThreads);
  hipStream_t s = (hipStream_t)stream;
  if (exact) {
    hipLaunchKernelGGL(replay_generic<true>, grid, block, smem, s, a);
  } else if (fast) {
    hipLaunchKernelGGL(replay_f32_128, grid, block, smem, s, a);
  } else {
    hipLaunchKernelGGL(replay_generic<false>, grid, block, smem, s, a);
  }
  DFLASH_HIP_OK(hipGetLastError());
  return DFLASH_OK;
}
