// GatedDeltaNet tape replay for gfx950 (MI355X).
//
// Counterpart of the reference's `tape_replay{,_vec}{,_mask}` Metal kernels
// (dflash_mlx/kernels.py:227-325, dispatcher :361-407; array-op form :328-358):
// re-apply the first `steps` recorded (k_t, delta_t, g_t) updates to a recurrent
// state S[Dv][Dk] (Dk contiguous),
//     S[dv][dk] <- g_t * S[dv][dk] + k_t[dk] * delta_t[dv].
//
// The operation moves 2*Dv*Dk*4 bytes of state per head and almost nothing
// else, so it is laid out for HBM streaming:
//  * one workgroup per (slot, value head); the whole 64 KiB tile of a 128x128
//    head is in flight at once, in and out in full 128-byte lines;
//  * the tape (k, delta, g of <= T steps) is staged once into LDS as fp32;
//  * for an fp32 state the T sequential sweeps are folded into a single one,
//      S_a = (prod g) S0 + sum_t delta_t (x) (c_t k_t),  c_t = prod_{u>t} g_u
//    (c_t folded into the staged k rows, per-Dk gates included).  For 128x128
//    that is a rank-16 update which runs on the fp32 matrix cores; as scalar
//    FMAs it costs more time than the memory traffic of the head.  bf16/fp16
//    states, which the reference rounds after every step (kernels.py:281-283),
//    and callers that ask for it keep the step-by-step order;
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
  // the conv window of the same layer, rebuilt by workgroups behind the replay's (none: conv_keep 0)
  const char* conv_prev;
  const char* conv_qkv;
  char* conv_out;
  size_t conv_row_bytes;
  int conv_keep, conv_vec16;
  int replay_blocks;  // slots * Hv
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

// Workgroups beyond the replay's own rebuild the conv window, one output row each.  True if this
// workgroup was one of them (and is done).
__device__ __forceinline__ bool conv_window_workgroup(const ReplayArgs& a) {
  if ((int)blockIdx.x < a.replay_blocks) return false;
  const int b = (int)blockIdx.x - a.replay_blocks;
  const int slot = b / a.conv_keep, j = b % a.conv_keep;
  const int steps = a.steps_dev ? a.steps_dev[slot] : a.steps_host;
  if (a.conv_vec16) conv_rebuild_row<uint4>(a.conv_prev, a.conv_qkv, a.conv_out, steps, a.T, a.conv_keep, a.conv_row_bytes, slot, j);
  else conv_rebuild_row<unsigned char>(a.conv_prev, a.conv_qkv, a.conv_out, steps, a.T, a.conv_keep, a.conv_row_bytes, slot, j);
  return true;
}

// ---------------------------------------------------------------------------
// fp32 state, Dk = Dv = 128, T <= 16: the folded sweep as a rank-16 update on the matrix cores.
//   S_out^T = diag(prod g) S_in^T + K'^T Delta,   K'[t][dk] = c_t[dk] k_t[dk]  (16 steps = 4 MFMAs
// of 16 x 16 x 4 fp32 per 16 x 16 tile).  As scalar FMAs the update costs a wave 1024
// instructions (4400 cycles) per head; with every workgroup of a CU reaching that phase at the
// same time the memory pipes idle meanwhile.  The state sits in registers in accumulator layout
// (see swap_row_bit) and goes in and out in full 128-byte lines.
// LDS (floats): sK[16][kPad] | sD[16][kPad] | sG[16][128] or [16] | sGt[128]
// ---------------------------------------------------------------------------
constexpr int kPad = 132;  // row stride of the staged tables: step rows fall on different banks
constexpr size_t replay_f32_128_lds_floats(bool g_per_dk) {
  return 2 * 16 * kPad + (g_per_dk ? 16 * 128 : 16) + 128;
}

// st (accumulator layout) <- diag(sGt) st + K'^T Delta over the first 4 NB steps; MFMA j of a tile
// covers steps 4 j + kq.
template <int NB>
__device__ __forceinline__ void rank_update(f32x4_t (&st)[2][8], const float* sK, const float* sD, const float* sGt,
                                            int wave, int li, int kq) {
  float dB[2][NB > 0 ? NB : 1];  // delta[step][32 wave + 16 t2 + li]
#pragma unroll
  for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
    for (int j = 0; j < NB; ++j) dB[t2][j] = sD[(4 * j + kq) * kPad + 32 * wave + 16 * t2 + li];
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    float kA[NB > 0 ? NB : 1];  // K'[step][16 c + li]
#pragma unroll
    for (int j = 0; j < NB; ++j) kA[j] = sK[(4 * j + kq) * kPad + 16 * c + li];
    const float4 gt4 = *reinterpret_cast<const float4*>(sGt + 16 * c + 4 * kq);
    const f32x4_t gt = {gt4.x, gt4.y, gt4.z, gt4.w};
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
      f32x4_t acc = st[t2][c] * gt;
#pragma unroll
      for (int j = 0; j < NB; ++j) acc = mfma4(kA[j], dB[t2][j], acc);
      st[t2][c] = acc;
    }
  }
}

template <bool TAPE_WIDE, bool K_WIDE>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(3, 3))) void replay_f32_128(ReplayArgs a) {
  extern __shared__ float smem[];
  float* sK = smem;
  float* sD = sK + 16 * kPad;
  float* sG = sD + 16 * kPad;
  float* sGt = sG + (a.g_per_dk ? 16 * 128 : 16);
  if (conv_window_workgroup(a)) return;
  const int slot = blockIdx.x / a.Hv, hv = blockIdx.x % a.Hv;
  const int n = slot_steps(a, slot);
  const int tid = threadIdx.x, lane = tid & 63, li = lane & 15, kq = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  const f32x4_t* in = reinterpret_cast<const f32x4_t*>(a.state_in) + (size_t)blockIdx.x * (128 * 32);
  f32x4_t* out = reinterpret_cast<f32x4_t*>(a.state_out) + (size_t)blockIdx.x * (128 * 32);

  // The tape is asked for first and the state right behind it: loads return in issue order,
  // so the tape is in LDS and the gates are folded while the 64 KiB of state are still on
  // their way, instead of the state waiting in registers for the tape.  Every request goes out
  // before anything is awaited: thread (t = tid / 16, seg = tid % 16) fetches eight elements of
  // step t as raw bits, and what the bits mean (dtype, mask) is sorted out afterwards.
  // Rows are fetched whether accepted or not (every row below T exists): the accepted length
  // may itself still be on its way from device memory, and nothing here waits for it.
  const int t = tid >> 4, seg = tid & 15;
  const bool row = t < a.T;
  const bool g_wide = a.g_dtype == DFLASH_FP32;
  // raw bytes and bits in plain registers; nothing is computed from them until the state has
  // been asked for (see the fence below)
  typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;
  u32x4_t rd0 = {0u, 0u, 0u, 0u}, rd1 = rd0, rk0 = rd0, rk1 = rd0, rg0 = rd0, rg1 = rd0;
  uint32_t mask_t = 1u, mask_g = 1u, g1_bits = 0u;
  {
    const int hk = hv / (a.Hv / a.Hk);
    const size_t slotT = (size_t)slot * a.T;
    if (row) {
      const size_t d_at = ((slotT + t) * a.Hv + hv) * 128 + 8 * seg;
      const size_t k_at = ((slotT + t) * a.Hk + hk) * 128 + 8 * seg;
      if (TAPE_WIDE) {
        rd0 = reinterpret_cast<const u32x4_t*>((const float*)a.tape + d_at)[0];
        rd1 = reinterpret_cast<const u32x4_t*>((const float*)a.tape + d_at)[1];
      } else {
        rd0 = *reinterpret_cast<const u32x4_t*>((const uint16_t*)a.tape + d_at);
      }
      if (K_WIDE) {
        rk0 = reinterpret_cast<const u32x4_t*>((const float*)a.k + k_at)[0];
        rk1 = reinterpret_cast<const u32x4_t*>((const float*)a.k + k_at)[1];
      } else {
        rk0 = *reinterpret_cast<const u32x4_t*>((const uint16_t*)a.k + k_at);
      }
      if (a.mask != nullptr) mask_t = a.mask[slotT + t];
      if (a.g_per_dk) {
        if (g_wide) {
          rg0 = reinterpret_cast<const u32x4_t*>((const float*)a.g + d_at)[0];
          rg1 = reinterpret_cast<const u32x4_t*>((const float*)a.g + d_at)[1];
        } else {
          rg0 = *reinterpret_cast<const u32x4_t*>((const uint16_t*)a.g + d_at);
        }
      }
    }
    if (!a.g_per_dk && tid < a.T && tid < 16) {  // thread t < 16 also fetches the gate of step t
      const size_t at = (slotT + tid) * a.Hv + hv;
      if (g_wide) {
        g1_bits = ((const uint32_t*)a.g)[at];
      } else {
        g1_bits = ((const uint16_t*)a.g)[at];
      }
      if (a.mask != nullptr) mask_g = a.mask[slotT + tid];
    }
  }

  f32x4_t st[2][8];
#pragma unroll
  for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
    for (int c = 0; c < 8; ++c) st[t2][c] = __builtin_nontemporal_load(&in[memory_index(wave, li, kq, t2, c)]);

  // Fence: the state's loads are out before any of the tape's values is looked at, so the
  // wait that the first use brings covers the tape only (loads return in issue order).
  asm volatile("" : "+v"(rd0), "+v"(rd1), "+v"(rk0), "+v"(rk1), "+v"(rg0), "+v"(rg1), "+v"(mask_t), "+v"(mask_g),
               "+v"(g1_bits)::"memory");

  // masked and missing steps are (delta = 0, k = 0, g = 1): no-op steps
  {
    const bool keep = t < n && mask_t != 0;
    Raw8<TAPE_WIDE> rd;
    Raw8<K_WIDE> rk;
    const u32x4_t zero = {0u, 0u, 0u, 0u};
    auto as_uint4 = [](u32x4_t v) { return uint4{v.x, v.y, v.z, v.w}; };
    rd.w[0] = as_uint4(keep ? rd0 : zero);
    rd.w[TAPE_WIDE ? 1 : 0] = as_uint4(keep ? (TAPE_WIDE ? rd1 : rd0) : zero);
    rk.w[0] = as_uint4(keep ? rk0 : zero);
    rk.w[K_WIDE ? 1 : 0] = as_uint4(keep ? (K_WIDE ? rk1 : rk0) : zero);
    raw8_to_lds<TAPE_WIDE>(rd, a.tape_dtype, sD + t * kPad + 8 * seg);
    raw8_to_lds<K_WIDE>(rk, a.k_dtype, sK + t * kPad + 8 * seg);
    if (a.g_per_dk) {
      float* dst = sG + t * 128 + 8 * seg;
      if (!keep) {
        reinterpret_cast<float4*>(dst)[0] = reinterpret_cast<float4*>(dst)[1] = float4{1.f, 1.f, 1.f, 1.f};
      } else if (g_wide) {
        Raw8<true> rg;
        rg.w[0] = as_uint4(rg0), rg.w[1] = as_uint4(rg1);
        raw8_to_lds<true>(rg, a.g_dtype, dst);
      } else {
        Raw8<false> rg;
        rg.w[0] = as_uint4(rg0);
        raw8_to_lds<false>(rg, a.g_dtype, dst);
      }
    } else if (tid < 16) {
      const bool on = tid < n && mask_g != 0;
      sG[tid] = !on ? 1.f : a.g_dtype == DFLASH_BF16 ? bf16_bits_to_f32(g1_bits)
                          : a.g_dtype == DFLASH_FP16 ? f16_bits_to_f32(g1_bits) : __uint_as_float(g1_bits);
    }
  }
  __syncthreads();
  // suffix products of the gates into the k rows; their total into sGt
  if (tid < 128) {
    float c = 1.f;
    for (int t = n - 1; t >= 0; --t) {
      sK[t * kPad + tid] *= c;
      c *= a.g_per_dk ? sG[t * 128 + tid] : sG[t];
    }
    sGt[tid] = c;
  }
  __syncthreads();

#pragma unroll
  for (int m = 0; m < 4; ++m) {
    swap_row_bit(st[0][2 * m], st[0][2 * m + 1]);
    swap_row_bit(st[1][2 * m], st[1][2 * m + 1]);
  }
  // n is uniform over the workgroup: blocks of four steps beyond it are skipped
  switch ((n + 3) >> 2) {
    case 0: rank_update<0>(st, sK, sD, sGt, wave, li, kq); break;
    case 1: rank_update<1>(st, sK, sD, sGt, wave, li, kq); break;
    case 2: rank_update<2>(st, sK, sD, sGt, wave, li, kq); break;
    case 3: rank_update<3>(st, sK, sD, sGt, wave, li, kq); break;
    default: rank_update<4>(st, sK, sD, sGt, wave, li, kq); break;
  }
#pragma unroll
  for (int m = 0; m < 4; ++m) {
    swap_row_bit(st[0][2 * m], st[0][2 * m + 1]);
    swap_row_bit(st[1][2 * m], st[1][2 * m + 1]);
  }
#pragma unroll
  for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
    for (int c = 0; c < 8; ++c) __builtin_nontemporal_store(st[t2][c], &out[memory_index(wave, li, kq, t2, c)]);
}

// ---------------------------------------------------------------------------
// Generic shapes / dtypes.  EXACT = step-by-step order with a round-trip through
// the state dtype after every step; otherwise the folded single sweep (fp32 state).
// ---------------------------------------------------------------------------
template <bool EXACT>
__global__ __launch_bounds__(kThreads) void replay_generic(ReplayArgs a) {
  extern __shared__ float smem[];
  if (conv_window_workgroup(a)) return;
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

namespace dflash {
namespace {
// The replay launch; with qkv != nullptr the conv window of the same slots rides along
// (conv_prev [slots, keep, C] or NULL, qkv [slots, T, C], conv_out [slots, keep, C]).
int replay_launch(const void* tape, const void* k, const void* g, const void* state_in, void* state_out,
                  const int32_t* steps_dev, int steps_host, const uint8_t* mask, int slots, int T, int Hk,
                  int Hv, int Dk, int Dv, int state_dtype, int tape_dtype, int k_dtype, int g_dtype,
                  int g_per_dk, int exact_order, const void* conv_prev, const void* qkv, void* conv_out,
                  int keep, int C, int qkv_elem_bytes, void* stream) {
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
  // the 128 x 128 kernel fetches tape, k and per-element gates 16 bytes at a time
  const bool aligned16 = (((uintptr_t)tape | (uintptr_t)k | (g_per_dk ? (uintptr_t)g : 0)) % 16) == 0;
  const bool fast = !exact && Dk == 128 && Dv == 128 && T <= 16 && aligned16;
  const size_t Tl = fast ? 16 : (size_t)T;
  const size_t smem_floats = fast ? replay_f32_128_lds_floats(g_per_dk != 0)
                                  : (size_t)Dv * Tl + Tl * Dk + Tl * (g_per_dk ? Dk : 1) + (size_t)Dk;
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
  a.replay_blocks = slots * Hv;
  a.conv_prev = a.conv_qkv = nullptr; a.conv_out = nullptr; a.conv_row_bytes = 0; a.conv_keep = a.conv_vec16 = 0;
  long long conv_blocks = 0;
  if (qkv != nullptr) {
    DFLASH_REQUIRE(conv_out && conv_out != conv_prev, DFLASH_ERR_ARG,
                   "dflash_rollback_layer: conv_out must be given and must not alias conv_prev");
    DFLASH_REQUIRE(T > 0 && keep > 0 && C > 0 && qkv_elem_bytes > 0, DFLASH_ERR_SHAPE,
                   "dflash_rollback_layer: non-positive dimension of the conv window");
    a.conv_prev = (const char*)conv_prev; a.conv_qkv = (const char*)qkv; a.conv_out = (char*)conv_out;
    a.conv_row_bytes = (size_t)C * qkv_elem_bytes;
    a.conv_keep = keep;
    a.conv_vec16 = a.conv_row_bytes % 16 == 0 && (uintptr_t)qkv % 16 == 0 && (uintptr_t)conv_out % 16 == 0 &&
                   (uintptr_t)conv_prev % 16 == 0;
    conv_blocks = (long long)slots * keep;
    DFLASH_REQUIRE((long long)slots * Hv + conv_blocks < (1ll << 31), DFLASH_ERR_SHAPE,
                   "dflash_rollback_layer: too many workgroups");
  }

  const dim3 grid((unsigned)(slots * Hv + conv_blocks)), block(kThreads);
  hipStream_t s = (hipStream_t)stream;
  if (exact) {
    hipLaunchKernelGGL(replay_generic<true>, grid, block, smem, s, a);
  } else if (fast) {
    const bool tw = tape_dtype == DFLASH_FP32, kw = k_dtype == DFLASH_FP32;
    if (tw && kw) hipLaunchKernelGGL((replay_f32_128<true, true>), grid, block, smem, s, a);
    else if (tw) hipLaunchKernelGGL((replay_f32_128<true, false>), grid, block, smem, s, a);
    else if (kw) hipLaunchKernelGGL((replay_f32_128<false, true>), grid, block, smem, s, a);
    else hipLaunchKernelGGL((replay_f32_128<false, false>), grid, block, smem, s, a);
  } else {
    hipLaunchKernelGGL(replay_generic<false>, grid, block, smem, s, a);
  }
  DFLASH_HIP_OK(hipGetLastError());
  return DFLASH_OK;
}
}  // namespace
}  // namespace dflash

extern "C" int dflash_tape_replay(const void* tape, const void* k, const void* g,
                                  const void* state_in, void* state_out, const int32_t* steps_dev,
                                  int steps_host, const uint8_t* mask, int slots, int T, int Hk,
                                  int Hv, int Dk, int Dv, int state_dtype, int tape_dtype,
                                  int k_dtype, int g_dtype, int g_per_dk, int exact_order,
                                  void* stream) {
  return dflash::replay_launch(tape, k, g, state_in, state_out, steps_dev, steps_host, mask, slots, T, Hk, Hv, Dk,
                               Dv, state_dtype, tape_dtype, k_dtype, g_dtype, g_per_dk, exact_order, nullptr,
                               nullptr, nullptr, 0, 0, 0, stream);
}

extern "C" int dflash_rollback_layer(const void* tape, const void* k, const void* g, const void* state_in,
                                     void* state_out, const void* conv_prev, const void* qkv, void* conv_out,
                                     const int32_t* steps_dev, int steps_host, int slots, int T, int Hk,
                                     int Hv, int Dk, int Dv, int state_dtype, int tape_dtype, int k_dtype,
                                     int g_dtype, int g_per_dk, int exact_order, int keep, int C,
                                     int qkv_elem_bytes, void* stream) {
  const bool window = qkv != nullptr && keep > 0;
  return dflash::replay_launch(tape, k, g, state_in, state_out, steps_dev, steps_host, nullptr, slots, T, Hk, Hv, Dk,
                               Dv, state_dtype, tape_dtype, k_dtype, g_dtype, g_per_dk, exact_order,
                               window ? conv_prev : nullptr, window ? qkv : nullptr, window ? conv_out : nullptr,
                               window ? keep : 0, window ? C : 0, window ? qkv_elem_bytes : 0, stream);
}
