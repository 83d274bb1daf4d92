// GatedDeltaNet forward over a block of T tokens that also records the innovation tape,
// for gfx950 (MI355X).
//
// Counterpart of the reference's `gated_delta_tape{,_vec}{,_mask}` Metal kernels
// (dflash_mlx/kernels.py:12-127; array-op form :131-173; dispatcher :176-224): for every
// (batch slot, value head), with the state S[Dv][Dk] (Dk contiguous) and for t = 0..T-1,
//     S      <- g_t * S                      (g_t a scalar per head, or one value per dk)
//     kv     =  S k_t                        (a value per dv)
//     delta  =  (v_t - kv) * beta_t
//     S      <- S + delta (x) k_t
//     y_t    =  S q_t
//     tape_t =  delta                        (fp32)
// and S rounded through the state dtype after every step (kernels.py:96-98; a no-op for an
// fp32 state).  A step whose mask byte is zero leaves S alone and gives y_t = tape_t = 0.
// The tape, with k and g, is what dflash_tape_replay needs to rebuild the state after any
// prefix of the block.
//
// Like the replay, the operation moves the state once in and once out and little else, but
// it is sequential in t, needs two reductions over dk per step, and at 16 steps its
// arithmetic costs about as much as its memory traffic.  Layout for 128 x 128 heads: one
// workgroup of 4 waves per (slot, head); a lane owns 4 rows x 16 columns of S (rows
// 32*wave + 4*(lane/8) + i; columns 4*(lane%8) + 32*c + {0..3}, c = 0..3), so that
//  * a row of S is spread over 8 neighbouring lanes: a reduction over dk is three DPP steps,
//    every lane ends up with the sums and nothing goes through LDS;
//  * every wave load or store of S is eight runs of 128 contiguous bytes;
//  * y_t = (g S) q + (k . q) delta, so one pass over S yields both sums of a step and one
//    reduction round serves both;
//  * with one gate per head and an fp32 state the decay is not applied to S at all: the
//    kernel keeps S / c with c = prod g, scales the two sums and delta instead, and
//    multiplies c back in once at the end (renormalising if c gets very small).
// q, k, v, g, beta of the block are staged once in LDS as fp32.
#include "dflash_common.h"
#include <cstdlib>

namespace dflash {
namespace {

constexpr int kThreads = 256;

struct GdnArgs {
  const void* q;
  const void* k;
  const void* v;
  const void* g;
  const void* beta;
  const void* state_in;
  void* state_out;
  void* y;
  float* tape;
  const uint8_t* mask;
  int T, Hk, Hv, Dk, Dv;
  int in_dtype, g_dtype, beta_dtype, state_dtype, g_per_dk;
  // gated output norm fused behind the recurrence (block kernel only): y is then
  // silu(z) * rms_norm(recurrence output, norm_weight), z laid out like y
  const void* z;
  const void* norm_weight;  // [Dv]
  int weight_dtype;
  float eps;
};

// v + (v of the lane the DPP control names): butterfly steps inside a row of 16 lanes -
// quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror (lanes of an aligned group of 8),
// row_mirror (the two groups of 8).
template <int CTRL>
__device__ __forceinline__ float add_dpp(float v) {
  const int o = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true);
  return v + __int_as_float(o);
}
__device__ __forceinline__ float sum_over_8(float v) {
  v = add_dpp<0xB1>(v);
  v = add_dpp<0x4E>(v);
  v = add_dpp<0x141>(v);
  return v;
}
__device__ __forceinline__ float sum_over_16(float v) { return add_dpp<0x140>(sum_over_8(v)); }

__device__ __forceinline__ float dot4(const f32x4_t& s, const float4& k) {
  return s.x * k.x + s.y * k.y + s.z * k.z + s.w * k.w;
}

// ---------------------------------------------------------------------------
// Dk = Dv = 128.  LDS (floats): sQ[T][128] | sK[T][128] | sV[T][128] | sG[T][128 or 1] |
// sBeta[T] | sKQ[T].  FOLD: keep S / prod(g) instead of applying the decay (one gate per
// head, fp32 state only).
// ---------------------------------------------------------------------------
template <bool VECG, bool FOLD>
__global__ __launch_bounds__(kThreads) void gdn_forward_128(GdnArgs a) {
  static_assert(!(VECG && FOLD), "the folded decay needs one gate per head");
  extern __shared__ float smem[];
  const int T = a.T;
  float* sQ = smem;
  float* sK = sQ + T * 128;
  float* sV = sK + T * 128;
  float* sG = sV + T * 128;
  float* sBeta = sG + T * (VECG ? 128 : 1);
  float* sKQ = sBeta + T;

  const int slot = blockIdx.x / a.Hv, hv = blockIdx.x % a.Hv;
  const int hk = hv / (a.Hv / a.Hk);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c3 = lane & 7;
  const int row0 = 32 * wave + 4 * (lane >> 3);  // this lane's rows: row0 .. row0 + 3
  const size_t slotT = (size_t)slot * T;
  const bool f32_state = FOLD || a.state_dtype == DFLASH_FP32;

  // ---- state in: float4 columns c3 + 8c (c = 0..3) of 4 rows --------------------------------
  const size_t sbase = (size_t)blockIdx.x * 128 * 128;
  f32x4_t st[4][4];
  if (f32_state) {
    const f32x4_t* in = reinterpret_cast<const f32x4_t*>((const float*)a.state_in + sbase);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int c = 0; c < 4; ++c) st[i][c] = __builtin_nontemporal_load(&in[(row0 + i) * 32 + c3 + 8 * c]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          st[i][c][e] = load_as_f32(a.state_in, sbase + (size_t)(row0 + i) * 128 + 4 * (c3 + 8 * c) + e,
                                    a.state_dtype);
  }

  // ---- stage the block ---------------------------------------------------------------------
  for (int i = tid; i < T * 128; i += kThreads) {
    const int t = i >> 7, d = i & 127;
    sQ[i] = load_as_f32(a.q, ((slotT + t) * a.Hk + hk) * 128 + d, a.in_dtype);
    sK[i] = load_as_f32(a.k, ((slotT + t) * a.Hk + hk) * 128 + d, a.in_dtype);
    sV[i] = load_as_f32(a.v, ((slotT + t) * a.Hv + hv) * 128 + d, a.in_dtype);
    if (VECG) sG[i] = load_as_f32(a.g, ((slotT + t) * a.Hv + hv) * 128 + d, a.g_dtype);
  }
  for (int t = tid; t < T; t += kThreads) {
    if (!VECG) sG[t] = load_as_f32(a.g, (slotT + t) * a.Hv + hv, a.g_dtype);
    sBeta[t] = load_as_f32(a.beta, (slotT + t) * a.Hv + hv, a.beta_dtype);
  }
  __syncthreads();
  // k_t . q_t: 16 lanes per step, 8 products each
  for (int t = tid >> 4; t < T; t += kThreads / 16) {
    const int c16 = tid & 15;
    float s = 0.f;
#pragma unroll
    for (int c = 0; c < 8; ++c) s += sK[t * 128 + 8 * c16 + c] * sQ[t * 128 + 8 * c16 + c];
    s = sum_over_16(s);
    if (c16 == 0) sKQ[t] = s;
  }
  __syncthreads();

  float cum = 1.f;  // FOLD: the registers hold S / cum
  const size_t obase = (size_t)slot * T * a.Hv * 128 + (size_t)hv * 128;  // + t * Hv * 128 + dv
  for (int t = 0; t < T; ++t) {
    float delta[4], yv[4];
    const bool on = a.mask == nullptr || a.mask[slotT + t] != 0;
    if (on) {
      float4 kk[4], qq[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        kk[c] = reinterpret_cast<const float4*>(sK + t * 128)[c3 + 8 * c];
        qq[c] = reinterpret_cast<const float4*>(sQ + t * 128)[c3 + 8 * c];
      }
      const float4 v4 = *reinterpret_cast<const float4*>(sV + t * 128 + row0);
      const float vv[4] = {v4.x, v4.y, v4.z, v4.w};
      const float beta = sBeta[t], kq = sKQ[t];
      if (FOLD) {
        cum *= sG[t];
        if (cum < 1e-12f) {  // same for the whole workgroup: put the scale back into S
#pragma unroll
          for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int c = 0; c < 4; ++c) st[i][c] *= cum;
          cum = 1.f;
        }
      } else {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          f32x4_t g4;
          if (VECG) {
            const float4 g = reinterpret_cast<const float4*>(sG + t * 128)[c3 + 8 * c];
            g4 = f32x4_t{g.x, g.y, g.z, g.w};
          } else {
            const float g = sG[t];
            g4 = f32x4_t{g, g, g, g};
          }
#pragma unroll
          for (int i = 0; i < 4; ++i) st[i][c] *= g4;
        }
      }
      float pk[4], pq[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        pk[i] = (dot4(st[i][0], kk[0]) + dot4(st[i][1], kk[1])) + (dot4(st[i][2], kk[2]) + dot4(st[i][3], kk[3]));
        pq[i] = (dot4(st[i][0], qq[0]) + dot4(st[i][1], qq[1])) + (dot4(st[i][2], qq[2]) + dot4(st[i][3], qq[3]));
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        pk[i] = sum_over_8(pk[i]);
        pq[i] = sum_over_8(pq[i]);
      }
      const float rcum = FOLD ? 1.f / cum : 1.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (FOLD) {
          pk[i] *= cum;
          pq[i] *= cum;
        }
        delta[i] = (vv[i] - pk[i]) * beta;
        yv[i] = pq[i] + kq * delta[i];
        const float d = FOLD ? delta[i] * rcum : delta[i];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          st[i][c].x += kk[c].x * d;
          st[i][c].y += kk[c].y * d;
          st[i][c].z += kk[c].z * d;
          st[i][c].w += kk[c].w * d;
        }
      }
      if (!f32_state) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int e = 0; e < 4; ++e) st[i][c][e] = round_through(st[i][c][e], a.state_dtype);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) delta[i] = 0.f, yv[i] = 0.f;
    }
    // lane c3 = i of each group of 8 lanes writes the outputs of row row0 + i
    float d_out = delta[0], y_out = yv[0];
#pragma unroll
    for (int i = 1; i < 4; ++i) {
      d_out = c3 == i ? delta[i] : d_out;
      y_out = c3 == i ? yv[i] : y_out;
    }
    if (c3 < 4) {
      const size_t o = obase + (size_t)t * a.Hv * 128 + row0 + c3;
      a.tape[o] = d_out;
      store_from_f32(a.y, o, y_out, a.in_dtype);
    }
  }

  // ---- state out ----------------------------------------------------------------------------
  if (f32_state) {
    f32x4_t* out = reinterpret_cast<f32x4_t*>((float*)a.state_out + sbase);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        if (FOLD) st[i][c] *= cum;
        __builtin_nontemporal_store(st[i][c], &out[(row0 + i) * 32 + c3 + 8 * c]);
      }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          store_from_f32(a.state_out, sbase + (size_t)(row0 + i) * 128 + 4 * (c3 + 8 * c) + e, st[i][c][e],
                         a.state_dtype);
  }
}

// ---------------------------------------------------------------------------
// Dk = Dv = 128, T <= 16, one gate per head, fp32 state: the block in closed form.
// With c_t = prod_{u<=t} g_u (masked steps: g = 1, beta = 0) the recurrence unrolls to
//     kv_t    = c_t (S0 k_t) + sum_{s<t}  (c_t/c_s) (k_s.k_t) delta_s
//     delta_t = beta_t (v_t - kv_t)
//     y_t     = c_t (S0 q_t) + sum_{s<=t} (c_t/c_s) (k_s.q_t) delta_s
//     S_T     = c_T S0 + sum_s (c_T/c_s) delta_s (x) k_s
// In matrix form, with U = S0 K^T, W = S0 Q^T (Dv x T), L[t][s] = beta_t (c_t/c_s)(k_s.k_t) for
// s < t and Lq[t][s] = (c_t/c_s)(k_s.q_t) for s <= t:
//     Delta = R (I + L)^-T with R[dv][t] = beta_t (v_t[dv] - c_t U[dv][t]),
//     Y = c W + Delta Lq^T,     S_T^T = c_T S0^T + K^T diag(c_T/c_s) Delta^T.
// Every product runs on the matrix cores (v_mfma_f32_16x16x4_f32; with bf16 q and k the three
// big ones on the bf16 matrix cores, see split_bf16); the only serial part
// is the inverse of the T x T unit triangular matrix, once per head.  The arithmetic per
// state element drops from ~5 T vector operations to ~1.5 T matrix-core operations, which
// leaves the kernel bound by the state traffic.
//
// MFMA 16x16x4 lanes: A lane l holds A[i = l % 16][k = l / 16], B lane l holds B[k = l / 16]
// [j = l % 16], accumulator register r of lane l is C[4 (l / 16) + r][l % 16].
// Lane (li = lane % 16, kq = lane / 16) of wave w keeps S rows 32w + 16a + li (a = 0, 1),
// columns 16c + 4kq + e (c = 0..7, e = 0..3).  As the A operand of S0 K^T, component e of
// chunk c pairs with k_t[16c + 4kq + e] on the B side: the columns are only summed in another
// order.  As the accumulator of the transposed update (rows = Dk, columns = Dv) the same
// registers are C[16c + 4kq + e][row li], so the new state lands where the old one was.
// ---------------------------------------------------------------------------
constexpr int kKPad = 132;  // row pitch of K and Q in LDS, in floats
constexpr int kRPad = 17;   // row pitch of R
constexpr int kOffK = 0;
constexpr int kOffQ = kOffK + 16 * kKPad;  // Q, then Delta[t][dv]
constexpr int kOffV = kOffQ + 16 * kKPad;
constexpr int kOffR = kOffV + 16 * 128;
constexpr int kOffRat = kOffR + 128 * kRPad;  // c_t / c_s, 0 above the diagonal
constexpr int kOffLq = kOffRat + 256;
constexpr int kOffM = kOffLq + 256;  // (I + L)^-1
constexpr int kOffC = kOffM + 256;
constexpr int kOffBeta = kOffC + 16;   // 0 for masked and missing steps
constexpr int kOffGate = kOffBeta + 16;  // 1 for masked and missing steps
constexpr int kOffOn = kOffGate + 16;    // 1 for steps that count, 0 for masked and missing ones
constexpr int kOffSS = kOffOn + 16;      // [wave][step]: a wave's share of a step's sum of squares
constexpr int kChunkLdsFloats = kOffSS + 64;

// Four consecutive elements at element i (a multiple of 4) of a 16-byte aligned array.
__device__ __forceinline__ void store4_from_f32(void* p, size_t i, f32x4_t v, int dt) {
  if (dt == DFLASH_FP32) {
    *reinterpret_cast<f32x4_t*>((float*)p + i) = v;
  } else if (dt == DFLASH_BF16) {
    *reinterpret_cast<uint2*>((uint16_t*)p + i) = uint2{f32_to_bf16_bits(v.x) | (f32_to_bf16_bits(v.y) << 16),
                                                        f32_to_bf16_bits(v.z) | (f32_to_bf16_bits(v.w) << 16)};
  } else {
    *reinterpret_cast<uint2*>((uint16_t*)p + i) = uint2{f32_to_f16_bits(v.x) | (f32_to_f16_bits(v.y) << 16),
                                                        f32_to_f16_bits(v.z) | (f32_to_f16_bits(v.w) << 16)};
  }
}
// The same for values that already are representable in dt (the bits are taken, not rounded).
__device__ __forceinline__ void store4_rounded(void* p, size_t i, f32x4_t v, int dt) {
  if (dt == DFLASH_BF16) {
    *reinterpret_cast<uint2*>((uint16_t*)p + i) =
        uint2{(__float_as_uint(v.x) >> 16) | (__float_as_uint(v.y) & 0xffff0000u),
              (__float_as_uint(v.z) >> 16) | (__float_as_uint(v.w) & 0xffff0000u)};
  } else {
    store4_from_f32(p, i, v, dt);
  }
}
// ---- exact products on the 16-bit matrix cores ---------------------------------------------
// An fp32 value is the sum of three bf16 values (its leading 8 significant bits, the next 8 of
// what is left, and the rest: 24 bits in all, each piece cut off, not rounded, so every
// difference is exact), and a bf16 times a bf16 is exact in fp32.  A product of an fp32 matrix
// with a matrix whose entries are bf16 numbers can therefore run as three passes of
// v_mfma_f32_16x16x32_bf16 (9 ns for 32 steps of the sum) instead of eight of
// v_mfma_f32_16x16x4_f32 (16 ns for 4 steps): the same products, summed in fp32 in another order.
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
// the upper halves of a and b (a in the low half): two bf16 numbers, cut off
__device__ __forceinline__ uint32_t upper_halves(float a, float b) {
  return __builtin_amdgcn_perm(__float_as_uint(b), __float_as_uint(a), 0x07060302u);
}
__device__ __forceinline__ float below_bf16(float v) {  // v minus its leading 8 significant bits
  return v - __uint_as_float(__float_as_uint(v) & 0xffff0000u);
}
template <int N>
struct Pieces {  // three bf16 pieces of N fp32 values, packed in pairs
  uint32_t hi[N / 2], mid[N / 2], lo[N / 2];
};
template <int N>
__device__ __forceinline__ Pieces<N> split_bf16(const float (&f)[N]) {
  Pieces<N> p;
  float r1[N], r2[N];
#pragma unroll
  for (int j = 0; j < N; ++j) r1[j] = below_bf16(f[j]), r2[j] = below_bf16(r1[j]);
#pragma unroll
  for (int j = 0; j < N / 2; ++j) {
    p.hi[j] = upper_halves(f[2 * j], f[2 * j + 1]);
    p.mid[j] = upper_halves(r1[2 * j], r1[2 * j + 1]);
    p.lo[j] = upper_halves(r2[2 * j], r2[2 * j + 1]);
  }
  return p;
}
__device__ __forceinline__ f32x4_t mfma32_bf16(const uint32_t (&a)[4], const uint32_t (&b)[4], f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, uint4{a[0], a[1], a[2], a[3]}),
                                                 __builtin_bit_cast(bf16x8_t, uint4{b[0], b[1], b[2], b[3]}), c, 0, 0, 0);
}
__device__ __forceinline__ f32x4_t mfma16_bf16(const uint32_t (&a)[2], const uint32_t (&b)[2], f32x4_t c) {
  return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4_t, uint2{a[0], a[1]}),
                                                   __builtin_bit_cast(s16x4_t, uint2{b[0], b[1]}), c, 0, 0, 0);
}

// What one (slot, head) item brings in from memory, as it sits in registers while in flight.
template <bool WIDE>
struct Incoming {
  Raw8<WIDE> k, q, v;
  uint32_t gate_bits, beta_bits, mask_byte;  // of step tid (threads below 16), as loaded
  // fused output norm: this lane's four columns of z (step li) and of the norm weight per row tile
  uint2 z2[2], w2[2];    // 16-bit elements
  f32x4_t z4[2], w4[2];  // fp32 elements
  f32x4_t st[2][8];
};
template <bool WIDE, bool NORM>
__device__ __forceinline__ void issue_item_loads(const GdnArgs& a, int item, int tid, Incoming<WIDE>& in) {
  const int T = a.T;
  const int slot = item / a.Hv, hv = item % a.Hv, hk = hv / (a.Hv / a.Hk);
  const size_t slotT = (size_t)slot * T;
  const int lane = tid & 63, wave = tid >> 6, li = lane & 15, kq = lane >> 4;
  // the block's operands first, the state behind them: loads complete in order
#pragma unroll
  for (int j = 0; j < (WIDE ? 2 : 1); ++j) in.k.w[j] = in.q.w[j] = in.v.w[j] = uint4{0u, 0u, 0u, 0u};
  const int t = tid >> 4, seg = tid & 15;
  if (t < T) {
    const size_t kq_at = ((slotT + t) * a.Hk + hk) * 128 + 8 * seg;
    const size_t v_at = ((slotT + t) * a.Hv + hv) * 128 + 8 * seg;
    in.k = load8_raw<WIDE>(a.k, kq_at);
    in.q = load8_raw<WIDE>(a.q, kq_at);
    in.v = load8_raw<WIDE>(a.v, v_at);
  }
  // gate, beta and mask of step tid as raw bits: whether the step counts is decided once the
  // state has been asked for, so that no request waits for another one's answer
  in.gate_bits = in.beta_bits = 0u;
  in.mask_byte = 1u;
  if (tid < T && tid < 16) {
    const size_t at = (slotT + tid) * a.Hv + hv;
    if (a.g_dtype == DFLASH_FP32) {
      in.gate_bits = ((const uint32_t*)a.g)[at];
    } else {
      in.gate_bits = ((const uint16_t*)a.g)[at];
    }
    if (a.beta_dtype == DFLASH_FP32) {
      in.beta_bits = ((const uint32_t*)a.beta)[at];
    } else {
      in.beta_bits = ((const uint16_t*)a.beta)[at];
    }
    if (a.mask != nullptr) in.mask_byte = a.mask[slotT + tid];
  }
  if (NORM) {
    // ahead of the state, like every load whose width depends on a dtype: behind it, the branch
    // around such a load would leave the number of loads in flight unknown at the first wait
    const int tz = li < T ? li : T - 1;
    const size_t zb = ((slotT + tz) * a.Hv + hv) * 128;
    const bool wwide = a.weight_dtype == DFLASH_FP32;
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
      const int col = 32 * wave + 16 * t2 + 4 * kq;
      if (WIDE) {
        in.z4[t2] = *reinterpret_cast<const f32x4_t*>((const float*)a.z + zb + col);
      } else {
        in.z2[t2] = *reinterpret_cast<const uint2*>((const uint16_t*)a.z + zb + col);
      }
      if (wwide) {
        in.w4[t2] = *reinterpret_cast<const f32x4_t*>((const float*)a.norm_weight + col);
      } else {
        in.w2[t2] = *reinterpret_cast<const uint2*>((const uint16_t*)a.norm_weight + col);
      }
    }
  }
  const f32x4_t* src = reinterpret_cast<const f32x4_t*>((const float*)a.state_in + (size_t)item * 128 * 128);
#pragma unroll
  for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
    for (int c = 0; c < 8; ++c)
      in.st[t2][c] = __builtin_nontemporal_load(&src[memory_index(wave, li, kq, t2, c)]);
  // Fence: everything above is on its way before the first of these values is looked at.
  asm volatile("" : "+v"(in.gate_bits), "+v"(in.beta_bits), "+v"(in.mask_byte)::"memory");
}
__device__ __forceinline__ float bits_as_f32(uint32_t bits, int dt) {
  return dt == DFLASH_BF16 ? bf16_bits_to_f32(bits) : dt == DFLASH_FP16 ? f16_bits_to_f32(bits) : __uint_as_float(bits);
}

// One workgroup per (slot, head); the register cap keeps at least three on a compute unit.
// SPLIT: q and k are bf16 arrays; the products with S0 and the state update run on the bf16
// matrix cores with the fp32 factor in three exact pieces (see split_bf16).
template <bool WIDE, bool NORM, bool SPLIT>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(3, 3))) void gdn_forward_chunk_128(GdnArgs a) {
  extern __shared__ __align__(16) float smem[];
  float* sK = smem + kOffK;
  float* sQ = smem + kOffQ;
  float* sD = smem + kOffQ;
  float* sV = smem + kOffV;
  float* sR = smem + kOffR;
  float* sRat = smem + kOffRat;
  float* sLq = smem + kOffLq;
  float* sM = smem + kOffM;
  float* sC = smem + kOffC;
  float* sBeta = smem + kOffBeta;
  float* sGate = smem + kOffGate;
  float* sOn = smem + kOffOn;
  float* sSS = smem + kOffSS;

  const int T = a.T;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: branches on it are real branches
  const int li = lane & 15, kq = lane >> 4;

  Incoming<WIDE> cur;
  const int item = blockIdx.x;
  issue_item_loads<WIDE, NORM>(a, item, tid, cur);
  const int slot = item / a.Hv, hv = item % a.Hv;
  const size_t slotT = (size_t)slot * T;
  const size_t sbase = (size_t)item * 128 * 128;
  f32x4_t (&st)[2][8] = cur.st;
  uint2 (&z2)[2] = cur.z2, (&w2)[2] = cur.w2;
  f32x4_t (&z4)[2] = cur.z4, (&w4)[2] = cur.w4;
  {
    const int t = tid >> 4, seg = tid & 15;
    raw8_to_lds(cur.k, a.in_dtype, sK + t * kKPad + 8 * seg);
    raw8_to_lds(cur.q, a.in_dtype, sQ + t * kKPad + 8 * seg);
    raw8_to_lds(cur.v, a.in_dtype, sV + t * 128 + 8 * seg);
  }
  if (tid < 16) {
    const bool on = tid < T && cur.mask_byte != 0;  // masked and missing steps: gate 1, beta 0
    sGate[tid] = on ? bits_as_f32(cur.gate_bits, a.g_dtype) : 1.f;
    sBeta[tid] = on ? bits_as_f32(cur.beta_bits, a.beta_dtype) : 0.f;
    sOn[tid] = on ? 1.f : 0.f;
  }
  __syncthreads();
  {  // c_t / c_s = prod_{s < u <= t} g_u for s <= t, and c_t itself
    const int t = tid >> 4, sx = tid & 15;
    float gates[16];
#pragma unroll
    for (int u = 0; u < 16; u += 4) {
      const float4 g4 = *reinterpret_cast<const float4*>(sGate + u);
      gates[u] = g4.x, gates[u + 1] = g4.y, gates[u + 2] = g4.z, gates[u + 3] = g4.w;
    }
    float r = sx <= t ? 1.f : 0.f;
#pragma unroll
    for (int u = 1; u < 16; ++u) r *= (u > sx && u <= t) ? gates[u] : 1.f;
    sRat[tid] = r;
    if (sx == 0) sC[t] = r * gates[0];
  }
  __syncthreads();

  // ---- U = S0 K^T, W = S0 Q^T (every wave, its 32 rows); K K^T (wave 1), K Q^T (wave 2) -------
#pragma unroll
  for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
    for (int m = 0; m < 4; ++m) swap_row_bit(st[t2][2 * m], st[t2][2 * m + 1]);
  f32x4_t U[2], W[2], X = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int t2 = 0; t2 < 2; ++t2) U[t2] = f32x4_t{0.f, 0.f, 0.f, 0.f}, W[t2] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  if constexpr (SPLIT) {
    // Element j = 4h + e (h = 0, 1) of a lane's operand is column 16 (2C + h) + 4kq + e: the 32
    // columns 32C .. 32C + 31 over the four lane groups, the same on both sides of a product.
#pragma unroll
    for (int C = 0; C < 4; ++C) {
      uint32_t kb[4], qb[4];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const float4 kf4 = *reinterpret_cast<const float4*>(sK + li * kKPad + 16 * (2 * C + h) + 4 * kq);
        const float4 qf4 = *reinterpret_cast<const float4*>(sQ + li * kKPad + 16 * (2 * C + h) + 4 * kq);
        kb[2 * h] = upper_halves(kf4.x, kf4.y), kb[2 * h + 1] = upper_halves(kf4.z, kf4.w);
        qb[2 * h] = upper_halves(qf4.x, qf4.y), qb[2 * h + 1] = upper_halves(qf4.z, qf4.w);
      }
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) {
        const float f[8] = {st[t2][2 * C][0],     st[t2][2 * C][1],     st[t2][2 * C][2],     st[t2][2 * C][3],
                            st[t2][2 * C + 1][0], st[t2][2 * C + 1][1], st[t2][2 * C + 1][2], st[t2][2 * C + 1][3]};
        const Pieces<8> sp = split_bf16(f);
        U[t2] = mfma32_bf16(sp.lo, kb, U[t2]);
        W[t2] = mfma32_bf16(sp.lo, qb, W[t2]);
        U[t2] = mfma32_bf16(sp.mid, kb, U[t2]);
        W[t2] = mfma32_bf16(sp.mid, qb, W[t2]);
        U[t2] = mfma32_bf16(sp.hi, kb, U[t2]);
        W[t2] = mfma32_bf16(sp.hi, qb, W[t2]);
      }
      if (wave == 1) X = mfma32_bf16(kb, kb, X);  // [s][t] = k_s . k_t
      if (wave == 2) X = mfma32_bf16(kb, qb, X);  // [s][t] = k_s . q_t
    }
  } else {
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      const float4 kf4 = *reinterpret_cast<const float4*>(sK + li * kKPad + 16 * c + 4 * kq);
      const float4 qf4 = *reinterpret_cast<const float4*>(sQ + li * kKPad + 16 * c + 4 * kq);
      const float kf[4] = {kf4.x, kf4.y, kf4.z, kf4.w};
      const float qf[4] = {qf4.x, qf4.y, qf4.z, qf4.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
#pragma unroll
        for (int t2 = 0; t2 < 2; ++t2) {
          U[t2] = mfma4(st[t2][c][e], kf[e], U[t2]);
          W[t2] = mfma4(st[t2][c][e], qf[e], W[t2]);
        }
        if (wave == 1) X = mfma4(kf[e], kf[e], X);  // [s][t] = k_s . k_t
        if (wave == 2) X = mfma4(kf[e], qf[e], X);  // [s][t] = k_s . q_t
      }
    }
  }
  {
    const int t = li;
    const float ct = sC[t], bt = sBeta[t];
    float Lr[4];  // wave 1: L[t][4kq + r], wave 2: Lq[t][4kq + r]
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int sx = 4 * kq + r;
      const float rat = sRat[t * 16 + sx];  // 0 for s > t
      Lr[r] = wave == 1 ? (sx < t ? bt * rat * X[r] : 0.f) : rat * X[r];
      if (wave == 2) sLq[t * 16 + sx] = Lr[r];
    }
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
      const int row0 = 32 * wave + 16 * t2 + 4 * kq;
      const float4 v4 = *reinterpret_cast<const float4*>(sV + t * 128 + row0);
      sR[(row0 + 0) * kRPad + t] = bt * (v4.x - ct * U[t2][0]);
      sR[(row0 + 1) * kRPad + t] = bt * (v4.y - ct * U[t2][1]);
      sR[(row0 + 2) * kRPad + t] = bt * (v4.z - ct * U[t2][2]);
      sR[(row0 + 3) * kRPad + t] = bt * (v4.w - ct * U[t2][3]);
    }
    // ---- M = (I + L)^-1 by forward substitution, column li per lane.  L[t][s] sits in lane
    // 16 (s / 4) + t, register s % 4 of this wave and reaches the others through v_readlane.
    if (wave == 1) {
      float x[16];
#pragma unroll
      for (int tt = 0; tt < 16; ++tt) {
        float acc = tt == li ? 1.f : 0.f;
#pragma unroll
        for (int sx = 0; sx < tt; ++sx) {
          const float l = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(Lr[sx & 3]), 16 * (sx >> 2) + tt));
          acc -= l * x[sx];
        }
        x[tt] = acc;
        if (kq == 0) sM[tt * 16 + li] = acc;
      }
    }
  }
  __syncthreads();  // Lq, R and M are complete; nobody reads Q any more

  // ---- Delta = R M^T: rows of this wave, accumulator (row 4kq + r, column t = li) ---------------
  f32x4_t D[2];
#pragma unroll
  for (int t2 = 0; t2 < 2; ++t2) {
    D[t2] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < 4; ++j)
      D[t2] = mfma4(sR[(32 * wave + 16 * t2 + li) * kRPad + 4 * j + kq], sM[li * 16 + 4 * j + kq], D[t2]);
  }
  const size_t obase = ((slotT + li) * a.Hv + hv) * 128;  // step li of this head in y and the tape
#pragma unroll
  for (int t2 = 0; t2 < 2; ++t2) {
    const int row0 = 32 * wave + 16 * t2 + 4 * kq;
    *reinterpret_cast<f32x4_t*>(sD + li * 128 + row0) = D[t2];
  }
  {
    // the tape leaves from LDS in full 128-byte lines: lane (t, q) stores this wave's rows
    // 32 wave + 8 q ..+7 of step t (the matrix-core layout would give 64-byte pieces)
    const int t = lane >> 2, dv0 = 32 * wave + 8 * (lane & 3);
    if (t < T) {
      float* dst = a.tape + ((slotT + t) * a.Hv + hv) * 128 + dv0;
      *reinterpret_cast<f32x4_t*>(dst) = *reinterpret_cast<const f32x4_t*>(sD + t * 128 + dv0);
      *reinterpret_cast<f32x4_t*>(dst + 4) = *reinterpret_cast<const f32x4_t*>(sD + t * 128 + dv0 + 4);
    }
  }
  __syncthreads();

  // ---- Y = c W + Delta Lq^T -----------------------------------------------------------------------
  float Yn[2][4];  // fused norm: Y rounded to the array dtype, kept until every wave's sum of squares is in
  float dA[2][4];  // Delta[row 16 t2 + li][s = 4j + kq]
#pragma unroll
  for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
    for (int j = 0; j < 4; ++j) dA[t2][j] = sD[(4 * j + kq) * 128 + 32 * wave + 16 * t2 + li];
  {
    const float ct = sC[li];
    const bool on = sOn[li] != 0.f;
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
      f32x4_t Y = W[t2] * ct;
#pragma unroll
      for (int j = 0; j < 4; ++j) Y = mfma4(dA[t2][j], sLq[li * 16 + 4 * j + kq], Y);
      if (!on) Y = f32x4_t{0.f, 0.f, 0.f, 0.f};
      if (!NORM) {
        if (li < T) store4_from_f32(a.y, obase + 32 * wave + 16 * t2 + 4 * kq, Y, a.in_dtype);
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) Yn[t2][r] = round_through(Y[r], a.in_dtype);  // the recurrence's output, as an array
      }
    }
    if (NORM) {
      // this wave's 32 columns of step li: 8 per lane, the four lanes (li, kq) of a step added up
      float ss = 0.f;
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
        for (int r = 0; r < 4; ++r) ss += Yn[t2][r] * Yn[t2][r];
      ss += __shfl_xor(ss, 16, 64);
      ss += __shfl_xor(ss, 32, 64);
      if (kq == 0) sSS[16 * wave + li] = ss;  // read after the state update, behind its barrier
    }
  }

  // ---- S_T^T = c_T S0^T + K^T diag(c_T / c_s) Delta^T -----------------------------------------------
  {
    const float cT = sC[T - 1];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float cf = sRat[(T - 1) * 16 + 4 * j + kq];  // 0 beyond step T - 1
      dA[0][j] *= cf;
      dA[1][j] *= cf;
    }
    Pieces<4> dp[2];  // SPLIT: the scaled Delta in pieces; element j of a lane's operand is step 4j + kq
    if constexpr (SPLIT) {
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) dp[t2] = split_bf16(dA[t2]);
    }
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      float kA[4];  // K[s = 4j + kq][16c + li]
#pragma unroll
      for (int j = 0; j < 4; ++j) kA[j] = sK[(4 * j + kq) * kKPad + 16 * c + li];
      const uint32_t ka[2] = {upper_halves(kA[0], kA[1]), upper_halves(kA[2], kA[3])};
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) {
        f32x4_t acc = st[t2][c] * cT;
        if constexpr (SPLIT) {
          acc = mfma16_bf16(ka, dp[t2].lo, acc);
          acc = mfma16_bf16(ka, dp[t2].mid, acc);
          acc = mfma16_bf16(ka, dp[t2].hi, acc);
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) acc = mfma4(kA[j], dA[t2][j], acc);
        }
        st[t2][c] = acc;
      }
    }
  }
  if (NORM) {
    // silu(z) * rms_norm(y, weight) with the rounding points of the separate operators: y, the
    // normalised and weighted y, sigmoid(z), z * sigmoid(z) and the product are arrays of the
    // input dtype; sums and the reciprocal root are fp32.
    // a bare barrier: __syncthreads() would also wait until every store issued so far has been
    // acknowledged, and the stores of the state are about to follow
    asm volatile("s_waitcnt lgkmcnt(0)\n s_barrier" ::: "memory");
    const float total = sSS[li] + sSS[16 + li] + sSS[32 + li] + sSS[48 + li];
    float zf[2][4], wf[2][4];
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
      if (WIDE) {
#pragma unroll
        for (int r = 0; r < 4; ++r) zf[t2][r] = z4[t2][r];
      } else {
        const uint32_t h[4] = {z2[t2].x & 0xFFFFu, z2[t2].x >> 16, z2[t2].y & 0xFFFFu, z2[t2].y >> 16};
#pragma unroll
        for (int r = 0; r < 4; ++r) zf[t2][r] = bits_as_f32(h[r], a.in_dtype);
      }
      if (a.weight_dtype == DFLASH_FP32) {
#pragma unroll
        for (int r = 0; r < 4; ++r) wf[t2][r] = w4[t2][r];
      } else {
        const uint32_t h[4] = {w2[t2].x & 0xFFFFu, w2[t2].x >> 16, w2[t2].y & 0xFFFFu, w2[t2].y >> 16};
#pragma unroll
        for (int r = 0; r < 4; ++r) wf[t2][r] = bits_as_f32(h[r], a.weight_dtype);
      }
    }
    // A head's launch occupies one compute unit in eight, so whatever this tail costs per lane is
    // added to the layer's latency in full: the 16-bit dtypes take the hardware's exp2,
    // reciprocal and reciprocal root (each within an ulp of fp32, far below half an ulp of a
    // 16-bit array) and a rounding written out for the dtype; fp32 arrays keep the library forms.
    auto finish = [&](auto rnd, auto sigmoid, float inv_rms) __attribute__((always_inline)) {
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) {
        f32x4_t o;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float normed = rnd(Yn[t2][r] * inv_rms * wf[t2][r]);
          o[r] = rnd(rnd(zf[t2][r] * rnd(sigmoid(zf[t2][r]))) * normed);
        }
        if (li < T) store4_rounded(a.y, obase + 32 * wave + 16 * t2 + 4 * kq, o, a.in_dtype);
      }
    };
    auto fast_sigmoid = [](float x) { return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504088896341f * x)); };
    if (a.in_dtype == DFLASH_BF16) {
      finish([](float v) { uint32_t u = __float_as_uint(v); u += 0x7fffu + ((u >> 16) & 1u); return __uint_as_float(u & 0xffff0000u); },
             fast_sigmoid, __builtin_amdgcn_rsqf(total * (1.0f / 128.0f) + a.eps));
    } else if (a.in_dtype == DFLASH_FP16) {
      finish([](float v) { return (float)(_Float16)v; }, fast_sigmoid, __builtin_amdgcn_rsqf(total * (1.0f / 128.0f) + a.eps));
    } else {
      finish([](float v) { return v; }, [](float x) { return 1.0f / (1.0f + expf(-x)); },
             1.0f / sqrtf(total / 128.0f + a.eps));
    }
  }
  {
    f32x4_t* out = reinterpret_cast<f32x4_t*>((float*)a.state_out + sbase);
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
      for (int m = 0; m < 4; ++m) swap_row_bit(st[t2][2 * m], st[t2][2 * m + 1]);
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
      for (int c = 0; c < 8; ++c)
        __builtin_nontemporal_store(st[t2][c], &out[memory_index(wave, li, kq, t2, c)]);
  }
}

// ---------------------------------------------------------------------------
// Any Dk, Dv: one workgroup per (slot, head), a thread walks whole rows of S, which lives in
// state_out between steps (so it is rounded through the state dtype after every step by
// construction).  Slow and simple; the 128 x 128 kernel above is the one that is measured.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void gdn_forward_generic(GdnArgs a) {
  const int slot = blockIdx.x / a.Hv, hv = blockIdx.x % a.Hv;
  const int hk = hv / (a.Hv / a.Hk);
  const size_t slotT = (size_t)slot * a.T;
  const size_t sbase = (size_t)blockIdx.x * a.Dv * a.Dk;
  for (int dv = threadIdx.x; dv < a.Dv; dv += kThreads) {
    const size_t row = sbase + (size_t)dv * a.Dk;
    for (int dk = 0; dk < a.Dk; ++dk)
      store_from_f32(a.state_out, row + dk, load_as_f32(a.state_in, row + dk, a.state_dtype), a.state_dtype);
    for (int t = 0; t < a.T; ++t) {
      const size_t o = ((slotT + t) * a.Hv + hv) * a.Dv + dv;
      float delta = 0.f, y = 0.f;
      if (a.mask == nullptr || a.mask[slotT + t] != 0) {
        const size_t kq0 = ((slotT + t) * a.Hk + hk) * a.Dk;
        const size_t g0 = a.g_per_dk ? ((slotT + t) * a.Hv + hv) * a.Dk : (slotT + t) * a.Hv + hv;
        float kv = 0.f;
        for (int dk = 0; dk < a.Dk; ++dk) {
          const float g = load_as_f32(a.g, a.g_per_dk ? g0 + dk : g0, a.g_dtype);
          kv += load_as_f32(a.state_out, row + dk, a.state_dtype) * g * load_as_f32(a.k, kq0 + dk, a.in_dtype);
        }
        delta = (load_as_f32(a.v, o, a.in_dtype) - kv) * load_as_f32(a.beta, (slotT + t) * a.Hv + hv, a.beta_dtype);
        for (int dk = 0; dk < a.Dk; ++dk) {
          const float g = load_as_f32(a.g, a.g_per_dk ? g0 + dk : g0, a.g_dtype);
          const float s = load_as_f32(a.state_out, row + dk, a.state_dtype) * g +
                          load_as_f32(a.k, kq0 + dk, a.in_dtype) * delta;
          y += s * load_as_f32(a.q, kq0 + dk, a.in_dtype);
          store_from_f32(a.state_out, row + dk, s, a.state_dtype);
        }
      }
      a.tape[o] = delta;
      store_from_f32(a.y, o, y, a.in_dtype);
    }
  }
}

}  // namespace
}  // namespace dflash

namespace dflash {
namespace {

// Shared body of the two entry points; z == nullptr: no output norm.
int gdn_forward_launch(const char* who, const void* q, const void* k, const void* v, const void* g, const void* beta,
                       const void* state_in, void* state_out, void* y, float* tape, const uint8_t* mask,
                       const void* z, const void* norm_weight, int weight_dtype, float eps, int slots, int T, int Hk,
                       int Hv, int Dk, int Dv, int in_dtype, int g_dtype, int beta_dtype, int state_dtype,
                       int g_per_dk, void* stream) {
  DFLASH_REQUIRE(q && k && v && g && beta && state_in && state_out && y && tape, DFLASH_ERR_ARG, "%s: null operand", who);
  DFLASH_REQUIRE(state_in != state_out, DFLASH_ERR_ARG, "%s: state_out must not alias state_in", who);
  auto ok = [](int dt) { return dt == DFLASH_BF16 || dt == DFLASH_FP16 || dt == DFLASH_FP32; };
  DFLASH_REQUIRE(ok(in_dtype) && ok(g_dtype) && ok(beta_dtype) && ok(state_dtype) && (!z || ok(weight_dtype)),
                 DFLASH_ERR_ARG, "%s: unknown dtype code", who);
  DFLASH_REQUIRE(slots >= 0 && T >= 0 && Hk > 0 && Hv > 0 && Dk > 0 && Dv > 0, DFLASH_ERR_SHAPE,
                 "%s: non-positive dimension", who);
  DFLASH_REQUIRE(Hv % Hk == 0, DFLASH_ERR_SHAPE, "%s: cannot align K heads %d to V heads %d", who, Hk, Hv);
  DFLASH_REQUIRE((long long)slots * Hv < (1ll << 31), DFLASH_ERR_SHAPE, "%s: too many (slot, head) pairs", who);
  DFLASH_REQUIRE(!z || (norm_weight && Dv % 64 == 0 && Dv <= 256), DFLASH_ERR_SHAPE,
                 "%s: the output norm needs a weight and a row length that is a multiple of 64 up to 256, got %d", who, Dv);
  if (slots == 0) return DFLASH_OK;

  GdnArgs a;
  a.q = q; a.k = k; a.v = v; a.g = g; a.beta = beta; a.state_in = state_in; a.state_out = state_out;
  a.y = y; a.tape = tape; a.mask = mask;
  a.T = T; a.Hk = Hk; a.Hv = Hv; a.Dk = Dk; a.Dv = Dv;
  a.in_dtype = in_dtype; a.g_dtype = g_dtype; a.beta_dtype = beta_dtype; a.state_dtype = state_dtype;
  a.g_per_dk = g_per_dk ? 1 : 0;
  a.z = z; a.norm_weight = norm_weight; a.weight_dtype = weight_dtype; a.eps = eps;

  const dim3 grid((unsigned)(slots * Hv)), block(kThreads);
  hipStream_t s = (hipStream_t)stream;
  const size_t smem = ((size_t)T * 128 * 3 + (size_t)T * (g_per_dk ? 128 : 1) + 2 * (size_t)T) * sizeof(float);
  const bool fast = Dk == 128 && Dv == 128 && T >= 1 && smem <= 64 * 1024 &&
                    (state_dtype != DFLASH_FP32 ||
                     (((uintptr_t)state_in % 16) == 0 && ((uintptr_t)state_out % 16) == 0));
  const bool no_chunk = option(DFLASH_OPT_GDN_STEP_BY_STEP) != 0;  // (tests of one kernel against the other)
  const bool aligned16 = (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)y | (uintptr_t)tape |
                           (uintptr_t)z | (uintptr_t)norm_weight) % 16) == 0;
  const bool chunk = fast && !g_per_dk && state_dtype == DFLASH_FP32 && T <= 16 && aligned16 && !no_chunk;
  bool norm_done = false;
  if (chunk) {
    const size_t lds = kChunkLdsFloats * sizeof(float);
    const bool wide = in_dtype == DFLASH_FP32;
    const bool split = in_dtype == DFLASH_BF16;  // q and k are bf16 numbers: exact products on the bf16 matrix cores
    if (z) {
      if (wide) hipLaunchKernelGGL((gdn_forward_chunk_128<true, true, false>), grid, block, lds, s, a);
      else if (split) hipLaunchKernelGGL((gdn_forward_chunk_128<false, true, true>), grid, block, lds, s, a);
      else hipLaunchKernelGGL((gdn_forward_chunk_128<false, true, false>), grid, block, lds, s, a);
      norm_done = true;
    } else {
      if (wide) hipLaunchKernelGGL((gdn_forward_chunk_128<true, false, false>), grid, block, lds, s, a);
      else if (split) hipLaunchKernelGGL((gdn_forward_chunk_128<false, false, true>), grid, block, lds, s, a);
      else hipLaunchKernelGGL((gdn_forward_chunk_128<false, false, false>), grid, block, lds, s, a);
    }
  } else if (fast) {
    if (g_per_dk) {
      hipLaunchKernelGGL((gdn_forward_128<true, false>), grid, block, smem, s, a);
    } else if (state_dtype == DFLASH_FP32) {
      hipLaunchKernelGGL((gdn_forward_128<false, true>), grid, block, smem, s, a);
    } else {
      hipLaunchKernelGGL((gdn_forward_128<false, false>), grid, block, smem, s, a);
    }
  } else {
    hipLaunchKernelGGL(gdn_forward_generic, grid, block, 0, s, a);
  }
  DFLASH_HIP_OK(hipGetLastError());
  if (z && !norm_done)  // the other kernels leave the recurrence's output in y: normalise it in place
    return dflash_gdn_gated_norm(y, z, norm_weight, y, (long long)slots * T * Hv, Dv, in_dtype, weight_dtype, eps,
                                 stream);
  return DFLASH_OK;
}

}  // namespace
}  // namespace dflash

extern "C" int dflash_gdn_forward_tape(const void* q, const void* k, const void* v, const void* g,
                                       const void* beta, const void* state_in, void* state_out,
                                       void* y, float* tape, const uint8_t* mask, int slots, int T,
                                       int Hk, int Hv, int Dk, int Dv, int in_dtype, int g_dtype,
                                       int beta_dtype, int state_dtype, int g_per_dk, void* stream) {
  return dflash::gdn_forward_launch("dflash_gdn_forward_tape", q, k, v, g, beta, state_in, state_out, y, tape, mask,
                                    nullptr, nullptr, DFLASH_FP32, 0.f, slots, T, Hk, Hv, Dk, Dv, in_dtype, g_dtype,
                                    beta_dtype, state_dtype, g_per_dk, stream);
}

extern "C" int dflash_gdn_forward_tape_norm(const void* q, const void* k, const void* v, const void* g,
                                            const void* beta, const void* state_in, void* state_out,
                                            const void* z, const void* norm_weight, void* out, float* tape,
                                            const uint8_t* mask, int slots, int T, int Hk, int Hv, int Dk, int Dv,
                                            int in_dtype, int g_dtype, int beta_dtype, int state_dtype,
                                            int weight_dtype, int g_per_dk, float eps, void* stream) {
  DFLASH_REQUIRE(z && norm_weight, DFLASH_ERR_ARG, "dflash_gdn_forward_tape_norm: null z or norm weight");
  return dflash::gdn_forward_launch("dflash_gdn_forward_tape_norm", q, k, v, g, beta, state_in, state_out, out, tape,
                                    mask, z, norm_weight, weight_dtype, eps, slots, T, Hk, Hv, Dk, Dv, in_dtype,
                                    g_dtype, beta_dtype, state_dtype, g_per_dk, stream);
}
