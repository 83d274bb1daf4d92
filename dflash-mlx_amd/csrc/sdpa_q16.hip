// Exact attention for a verify block of 16 queries over a long KV cache, gfx950.
//
// Replaces the two Metal kernels of dflash_mlx/kernels.py:442-655 (`batched_sdpa_2pass_partials`
// and `batched_sdpa_2pass_reduce`) behind `batched_sdpa_2pass_exact` (:658-761): for every
// batch b, query head hq (key/value head hk = hq / (Hq / Hk)) and query position i < 16
//     out[i] = softmax_n( scale * q[i] . k[n] + mask[i][n] ) v[n]
// over the keys n <= N - 16 + i (the block's own causal rule, kernels.py:517) whose mask value,
// if a mask is given, is not the dtype's lowest finite value (:452-454); rows without any key
// give 0 (:617).
//
// The path is bound by reading K and V once (2 * N * D * 2 bytes per key/value head; at
// N = 4096, D = 256, 8 heads: 33.7 MB per layer).  So the 16 queries of ALL query heads of a
// key/value head are served from one pass over its keys: a workgroup takes one (batch,
// key/value head, range of keys), wave w holds the 16 queries of query head hk * G + w, and
// K / V tiles of 32 keys go through LDS once for all waves.
//
// Matrix-core layout (v_mfma_f32_16x16x32 bf16 / f16; A lane l = A[l % 16][8 (l / 16) ..+7],
// B lane l = B[8 (l / 16) ..+7][l % 16], accumulator r of lane l = C[4 (l / 16) + r][l % 16]):
//   S^T = K Q^T : A = K tile rows (keys), B = Q (held in registers for the whole kernel);
//                 lane (j, kb) ends up with query j's scores for keys 4 kb + r of each
//                 16-key half: the softmax state (max, sum, rescale factor) is per lane;
//   O^T = V^T P^T: those scores, exponentiated and packed, ARE the B operand (k-slot e <-> key
//                 4 kb + e, slot 4 + e <-> key 16 + 4 kb + e), and the A operand with the same
//                 key order comes from the row-major V tile through ds_read_b64_tr_b16: within
//                 a group of 16 lanes, source lane 4 e + q supplies 8 bytes and lane t receives
//                 element t % 4 of source lanes t / 4, 4 + t / 4, 8 + t / 4, 12 + t / 4 - so source
//                 lane 4 e + q points at V[key 4 kb + e][16 c + 4 q ..+3] and lane t receives
//                 column 16 c + t of four keys.  No transposed copy of V or P is ever stored.
// Ranges of keys (splits) write partial outputs in the input dtype (kernels.py:556-558) with their
// fp32 max and sum; a second kernel merges them (the reference's second pass).
#include "dflash_common.h"

#include <cmath>
#include <cstdlib>
#include <type_traits>

namespace dflash {
namespace {

constexpr int kTileKeys = 32;
constexpr int kThreads = 512;   // eight waves
constexpr int kPadElems = 8;      // 16 bytes: rows of a tile start 16 bytes apart modulo 128
// Score of a key that is not used: below every score a used key can have (a used key may carry
// the dtype's lowest finite value as its mask, -3.39e38 for bf16).
constexpr float kMasked = -3.4028234663852886e38f;

typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

struct SdpaArgs {
  const uint16_t* q;     // [B, Hq, 16, D]
  const uint16_t* k;     // [B, Hk, N, D] through strides (elements), D contiguous
  const uint16_t* v;
  const uint16_t* mask;  // [B, Hq, 16, N] additive, in the input dtype, or null
  uint16_t* out;         // [B, Hq, 16, D]
  uint16_t* part_o;      // [splits, B * Hq, 16, D] in the input dtype, as the reference keeps them
  float* part_ml;        // [splits, B * Hq, 16, 2]  (max, sum)
  long long k_batch_stride, k_head_stride, k_seq_stride;
  long long v_batch_stride, v_head_stride, v_seq_stride;
  int B, Hq, Hk, N, G, splits, keys_per_split;
  float scale, lowest;   // lowest finite value of the input dtype
};

template <bool FP16>
__device__ __forceinline__ f32x4_t mfma32(uint4 a, uint4 b, f32x4_t c) {
  if (FP16) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c,
                                                  0, 0, 0);
  }
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c,
                                                 0, 0, 0);
}

template <bool FP16>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  const f32x2_t f = {lo, hi};
  if (FP16) return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2_t));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
}

template <bool FP16>
__device__ __forceinline__ float elem_to_f32(uint16_t h) {
  return FP16 ? f16_bits_to_f32(h) : bf16_bits_to_f32(h);
}

// One workgroup per (batch, key/value head, split).  Wave w serves query head w % G and the
// columns [slice * D / CS, (slice + 1) * D / CS) of the output, slice = w / G: with few query
// heads per key/value head the output columns are split over CS waves (each repeats the cheap
// K Q^T) so that a SIMD has more than one wave to switch between.  Every launch has kThreads
// threads: waves beyond G * CS move tiles only.
template <int D, bool FP16, int CS, bool MASK>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void sdpa_q16_kernel(SdpaArgs a) {
  constexpr int kCols = D / 16 / CS;          // 16-column chunks of the output per wave
  constexpr int P = D + kPadElems;            // row pitch of a tile in LDS, elements
  constexpr int kTileElems = kTileKeys * P;   // one K or V tile
  constexpr int kChunks = kTileKeys * D / 8;  // 16-byte pieces of a tile
  constexpr int kLoads = kChunks / kThreads;  // per thread: every launch has kThreads threads
  extern __shared__ __align__(16) uint16_t lds[];  // [2][K tile | V tile]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int split = blockIdx.x % a.splits;
  const int bh = blockIdx.x / a.splits;
  const int b = bh / a.Hk, hk = bh % a.Hk;
  const int n_begin = split * a.keys_per_split;
  const int n_end = n_begin + a.keys_per_split < a.N ? n_begin + a.keys_per_split : a.N;
  const int j = lane & 15, kb = lane >> 4;
  const bool computes = wave < a.G * CS;  // the other waves only move tiles
  const int slice = computes ? wave / a.G : 0;
  const int hq = hk * a.G + (computes ? wave % a.G : 0);
  const size_t qrow = ((size_t)b * a.Hq + hq) * 16 + j;  // this lane's query

  const uint16_t* kbase = a.k + (size_t)b * a.k_batch_stride + (size_t)hk * a.k_head_stride;
  const uint16_t* vbase = a.v + (size_t)b * a.v_batch_stride + (size_t)hk * a.v_head_stride;

  // ---- tile movement: global -> registers -> LDS.  Two register stages: the loads of tile i + 2
  // are issued before the arithmetic of tile i, and tile i + 1 goes from its registers to LDS
  // after it, a full tile after its loads were issued.  Nothing here is conditional: rows past
  // the end of the range repeat its last row (their scores are masked, their weights zero) and a
  // tile past the end is fetched and dropped, so that the number of loads in flight at every wait
  // is known when the kernel is compiled and a wait covers the older tile only. -----------------
  typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;  // a native vector: plain loads and stores
  struct Stage {
    u32x4_t k[kLoads], v[kLoads];
  };
  Stage stage0, stage1;
  auto fetch = [&](Stage& st, int n0) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const int c = tid + i * kThreads;
      const int key = c / (D / 8), piece = c % (D / 8);
      const int n = n0 + key < n_end ? n0 + key : n_end - 1;
      st.k[i] = *reinterpret_cast<const u32x4_t*>(kbase + (size_t)n * a.k_seq_stride + 8 * piece);
      st.v[i] = *reinterpret_cast<const u32x4_t*>(vbase + (size_t)n * a.v_seq_stride + 8 * piece);
    }
  };
  auto stash = [&](const Stage& st, int buf) __attribute__((always_inline)) {
    uint16_t* sk = lds + buf * 2 * kTileElems;
    uint16_t* sv = sk + kTileElems;
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const int c = tid + i * kThreads;
      const int key = c / (D / 8), piece = c % (D / 8);
      *reinterpret_cast<u32x4_t*>(sk + key * P + 8 * piece) = st.k[i];
      *reinterpret_cast<u32x4_t*>(sv + key * P + 8 * piece) = st.v[i];
    }
  };

  // ---- this wave's queries, as the B operand of K Q^T -----------------------------------------
  uint4 qreg[D / 32];
#pragma unroll
  for (int s = 0; s < D / 32; ++s)
    qreg[s] = computes ? *reinterpret_cast<const uint4*>(a.q + qrow * D + 32 * s + 8 * kb) : uint4{0u, 0u, 0u, 0u};
  // (asked for ahead of the tiles: loads return in order, and the first product needs these)

  fetch(stage0, n_begin);
  fetch(stage1, n_begin + kTileKeys);

  f32x4_t O[kCols];
#pragma unroll
  for (int c = 0; c < kCols; ++c) O[c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m_run = kMasked, l_run = 0.f;  // l_run: this lane's keys only, merged at the end

  auto compute_tile = [&](int buf, int n0) __attribute__((always_inline)) {
    if (computes) {
      const uint16_t* sk = lds + buf * 2 * kTileElems;
      const uint16_t* sv = sk + kTileElems;
      // S^T = K Q^T for the two 16-key halves of the tile
      // (all reads of the tile are issued before the first product: one LDS latency, not sixteen)
      uint4 kf[2][D / 32];
#pragma unroll
      for (int s = 0; s < D / 32; ++s)
#pragma unroll
        for (int t = 0; t < 2; ++t) kf[t][s] = *reinterpret_cast<const uint4*>(sk + (16 * t + j) * P + 32 * s + 8 * kb);
      f32x4_t st[2] = {f32x4_t{0.f, 0.f, 0.f, 0.f}, f32x4_t{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
      for (int s = 0; s < D / 32; ++s)
#pragma unroll
        for (int t = 0; t < 2; ++t) st[t] = mfma32<FP16>(kf[t][s], qreg[s], st[t]);
      // scores of query j for keys n0 + 16 t + 4 kb + r
      float x[8];
      bool use[8];
      float m_tile = kMasked;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int n = n0 + 16 * t + 4 * kb + r;
          bool ok = n < n_end && n <= a.N - 16 + j;
          float s = st[t][r] * a.scale;
          if (MASK && ok) {
            const float mv = elem_to_f32<FP16>(a.mask[qrow * a.N + n]);
            ok = mv >= a.lowest;
            s += mv;
          }
          use[4 * t + r] = ok;
          x[4 * t + r] = ok ? s : kMasked;
          m_tile = fmaxf(m_tile, x[4 * t + r]);
        }
      }
      m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 16, 64));
      m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32, 64));
      const float m_new = fmaxf(m_run, m_tile);
      const float factor = __expf(m_run - m_new);  // 1 while nothing has been seen (both masked)
      float p[8], sum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        p[e] = use[e] ? __expf(x[e] - m_new) : 0.f;
        sum += p[e];
      }
      l_run = l_run * factor + sum;
      m_run = m_new;
      if (__any(factor != 1.f)) {
#pragma unroll
        for (int c = 0; c < kCols; ++c) O[c] *= factor;
      }
      const uint4 pb = {pack2<FP16>(p[0], p[1]), pack2<FP16>(p[2], p[3]), pack2<FP16>(p[4], p[5]),
                        pack2<FP16>(p[6], p[7])};
      // O^T += V^T P^T, 16 columns of V at a time
      const int src = lane & 15;  // source lane inside the group of 16: key 4 kb + src / 4, columns 4 (src % 4) ..+3
      const uint16_t* vrow = sv + (4 * kb + (src >> 2)) * P + 4 * (src & 3) + 16 * kCols * slice;
      typedef __attribute__((address_space(3))) s16x4_t lds_s16x4;
      s16x4_t lo[kCols], hi[kCols];
#pragma unroll
      for (int c = 0; c < kCols; ++c) {
        lo[c] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(vrow + 16 * c));
        hi[c] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(vrow + 16 * P + 16 * c));
      }
#pragma unroll
      for (int c = 0; c < kCols; ++c) {
        const uint2 lo2 = __builtin_bit_cast(uint2, lo[c]), hi2 = __builtin_bit_cast(uint2, hi[c]);
        O[c] = mfma32<FP16>(uint4{lo2.x, lo2.y, hi2.x, hi2.y}, pb, O[c]);
      }
    }

  };

  stash(stage0, 0);
  __syncthreads();
  for (int n0 = n_begin; n0 < n_end; n0 += 2 * kTileKeys) {
    // even tile in buffer 0; stage 1 holds the next tile, stage 0 is free
    fetch(stage0, n0 + 2 * kTileKeys);
    compute_tile(0, n0);
    stash(stage1, 1);
    __syncthreads();
    if (n0 + kTileKeys >= n_end) break;
    // odd tile in buffer 1; stage 0 holds the next tile, stage 1 is free
    fetch(stage1, n0 + 3 * kTileKeys);
    compute_tile(1, n0 + kTileKeys);
    stash(stage0, 0);
    __syncthreads();
  }

  if (!computes) return;
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
  // accumulator r of chunk c is column 16 (kCols slice + c) + 4 kb + r of query j
  const int col0 = 16 * kCols * slice + 4 * kb;
  if (a.splits == 1) {
    const float inv = l_run > 0.f ? 1.f / l_run : 1.f;
#pragma unroll
    for (int c = 0; c < kCols; ++c) {
      const uint2 o = {pack2<FP16>(O[c][0] * inv, O[c][1] * inv), pack2<FP16>(O[c][2] * inv, O[c][3] * inv)};
      *reinterpret_cast<uint2*>(a.out + qrow * D + col0 + 16 * c) = o;
    }
  } else {
    const size_t prow = (size_t)split * a.B * a.Hq * 16 + qrow;
#pragma unroll
    for (int c = 0; c < kCols; ++c)
      *reinterpret_cast<uint2*>(a.part_o + prow * D + col0 + 16 * c) =
          uint2{pack2<FP16>(O[c][0], O[c][1]), pack2<FP16>(O[c][2], O[c][3])};
    if (kb == 0 && slice == 0) *reinterpret_cast<f32x2_t*>(a.part_ml + prow * 2) = f32x2_t{m_run, l_run};
  }
}

// Second pass: one workgroup of 256 threads per query row.  Thread (g, c) adds the partial
// outputs of the splits s = g, g + 4, ... for 4 output columns; the weights exp(m_s - m) and the
// total sum are worked out once, by the first wave.
constexpr int kMaxSplits = 256;
template <bool FP16>
__global__ __launch_bounds__(256) void sdpa_q16_merge_kernel(SdpaArgs a, int D) {
  __shared__ float weight[kMaxSplits];
  __shared__ float total;
  __shared__ f32x4_t acc[4][64];
  const size_t row = blockIdx.x;  // (b * Hq + hq) * 16 + i
  const size_t rows = (size_t)a.B * a.Hq * 16;
  const int tid = threadIdx.x, c4 = tid & 63, g = tid >> 6;
  const bool col = 4 * c4 < D;
  // Group g adds up splits g, g + 4, ...; eight of them per round.  The first round's partial
  // outputs are asked for before anything else, and every round asks for all eight before it
  // uses one: a split's answer takes a microsecond, and there are up to 64 per group.
  constexpr int kRound = 8;
  uint2 h[kRound];
  auto issue_round = [&](int s0) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < kRound; ++j) {
      const int s = s0 + 4 * j;
      h[j] = uint2{0u, 0u};
      if (col && s < a.splits) h[j] = *reinterpret_cast<const uint2*>(a.part_o + ((size_t)s * rows + row) * D + 4 * c4);
    }
  };
  issue_round(g);
  if (tid < 64) {
    f32x2_t ml[kMaxSplits / 64];
#pragma unroll
    for (int j = 0; j < kMaxSplits / 64; ++j) {
      const int s = tid + 64 * j;
      ml[j] = f32x2_t{kMasked, 0.f};
      if (s < a.splits) ml[j] = *reinterpret_cast<const f32x2_t*>(a.part_ml + ((size_t)s * rows + row) * 2);
    }
    float m = kMasked;
#pragma unroll
    for (int j = 0; j < kMaxSplits / 64; ++j) m = fmaxf(m, ml[j][0]);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    float l = 0.f;
#pragma unroll
    for (int j = 0; j < kMaxSplits / 64; ++j) {
      const int s = tid + 64 * j;
      if (s < a.splits) {
        const float w = __expf(ml[j][0] - m);
        weight[s] = w;
        l += w * ml[j][1];
      }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) l += __shfl_xor(l, off, 64);
    if (tid == 0) total = l;
  }
  __syncthreads();
  f32x4_t o = {0.f, 0.f, 0.f, 0.f};
  for (int s0 = g; s0 < a.splits; s0 += 4 * kRound) {
    if (s0 != g) issue_round(s0);
#pragma unroll
    for (int j = 0; j < kRound; ++j) {
      const int s = s0 + 4 * j;
      if (s < a.splits) {
        const f32x4_t v = {elem_to_f32<FP16>((uint16_t)h[j].x), elem_to_f32<FP16>((uint16_t)(h[j].x >> 16)),
                           elem_to_f32<FP16>((uint16_t)h[j].y), elem_to_f32<FP16>((uint16_t)(h[j].y >> 16))};
        o += v * weight[s];
      }
    }
  }
  acc[g][c4] = o;
  __syncthreads();
  if (g == 0 && col) {
    o = acc[0][c4] + acc[1][c4] + acc[2][c4] + acc[3][c4];
    const float inv = total > 0.f ? 1.f / total : 1.f;
    const uint2 packed = {pack2<FP16>(o[0] * inv, o[1] * inv), pack2<FP16>(o[2] * inv, o[3] * inv)};
    *reinterpret_cast<uint2*>(a.out + row * D + 4 * c4) = packed;
  }
}

int pick_splits(int B, int Hk, int N, int* keys_per_split) {
  // About one workgroup per compute unit, and never less than 128 keys per split: every split
  // adds B * Hq * 16 * (2 D + 8) bytes of partial results, written once and read once.
  // DFLASH_OPT_SDPA_SPLITS = n asks for n ranges instead (tests)
  const int forced = option(DFLASH_OPT_SDPA_SPLITS);
  int want = forced > 0 ? forced : (256 + B * Hk - 1) / (B * Hk);
  const int most = (N + 127) / 128;
  if (want > most) want = most;
  if (want > kMaxSplits) want = kMaxSplits;
  if (want < 1) want = 1;
  int per = (N + want - 1) / want;
  per = (per + kTileKeys - 1) / kTileKeys * kTileKeys;
  *keys_per_split = per;
  return (N + per - 1) / per;  // no empty split
}

}  // namespace
}  // namespace dflash

extern "C" size_t dflash_sdpa_q16_workspace_bytes(int B, int Hq, int Hk, int N, int D) {
  using namespace dflash;
  if (B <= 0 || Hq <= 0 || Hk <= 0 || N <= 0 || D <= 0) return 0;
  int per = 0;
  const int splits = pick_splits(B, Hk, N, &per);
  if (splits == 1) return 0;
  return (size_t)splits * B * Hq * 16 * (D * sizeof(uint16_t) + 2 * sizeof(float));
}

extern "C" int dflash_sdpa_q16(const void* q, const void* k, const void* v, const void* mask, void* out,
                               void* workspace, size_t workspace_bytes, int B, int Hq, int Hk, int N, int D,
                               long long k_batch_stride, long long k_head_stride, long long k_seq_stride,
                               long long v_batch_stride, long long v_head_stride, long long v_seq_stride,
                               float scale, int dtype, void* stream) {
  using namespace dflash;
  DFLASH_REQUIRE(q && k && v && out, DFLASH_ERR_ARG, "dflash_sdpa_q16: null operand");
  DFLASH_REQUIRE(dtype == DFLASH_BF16 || dtype == DFLASH_FP16, DFLASH_ERR_ARG,
                 "dflash_sdpa_q16: bf16 or fp16 only");
  DFLASH_REQUIRE(D == 128 || D == 256, DFLASH_ERR_SHAPE, "dflash_sdpa_q16: head dim %d (128 or 256)", D);
  DFLASH_REQUIRE(B > 0 && Hq > 0 && Hk > 0 && N >= 16 && Hq % Hk == 0 && Hq / Hk <= 8, DFLASH_ERR_SHAPE,
                 "dflash_sdpa_q16: B %d, Hq %d, Hk %d, N %d (Hq a multiple of Hk, at most 8 times; N >= 16)", B, Hq,
                 Hk, N);
  DFLASH_REQUIRE(k_seq_stride >= D && v_seq_stride >= D && k_seq_stride % 8 == 0 && v_seq_stride % 8 == 0 &&
                     k_head_stride % 8 == 0 && v_head_stride % 8 == 0 && k_batch_stride % 8 == 0 &&
                     v_batch_stride % 8 == 0,
                 DFLASH_ERR_SHAPE, "dflash_sdpa_q16: strides must keep rows 16-byte aligned");
  DFLASH_REQUIRE((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) % 16) == 0, DFLASH_ERR_ARG,
                 "dflash_sdpa_q16: operands must be 16-byte aligned");
  DFLASH_REQUIRE((long long)B * Hq * 16 < (1ll << 31) && (long long)B * Hk * ((N + 127) / 128) < (1ll << 31),
                 DFLASH_ERR_SHAPE, "dflash_sdpa_q16: too many rows");

  SdpaArgs a;
  a.q = (const uint16_t*)q; a.k = (const uint16_t*)k; a.v = (const uint16_t*)v; a.mask = (const uint16_t*)mask;
  a.out = (uint16_t*)out;
  a.k_batch_stride = k_batch_stride; a.k_head_stride = k_head_stride; a.k_seq_stride = k_seq_stride;
  a.v_batch_stride = v_batch_stride; a.v_head_stride = v_head_stride; a.v_seq_stride = v_seq_stride;
  a.B = B; a.Hq = Hq; a.Hk = Hk; a.N = N; a.G = Hq / Hk;
  a.splits = pick_splits(B, Hk, N, &a.keys_per_split);
  a.scale = scale;
  a.lowest = dtype == DFLASH_FP16 ? -65504.0f : -3.3895313892515355e38f;
  a.part_o = nullptr;
  a.part_ml = nullptr;
  if (a.splits > 1) {
    const size_t need = (size_t)a.splits * B * Hq * 16 * (D * sizeof(uint16_t) + 2 * sizeof(float));
    DFLASH_REQUIRE(workspace && workspace_bytes >= need && ((uintptr_t)workspace % 16) == 0, DFLASH_ERR_WORKSPACE,
                   "dflash_sdpa_q16: workspace of %zu bytes needed, %zu given", need,
                   workspace ? workspace_bytes : (size_t)0);
    a.part_ml = (float*)workspace;   // [splits, rows, 2] fp32 first: keeps both arrays 16-byte aligned
    a.part_o = (uint16_t*)(a.part_ml + (size_t)a.splits * B * Hq * 16 * 2);
  }

  hipStream_t s = (hipStream_t)stream;
  // column split: as many waves as fit eight, in powers of two
  const int cs = a.G <= 2 ? 4 : a.G <= 4 ? 2 : 1;
  const size_t lds_bytes = (size_t)2 * 2 * kTileKeys * (D + kPadElems) * sizeof(uint16_t);
  const bool f16 = dtype == DFLASH_FP16;
#define DFLASH_SDPA_ROW(D_, F_, M_)                                                                      \
  {(const void*)sdpa_q16_kernel<D_, F_, 1, M_>, (const void*)sdpa_q16_kernel<D_, F_, 2, M_>, \
   (const void*)sdpa_q16_kernel<D_, F_, 4, M_>}
  const void* table[2][2][2][3] = {
      {{DFLASH_SDPA_ROW(128, false, false), DFLASH_SDPA_ROW(128, false, true)},
       {DFLASH_SDPA_ROW(128, true, false), DFLASH_SDPA_ROW(128, true, true)}},
      {{DFLASH_SDPA_ROW(256, false, false), DFLASH_SDPA_ROW(256, false, true)},
       {DFLASH_SDPA_ROW(256, true, false), DFLASH_SDPA_ROW(256, true, true)}}};
#undef DFLASH_SDPA_ROW
  const bool masked = mask != nullptr;
  const int ics = cs == 1 ? 0 : cs == 2 ? 1 : 2;
  void* args[] = {&a};
  const int slot = current_device_slot();
  {
    const void* fn = table[D == 256][f16][masked][ics];
    // the attribute belongs to the device's copy of the kernel: once per device and kernel
    static bool attr_set[kMaxDevices][24] = {};
    const int idx = (((D == 256) * 2 + f16) * 2 + masked) * 3 + ics;
    if (!attr_set[slot][idx] || slot == kMaxDevices - 1) {
      DFLASH_HIP_OK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
      attr_set[slot][idx] = true;
    }
    DFLASH_HIP_OK(hipLaunchKernel(fn, dim3((unsigned)(B * Hk * a.splits)), dim3(kThreads), args, lds_bytes, s));
  }
  if (a.splits > 1) {
    if (dtype == DFLASH_FP16) {
      hipLaunchKernelGGL(sdpa_q16_merge_kernel<true>, dim3((unsigned)(B * Hq * 16)), dim3(256), 0, s, a, D);
    } else {
      hipLaunchKernelGGL(sdpa_q16_merge_kernel<false>, dim3((unsigned)(B * Hq * 16)), dim3(256), 0, s, a, D);
    }
    DFLASH_HIP_OK(hipGetLastError());
  }
  return DFLASH_OK;
}
