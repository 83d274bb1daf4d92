// Chained M=16 int4 qmm for gfx950: several matrices in ONE launch.
//
// A verify step calls the quantized matmul once per projection (dflash_mlx/verify_linear.py:
// 103-143, five times per layer), and a launch of the streaming kernel (qmm_m16_stream.hip)
// spends more time around its weight stream than in it: the gap between two kernels of a
// stream, the first memory round trips of cold workgroups, the split-K hand-over at the end.
// This kernel runs a list of problems  y_p[16, N_p] = x_p[16, K_p] . (s*q + b)_p^T  back to back
// inside one persistent grid.  Every problem is divided among the workgroups exactly as a
// launch of its own would divide it (same grid rule, same unit ranges, same order of partial
// sums: results are bit for bit those of separate launches), but the ring of LDS slots never
// drains: while the workers of a workgroup finish problem p and hand over its partial tiles,
// its loaders already stream the first units of problem p + 1.  Weights never depend on
// activations; only x does:
//
//  * a problem whose x is the y of an earlier problem of the chain (wait_for) has its codes,
//    scales and biases prefetched like any other, its x loads held back until the earlier
//    problem's row blocks have all been stored (a counter per problem, bumped at agent scope
//    after the stores are acknowledged; x is then read around the L2, which is per XCD).  The
//    wait is bounded: after spin_limit polls a workgroup records an error word, goes on with
//    whatever x holds, and the launch ends normally.
//  * an epilogue turns a gate/up pair into the MLP's hidden activation inside the launch:
//    the matrix holds gate rows then up rows, a row block takes 64 rows of each, and the
//    workgroup that finishes it stores silu(gate) * up (every operator of x * sigmoid(x) * up
//    rounded to the activation type, as separate operators would) - which the down projection
//    then waits for.
//
// Everything else - units of 128 rows x 256 k, 8 worker + 4 loader waves, direct-to-LDS loads
// into a ring, hand-written LDS reads, bare barriers - is the streaming kernel's, see there.
#include <cstdlib>

#include "dflash_common.h"
#include "qmm_stream_device.h"

namespace dflash {
namespace stream {

constexpr int kMaxChain = DFLASH_QMM_CHAIN_MAX;
#ifndef DFLASH_CHAIN_AHEAD
#define DFLASH_CHAIN_AHEAD 3
#endif
constexpr int kChainAhead = DFLASH_CHAIN_AHEAD;  // units issued beyond the one being consumed
// LDS behind the two rings: last-arriver flags, the up half of an epilogue row block (4 tiles of
// 1 KiB) for each of the two row blocks a workgroup can be last at, the table of ranges.
constexpr int kChainFlags = kLdsBytes;
constexpr int kChainExchange = kChainFlags + 64;
constexpr int kChainTable = kChainExchange + 2 * 4096;  // 48 bytes per problem: its Range
constexpr int kLdsBytesChain = kChainTable + 48 * kMaxChain;  // 152.8 KiB
// The last words of the 64 KiB counter block: launch bookkeeping of chains.
constexpr int kChainStatusWord = 16384 - 64;  // [0] exit counter, [1] error word
constexpr int kChainDoneWord = kChainStatusWord + 8;  // [kMaxChain] row blocks stored, per problem
constexpr int kChainCounterWords = kChainStatusWord;

struct ChainProblem {
  const uint16_t* x;
  const uint32_t* w;
  const uint16_t* scales;
  const uint16_t* biases;
  uint16_t* y;
  int K, N;          // N counts the rows of w (gate and up rows for the epilogue)
  int grid;          // workgroups that take part: what a launch of its own would use
  int counter_base;  // first arrival counter of this problem
  int partial_base;  // first partial tile of this problem (tiles of kPartialFloats floats)
  int wait_for;      // earlier problem whose y is this x, or -1
  int epilogue;      // DFLASH_QMM_EPILOGUE_*
  int signal;        // a later problem waits for this one
};
struct ChainParams {
  ChainProblem prob[kMaxChain];
  int count;
  float* partials;
  uint32_t* counters;
  int has_deps;
  int spin_limit;
  int joint;  // the problems' units laid end to end and divided as ONE range (independent problems only)
};

// The kernel reads its argument block in place, through the constant address space: a
// reference to a by-value struct argument that is indexed at run time would make the compiler
// copy the whole block into per-thread memory.
typedef const __attribute__((address_space(4))) ChainProblem CProblem;
typedef const __attribute__((address_space(4))) ChainParams CParams;

// How one problem is divided: this workgroup's range of units, or wg < 0 if it has none.
// `off` and `total` place the problem's units on the line that `grid` workgroups divide: the
// problem's own units (off 0, total = units) or, in the joint form, the units of all problems
// end to end (off = units of the problems before it, total = all of them).
struct Range {
  int stages, RB, units, grid, wg;
  int u0, u1, rb0, st0;
  int off, total;
};
__device__ __forceinline__ Range problem_range(CParams& p, int i, int block, int nblocks) {
  CProblem& q = p.prob[i];
  Range r;
  r.stages = q.K / kUnitK;
  r.RB = (q.N + kRows - 1) / kRows;
  r.units = r.RB * r.stages;
  r.off = 0;
  r.total = r.units;
  r.u0 = r.u1 = r.rb0 = r.st0 = 0;
  if (p.joint) {
    // One range per workgroup over all problems: nearly every row block is computed by one
    // workgroup from end to end, only the row blocks at the ends of a range are shared.
    int off = 0, total = 0;
    for (int j = 0; j < p.count; ++j) {
      const int u = ((p.prob[j].N + kRows - 1) / kRows) * (p.prob[j].K / kUnitK);
      off += j < i ? u : 0;
      total += u;
    }
    r.off = off;
    r.total = total;
    // (no more workgroups than units: every workgroup between two contributors of a row block
    // must be a contributor itself)
    const int grid = nblocks < total ? nblocks : total;
    r.grid = grid;
    const int wg = grid == nblocks && nblocks % 8 == 0 ? (block % 8) * (nblocks / 8) + block / 8 : block;  // XCD-major, as below
    int a = 0, b = 0;
    if (wg < grid) {
      a = range_begin(total, wg, grid) - off, b = range_begin(total, wg + 1, grid) - off;
      a = a < 0 ? 0 : (a > r.units ? r.units : a);
      b = b < 0 ? 0 : (b > r.units ? r.units : b);
    }
    r.wg = a < b ? wg : -1;
    if (r.wg >= 0) {
      r.u0 = a;
      r.u1 = b;
      r.rb0 = a / r.stages;
      r.st0 = a - r.rb0 * r.stages;
    }
    return r;
  }
  r.grid = q.grid;
  // Workgroups are dealt to the eight XCDs in turn (block % 8); unit ranges follow the XCD-major
  // order, so that the neighbours that share a row block sit behind one L2 (as a launch of its
  // own with `grid` workgroups would place them).
  if (r.grid % 8 == 0 && nblocks % 8 == 0) {
    const int per = r.grid / 8, slot = block / 8;
    r.wg = slot < per ? (block % 8) * per + slot : -1;
  } else {
    r.wg = block < r.grid ? block : -1;
  }
  if (r.wg >= 0) {
    r.u0 = range_begin(r.units, r.wg, r.grid);
    r.u1 = range_begin(r.units, r.wg + 1, r.grid);
    r.rb0 = r.u0 / r.stages;
    r.st0 = r.u0 - r.rb0 * r.stages;
  }
  return r;
}

// The Range of problem i from the table in LDS (hand-written reads: see the file header of
// qmm_m16_stream.hip).  All values are the same in every lane.
__device__ __forceinline__ Range read_range(uint32_t lds0, int i) {
  u32x4_t a, b;
  u32x2_t c;
  const uint32_t addr = lds0 + kChainTable + i * 48;
  asm volatile("ds_read_b128 %0, %3\n ds_read_b128 %1, %3 offset:16\n ds_read_b64 %2, %3 offset:32\n s_waitcnt lgkmcnt(0)"
               : "=&v"(a), "=&v"(b), "=&v"(c)
               : "v"(addr)
               : "memory");
  Range r;
  r.wg = __builtin_amdgcn_readfirstlane((int)a.x);
  r.u0 = __builtin_amdgcn_readfirstlane((int)a.y);
  r.u1 = __builtin_amdgcn_readfirstlane((int)a.z);
  r.rb0 = __builtin_amdgcn_readfirstlane((int)a.w);
  r.st0 = __builtin_amdgcn_readfirstlane((int)b.x);
  r.stages = __builtin_amdgcn_readfirstlane((int)b.y);
  r.units = __builtin_amdgcn_readfirstlane((int)b.z);
  r.grid = __builtin_amdgcn_readfirstlane((int)b.w);
  r.off = __builtin_amdgcn_readfirstlane((int)c.x);
  r.total = __builtin_amdgcn_readfirstlane((int)c.y);
  r.RB = r.units / r.stages;
  return r;
}

// wait_loads() rounded down to the thresholds that occur in steady state (one or two units
// issued behind the one waited for, each 6 loads, 8 with its scales and biases): waiting for
// fewer outstanding loads than allowed is always safe, and the full switch costs the wave tens
// of instructions per unit.
__device__ __forceinline__ void wait_loads_coarse(int n) {
  if (n >= 12) {
    if (n >= 20) __builtin_amdgcn_s_waitcnt(0x0F70 | (20 & 15) | ((20 >> 4) << 14));
    else if (n >= 18) __builtin_amdgcn_s_waitcnt(0x0F70 | (18 & 15) | ((18 >> 4) << 14));
    else if (n >= 14) __builtin_amdgcn_s_waitcnt(0x0F70 | 14);
    else __builtin_amdgcn_s_waitcnt(0x0F70 | 12);
  } else {
    if (n >= 8) __builtin_amdgcn_s_waitcnt(0x0F70 | 8);
    else if (n >= 6) __builtin_amdgcn_s_waitcnt(0x0F70 | 6);
    else __builtin_amdgcn_s_waitcnt(0x0F70);
  }
}

// The hand-over of a problem's shared row blocks needs three memory round trips.  Where nothing
// waits for the result they are spread over the first units of the workgroup's next problem
// instead of being sat out: not for a problem that another one waits for or that has an
// epilogue (their outputs are needed at once / take one more barrier), and only if the next
// problem this workgroup takes part in has its x at hand and at least kHandoverSumUnit + 1 units
// here.  Loaders and workers decide alike: the rule fixes the barriers of the hand-over.
constexpr int kHandoverArriveUnit = 1;  // unit of the next problem at whose barrier the arrival counters are bumped
constexpr int kHandoverSumUnit = 3;     // ... and at whose barrier the last to arrive adds the partial tiles
__device__ __forceinline__ bool handover_deferred(CParams& p, uint32_t lds0, int cp) {
  if (p.prob[cp].signal || p.prob[cp].epilogue != DFLASH_QMM_EPILOGUE_NONE) return false;
  for (int nx = cp + 1; nx < p.count; ++nx) {
    const Range r = read_range(lds0, nx);
    if (r.wg < 0) continue;
    return p.prob[nx].wait_for < 0 && r.u1 - r.u0 > kHandoverSumUnit;
  }
  return false;
}

// Row of w behind row v (0..127) of row block rb.  Plain: 128 rb + v.  Epilogue: the first 64
// rows are gate rows 64 rb .., the other 64 the up rows of the same output columns.
__device__ __forceinline__ int weight_row(CProblem& q, int rb, int v) {
  if (q.epilogue == DFLASH_QMM_EPILOGUE_SILU_MUL) {
    const int half_rows = q.N >> 1;
    int r = 64 * rb + (v & 63);
    r = r < half_rows ? r : half_rows - 1;
    return v < 64 ? r : half_rows + r;
  }
  const int r = kRows * rb + v;
  return r < q.N ? r : q.N - 1;
}

__device__ __forceinline__ void load16_to_lds_coherent(const void* gptr, char* lds_base) {
  __builtin_amdgcn_global_load_lds((global_cvoid_t*)gptr, (lds_void_t*)lds_base, 16, 0, 16);  // sc1
}

#ifdef DFLASH_CHAIN_STAMPS
// Experiment builds only: per workgroup, wave 0 (a worker) and wave 8 (a loader) record the
// constant-rate wall clock at every unit.  [block][role][slot]
#if DFLASH_CHAIN_STAMPS == 3  // per problem only, every workgroup: [block][problem * 4 + event]
constexpr int kStampSlots = 64;
__device__ unsigned long long g_stamps[256][1][kStampSlots];
#define DFLASH_STAMP(role, idx)                                                          \
  do {                                                                                   \
    if (lane == 0 && (role) == 12 && (idx) < kStampSlots && blockIdx.x < 256)            \
      g_stamps[blockIdx.x][0][idx] = wall_clock64();                                     \
  } while (0)
#else
constexpr int kStampSlots = 512;
__device__ unsigned long long g_stamps[64][13][kStampSlots];
#define DFLASH_STAMP(role, idx)                                                          \
  do {                                                                                   \
    if (lane == 0 && (idx) < kStampSlots && blockIdx.x < 64)                             \
      g_stamps[blockIdx.x][role][idx] = wall_clock64();                                  \
  } while (0)
#endif
#else
#define DFLASH_STAMP(role, idx) do {} while (0)
#endif

template <bool FP16>
__device__ __forceinline__ float silu_mul(float g, float u) {
  using A = Act<FP16>;
  // silu(g) * u as the array operators x * sigmoid(x) and * give it: the factors as the
  // activation type holds them between the projections and the activation, then the sigmoid,
  // its product with g and the product with u each rounded to that type (the last one by the
  // store).  Same form as the GatedDeltaNet glue kernels use.
  g = A::to_f32(A::from_f32(g));
  u = A::to_f32(A::from_f32(u));
  const float sig = A::to_f32(A::from_f32(1.0f / (1.0f + expf(-g))));
  const float s = A::to_f32(A::from_f32(g * sig));
  return s * u;
}

// Packed images (see qmm_pack_kernel in qmm_m16_stream.hip) of a gate/up matrix for the silu-mul
// epilogue: row block rb holds gate rows 64 rb .. 64 rb + 63 followed by the up rows of the same
// output columns - weight_row() below as a layout.  One thread per 16 bytes of output.
__global__ __launch_bounds__(256) void qmm_pack_gate_up_kernel(const uint32_t* __restrict__ w,
                                                               const uint16_t* __restrict__ scales,
                                                               const uint16_t* __restrict__ biases,
                                                               uint4* __restrict__ w_out, uint4* __restrict__ s_out,
                                                               uint4* __restrict__ b_out, int K, int N) {
  const int stages = K / kUnitK, chunks = stages / 4;
  const int half_rows = N >> 1;
  const int RB = (half_rows + 63) / 64;
  const size_t code_granules = (size_t)RB * stages * (kPackedUnitBytes / 16);
  const size_t sb_granules = (size_t)RB * chunks * (kPackedChunkBytes / 16);
  const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  auto source_row = [&](int rb, int v) {
    int r = 64 * rb + (v & 63);
    r = r < half_rows ? r : half_rows - 1;
    return v < 64 ? r : half_rows + r;
  };
  if (t < code_granules) {
    const int lane = (int)(t & 63), q = (int)((t >> 6) & 15);
    const size_t unit = t >> 10;
    const int st = (int)(unit % stages), rb = (int)(unit / stages);
    const int r8 = lane >> 3;
    const int row = source_row(rb, 8 * q + r8);
    const int g = (lane & 7) ^ (((r8 >> 1) & 3) << 1);
    w_out[t] = *reinterpret_cast<const uint4*>((const char*)w + (size_t)row * (K >> 1) + st * (kUnitK / 2) + g * 16);
  } else if (t < code_granules + 2 * sb_granules) {
    size_t u = t - code_granules;
    const bool is_bias = u >= sb_granules;
    if (is_bias) u -= sb_granules;
    const int lane = (int)(u & 63), part = (int)((u >> 6) & 3);
    const size_t chunk = u >> 8;
    const int c = (int)(chunk % chunks), rb = (int)(chunk / chunks);
    const int row = source_row(rb, 32 * part + (lane >> 1));
    const char* src = (const char*)(is_bias ? biases : scales) + ((size_t)row * (K / kGS) + c * 16) * 2 + (lane & 1) * 16;
    (is_bias ? b_out : s_out)[u] = *reinterpret_cast<const uint4*>(src);
  }
}

// PACKED: w, scales, biases of every problem are the packed images of dflash_qmm_m16_pack (a
// property of the launch, so that the loaders carry no per-problem strides in registers).
template <bool ACT_FP16, bool SB_FP16, bool PACKED>
__global__ __launch_bounds__(kThreads, 1) void qmm_chain_kernel(ChainParams by_value) {
  using A = Act<ACT_FP16>;
  (void)by_value;  // the first (and only) argument: offset 0 of the argument block
  CParams& p = *(CParams*)__builtin_amdgcn_kernarg_segment_ptr();
  constexpr int CHUNK = 4;
  constexpr int SBROW = 8 * CHUNK;
  extern __shared__ __attribute__((aligned(1024))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t lds0 = lds_address(lds);
  const int block = (int)blockIdx.x, nblocks = (int)gridDim.x;
  uint32_t* const status = p.counters + kChainStatusWord;
  uint32_t* const done = p.counters + kChainDoneWord;

  // How every problem is divided (this workgroup's range): computed once, lane i of wave 0 for
  // problem i, and kept in LDS; the waves look a problem up when they reach it.
  if (wave == 0 && lane < p.count) {
    const Range r = problem_range(p, lane, block, nblocks);
    int* t = reinterpret_cast<int*>(lds + kChainTable + lane * 48);
    t[0] = r.wg, t[1] = r.u0, t[2] = r.u1, t[3] = r.rb0, t[4] = r.st0, t[5] = r.stages, t[6] = r.units, t[7] = r.grid;
    t[8] = r.off, t[9] = r.total;
  }
  __syncthreads();

  // Both kinds of wave walk the same problems and units and pass the same barriers.  Per
  // problem this workgroup takes part in:
  //   one at its start (its first unit has landed),
  //   one per unit u (the next unit of the problem has landed; every worker holds unit u in
  //     registers, so the slot of unit u is free),
  //   when a row block ends with unit u: one more (the slot of unit u carries the cross-wave
  //     sum), and with an epilogue another one (the up half crosses to the gate half's waves),
  //   after the last unit, if a row block was shared with other workgroups: two more (partial
  //     tiles stored / arrival counters bumped), with an epilogue a third,
  //   if a later problem waits for this one: one more (outputs stored).

  if (wave >= kWaves) {
    // ================================ loader waves ====================================
    // See qmm_m16_stream.hip for which loader issues which 16-byte pieces of a unit.  The
    // workers wait for this wave at every unit, so its path from one barrier to the next is
    // kept short: 32-bit offsets from base pointers held in scalar registers, unit ranges read
    // from the table in LDS, waits rounded to a few thresholds.  (A loader may not spill: spill
    // traffic would count as loads of its own.)
    const int ld = wave - kWaves;
    const int w_r = lane >> 3;
    const int w_c = (lane & 7) ^ (((w_r >> 1) & 3) << 1);

    // ---- issue cursor: runs kChainAhead units ahead of the workers, across problems -----
    enum { NEED_OPEN, OPEN, PARKED, EXHAUSTED };
    int i_state = NEED_OPEN;
    int ip = -1;  // problem being issued
    int iu = 0, iu1 = 0, irb = 0, ist = 0, istages = 1;  // next unit to issue: index, end of range, row block, stage
    bool i_first = false;     // it is the first unit of this workgroup's range
    bool i_coherent = false;  // x of problem ip is written by this launch
    bool i_ready = true;      // ... and is known to be complete
    const char* bx = nullptr;  // arrays of problem ip
    const char* bw = nullptr;
    const char* bs = nullptr;
    const char* bb = nullptr;
    // byte offsets of this lane's pieces from the problem's x, w and scales (= biases) arrays
    // (named one by one: an array indexed inside these loops would be placed in memory)
    uint32_t xo0 = 0u, xo1 = 0u, wo0 = 0u, wo1 = 0u, wo2 = 0u, wo3 = 0u, so = 0u;
    // bytes from unit to unit / chunk to chunk of a row block
    constexpr uint32_t w_step = PACKED ? kPackedUnitBytes : kUnitK / 2;
    constexpr uint32_t sb_step = PACKED ? kPackedChunkBytes : CHUNK * kGroups * 2;
    int slot_i = 0, sb_slot_i = 0;
    int n_issued = 0, n_cons = 0;  // units issued / units whose barrier has passed
    int tot = 0;                   // loads this wave has issued
    int mark0 = 0, mark1 = 0, mark2 = 0, mark3 = 0, fifo_n = 0;  // `tot` after each of the last units issued, newest first; how many are not yet waited for
    int def_n = 0, def_slot = 0, def_st = 0;  // units of problem ip issued without their x

    auto set_row_block = [&](int rb) __attribute__((always_inline)) {
      CProblem& q = p.prob[ip];
      if constexpr (PACKED) {
        // every instruction of a wave moves 1 KiB of consecutive memory (see qmm_pack_kernel)
        const uint32_t unit0 = (uint32_t)rb * (uint32_t)(q.K / kUnitK) * kPackedUnitBytes + lane * 16;
        wo0 = unit0 + (ld + 0) * 1024, wo1 = unit0 + (ld + 4) * 1024, wo2 = unit0 + (ld + 8) * 1024, wo3 = unit0 + (ld + 12) * 1024;
        so = (uint32_t)rb * (uint32_t)(q.K / (kUnitK * 4)) * kPackedChunkBytes + ld * 1024 + lane * 16;
        return;
      }
      const uint32_t row_bytes = (uint32_t)q.K >> 1;
      wo0 = (uint32_t)weight_row(q, rb, 8 * (ld + 0) + w_r) * row_bytes + w_c * 16;
      wo1 = (uint32_t)weight_row(q, rb, 8 * (ld + 4) + w_r) * row_bytes + w_c * 16;
      wo2 = (uint32_t)weight_row(q, rb, 8 * (ld + 8) + w_r) * row_bytes + w_c * 16;
      wo3 = (uint32_t)weight_row(q, rb, 8 * (ld + 12) + w_r) * row_bytes + w_c * 16;
      so = (uint32_t)weight_row(q, rb, 32 * ld + (lane >> 1)) * (uint32_t)(q.K / kGS * 2) + (lane & 1) * 16;
    };
    auto issue_x = [&](int st, int slot) __attribute__((always_inline)) {
#ifdef DFLASH_CHAIN_NOX  // (timing experiments: the stream without the x loads; results are wrong)
      (void)st, (void)slot;
      return;
#endif
      char* dst = lds + slot * kSlotBytes + kXOffset + ld * 1024;
      const uint32_t step = (uint32_t)st * (kUnitK * 2);
      if (i_coherent) {
        load16_to_lds_coherent(bx + (xo0 + step), dst);
        load16_to_lds_coherent(bx + (xo1 + step), dst + 4096);
      } else {
        load16_to_lds(bx + (xo0 + step), dst);
        load16_to_lds(bx + (xo1 + step), dst + 4096);
      }
      tot += 2;
    };
    // Keeps kChainAhead units issued beyond the one being consumed.
    auto top_up = [&]() __attribute__((always_inline)) {
#pragma unroll 1
      while (n_issued - n_cons < kChainAhead) {
        if (i_state == NEED_OPEN) {
          i_state = EXHAUSTED;
          while (++ip < p.count) {
            const Range r = read_range(lds0, ip);
            if (r.wg >= 0) {
              iu = r.u0, iu1 = r.u1, irb = r.rb0, ist = r.st0, istages = r.stages;
              i_state = OPEN;
              break;
            }
          }
          if (i_state == OPEN) {
            CProblem& q = p.prob[ip];
            bx = (const char*)q.x, bw = (const char*)q.w, bs = (const char*)q.scales, bb = (const char*)q.biases;
            i_first = true;
            i_coherent = q.wait_for >= 0;
            i_ready = !i_coherent;
            // x: instruction i of 8 moves group i >> 1, k-blocks 2 (i & 1) and 2 (i & 1) + 1; this
            // loader issues i = ld and ld + 4
            const int xrow = lane & 15;
            const uint32_t xbase = (uint32_t)(xrow * q.K + (2 * (ld & 1) + (lane >> 5)) * 16 + ((lane >> 4) & 1) * 8);
            xo0 = (xbase + (uint32_t)((ld >> 1) * kGS)) * 2u;
            xo1 = (xbase + (uint32_t)(((ld + 4) >> 1) * kGS)) * 2u;
            set_row_block(irb);
          }
        }
        if (i_state != OPEN) break;
        // ---- one unit: scales/biases with the first unit of a chunk or of the range, x unless
        // it is still being computed, codes
        char* slot = lds + slot_i * kSlotBytes;
        if ((ist & (CHUNK - 1)) == 0 || i_first) {
          char* sb = lds + kSbOffset + sb_slot_i * kSbSlotBytes;
          const uint32_t off = so + (uint32_t)(ist / CHUNK) * sb_step;
          load16_to_lds(bs + off, sb + ld * 1024);
          load16_to_lds(bb + off, sb + kSbArrayBytes + ld * 1024);
          tot += 2;
          if (++sb_slot_i == kSbDepth) sb_slot_i = 0;
        }
        i_first = false;
        if (i_ready) {
          issue_x(ist, slot_i);
        } else {
          if (def_n == 0) def_slot = slot_i, def_st = ist;
          ++def_n;
        }
        {
          const uint32_t step = (uint32_t)ist * w_step;
          char* dst = slot + ld * 1024;
          load16_to_lds_stream(bw + (wo0 + step), dst);
          load16_to_lds_stream(bw + (wo1 + step), dst + 4096);
          load16_to_lds_stream(bw + (wo2 + step), dst + 8192);
          load16_to_lds_stream(bw + (wo3 + step), dst + 12288);
        }
        tot += 4;
        // remember where this unit's loads end: newest first
        mark3 = mark2, mark2 = mark1, mark1 = mark0, mark0 = tot;
        ++fifo_n;
        ++n_issued;
        if (++slot_i == kDepth) slot_i = 0;
        if (++iu == iu1) {
          // A problem with held-back x loads keeps the cursor until they have been issued: the
          // cursor never enters a second problem whose x is still being computed.
          i_state = def_n == 0 ? NEED_OPEN : PARKED;
        } else if (++ist == istages) {
          ist = 0;
          ++irb;
          set_row_block(irb);
        }
      }
    };
    // Waits until this loader's part of the oldest unit not yet waited for has landed.
    auto wait_oldest = [&]() __attribute__((always_inline)) {
      const int oldest = fifo_n == 1 ? mark0 : fifo_n == 2 ? mark1 : fifo_n == 3 ? mark2 : mark3;
      wait_loads_coarse(tot - oldest);
      --fifo_n;
    };

#ifdef DFLASH_CHAIN_STAMPS
    int st_idx = 0;
#endif
#pragma unroll 1
    for (int cp = 0; cp < p.count; ++cp) {
      const Range cr = read_range(lds0, cp);
      if (cr.wg < 0) continue;
      top_up();
      if (p.prob[cp].wait_for >= 0) {
        // The x of problem cp is the y of an earlier problem: wait (bounded) until all its row
        // blocks have been stored, then issue the x loads that were held back.  The issue
        // cursor is on problem cp (inside it, or parked at its end).
        CProblem& q = p.prob[cp];
        const uint32_t want = (uint32_t)((p.prob[q.wait_for].N + kRows - 1) / kRows);  // its row blocks
        int polls = 0;
        while (__hip_atomic_load(&done[q.wait_for], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < want) {
          if (++polls > p.spin_limit) {
            if (lane == 0 && ld == 0)
              __hip_atomic_store(&status[1], (uint32_t)(cp + 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
          }
          __builtin_amdgcn_s_sleep(8);
        }
        if (ip == cp) {
          int st = def_st, slot = def_slot;
#pragma unroll 1
          for (int j = 0; j < def_n; ++j) {
            issue_x(st, slot);
            if (++st == istages) st = 0;
            if (++slot == kDepth) slot = 0;
          }
          // Nothing but held-back units is waiting to be waited for (every unit of the problems
          // before cp has been consumed), and they end with the x loads just issued.
          mark0 = mark1 = mark2 = mark3 = tot;
          def_n = 0;
          i_ready = true;
          if (i_state == PARKED) i_state = NEED_OPEN;
        }
      }
      wait_oldest();
      asm volatile("s_barrier" ::: "memory");  // the first unit of problem cp has landed
      const bool epi = p.prob[cp].epilogue == DFLASH_QMM_EPILOGUE_SILU_MUL;
      int rb_left = cr.stages - cr.st0;
      int in_rb = 0;
      bool any_shared = false;
#pragma unroll 1
      for (int u = cr.u0; u < cr.u1; ++u) {
        // ---- the common case in a loop of its own -------------------------------------------
        // Units in the interior of a row block, for both cursors: per unit one wait, one
        // barrier and the loads of one unit, nothing else.  The general code below does the
        // same thing one unit at a time and handles everything that can happen at a boundary.
        if (n_issued - n_cons == kChainAhead && i_state == OPEN && i_ready && fifo_n == 2) {
          int n = rb_left - 1;
          n = n < cr.u1 - 1 - u ? n : cr.u1 - 1 - u;
          n = n < iu1 - iu - 1 ? n : iu1 - iu - 1;
          n = n < istages - ist - 1 ? n : istages - ist - 1;
          if (n > 0) {
            bool newest_had_sb = mark0 - mark1 == 8;  // loads of the unit issued last: 6, or 8 with scales and biases
            int sb_issued = 0;
            uint32_t slot_off = (uint32_t)slot_i * kSlotBytes + ld * 1024;
            uint32_t sb_off = kSbOffset + (uint32_t)sb_slot_i * kSbSlotBytes + ld * 1024;
            uint32_t w_off = (uint32_t)ist * w_step, x_step = (uint32_t)ist * (kUnitK * 2);
            int st = ist;
#pragma unroll 1
            for (int k = 0; k < n; ++k) {
              // unit u + 1 has landed once at most the newest unit's loads are outstanding
              if (newest_had_sb) __builtin_amdgcn_s_waitcnt(0x0F70 | 8);
              else __builtin_amdgcn_s_waitcnt(0x0F70 | 6);
              asm volatile("s_barrier" ::: "memory");
              newest_had_sb = (st & (CHUNK - 1)) == 0;
              if (newest_had_sb) {
                const uint32_t off = so + (uint32_t)(st / CHUNK) * sb_step;
                load16_to_lds(bs + off, lds + sb_off);
                load16_to_lds(bb + off, lds + sb_off + kSbArrayBytes);
                ++sb_issued;
                sb_off += kSbSlotBytes;
                if (sb_off >= kSbOffset + kSbDepth * kSbSlotBytes) sb_off -= kSbDepth * kSbSlotBytes;
              }
              char* dst = lds + slot_off;
              if (i_coherent) {
                load16_to_lds_coherent(bx + (xo0 + x_step), dst + kXOffset);
                load16_to_lds_coherent(bx + (xo1 + x_step), dst + kXOffset + 4096);
              } else {
                load16_to_lds(bx + (xo0 + x_step), dst + kXOffset);
                load16_to_lds(bx + (xo1 + x_step), dst + kXOffset + 4096);
              }
              load16_to_lds_stream(bw + (wo0 + w_off), dst);
              load16_to_lds_stream(bw + (wo1 + w_off), dst + 4096);
              load16_to_lds_stream(bw + (wo2 + w_off), dst + 8192);
              load16_to_lds_stream(bw + (wo3 + w_off), dst + 12288);
              ++st;
              w_off += w_step;
              x_step += kUnitK * 2;
              slot_off += kSlotBytes;
              if (slot_off >= kDepth * kSlotBytes) slot_off -= kDepth * kSlotBytes;
            }
            // the books, all at once
            ist = st, iu += n;
            slot_i = (slot_i + n) % kDepth;
            sb_slot_i = (sb_slot_i + sb_issued) % kSbDepth;
            tot += 6 * n + 2 * sb_issued;
            mark0 = tot, mark1 = tot - (newest_had_sb ? 8 : 6);  // the two units not yet waited for
            n_issued += n, n_cons += n;
            u += n, rb_left -= n, in_rb += n;
          }
        }
        // unit u + 1 has landed, and every worker holds unit u in registers: its slot is free
#if defined(DFLASH_CHAIN_STAMPS) && DFLASH_CHAIN_STAMPS == 2
        if (ld == 0) DFLASH_STAMP(8, st_idx);
#endif
        if (u + 1 < cr.u1) wait_oldest();
#if defined(DFLASH_CHAIN_STAMPS) && DFLASH_CHAIN_STAMPS == 2
        if (ld == 0) DFLASH_STAMP(9, st_idx);
#elif defined(DFLASH_CHAIN_STAMPS)
        DFLASH_STAMP(wave, st_idx); ++st_idx;
#endif
        asm volatile("s_barrier" ::: "memory");
#if defined(DFLASH_CHAIN_STAMPS) && DFLASH_CHAIN_STAMPS == 2
        if (ld == 0) DFLASH_STAMP(10, st_idx);
#endif
        ++n_cons;
        top_up();
#if defined(DFLASH_CHAIN_STAMPS) && DFLASH_CHAIN_STAMPS == 2
        if (ld == 0) { DFLASH_STAMP(11, st_idx); ++st_idx; }
#endif
        ++in_rb;
        if (--rb_left == 0 || u + 1 == cr.u1) {
          asm volatile("s_barrier" ::: "memory");
          if (epi) asm volatile("s_barrier" ::: "memory");
#ifndef DFLASH_CHAIN_NOHANDOVER
          if (in_rb != cr.stages) any_shared = true;
#endif
          in_rb = 0;
          rb_left = cr.stages;
        }
      }
      if (any_shared && !handover_deferred(p, lds0, cp)) {
        asm volatile("s_barrier" ::: "memory");
        asm volatile("s_barrier" ::: "memory");
        if (epi) asm volatile("s_barrier" ::: "memory");
      }
      if (p.prob[cp].signal) asm volatile("s_barrier" ::: "memory");
    }
    return;
  }

  // Contributors of row block rb of a problem divided as `rx`: the workgroups whose ranges
  // intersect [lo, lo + stages) of the divided line; owner(v) = ceil((v+1)*grid/total) - 1 holds
  // unit v of it.
  auto contributors = [&](const Range& rx, int rb, int& lo_wg, int& hi_wg) __attribute__((always_inline)) {
    const int lo = rx.off + rb * rx.stages;
    lo_wg = (int)((((unsigned)lo + 1u) * (unsigned)rx.grid + rx.total - 1) / (unsigned)rx.total) - 1;
    hi_wg = (int)((((unsigned)(lo + rx.stages)) * (unsigned)rx.grid + rx.total - 1) / (unsigned)rx.total) - 1;
  };

  // ================================== worker waves ====================================
  const int col = lane & 15;
  const int kblk = lane >> 4;
  const uint4 ones = make_uint4(A::kOnes, A::kOnes, A::kOnes, A::kOnes);
  uint32_t mask = 0x000F000Fu, magic = A::kMagic;
  asm volatile("" : "+s"(mask), "+v"(magic));
  const int grp = wave & 3;    // quantisation group of the unit this wave works on
  const int half = wave >> 2;  // rows 64*half .. 64*half + 63: tiles j = 0..3
  const uint32_t xoff =
      lds0 + kXOffset + grp * 2048 + (kblk >> 1) * 1024 + (16 * (2 * (kblk & 1)) + col) * 16;
  const uint32_t wrow = 64 * half + col;
  const uint32_t woff =
      lds0 + wrow * 128 + ((grp ^ ((wrow >> 1) & 3)) << 5) + (kblk >> 1) * 16 + (kblk & 1) * 8;
  const uint32_t soff = lds0 + kSbOffset + wrow * SBROW + grp * 2;

  int rd_slot = 0;            // byte offset of the ring slot of the unit whose operands are fetched next
  int rd_sb = -kSbSlotBytes;  // byte offset of its scale/bias slot
  int cur_slot = 0;           // byte offset of the current unit's ring slot
  f32x4_t acc4[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) acc4[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  Operands op[2];
#ifdef DFLASH_CHAIN_STAMPS
  int wst_idx = 0;
#endif

  // ---- output of whole row blocks; `cpx` names the problem they belong to -------------------
  // Stores tile `wave` of row block rb.  Accumulator r of lane l is (m = 4*(l/16) + r,
  // column 16*wave + l%16) of the row block.  With the epilogue, waves 0..3 hold the gate
  // half and `up` the up half of the same 64 output columns; waves 4..7 store nothing.
  auto store_out = [&](int cpx, size_t index, float v) __attribute__((always_inline)) {
    CProblem& q = p.prob[cpx];
    const uint16_t bits = (uint16_t)A::from_f32(v);
    if (q.signal)
      __hip_atomic_store(&q.y[index], bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else
      q.y[index] = bits;
  };
  auto emit = [&](int cpx, int rb, const f32x4_t& acc) __attribute__((always_inline)) {
    const int n_out = p.prob[cpx].N;
    const int n = rb * kRows + 16 * wave + col;
    if (n >= n_out) return;
#pragma unroll
    for (int r = 0; r < 4; ++r) store_out(cpx, (size_t)(4 * kblk + r) * n_out + n, acc[r]);
  };
  auto emit_epilogue = [&](int cpx, int rb, const f32x4_t& gate, const f32x4_t& up) __attribute__((always_inline)) {
    const int n_out = p.prob[cpx].N >> 1;
    const int n = rb * 64 + 16 * wave + col;
    if (wave >= 4 || n >= n_out) return;
#pragma unroll
    for (int r = 0; r < 4; ++r)
      store_out(cpx, (size_t)(4 * kblk + r) * n_out + n, silu_mul<ACT_FP16>(gate[r], up[r]));
  };
  // The up half's waves (4..7) hand their tile to the gate half's (0..3) through LDS.
  auto exchange_write = [&](int which, const f32x4_t& acc) __attribute__((always_inline)) {
    if (wave >= 4) {
      const uint32_t addr = lds0 + kChainExchange + which * 4096 + (wave - 4) * 1024 + lane * 16;
      asm volatile("ds_write_b128 %0, %1\n s_waitcnt lgkmcnt(0)" : : "v"(addr), "v"(acc) : "memory");
    }
  };
  auto exchange_read = [&](int which) __attribute__((always_inline)) -> f32x4_t {
    f32x4_t v = f32x4_t{0.f, 0.f, 0.f, 0.f};
    if (wave < 4) {
      const uint32_t addr = lds0 + kChainExchange + which * 4096 + wave * 1024 + lane * 16;
      asm volatile("ds_read_b128 %0, %1\n s_waitcnt lgkmcnt(0)" : "=&v"(v) : "v"(addr) : "memory");
    }
    return v;
  };
  // ---- hand-over of a problem's shared row blocks `srb` (at most two: the one this workgroup's
  // range starts in and the one it ends in; see qmm_m16_stream.hip), in three steps:
  //   1. once every worker's partial stores have been acknowledged, and after a barrier: thread 0
  //      bumps the arrival counters (wrapping: the last arrival sees n-1 and leaves 0 behind);
  //   2. thread 0 waits for the counters' answers and leaves "last to arrive" flags in LDS;
  //   3. after a barrier: a workgroup that arrived last adds the partial tiles in contributor
  //      order and stores the result.
  // The steps run back to back at the end of the problem, or - where nothing waits for the
  // result - at the second and the fourth unit of the next problem, whose barriers then stand
  // between them and whose arithmetic hides the first two round trips.
  auto handover_arrive = [&](int cpx, const Range& rx, const int (&srb)[2], uint32_t (&prev)[2]) __attribute__((always_inline)) {
    if (tid == 0) {
      uint32_t* const counters = p.counters + p.prob[cpx].counter_base;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        prev[i] = 0u;
        if (srb[i] >= 0) {
          int lo_wg, hi_wg;
          contributors(rx, srb[i], lo_wg, hi_wg);
          prev[i] = atomicInc(&counters[srb[i]], (uint32_t)(hi_wg - lo_wg));
        }
      }
    }
  };
  auto handover_flags = [&](const Range& rx, const int (&srb)[2], uint32_t (&prev)[2]) __attribute__((always_inline)) {
    if (tid == 0) {
      asm volatile("s_waitcnt vmcnt(0)" : "+v"(prev[0]), "+v"(prev[1]) : : "memory");
      uint32_t flag[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        int lo_wg = 0, hi_wg = 0;
        if (srb[i] >= 0) contributors(rx, srb[i], lo_wg, hi_wg);
        flag[i] = (srb[i] >= 0 && prev[i] == (uint32_t)(hi_wg - lo_wg)) ? 1u : 0u;
      }
      asm volatile("ds_write_b32 %0, %1\n ds_write_b32 %0, %2 offset:4\n s_waitcnt lgkmcnt(0)"
                   :
                   : "v"(lds0 + kChainFlags), "v"(flag[0]), "v"(flag[1])
                   : "memory");
    }
  };
  // Returns the number of row blocks summed; `sum` keeps the totals (for the epilogue's second half).
  auto handover_reduce = [&](int cpx, const Range& rx, const int (&srb)[2], bool (&is_last)[2],
                             f32x4_t (&sum)[2], bool store) __attribute__((always_inline)) -> int {
    uint32_t last0, last1;
    asm volatile("ds_read_b32 %0, %2\n ds_read_b32 %1, %2 offset:4\n s_waitcnt lgkmcnt(0)"
                 : "=&v"(last0), "=&v"(last1)
                 : "v"(lds0 + kChainFlags)
                 : "memory");
    is_last[0] = __builtin_amdgcn_readfirstlane(last0) != 0;
    is_last[1] = __builtin_amdgcn_readfirstlane(last1) != 0;
    const float* const tiles = p.partials + (size_t)p.prob[cpx].partial_base * kPartialFloats;
    int summed = 0;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      sum[i] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      if (!is_last[i]) continue;
      int lo_wg, hi_wg;
      contributors(rx, srb[i], lo_wg, hi_wg);
      // Only the first contributor can have started before the row block (then the block is the
      // one its range ends in, slot 1); every later one starts inside it (slot 0).
      // (in the joint form its range may begin in an earlier problem: here it then begins with
      // row block 0)
      const int first_begin = range_begin(rx.total, lo_wg, rx.grid) - rx.off;
      const int which_first = (first_begin > 0 ? first_begin : 0) < srb[i] * rx.stages ? 1 : 0;
      for (int wg0 = lo_wg; wg0 <= hi_wg; wg0 += 8) {
        const float* src[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int w = wg0 + j <= hi_wg ? wg0 + j : hi_wg;  // surplus slots re-read the last tile
          src[j] = tiles + ((size_t)w * 2 + (w == lo_wg ? which_first : 0)) * kPartialFloats + tid * 4;
        }
        f32x4_t v[8];
        load_partials8(src, v);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          if (wg0 + j <= hi_wg) {
#pragma unroll
            for (int r = 0; r < 4; ++r) sum[i][r] += v[j][r];
            // the workspace is left zero-filled: the streaming kernel, which may share it, takes
            // a non-zero word in a slot of its own for a partial tile that has arrived
            store_partial(const_cast<float*>(src[j]), f32x4_t{0.f, 0.f, 0.f, 0.f});
          }
        }
      }
      if (store) emit(cpx, srb[i], sum[i]);
      ++summed;
    }
    return summed;
  };

  // a hand-over that is spread over the first units of the next problem
  int ho_cp = -1;           // the problem it belongs to (-1: none)
  int ho_rb[2] = {-1, -1};  // its shared row blocks
  uint32_t ho_prev[2] = {0u, 0u};

#pragma unroll 1
  for (int cp = 0; cp < p.count; ++cp) {
    const Range cr = read_range(lds0, cp);
    if (cr.wg < 0) continue;
    CProblem& q = p.prob[cp];
    const bool epi = q.epilogue == DFLASH_QMM_EPILOGUE_SILU_MUL;
    float* const partials = p.partials + (size_t)q.partial_base * kPartialFloats;
    int emitted = 0;  // row blocks of this problem whose output this workgroup has stored

    int rd_q = cr.st0 % CHUNK;
    bool rd_first = true;
    uint32_t rd_x, rd_w, rd_s;
    auto next_addresses = [&]() __attribute__((always_inline)) {
      if (rd_q == 0 || rd_first) {
        rd_sb += kSbSlotBytes;
        if (rd_sb == kSbDepth * kSbSlotBytes) rd_sb = 0;
        rd_first = false;
      }
      rd_x = xoff + rd_slot;
      rd_w = woff + rd_slot;
      rd_s = soff + rd_sb + rd_q * 8;
      rd_slot += kSlotBytes;
      if (rd_slot == kDepth * kSlotBytes) rd_slot = 0;
      rd_q = (rd_q + 1) & (CHUNK - 1);
    };

    asm volatile("s_barrier" ::: "memory");  // the first unit of this problem has landed
#ifdef DFLASH_CHAIN_STAMPS
    if (wave == 0) DFLASH_STAMP(12, cp * 4 + 0);
#endif
#pragma unroll
    for (int j = 0; j < 4; ++j) acc4[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    next_addresses();
    operands_issue_piece<0, SBROW>(rd_x, rd_w, rd_s, op[0], acc4[0]);
    operands_issue_piece<1, SBROW>(rd_x, rd_w, rd_s, op[0], acc4[0]);
    operands_issue_piece<2, SBROW>(rd_x, rd_w, rd_s, op[0], acc4[0]);
    operands_issue_piece<3, SBROW>(rd_x, rd_w, rd_s, op[0], acc4[0]);
    operands_wait(op[0], acc4[0], acc4[1], acc4[2], acc4[3]);
    // The second operand set holds nothing yet (it is filled while the first unit is worked
    // on): saying so keeps its registers free across the problem boundary.
    asm volatile("" : "=v"(op[1].f0), "=v"(op[1].f1), "=v"(op[1].wq[0]), "=v"(op[1].wq[1]), "=v"(op[1].wq[2]),
                 "=v"(op[1].wq[3]));
    asm volatile("" : "=v"(op[1].sv[0]), "=v"(op[1].sv[1]), "=v"(op[1].sv[2]), "=v"(op[1].sv[3]),
                 "=v"(op[1].bv[0]), "=v"(op[1].bv[1]), "=v"(op[1].bv[2]), "=v"(op[1].bv[3]));

    int left = cr.u1 - cr.u0;         // units still to consume, the current one included
    int rb_left = cr.stages - cr.st0;  // same, within the current row block
    int in_rb = 0;                     // units of the current row block this workgroup has done
    int rb = cr.rb0;
    int shared_rb[2] = {-1, -1};       // row blocks whose partial tiles I have stored
    int unit_no = 0;                   // units of this problem consumed so far

#pragma unroll 1
    while (left > 0) {
#pragma unroll
      for (int par = 0; par < 2; ++par) {
        if (left > 0) {
          Operands& cur = op[par];
          Operands& nxt = op[par ^ 1];
          // ---- the previous problem's hand-over, between this problem's barriers ---------
          if (ho_cp >= 0) {
            if (unit_no == kHandoverArriveUnit) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // partial stores acknowledged
            if (unit_no == kHandoverSumUnit) handover_flags(read_range(lds0, ho_cp), ho_rb, ho_prev);
          }
#ifdef DFLASH_CHAIN_STAMPS
          DFLASH_STAMP(wave, wst_idx);
#endif
          asm volatile("s_barrier" ::: "memory");
#ifdef DFLASH_CHAIN_STAMPS
          ++wst_idx;
#endif
          if (ho_cp >= 0) {
            if (unit_no == kHandoverArriveUnit) handover_arrive(ho_cp, read_range(lds0, ho_cp), ho_rb, ho_prev);
            if (unit_no == kHandoverSumUnit) {
              bool is_last[2];
              f32x4_t sum[2];
              handover_reduce(ho_cp, read_range(lds0, ho_cp), ho_rb, is_last, sum, true);
              ho_cp = -1;
            }
          }
          const bool fetch = left > 1;
          if (fetch) next_addresses();
#ifndef DFLASH_CHAIN_NOCOMPUTE  // (timing experiments: the stream without the arithmetic; results are wrong)
          consume_unit<ACT_FP16, SB_FP16, SBROW>(cur, nxt, fetch, rd_x, rd_w, rd_s, acc4, ones, mask, magic);
          if (fetch) operands_wait(nxt, acc4[0], acc4[1], acc4[2], acc4[3]);
#endif
          --left;
          ++in_rb;
          ++unit_no;
          if (--rb_left == 0 || left == 0) {
            // ---- a row block ends inside my range -------------------------------------------
            const uint32_t sbase = lds0 + cur_slot;
            reduce_groups_write(sbase, acc4, wave, lane);
            asm volatile("s_barrier" ::: "memory");
            const f32x4_t acc = reduce_groups_read(sbase, acc4, wave, lane);
#pragma unroll
            for (int j = 0; j < 4; ++j) acc4[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            const bool whole = in_rb == cr.stages;
            if (epi) {
              if (whole) exchange_write(0, acc);
              asm volatile("s_barrier" ::: "memory");
              if (whole) emit_epilogue(cp, rb, acc, exchange_read(0));
            } else if (whole) {
              emit(cp, rb, acc);
            }
            if (whole) {
              ++emitted;
            } else {
              // Other workgroups hold the rest of this row block: partial slot 0 for the row
              // block my range starts in, slot 1 for the one it ends in.
              const int which = rb == cr.rb0 ? 0 : 1;
#ifndef DFLASH_CHAIN_NOHANDOVER  // (timing experiments: shared row blocks are dropped; results are wrong)
              store_partial(partials + ((size_t)cr.wg * 2 + which) * kPartialFloats + tid * 4, acc);
              shared_rb[which] = rb;
#else
              (void)which;
#endif
            }
            ++rb;
            in_rb = 0;
            rb_left = cr.stages;
          }
          cur_slot += kSlotBytes;
          if (cur_slot == kDepth * kSlotBytes) cur_slot = 0;
        }
      }
      // an odd number of units leaves the operands of the next problem's first unit to op[0]
    }

#ifdef DFLASH_CHAIN_STAMPS
    if (wave == 0) DFLASH_STAMP(12, cp * 4 + 1);
#endif
    if (shared_rb[0] >= 0 || shared_rb[1] >= 0) {
      if (handover_deferred(p, lds0, cp)) {
        // the next problem's first units carry it
        ho_cp = cp, ho_rb[0] = shared_rb[0], ho_rb[1] = shared_rb[1];
      } else {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        asm volatile("s_barrier" ::: "memory");
        uint32_t prev[2];
        handover_arrive(cp, cr, shared_rb, prev);
        handover_flags(cr, shared_rb, prev);
        asm volatile("s_barrier" ::: "memory");
        bool is_last[2];
        f32x4_t sum[2];
        emitted += handover_reduce(cp, cr, shared_rb, is_last, sum, !epi);
        if (epi) {
#pragma unroll
          for (int i = 0; i < 2; ++i)
            if (is_last[i]) exchange_write(i, sum[i]);
          asm volatile("s_barrier" ::: "memory");
#pragma unroll
          for (int i = 0; i < 2; ++i)
            if (is_last[i]) emit_epilogue(cp, shared_rb[i], sum[i], exchange_read(i));
        }
      }
    }

#ifdef DFLASH_CHAIN_STAMPS
    if (wave == 0) DFLASH_STAMP(12, cp * 4 + 2);
#endif
    if (q.signal) {
      // every worker's output stores acknowledged, then one bump of the problem's counter
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      asm volatile("s_barrier" ::: "memory");
      if (tid == 0 && emitted > 0)
        __hip_atomic_fetch_add(&done[cp], (uint32_t)emitted, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  if (p.has_deps && tid == 0) {
    // The last workgroup to leave puts the problems' counters back to zero for the next launch
    // (every waiting workgroup has passed its waits by then).
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const uint32_t prev = atomicInc(&status[0], (uint32_t)(nblocks - 1));
    if (prev == (uint32_t)(nblocks - 1)) {
      for (int i = 0; i < p.count; ++i)
        __hip_atomic_store(&done[i], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

}  // namespace stream

// ---------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------
int qmm_stream_grid();
int qmm_stream_pick_grid(int units, int row_blocks, int cus);
bool qmm_stream_eligible(int K, int N, int group_size);

namespace {
bool chain_problem_ok(const dflash_qmm_problem& q, int group_size) {
  if (!qmm_stream_eligible(q.K, q.N, group_size) || q.K % (stream::kUnitK * 4) != 0) return false;
  if ((long long)q.N * q.K / 2 >= (1ll << 32)) return false;  // 32-bit byte offsets inside a matrix
  if (q.layout != DFLASH_QMM_LAYOUT_ROWS && q.layout != DFLASH_QMM_LAYOUT_PACKED) return false;
  if (q.epilogue == DFLASH_QMM_EPILOGUE_SILU_MUL) return q.N % 128 == 0;  // 64 rows of each half per row block
  return q.epilogue == DFLASH_QMM_EPILOGUE_NONE;
}
int chain_row_blocks(const dflash_qmm_problem& q) { return (q.N + stream::kRows - 1) / stream::kRows; }
}  // namespace

size_t qmm_chain_workspace_bytes(const dflash_qmm_problem* problems, int count, int group_size, int flags) {
  if (!problems || count <= 0 || count > stream::kMaxChain) return 0;
  const int cus = qmm_stream_grid();
  const bool joint = (flags & DFLASH_QMM_CHAIN_JOINT_SPLIT) != 0;
  size_t tiles = 0;
  for (int i = 0; i < count; ++i) {
    if (!chain_problem_ok(problems[i], group_size)) return 0;
    const int rbs = chain_row_blocks(problems[i]);
    tiles += 2 * (size_t)(joint ? cus : qmm_stream_pick_grid(rbs * (problems[i].K / stream::kUnitK), rbs, cus));
  }
  return (size_t)64 * 1024 + tiles * stream::kPartialFloats * sizeof(float);
}

int qmm_chain_launch(const dflash_qmm_problem* problems, int count, void* workspace,
                     size_t workspace_bytes, int group_size, int act_dtype, int sb_dtype,
                     int spin_limit, int flags, hipStream_t stream) {
  using namespace stream;
  DFLASH_REQUIRE(problems && count > 0, DFLASH_ERR_ARG, "dflash_qmm_m16_chain: no problems");
  DFLASH_REQUIRE((flags & ~DFLASH_QMM_CHAIN_JOINT_SPLIT) == 0, DFLASH_ERR_ARG, "dflash_qmm_m16_chain: flags %d", flags);
  const bool joint = (flags & DFLASH_QMM_CHAIN_JOINT_SPLIT) != 0;
  DFLASH_REQUIRE(count <= kMaxChain, DFLASH_ERR_SHAPE, "dflash_qmm_m16_chain: at most %d problems per launch, got %d",
                 kMaxChain, count);
  ChainParams p{};
  const int cus = qmm_stream_grid();
  int counters = 0, tiles = 0;
  for (int i = 0; i < count; ++i) {
    const dflash_qmm_problem& q = problems[i];
    DFLASH_REQUIRE(q.x && q.w_q && q.scales && q.biases && q.y, DFLASH_ERR_ARG,
                   "dflash_qmm_m16_chain: null operand in problem %d", i);
    DFLASH_REQUIRE(chain_problem_ok(q, group_size), DFLASH_ERR_SHAPE,
                   "dflash_qmm_m16_chain: problem %d needs group_size 64, K %% 1024 == 0, N %% 16 == 0 "
                   "(N %% 128 == 0 with an epilogue), less than 4 GiB of codes, a known epilogue and layout "
                   "(K=%d N=%d gs=%d epilogue=%d layout=%d)",
                   i, q.K, q.N, group_size, q.epilogue, q.layout);
    DFLASH_REQUIRE(((uintptr_t)q.x % 16) == 0 && ((uintptr_t)q.w_q % 16) == 0 && ((uintptr_t)q.scales % 16) == 0 &&
                       ((uintptr_t)q.biases % 16) == 0,
                   DFLASH_ERR_ARG, "dflash_qmm_m16_chain: operands of problem %d must be 16-byte aligned", i);
    DFLASH_REQUIRE(q.wait_for >= -1 && q.wait_for < i, DFLASH_ERR_ARG,
                   "dflash_qmm_m16_chain: problem %d can only wait for an earlier problem (wait_for=%d)", i,
                   q.wait_for);
    DFLASH_REQUIRE(!(joint && q.wait_for >= 0), DFLASH_ERR_ARG,
                   "dflash_qmm_m16_chain: the joint split is for independent problems (problem %d waits for %d): "
                   "a workgroup whose range lies in a later problem would sit waiting from the start", i, q.wait_for);
    if (q.wait_for >= 0) {
      const dflash_qmm_problem& src = problems[q.wait_for];
      const int src_cols = src.epilogue == DFLASH_QMM_EPILOGUE_SILU_MUL ? src.N / 2 : src.N;
      DFLASH_REQUIRE(q.x == src.y && q.K == src_cols, DFLASH_ERR_ARG,
                     "dflash_qmm_m16_chain: problem %d waits for problem %d, so its x must be that problem's y "
                     "[16, %d] (K=%d)", i, q.wait_for, src_cols, q.K);
      p.prob[q.wait_for].signal = 1;
      p.has_deps = 1;
    }
    ChainProblem& d = p.prob[i];
    d.x = (const uint16_t*)q.x;
    d.w = q.w_q;
    d.scales = (const uint16_t*)q.scales;
    d.biases = (const uint16_t*)q.biases;
    d.y = (uint16_t*)q.y;
    d.K = q.K;
    d.N = q.N;
    const int rbs = chain_row_blocks(q);
    d.grid = joint ? cus : qmm_stream_pick_grid(rbs * (q.K / kUnitK), rbs, cus);
    d.counter_base = counters;
    d.partial_base = tiles;
    d.wait_for = q.wait_for;
    d.epilogue = q.epilogue;
    DFLASH_REQUIRE(q.layout == problems[0].layout, DFLASH_ERR_ARG,
                   "dflash_qmm_m16_chain: all problems of a launch share one weight layout (problem %d)", i);
    counters += rbs;
    tiles += 2 * d.grid;
  }
  DFLASH_REQUIRE(counters <= kChainCounterWords, DFLASH_ERR_SHAPE,
                 "dflash_qmm_m16_chain: %d row blocks in one chain, at most %d", counters, kChainCounterWords);
  const size_t need = (size_t)64 * 1024 + (size_t)tiles * kPartialFloats * sizeof(float);
  DFLASH_REQUIRE(workspace && workspace_bytes >= need, DFLASH_ERR_WORKSPACE,
                 "dflash_qmm_m16_chain: workspace of %zu bytes needed, %zu given", need,
                 workspace ? workspace_bytes : (size_t)0);
  p.count = count;
  p.counters = (uint32_t*)workspace;
  p.partials = (float*)((char*)workspace + 64 * 1024);
  p.spin_limit = spin_limit > 0 ? spin_limit : (1 << 22);
  p.joint = joint ? 1 : 0;

  const bool a16 = act_dtype == DFLASH_FP16, s16 = sb_dtype == DFLASH_FP16;
  const bool packed = problems[0].layout == DFLASH_QMM_LAYOUT_PACKED;
  const void* const table[2][2][2] = {
      {{(const void*)qmm_chain_kernel<false, false, false>, (const void*)qmm_chain_kernel<false, false, true>},
       {(const void*)qmm_chain_kernel<false, true, false>, (const void*)qmm_chain_kernel<false, true, true>}},
      {{(const void*)qmm_chain_kernel<true, false, false>, (const void*)qmm_chain_kernel<true, false, true>},
       {(const void*)qmm_chain_kernel<true, true, false>, (const void*)qmm_chain_kernel<true, true, true>}}};
  const void* fn = table[a16][s16][packed];
  static bool attr_set[kMaxDevices][8] = {};
  const int idx = (a16 ? 4 : 0) + (s16 ? 2 : 0) + (packed ? 1 : 0);
  const int slot = current_device_slot();
  if (!attr_set[slot][idx] || slot == kMaxDevices - 1) {
    DFLASH_HIP_OK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytesChain));
    attr_set[slot][idx] = true;
  }
  void* args[] = {&p};
  // every workgroup must be resident at once (waits between problems): one per CU at most
  DFLASH_HIP_OK(hipLaunchKernel(fn, dim3(cus), dim3(kThreads), args, kLdsBytesChain, stream));
  return DFLASH_OK;
}

}  // namespace dflash

#ifdef DFLASH_CHAIN_STAMPS
extern "C" int dflash_debug_read_stamps(unsigned long long* out_host) {
  return (int)hipMemcpyFromSymbol(out_host, HIP_SYMBOL(dflash::stream::g_stamps),
                                  sizeof(dflash::stream::g_stamps));
}
#endif

extern "C" int dflash_qmm_m16_pack_gate_up(const uint32_t* w_q, const void* scales, const void* biases,
                                           void* codes_out, void* scales_out, void* biases_out, int K, int N,
                                           int group_size, void* stream) {
  using namespace dflash;
  using namespace dflash::stream;
  DFLASH_REQUIRE(w_q && scales && biases && codes_out && scales_out && biases_out, DFLASH_ERR_ARG,
                 "dflash_qmm_m16_pack_gate_up: null operand");
  DFLASH_REQUIRE(group_size == 64 && K > 0 && K % (kUnitK * 4) == 0 && N > 0 && N % 128 == 0, DFLASH_ERR_SHAPE,
                 "dflash_qmm_m16_pack_gate_up: group_size 64, K %% 1024 == 0 and N %% 128 == 0 (gate rows then up rows) "
                 "(K=%d N=%d gs=%d)", K, N, group_size);
  DFLASH_REQUIRE(((uintptr_t)w_q % 16) == 0 && ((uintptr_t)scales % 16) == 0 && ((uintptr_t)biases % 16) == 0 &&
                     ((uintptr_t)codes_out % 16) == 0 && ((uintptr_t)scales_out % 16) == 0 &&
                     ((uintptr_t)biases_out % 16) == 0,
                 DFLASH_ERR_ARG, "dflash_qmm_m16_pack_gate_up: operands must be 16-byte aligned");
  const size_t RB = (size_t)(N / 2 + 63) / 64, stages = (size_t)K / kUnitK;
  const size_t threads = (RB * stages * kPackedUnitBytes + 2 * RB * (stages / 4) * kPackedChunkBytes) / 16;
  hipLaunchKernelGGL(qmm_pack_gate_up_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, w_q, (const uint16_t*)scales, (const uint16_t*)biases, (uint4*)codes_out,
                     (uint4*)scales_out, (uint4*)biases_out, K, N);
  DFLASH_HIP_OK(hipGetLastError());
  return DFLASH_OK;
}

extern "C" size_t dflash_qmm_m16_chain_workspace_bytes(const dflash_qmm_problem* problems, int count,
                                                       int group_size, int flags) {
  return dflash::qmm_chain_workspace_bytes(problems, count, group_size, flags);
}

extern "C" int dflash_qmm_m16_chain(const dflash_qmm_problem* problems, int count, void* workspace,
                                    size_t workspace_bytes, int group_size, int act_dtype, int sb_dtype,
                                    int spin_limit, int flags, void* stream) {
  using namespace dflash;
  DFLASH_REQUIRE(act_dtype == DFLASH_BF16 || act_dtype == DFLASH_FP16, DFLASH_ERR_ARG,
                 "dflash_qmm_m16_chain: act_dtype %d is not bf16/fp16", act_dtype);
  DFLASH_REQUIRE(sb_dtype == DFLASH_BF16 || sb_dtype == DFLASH_FP16, DFLASH_ERR_ARG,
                 "dflash_qmm_m16_chain: sb_dtype %d is not bf16/fp16", sb_dtype);
  return qmm_chain_launch(problems, count, workspace, workspace_bytes, group_size, act_dtype, sb_dtype,
                          spin_limit, flags, (hipStream_t)stream);
}
