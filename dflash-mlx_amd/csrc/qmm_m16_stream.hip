// Streaming M=16 int4 qmm for gfx950: persistent workgroups, LDS-staged weights.
//
// y[16,N] = x[16,K] . (s*q + b)^T for group_size 64, K % 512 == 0, N % 16 == 0 - the
// shapes of the projections in the dense verify stacks - and its gathered form for MoE
// layers, y[p] = x[p] . (s*q + b)^T of expert ids[p] for up to 256 rows: rows that share an
// expert are taken 16 at a time as the M dimension, and the weights of the experts that
// have rows are streamed like one tall matrix.  Same arithmetic as
// qmm_m16.hip (MFMA 16x16x32 on raw codes, scale/bias applied per (column, group) to
// the fp32 accumulators); what differs is how bytes move and who moves them:
//
//  * The weight matrix is cut into units of 128 rows x 256 k (16 KiB of codes plus the
//    8 KiB slice of x they multiply; scales/biases come per chunk of four units).  Units
//    are numbered row-block-major and divided EVENLY among a persistent grid of at most one
//    workgroup per CU: every workgroup streams the same number of bytes (+-1 unit) whatever N
//    and K are, fills its load pipeline once, and there is no tail of half-empty rounds.  The
//    host prefers a grid that is a multiple of the number of row blocks when that costs at most
//    two units of range length (qmm_stream_pick_grid): no range then crosses a row block.
//  * A workgroup is 8 worker waves plus 4 loader waves.  Loaders do nothing but move units
//    global -> LDS with 16-byte direct loads (no VGPR staging; each instruction moves
//    128-byte row segments of 8 rows) into a ring of slots, a few units ahead of the
//    workers.  An instruction that finds the CU's load queue full sits in its issue stage;
//    in a loader that costs nothing, in a worker it would stop the arithmetic.  Granules
//    are XOR-swizzled inside a row so that MFMA-shaped reads spread over the LDS banks.
//  * Within a unit, worker w handles ONE quantisation group (w & 3) for 64 rows (four MFMA
//    tiles, rows 64*(w >> 2) ..): the x fragments and the row sums of x (an MFMA against
//    ones, already in accumulator layout) are shared by its four tiles.  The operands of
//    the next unit are read from LDS into a second register set while the current unit is
//    worked on, a few reads between one tile and the next.  The four workers that cover
//    the same rows add their accumulators through LDS only when a row block ends; after
//    that worker w holds tile w.
//  * A workgroup whose range covers all of K for a row block writes y directly.  Row
//    blocks shared between workgroups go through fp32 partial tiles in the workspace, in
//    ONE memory round trip: a partial tile is its own "ready" flag.  Slots read zero
//    between calls; a contributor stores its tile with every +0.0 written as -0.0, so that
//    no word of a stored tile has the bit pattern zero, and leaves.  One fixed contributor
//    per row block - the one with the highest block index, so that everything it waits for
//    was dispatched before it - keeps its own tile in registers, reads the others' slots
//    until every word is non-zero, adds the tiles in contributor order, rounds once, and
//    puts the slots back to zero.  Deterministic; the wait is bounded (a workgroup that
//    gives up records an error word in the workspace and the launch still ends).  Partials
//    are written through to / read from the level all XCDs share (sc1): no L2 write-back
//    fence is ever issued, nobody waits for a store to be acknowledged, and there is no
//    arrival counter whose answer somebody would have to wait for.
//
// The compiler orders every LDS access it can see behind ALL outstanding direct-to-LDS
// loads (s_waitcnt vmcnt(0)), and __syncthreads() carries a fence with the same effect;
// either would drain the ring on every unit.  The kernel therefore touches LDS only
// through hand-written instruction blocks and synchronises with bare s_barriers; a loader
// waits for "my part of unit v has landed" with an explicit vmcnt (loads retire in issue
// order, and the number a loader issues per unit is a closed form of the unit index).
// Every instruction a wave issues costs it at least four cycles, scalar bookkeeping
// included, so the per-unit paths are kept short: ring positions advance by addition,
// and the loaders and the workers run separate loops that meet only at the barriers.
#include <cstdlib>

#include "dflash_common.h"
#include "qmm_stream_device.h"

namespace dflash {
namespace stream {

struct Params {
  const uint16_t* x;
  const uint32_t* w;
  const uint16_t* scales;
  const uint16_t* biases;
  uint16_t* y;
  float* partials;     // [2 * grid][wave][lane][4] fp32; all zero between calls
  uint32_t* status;    // the 64 KiB block ahead of the partial tiles: [kErrorWord] is set when a wait gives up
  int spin_limit;      // polls of a row block's partial tiles before the adding workgroup gives up
#ifdef DFLASH_STREAM_STAMPS
  int stamp_slot;
#endif
  int K, N;
  int stages;          // K / 256
  int units;           // row blocks * stages (dense form; the gathered form counts its own)
  // gathered form: x, y [P, .], row p goes through the weights of expert expert_ids[p];
  // w, scales, biases hold E matrices of [N, .] back to back
  const int32_t* expert_ids;
  int P, E;
  // dense form, K % 1024 == 0: w, scales, biases hold the images qmm_pack_kernel writes - per
  // (row block, unit) the 16 KiB of codes in the order of the LDS slot, per (row block, chunk)
  // 4 KiB of scales and of biases - so that every load instruction of a wave moves 1 KiB of
  // consecutive memory
  int packed;
};

// Writes the packed images of one [N, K] matrix (K % 1024 == 0): one thread per 16 bytes of
// output.  Codes: granule (q, lane) of unit (rb, st) is granule (lane & 7) ^ sw(lane >> 3) of
// row 128 rb + 8 q + (lane >> 3), bytes 128 st .. 128 st + 127 - the lane order of the loader
// waves' instruction q.  Scales and biases: granule (part, lane) of chunk (rb, c) is granule
// lane & 1 of row 128 rb + 32 part + (lane >> 1), groups 16 c .. 16 c + 15.  Rows past N repeat
// row N - 1 (their products are never stored).
__global__ __launch_bounds__(256) void qmm_pack_kernel(const uint32_t* __restrict__ w,
                                                       const uint16_t* __restrict__ scales,
                                                       const uint16_t* __restrict__ biases,
                                                       uint4* __restrict__ w_out, uint4* __restrict__ s_out,
                                                       uint4* __restrict__ b_out, int K, int N) {
  const int stages = K / kUnitK, chunks = stages / 4;
  const int RB = (N + kRows - 1) / kRows;
  const size_t code_granules = (size_t)RB * stages * (kPackedUnitBytes / 16);
  const size_t sb_granules = (size_t)RB * chunks * (kPackedChunkBytes / 16);
  const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < code_granules) {
    const int lane = (int)(t & 63), q = (int)((t >> 6) & 15);
    const size_t unit = t >> 10;
    const int st = (int)(unit % stages), rb = (int)(unit / stages);
    const int r8 = lane >> 3;
    int row = rb * kRows + 8 * q + r8;
    row = row < N ? row : N - 1;
    const int g = (lane & 7) ^ (((r8 >> 1) & 3) << 1);
    w_out[t] = *reinterpret_cast<const uint4*>((const char*)w + (size_t)row * (K >> 1) + st * (kUnitK / 2) + g * 16);
  } else if (t < code_granules + 2 * sb_granules) {
    size_t u = t - code_granules;
    const bool is_bias = u >= sb_granules;
    if (is_bias) u -= sb_granules;
    const int lane = (int)(u & 63), part = (int)((u >> 6) & 3);
    const size_t chunk = u >> 8;
    const int c = (int)(chunk % chunks), rb = (int)(chunk / chunks);
    int row = rb * kRows + 32 * part + (lane >> 1);
    row = row < N ? row : N - 1;
    const char* src = (const char*)(is_bias ? biases : scales) + ((size_t)row * (K / kGS) + c * 16) * 2 + (lane & 1) * 16;
    (is_bias ? b_out : s_out)[u] = *reinterpret_cast<const uint4*>(src);
  }
}

#ifdef DFLASH_STREAM_STAMPS
// Experiment builds only: wall-clock stamps of wave 0 (a worker) and wave 8 (a loader) of every
// workgroup, for the last 64 launches.  [launch % 64][block][event]
__device__ unsigned long long g_sstamps[64][256][16];
#define DFLASH_SSTAMP(ev)                                                                     \
  do {                                                                                        \
    if (lane == 0 && (wave == 0 || wave == kWaves) && blockIdx.x < 256)                       \
      g_sstamps[p.stamp_slot & 63][blockIdx.x][ev] = wall_clock64();                         \
  } while (0)
#else
#define DFLASH_SSTAMP(ev) do {} while (0)
#endif

// CHUNK: units per scale/bias chunk (4, or 2 when K is a multiple of 512 only).
// GATHER: per-expert form.  Rows of x that share an expert are taken 16 at a time as one
// "entry"; an entry is a matrix problem of its own, [rows, K] x [N, K]^T, and the unit
// space is that of all entries back to back: virtual row block = entry * RB + row block.
template <bool ACT_FP16, bool SB_FP16, int CHUNK, bool GATHER>
__global__ __launch_bounds__(kThreads, 1) void qmm_stream_kernel(Params p) {
  using A = Act<ACT_FP16>;
  constexpr int SBROW = 8 * CHUNK;              // bytes of scales per row and chunk
  constexpr int kChunkLoads = CHUNK == 4 ? 2 : 1;  // loads per loader and chunk
  // The first unit is what a launch waits for longest, and its scales and biases (256 pieces
  // of 32 bytes, one DRAM access each) are the last of it to land.  The worker waves, which
  // have nothing to do until that unit is in LDS, ask for it as their first instructions -
  // about a microsecond before the loader waves have their pointers set up - and the loaders
  // start with the second unit.  CHUNK = 4: per worker lane one 16-byte load of scales or biases
  // (wave w < 4 the scales of rows 32 w .., the others the biases), one of x (instruction w of
  // the loaders' scheme) and two of codes (instructions 2 w, 2 w + 1).
  constexpr bool kWorkersFetchFirstChunk = CHUNK == 4;
  constexpr int kFirst = kWorkersFetchFirstChunk ? 1 : 0;  // units at the head of the range the loaders skip
  extern __shared__ __attribute__((aligned(1024))) char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t lds0 = lds_address(lds);
  if (wave == 0) DFLASH_SSTAMP(0);
  if (wave == kWaves) DFLASH_SSTAMP(8);
  const int RB = (p.N + kRows - 1) / kRows;  // row blocks of one matrix
  // bytes from one unit's codes to the next unit's of the same rows, and from chunk to chunk
  const bool packed = !GATHER && CHUNK == 4 && p.packed;
  const uint32_t w_unit_stride = packed ? kPackedUnitBytes : kUnitK / 2;
  const uint32_t sb_chunk_stride = packed ? kPackedChunkBytes : CHUNK * kGroups * 2;

  int units = p.units;
  if (GATHER) {
    // ---- entry tables (ordinary code: no direct-to-LDS load has been issued yet) ----------
    uint32_t* t_count = reinterpret_cast<uint32_t*>(lds + kTabOffset + kTabCount);
    uint32_t* t_entry = reinterpret_cast<uint32_t*>(lds + kTabOffset + kTabEntry);
    uint16_t* t_rows = reinterpret_cast<uint16_t*>(lds + kTabOffset + kTabRows);
    uint32_t* t_total = reinterpret_cast<uint32_t*>(lds + kTabOffset + kTabTotal);
    // Every workgroup builds the same tables: a row's place among the rows of its expert is
    // its rank by row index, not the order in which threads happen to get there (partial
    // tiles of one row block come from several workgroups and must agree on the rows).
    for (int e = tid; e < p.E; e += kThreads) t_count[e] = 0;
    int my_e = -1;
    if (tid < p.P) {
      const int e = p.expert_ids[tid];
      if (e >= 0 && e < p.E) my_e = e;
      t_entry[tid] = (uint32_t)my_e;  // the ids, until the entries are written below
    }
    __syncthreads();
    int my_pos = 0;
    if (my_e >= 0) {
      atomicAdd(&t_count[my_e], 1u);
      for (int j = 0; j < tid; ++j) my_pos += (t_entry[j] == (uint32_t)my_e) ? 1 : 0;
    }
    __syncthreads();
    if (wave == 0) {
      // exclusive scan of ceil(rows / 16) over the experts: first entry of each expert
      int carry = 0;
      for (int base = 0; base < p.E; base += 64) {
        const int e = base + lane;
        const int rows = e < p.E ? (int)t_count[e] : 0;
        const int n = (rows + 15) >> 4;
        int incl = n;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
          const int up = __shfl_up(incl, d, 64);
          if (lane >= d) incl += up;
        }
        if (e < p.E) t_count[e] = ((uint32_t)rows << 16) | (uint32_t)(carry + incl - n);
        carry += __shfl(incl, 63, 64);
      }
      if (lane == 0) *t_total = (uint32_t)carry;
    }
    __syncthreads();
    if (my_e >= 0) {
      const uint32_t c = t_count[my_e];
      const int rows = (int)(c >> 16), first = (int)(c & 0xFFFFu);
      const int ent = first + (my_pos >> 4), m = my_pos & 15;
      t_rows[ent * 16 + m] = (uint16_t)tid;
      if (m == 0) {
        const int left_rows = rows - (my_pos & ~15);
        t_entry[ent] = ((uint32_t)(left_rows < 16 ? left_rows : 16) << 16) | (uint32_t)my_e;
      }
    }
    __syncthreads();
    units = (int)*t_total * RB * p.stages;
    // A row whose expert id is outside [0, E) belongs to no entry: its output is zero (written
    // here, by the first workgroup, so that no row of y is left as it was found).
    if (blockIdx.x == 0 && tid < p.P && my_e < 0) {
      for (int n = 0; n < p.N; ++n) p.y[(size_t)tid * p.N + n] = 0;
    }
  }

  // Workgroups beyond the number of units leave; the others divide the units among
  // themselves, so every one of them has work and every contributor of a row block arrives.
  const int grid = (int)gridDim.x < units ? (int)gridDim.x : units;
  // Workgroups are handed to the eight XCDs in turn (b % 8), each with an L2 of its own, while
  // neighbours in unit order share the scale/bias lines and the partial tiles of the row block
  // they split: with a full grid, unit ranges follow the XCD-major order b % 8, b / 8, so that
  // neighbours mostly sit behind the same L2.
  const int xcds = 8;
  const int wg = (grid == (int)gridDim.x && grid % xcds == 0)
                     ? (int)(blockIdx.x % xcds) * (grid / xcds) + (int)(blockIdx.x / xcds)
                     : (int)blockIdx.x;
  if (wg >= grid) return;
  const int u0 = range_begin(units, wg, grid);
  const int u1 = range_begin(units, wg + 1, grid);
  const int rb0 = u0 / p.stages, st0 = u0 - rb0 * p.stages;  // (virtual) row block, stage

  // Where a virtual row block lives: entry, row block inside the matrix, expert, rows.
  struct Where {
    int entry, rb, expert, rows;
  };
  auto locate = [&](int vrb) __attribute__((always_inline)) -> Where {
    Where wh;
    if (GATHER) {
      wh.entry = vrb / RB;
      wh.rb = vrb - wh.entry * RB;
      const uint32_t e = lds_read_u32(lds0 + kTabOffset + kTabEntry + 4 * wh.entry);
      wh.expert = (int)(e & 0xFFFFu);
      wh.rows = (int)(e >> 16);
    } else {
      wh.entry = 0, wh.rb = vrb, wh.expert = 0, wh.rows = 16;
    }
    return wh;
  };

  // Both kinds of wave walk the same units and pass the same barriers:
  //   one before the loop (unit u0 has landed),
  //   one per unit u (unit u+1 has landed; every worker holds unit u in registers, so the
  //     slot of unit u is free),
  //   when a row block ends with unit u: one more (the slot of unit u carries the cross-wave
  //     sum),
  // (the hand-over of shared row blocks after the last unit involves the worker waves only,
  // each on its own: no barrier).

  if (wave >= kWaves) {
    // ================================ loader waves ====================================
    //  codes: 16 instructions cover 128 rows x 128 B; instruction q holds rows 8q..8q+7,
    //         lane = 8*row_in_8 + slot, and slot holds granule slot ^ sw(row) with
    //         sw(row) = ((row >> 1) & 3) << 1  (swaps 32-byte pairs, i.e. whole groups);
    //         loader l issues q = l, l+4, l+8, l+12
    //  x:     8 instructions; instruction i moves group i>>1, k-blocks 2*(i&1) and 2*(i&1)+1:
    //         lane = 16*(2*kbl + j) + m fetches x[m][64g + 16*(2*(i&1) + kbl) + 8j .. +7],
    //         64 contiguous bytes per row; loader l issues i = l, l+4
    //  scales/biases of a chunk, CHUNK = 4: 4 + 4 instructions of 32 rows, two 16-byte
    //         granules per row; loader l issues scales and biases of rows 32l..32l+31
    //         CHUNK = 2: 2 + 2 instructions of 64 rows, one granule per row; loaders 0, 1
    //         issue the scales of rows 0..63, 64..127, loaders 2, 3 the biases
    const int ld = wave - kWaves;
    const int G = p.K / kGS;
    const size_t row_bytes = (size_t)p.K >> 1;
    const int w_r = lane >> 3;
    const int w_c = (lane & 7) ^ (((w_r >> 1) & 3) << 1);
    const char* xp[2];   // x of this lane's row at stage 0
    const char* wp[4];   // codes of this lane's rows at stage 0 of the row block being issued
    const char* sbp[2];  // scales / biases of this lane's row, chunk 0 (CHUNK = 2: [0] only)
    auto set_row_block = [&](int vrb) __attribute__((always_inline)) {
      const Where wh = locate(vrb);
      const int row0 = wh.rb * kRows;
      const uint32_t* wmat = p.w + (size_t)wh.expert * p.N * (row_bytes >> 2);
      const uint16_t* smat = p.scales + (size_t)wh.expert * p.N * G;
      const uint16_t* bmat = p.biases + (size_t)wh.expert * p.N * G;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int row = row0 + 8 * (ld + 4 * i) + w_r;
        row = row < p.N ? row : p.N - 1;
        wp[i] = (const char*)wmat + (size_t)row * row_bytes + w_c * 16;
      }
      if (!GATHER && CHUNK == 4 && p.packed) {
        const char* img = (const char*)p.w + (size_t)wh.rb * p.stages * kPackedUnitBytes + lane * 16;
#pragma unroll
        for (int i = 0; i < 4; ++i) wp[i] = img + (ld + 4 * i) * 1024;
        const size_t sb_img = (size_t)wh.rb * (p.stages / 4) * kPackedChunkBytes + ld * 1024 + lane * 16;
        sbp[0] = (const char*)p.scales + sb_img;
        sbp[1] = (const char*)p.biases + sb_img;
      } else if (CHUNK == 4) {
        int row = row0 + 32 * ld + (lane >> 1);
        row = row < p.N ? row : p.N - 1;
        sbp[0] = (const char*)(smat + (size_t)row * G) + (lane & 1) * 16;
        sbp[1] = (const char*)(bmat + (size_t)row * G) + (lane & 1) * 16;
      } else {
        int row = row0 + 64 * (ld & 1) + lane;
        row = row < p.N ? row : p.N - 1;
        sbp[0] = (const char*)(((ld & 2) ? bmat : smat) + (size_t)row * G);
        sbp[1] = sbp[0];
      }
      // rows of x: the entry's rows in the order of its table; surplus rows of the MFMA tile
      // repeat the entry's first row (their results are never stored)
      int xrow = lane & 15;
      if (GATHER) {
        const int m = xrow < wh.rows ? xrow : 0;
        xrow = (int)lds_read_u16(lds0 + kTabOffset + kTabRows + 2 * (wh.entry * 16 + m));
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int xi = ld + 4 * i;
        xp[i] = (const char*)(p.x + (size_t)xrow * p.K + (xi >> 1) * kGS +
                              (2 * (xi & 1) + (lane >> 5)) * 16 + ((lane >> 4) & 1) * 8);
      }
    };

    int rb_i = rb0, st_i = st0;  // next unit to issue
    int issued = u0 + kFirst;
    int slot_i = kFirst;  // ring slot of the next unit to issue
    if (kFirst && ++st_i == p.stages) {
      st_i = 0;
      ++rb_i;
    }
    int sb_slot_i = kFirst;  // scale/bias slot of the next chunk to issue
    if (issued < u1 || !kFirst) set_row_block(rb_i);
    // Issues one unit: 6 loads (2 for x, 4 for codes), plus kChunkLoads with the first unit
    // of every scale/bias chunk and with the first unit of the range.
    auto issue_next = [&]() __attribute__((always_inline)) {
      char* slot = lds + slot_i * kSlotBytes;
      if ((st_i % CHUNK) == 0 || (!kFirst && issued == u0)) {
        char* sb = lds + kSbOffset + sb_slot_i * kSbSlotBytes;
        const size_t off = (size_t)(st_i / CHUNK) * sb_chunk_stride;
        if (CHUNK == 4) {
          load16_to_lds(sbp[0] + off, sb + ld * 1024);
          load16_to_lds(sbp[1] + off, sb + kSbArrayBytes + ld * 1024);
        } else {
          load16_to_lds(sbp[0] + off, sb + (ld >> 1) * kSbArrayBytes + (ld & 1) * 1024);
        }
        if (++sb_slot_i == kSbDepth) sb_slot_i = 0;
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
        load16_to_lds(xp[i] + (size_t)st_i * (kUnitK * 2), slot + kXOffset + (ld + 4 * i) * 1024);
#pragma unroll
      for (int i = 0; i < 4; ++i)
        load16_to_lds_stream(wp[i] + (size_t)st_i * w_unit_stride, slot + (ld + 4 * i) * 1024);
      ++issued;
      if (++slot_i == kDepth) slot_i = 0;
      if (++st_i == p.stages) {
        st_i = 0;
        ++rb_i;
        if (issued < u1) set_row_block(rb_i);
      }
    };
    // Loads this loader has issued for units u0..v.  Unit indices are global and the number
    // of stages is a multiple of CHUNK, so a unit starts a chunk iff its index is one.
    auto loads_through = [&](int v) __attribute__((always_inline)) -> int {
      return 6 * (v - u0 + 1 - kFirst) + kChunkLoads * (1 - kFirst + (v / CHUNK) - (u0 / CHUNK));
    };
    // Waits until this loader's part of unit v has landed (loads retire in issue order).
    auto wait_unit = [&](int v) __attribute__((always_inline)) {
      wait_loads(loads_through(issued - 1) - loads_through(v));
    };

    const int ahead = units < 4 * grid ? kAheadShort : kAhead;
    DFLASH_SSTAMP(9);
    for (int i = kFirst; i < ahead && issued < u1; ++i) issue_next();
    if (!kFirst) wait_unit(u0);
    DFLASH_SSTAMP(10);
    asm volatile("s_barrier" ::: "memory");
    DFLASH_SSTAMP(11);
    int rb_left = p.stages - st0;  // units of the current row block from unit u on
#pragma unroll 1
    for (int u = u0; u < u1; ++u) {
      const bool rb_ends = rb_left == 1 || u + 1 == u1;
      if (u + 1 < u1) wait_unit(u + 1);
      asm volatile("s_barrier" ::: "memory");
      // keep kAhead units issued beyond unit u; their slots are free: the ring has kDepth > kAhead
      // slots, and the slot of unit u itself (which may carry a cross-wave sum below) is only
      // refilled kDepth - kAhead units later
      const int limit = u + ahead;
      while (issued <= limit && issued < u1) issue_next();
      --rb_left;
      if (rb_ends) {
        asm volatile("s_barrier" ::: "memory");
        rb_left = p.stages;
      }
    }
    return;
  }

  // ================================== worker waves ====================================
  if (kWorkersFetchFirstChunk) {
    const Where wh = locate(rb0);
    const int G = p.K / kGS;
    const int part = wave & 3;
    int row = wh.rb * kRows + 32 * part + (lane >> 1);
    row = row < p.N ? row : p.N - 1;
    const uint16_t* mat = (wave < 4 ? p.scales : p.biases) + (size_t)wh.expert * p.N * G;
    const char* src = (const char*)(mat + (size_t)row * G) + (lane & 1) * 16 +
                      (size_t)(st0 / CHUNK) * (CHUNK * kGroups * 2);
    if (packed)
      src = (const char*)(wave < 4 ? p.scales : p.biases) +
            ((size_t)wh.rb * (p.stages / 4) + st0 / CHUNK) * kPackedChunkBytes + part * 1024 + lane * 16;
    load16_to_lds(src, lds + kSbOffset + (wave < 4 ? 0 : kSbArrayBytes) + part * 1024);
    // x: instruction `wave` of the loaders' scheme; codes: instructions 2 wave and 2 wave + 1
    int xrow = lane & 15;
    if (GATHER) {
      const int m = xrow < wh.rows ? xrow : 0;
      xrow = (int)lds_read_u16(lds0 + kTabOffset + kTabRows + 2 * (wh.entry * 16 + m));
    }
    const char* xsrc = (const char*)(p.x + (size_t)xrow * p.K + (wave >> 1) * kGS +
                                     (2 * (wave & 1) + (lane >> 5)) * 16 + ((lane >> 4) & 1) * 8) +
                       (size_t)st0 * (kUnitK * 2);
    load16_to_lds(xsrc, lds + kXOffset + wave * 1024);
    const size_t row_bytes = (size_t)p.K >> 1;
    const uint32_t* wmat = p.w + (size_t)wh.expert * p.N * (row_bytes >> 2);
    const int w_r = lane >> 3;
    const int w_c = (lane & 7) ^ (((w_r >> 1) & 3) << 1);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int q = 2 * wave + i;
      int wrow = wh.rb * kRows + 8 * q + w_r;
      wrow = wrow < p.N ? wrow : p.N - 1;
      const char* wsrc = (const char*)wmat + (size_t)wrow * row_bytes + w_c * 16 + (size_t)st0 * (kUnitK / 2);
      if (packed)
        wsrc = (const char*)p.w + ((size_t)wh.rb * p.stages + st0) * kPackedUnitBytes + q * 1024 + lane * 16;
      load16_to_lds_stream(wsrc, lds + q * 1024);
    }
  }
  const int col = lane & 15;
  const int kblk = lane >> 4;
  const uint4 ones = make_uint4(A::kOnes, A::kOnes, A::kOnes, A::kOnes);
  uint32_t mask = 0x000F000Fu, magic = A::kMagic;
  asm volatile("" : "+s"(mask), "+v"(magic));
  const int grp = wave & 3;   // quantisation group of the unit this wave works on
  const int half = wave >> 2; // rows 64*half .. 64*half + 63: tiles j = 0..3
  //   x fragment j of lane (m = col, kb = kblk) for group grp inside a slot: + j*256
  const uint32_t xoff =
      lds0 + kXOffset + grp * 2048 + (kblk >> 1) * 1024 + (16 * (2 * (kblk & 1)) + col) * 16;
  // codes of row 64*half + 16j + col: group grp sits in the 32-byte pair grp ^ ((row >> 1) & 3),
  // which does not depend on j; tile j is 2 KiB further
  const uint32_t wrow = 64 * half + col;
  const uint32_t woff =
      lds0 + wrow * 128 + ((grp ^ ((wrow >> 1) & 3)) << 5) + (kblk >> 1) * 16 + (kblk & 1) * 8;
  // scale of that row: SBROW bytes per row and chunk, four 16-bit values per unit; tile j is
  // 16 rows further, biases one array further
  const uint32_t soff = lds0 + kSbOffset + wrow * SBROW + grp * 2;

  // reading position: the unit whose operands are fetched next
  int rd_slot = 0;   // byte offset of its ring slot
  int rd_sb = -kSbSlotBytes;  // byte offset of its scale/bias slot
  int rd_q = st0 % CHUNK;     // its stage within the chunk
  bool rd_first = true;
  f32x4_t acc4[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) acc4[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  Operands op[2];

  // addresses of the next unit's operands, and the step to the unit after it
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

  // Output of a finished tile: accumulator r of lane l is (m = 4*(l/16) + r, n = 16*wave + l%16)
  // of the row block; in the gathered form m is a position in the entry's row table.
  auto emit = [&](int vrb, const f32x4_t& acc) __attribute__((always_inline)) {
    const Where wh = locate(vrb);
    const int n_out = wh.rb * kRows + 16 * wave + col;
    if (n_out >= p.N) return;
    if (GATHER) {
      const u32x2_t rr = lds_read_u64(lds0 + kTabOffset + kTabRows + 2 * (wh.entry * 16 + 4 * kblk));
      const uint32_t rows4[4] = {rr.x & 0xFFFFu, rr.x >> 16, rr.y & 0xFFFFu, rr.y >> 16};
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (4 * kblk + r < wh.rows) p.y[(size_t)rows4[r] * p.N + n_out] = (uint16_t)A::from_f32(acc[r]);
      }
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r) p.y[(size_t)(4 * kblk + r) * p.N + n_out] = (uint16_t)A::from_f32(acc[r]);
    }
  };

  DFLASH_SSTAMP(1);
  if (kWorkersFetchFirstChunk) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  DFLASH_SSTAMP(2);
  asm volatile("s_barrier" ::: "memory");
  DFLASH_SSTAMP(3);
  next_addresses();
  operands_issue_piece<0, SBROW>(rd_x, rd_w, rd_s, op[0], acc4[0]);
  operands_issue_piece<1, SBROW>(rd_x, rd_w, rd_s, op[0], acc4[0]);
  operands_issue_piece<2, SBROW>(rd_x, rd_w, rd_s, op[0], acc4[0]);
  operands_issue_piece<3, SBROW>(rd_x, rd_w, rd_s, op[0], acc4[0]);
  operands_wait(op[0], acc4[0], acc4[1], acc4[2], acc4[3]);

  int left = u1 - u0;            // units still to consume, the current one included
  int rb_left = p.stages - st0;  // same, within the current row block
  int in_rb = 0;                 // units of the current row block this workgroup has done
  int rb = rb0;
  int cur_slot = 0;              // byte offset of the current unit's ring slot
  int mine_rb[2] = {-1, -1};     // shared row blocks whose tiles I add (slot 0: the one my range starts in)
  f32x4_t mine0 = f32x4_t{0.f, 0.f, 0.f, 0.f}, mine1 = mine0;  // my own tiles of those row blocks

  // contributors of a row block: the workgroups whose ranges intersect [lo, lo+stages);
  // owner(v) = ceil((v+1)*grid/units) - 1 is the workgroup whose range holds unit v
  auto contributors = [&](int vrb, int& lo_wg, int& hi_wg) __attribute__((always_inline)) {
    const int lo = vrb * p.stages;
    lo_wg = (int)((((unsigned)lo + 1u) * (unsigned)grid + units - 1) / (unsigned)units) - 1;
    hi_wg = (int)((((unsigned)(lo + p.stages)) * (unsigned)grid + units - 1) / (unsigned)units) - 1;
  };
  // Who adds the tiles of a row block with contributors lo_wg..hi_wg: the one with the highest
  // block index.  Workgroups are dispatched in the order of their block indices, so all the
  // others are running or have finished when it starts: its wait cannot keep a workgroup it
  // waits for off the device.  Unit ranges in block order: the last contributor.  In the
  // XCD-major order (block = (wg % per) * 8 + wg / per, per = grid / 8) the block index grows
  // with wg inside a chunk of `per` ranges, and the last range of a chunk has the highest index
  // of all: the last contributor if the contributors sit in one chunk or end on its last range,
  // else the last range of the chunk before.
  const bool xcd_major = grid == (int)gridDim.x && grid % xcds == 0;
  auto adder_of = [&](int lo_wg, int hi_wg) __attribute__((always_inline)) -> int {
    if (!xcd_major) return hi_wg;
    const int per = grid / xcds;
    const int chunk = hi_wg / per;
    if (lo_wg / per == chunk || hi_wg - chunk * per == per - 1) return hi_wg;
    return chunk * per - 1;
  };
  auto slot_of = [&](int w, int which) __attribute__((always_inline)) -> float* {
    return p.partials + ((size_t)w * 2 + which) * kPartialFloats + tid * 4;
  };

#pragma unroll 1
  while (true) {
#pragma unroll
    for (int par = 0; par < 2; ++par) {
      Operands& cur = op[par];
      Operands& nxt = op[par ^ 1];
      asm volatile("s_barrier" ::: "memory");
      // The next unit's operands are read along the way.  After the last unit the same reads
      // are made once more, of the unit just consumed (valid LDS, results unused): with a
      // condition around them every tile would be a basic block of its own, and the compiler
      // could not run one tile's unpacking under another tile's matrix instructions.
      if (left > 1) next_addresses();
      consume_unit<ACT_FP16, SB_FP16, SBROW>(cur, nxt, true, rd_x, rd_w, rd_s, acc4, ones, mask, magic);
      operands_wait(nxt, acc4[0], acc4[1], acc4[2], acc4[3]);
      --left;
      ++in_rb;
#ifdef DFLASH_STREAM_STAMPS
      if (left + 1 == u1 - u0) DFLASH_SSTAMP(4);
#endif
      if (--rb_left == 0 || left == 0) {
        // ---- a row block ends inside my range ---------------------------------------------
        const uint32_t sbase = lds0 + cur_slot;
        reduce_groups_write(sbase, acc4, wave, lane);
        asm volatile("s_barrier" ::: "memory");
        const f32x4_t acc = reduce_groups_read(sbase, acc4, wave, lane);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc4[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        if (in_rb == p.stages) {
          emit(rb, acc);  // the whole row block was mine
        } else {
          // Other workgroups hold the rest of this row block.  A workgroup shares at most two
          // row blocks: the one its range starts in (partial slot 0) and the one it ends in
          // (slot 1); partial tiles are kept in accumulator layout.  The workgroup that adds
          // keeps its tile; every other one stores it and is done with the row block.
          const int which = rb == rb0 ? 0 : 1;
          int lo_wg, hi_wg;
          contributors(rb, lo_wg, hi_wg);
          if (adder_of(lo_wg, hi_wg) == wg) {
            mine_rb[which] = rb;
            if (which == 0) mine0 = acc;
            else mine1 = acc;
          } else {
            store_partial(slot_of(wg, which), nonzero_words(acc));
          }
        }
        ++rb;
        in_rb = 0;
        rb_left = p.stages;
      }
      cur_slot += kSlotBytes;
      if (cur_slot == kDepth * kSlotBytes) cur_slot = 0;
      if (left == 0) goto hand_over;
    }
  }
hand_over:
  DFLASH_SSTAMP(5);
  // ---- the row blocks whose tiles I add -----------------------------------------------------
  // Every wave on its own (its 1 KiB of every tile): read the other contributors' slots, eight
  // tiles at a time, until no word is zero; add in contributor order, my own tile in its place;
  // store the result; put the slots back to zero for the next call.
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    if (mine_rb[i] < 0) continue;
    int lo_wg, hi_wg;
    contributors(mine_rb[i], lo_wg, hi_wg);
    // Only the first contributor can have started before the row block (then the block is the
    // one its range ends in, slot 1); every later one starts inside it (slot 0).
    const int which_first = range_begin(units, lo_wg, grid) < mine_rb[i] * p.stages ? 1 : 0;
    const f32x4_t own = i == 0 ? mine0 : mine1;
    f32x4_t acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
    for (int wg0 = lo_wg; wg0 <= hi_wg; wg0 += 8) {  // more than eight contributors: long K, few rows
      const float* src[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int w = wg0 + j <= hi_wg ? wg0 + j : hi_wg;  // surplus slots re-read the last tile
        src[j] = slot_of(w, w == lo_wg ? which_first : 0);
      }
      f32x4_t v[8];
      int polls = 0;
      while (true) {
        load_partials8(src, v);
        uint32_t present = 1u;  // stays non-zero while no word of a tile I wait for is zero
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          if (wg0 + j <= hi_wg && wg0 + j != wg) {
            const u32x4_t bits = __builtin_bit_cast(u32x4_t, v[j]);
            present = min(present, min(min(bits.x, bits.y), min(bits.z, bits.w)));
          }
        }
        if (__builtin_amdgcn_ballot_w64(present == 0u) == 0ull) break;
        if (++polls > p.spin_limit) {
          // gives up: the launch ends, this row block's output is wrong, and the caller can tell
          if (lane == 0) __hip_atomic_store(&p.status[kErrorWord], 0x80000000u | (uint32_t)mine_rb[i],
                                            __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
        __builtin_amdgcn_s_sleep(2);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (wg0 + j <= hi_wg) {
          const bool me = wg0 + j == wg;
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[r] += me ? own[r] : v[j][r];
          if (!me) store_partial(const_cast<float*>(src[j]), f32x4_t{0.f, 0.f, 0.f, 0.f});
        }
      }
    }
    DFLASH_SSTAMP(6);
    emit(mine_rb[i], acc);
  }
  DFLASH_SSTAMP(7);
}

}  // namespace stream
}  // namespace dflash

// ---------------------------------------------------------------------------------
// Host side of the streaming kernel (called from dflash_qmm_m16 for eligible shapes).
// ---------------------------------------------------------------------------------
namespace dflash {

int qmm_stream_grid() {
  static int cus[kMaxDevices] = {};
  const int slot = current_device_slot();
  if (cus[slot] == 0 || slot == kMaxDevices - 1) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 256;
    cus[slot] = n > 0 ? (n > 1024 ? 1024 : n) : 256;
  }
  return cus[slot];
}

// Workgroups of a dense launch.  With one workgroup per CU the unit ranges end wherever
// units / CUs puts them, most workgroups work on two row blocks that others share, and a
// workgroup that arrives last at both ends the launch two hand-overs after its last unit.  A
// grid that is a multiple of the number of row blocks cuts every row block into the same
// whole number of ranges: one shared row block per workgroup, fewer contributors to each.
// Measured on the projections of the dense stacks that is worth about two units of streaming
// (5120x7168: 10.7 us with 224 workgroups against 11.8 us with 256; 17408x5120: 15.9 us with 240
// against 17.2 us), and among such grids with the same longest range the smaller one is faster
// (5120x5120: 200 workgroups 9.65 us, 240 9.94 us, 256 10.06 us).  Grids are kept multiples of
// eight, the number of XCDs the ranges are dealt over.
int qmm_stream_pick_grid(int units, int row_blocks, int cus) {
  if (cus > units) return units;
  constexpr int kUnalignedPenalty = 2;  // units
  int best = cus;
  int best_cost = (units + cus - 1) / cus + kUnalignedPenalty;
  if (cus % row_blocks == 0) best_cost -= kUnalignedPenalty;
  for (int g = row_blocks; g <= cus; g += row_blocks) {
    if (g % 8 != 0 || g == cus) continue;
    const int cost = (units + g - 1) / g;
    // ties go to the aligned grid, and among aligned grids to the smaller one
    if (cost < best_cost || (cost == best_cost && (best == cus || g < best))) {
      best = g;
      best_cost = cost;
    }
  }
  return best;
}

bool qmm_stream_eligible(int K, int N, int group_size) {
  // whole scale/bias chunks: K must be a multiple of two units
  if (group_size != 64 || K <= 0 || K % (stream::kUnitK * 2) != 0 || N <= 0 || N % 16 != 0) return false;
  const long long row_blocks = (N + stream::kRows - 1) / stream::kRows;
  const long long units = row_blocks * (K / stream::kUnitK);
  return units * 1024 < (1ll << 31) && row_blocks <= (64 * 1024) / 4;
}

bool qmm_stream_gather_eligible(int P, int K, int N, int E, int group_size) {
  if (!qmm_stream_eligible(K, N, group_size)) return false;
  const long long row_blocks = (N + stream::kRows - 1) / stream::kRows;
  // every row could be an entry of its own
  return P > 0 && P <= stream::kMaxEntries && E > 0 && E <= stream::kMaxExperts &&
         row_blocks * stream::kMaxEntries <= (64 * 1024) / 4 &&
         row_blocks * stream::kMaxEntries * (K / stream::kUnitK) * 1024 < (1ll << 31);
}

size_t qmm_stream_workspace_bytes(int N, int grid) {
  (void)N;
  return (size_t)64 * 1024 + (size_t)grid * 2 * stream::kPartialFloats * sizeof(float);
}

namespace {
template <bool GATHER>
const void* stream_kernel_for(bool a16, bool s16, bool chunk4) {
  using namespace stream;
#define DFLASH_STREAM_PICK(A16, S16)                                                      \
  if (a16 == A16 && s16 == S16)                                                           \
    return chunk4 ? (const void*)qmm_stream_kernel<A16, S16, 4, GATHER>                   \
                  : (const void*)qmm_stream_kernel<A16, S16, 2, GATHER>;
  DFLASH_STREAM_PICK(false, false)
  DFLASH_STREAM_PICK(false, true)
  DFLASH_STREAM_PICK(true, false)
  DFLASH_STREAM_PICK(true, true)
#undef DFLASH_STREAM_PICK
  return nullptr;
}

int launch_stream(stream::Params& p, bool gather, int grid, int act_dtype, int sb_dtype,
                  hipStream_t stream) {
  using namespace stream;
  const bool a16 = act_dtype == DFLASH_FP16, s16 = sb_dtype == DFLASH_FP16;
  const bool chunk4 = p.K % (kUnitK * 4) == 0;
  // (tests shorten the wait of the workgroups that add partial tiles to see them give up)
  p.spin_limit = option(DFLASH_OPT_QMM_SPIN_LIMIT) > 0 ? option(DFLASH_OPT_QMM_SPIN_LIMIT) : kSpinLimit;
  const void* fn = gather ? stream_kernel_for<true>(a16, s16, chunk4) : stream_kernel_for<false>(a16, s16, chunk4);
  const int lds_bytes = gather ? kLdsBytesGather : kLdsBytes;
  // the attribute belongs to the device's copy of the kernel: once per device and kernel
  static bool attr_set[kMaxDevices][16] = {};
  const int idx = (gather ? 8 : 0) + (chunk4 ? 4 : 0) + (a16 ? 2 : 0) + (s16 ? 1 : 0);
  const int slot = current_device_slot();
  if (!attr_set[slot][idx] || slot == kMaxDevices - 1) {
    DFLASH_HIP_OK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes));
    attr_set[slot][idx] = true;
  }
#ifdef DFLASH_STREAM_STAMPS
  static int launches = 0;
  p.stamp_slot = launches++;
#endif
  void* args[] = {&p};
  DFLASH_HIP_OK(hipLaunchKernel(fn, dim3(grid), dim3(kThreads), args, lds_bytes, stream));
  return DFLASH_OK;
}
}  // namespace

int qmm_stream_launch(const void* x, const uint32_t* w, const void* scales, const void* biases,
                      void* y, void* workspace, size_t workspace_bytes, int K, int N,
                      int act_dtype, int sb_dtype, hipStream_t stream) {
  using namespace stream;
  Params p{};
  p.x = (const uint16_t*)x;
  p.w = w;
  p.scales = (const uint16_t*)scales;
  p.biases = (const uint16_t*)biases;
  p.y = (uint16_t*)y;
  p.K = K;
  p.N = N;
  p.stages = K / kUnitK;
  p.units = ((N + kRows - 1) / kRows) * p.stages;
  const int grid = qmm_stream_pick_grid(p.units, p.units / p.stages, qmm_stream_grid());
  const size_t need = qmm_stream_workspace_bytes(N, grid);
  DFLASH_REQUIRE(workspace && workspace_bytes >= need, DFLASH_ERR_WORKSPACE,
                 "dflash_qmm_m16: workspace of %zu bytes needed, %zu given", need,
                 workspace ? workspace_bytes : (size_t)0);
  p.status = (uint32_t*)workspace;
  p.partials = (float*)((char*)workspace + 64 * 1024);
  return launch_stream(p, false, grid, act_dtype, sb_dtype, stream);
}

bool qmm_stream_packed_eligible(int K, int N, int group_size) {
  return qmm_stream_eligible(K, N, group_size) && K % (stream::kUnitK * 4) == 0;
}

void qmm_stream_packed_bytes(int K, int N, size_t* w_bytes, size_t* sb_bytes) {
  const size_t RB = (size_t)(N + stream::kRows - 1) / stream::kRows, stages = (size_t)K / stream::kUnitK;
  *w_bytes = RB * stages * stream::kPackedUnitBytes;
  *sb_bytes = RB * (stages / 4) * stream::kPackedChunkBytes;
}

int qmm_stream_pack(const uint32_t* w, const void* scales, const void* biases, void* w_out,
                    void* s_out, void* b_out, int K, int N, hipStream_t stream) {
  size_t wb, sb;
  qmm_stream_packed_bytes(K, N, &wb, &sb);
  const size_t threads = (wb + 2 * sb) / 16;
  hipLaunchKernelGGL(stream::qmm_pack_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream,
                     w, (const uint16_t*)scales, (const uint16_t*)biases, (uint4*)w_out, (uint4*)s_out,
                     (uint4*)b_out, K, N);
  DFLASH_HIP_OK(hipGetLastError());
  return DFLASH_OK;
}

int qmm_stream_packed_launch(const void* x, const void* w_img, const void* s_img, const void* b_img,
                             void* y, void* workspace, size_t workspace_bytes, int K, int N,
                             int act_dtype, int sb_dtype, hipStream_t stream) {
  using namespace stream;
  Params p{};
  p.x = (const uint16_t*)x;
  p.w = (const uint32_t*)w_img;
  p.scales = (const uint16_t*)s_img;
  p.biases = (const uint16_t*)b_img;
  p.y = (uint16_t*)y;
  p.K = K;
  p.N = N;
  p.stages = K / kUnitK;
  p.units = ((N + kRows - 1) / kRows) * p.stages;
  p.packed = 1;
  const int grid = qmm_stream_pick_grid(p.units, p.units / p.stages, qmm_stream_grid());
  const size_t need = qmm_stream_workspace_bytes(N, grid);
  DFLASH_REQUIRE(workspace && workspace_bytes >= need, DFLASH_ERR_WORKSPACE,
                 "dflash_qmm_m16_packed: workspace of %zu bytes needed, %zu given", need,
                 workspace ? workspace_bytes : (size_t)0);
  p.status = (uint32_t*)workspace;
  p.partials = (float*)((char*)workspace + 64 * 1024);
  return launch_stream(p, false, grid, act_dtype, sb_dtype, stream);
}

int qmm_stream_gather_launch(const void* x, const int32_t* expert_ids, const uint32_t* w,
                             const void* scales, const void* biases, void* y, void* workspace,
                             size_t workspace_bytes, int P, int K, int N, int E, int act_dtype,
                             int sb_dtype, hipStream_t stream) {
  using namespace stream;
  Params p{};
  p.x = (const uint16_t*)x;
  p.w = w;
  p.scales = (const uint16_t*)scales;
  p.biases = (const uint16_t*)biases;
  p.y = (uint16_t*)y;
  p.K = K;
  p.N = N;
  p.stages = K / kUnitK;
  p.units = 0;  // counted on the device from the routing
  p.expert_ids = expert_ids;
  p.P = P;
  p.E = E;
  // the number of entries is not known here: a full grid, workgroups without units leave
  const int grid = qmm_stream_grid();
  const size_t need = qmm_stream_workspace_bytes(N, grid);
  DFLASH_REQUIRE(workspace && workspace_bytes >= need, DFLASH_ERR_WORKSPACE,
                 "dflash_qmm_m16_gather: workspace of %zu bytes needed, %zu given", need,
                 workspace ? workspace_bytes : (size_t)0);
  p.status = (uint32_t*)workspace;
  p.partials = (float*)((char*)workspace + 64 * 1024);
  return launch_stream(p, true, grid, act_dtype, sb_dtype, stream);
}

}  // namespace dflash

#ifdef DFLASH_STREAM_STAMPS
extern "C" int dflash_debug_read_stream_stamps(unsigned long long* out_host) {
  return (int)hipMemcpyFromSymbol(out_host, HIP_SYMBOL(dflash::stream::g_sstamps), sizeof(dflash::stream::g_sstamps));
}
#endif
