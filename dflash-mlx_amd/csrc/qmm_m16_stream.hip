// Streaming M=16 int4 qmm for gfx950: persistent workgroups, LDS-staged weights.
//
// y[16,N] = x[16,K] . (s*q + b)^T for group_size 64, K % 1024 == 0, N % 16 == 0 -
// the shapes of the projections in the dense verify stacks.  Same arithmetic as
// qmm_m16.hip (MFMA 16x16x32 on raw codes, scale/bias applied per (column, group) to
// the fp32 accumulators); what differs is how bytes move:
//
//  * The weight matrix is cut into units of 128 rows x 256 k (16 KiB of codes plus the
//    8 KiB slice of x they multiply; scales/biases come per chunk of four units).  Units
//    are numbered row-block-major and divided EVENLY among a persistent grid of one
//    512-thread workgroup per CU: every CU streams the same number of bytes (+-1 unit)
//    whatever N and K are, fills its load pipeline once, and there is no tail of
//    half-empty rounds.
//  * Units go global -> LDS with 16-byte direct loads (no VGPR staging); each wave
//    instruction moves 128-byte row segments of 8 rows.  A 5-deep ring keeps four units
//    (96 KiB per CU) in flight while the fifth is consumed - HBM latency times bandwidth
//    is ~100 KiB per CU on this part.  Granules are XOR-swizzled inside a row so that the
//    MFMA-shaped reads spread evenly over the LDS banks.
//  * Work every wave would otherwise repeat is done once per unit, one unit ahead, by
//    waves 0-3: putting the x fragments into MFMA slot order (in place) and the per-group
//    row sums of x (an MFMA against ones, already in accumulator layout).
//  * Within a unit, wave w owns rows 16w..16w+15 (one MFMA tile) for all four
//    quantisation groups, so its accumulators never need a cross-wave reduction and a
//    finished row block goes from registers straight to memory.
//  * A workgroup whose range covers all of K for a row block writes y directly.
//    Row blocks shared between workgroups go through fp32 partial tiles in the
//    workspace; the last contributor to arrive (wrapping agent-scope counter)
//    adds them in contributor order and rounds once - deterministic, no spinning.
//    Partials are written through to / read from the level all XCDs share (sc1), so
//    that no L2 write-back fence is ever issued.
//
// The compiler orders every LDS access it can see behind ALL outstanding direct-to-LDS
// loads (s_waitcnt vmcnt(0)), and __syncthreads() carries a fence with the same effect;
// either would drain the ring on every unit.  The main loop therefore touches LDS only
// through hand-written instruction blocks and synchronises with a bare s_barrier plus
// an explicit vmcnt wait (loads retire in issue order and every wave issues the same
// number of them per unit: one for x, two for codes, plus one with each scale/bias chunk).
#include "dflash_common.h"

namespace dflash {
namespace stream {

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kRows = 128;   // rows per unit (16 per wave)
constexpr int kUnitK = 256;  // k per unit (four groups of 64)
constexpr int kGS = 64;
constexpr int kGroups = kUnitK / kGS;
constexpr int kDepth = 5;                      // ring slots of (codes + x)
constexpr int kWBytes = kRows * (kUnitK / 2);  // 16 KiB: 128 B per row
constexpr int kXBytes = 16 * kUnitK * 2;       // 8 KiB
constexpr int kXOffset = kWBytes;
constexpr int kSlotBytes = kWBytes + kXBytes;  // 24 KiB
// row sums of x per group in accumulator layout, for the unit in use and the next one
constexpr int kXsBytes = kGroups * 64 * 16;    // 4 KiB
constexpr int kXsOffset = kDepth * kSlotBytes;
// Scales and biases are staged per chunk of kChunk units (32 bytes per row and array):
// fetching them unit by unit would cost two 8-byte requests per row and unit, twice the
// number of memory requests the codes themselves need.
constexpr int kChunk = 4;
constexpr int kSbDepth = 3;
constexpr int kSbArrayBytes = kRows * kChunk * kGroups * 2;  // 4 KiB
constexpr int kSbSlotBytes = 2 * kSbArrayBytes;              // scales then biases
constexpr int kSbOffset = kXsOffset + 2 * kXsBytes;
constexpr int kLdsBytes = kSbOffset + kSbDepth * kSbSlotBytes;  // 152 KiB
constexpr int kPartialFloats = 16 * kRows;

template <bool FP16>
struct Act;
template <>
struct Act<false> {
  static constexpr uint32_t kMagic = 0x43004300u;  // bf16 128.0 twice: 0x4300|q == 128+q
  static constexpr float kOffset = 128.0f;
  static constexpr uint32_t kOnes = 0x3F803F80u;
  static __device__ __forceinline__ f32x4_t mfma(uint4 a, uint4 b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t from_f32(float v) { return f32_to_bf16_bits(v); }
  static __device__ __forceinline__ float to_f32(uint32_t h) { return bf16_bits_to_f32(h); }
};
template <>
struct Act<true> {
  static constexpr uint32_t kMagic = 0x64006400u;  // fp16 1024.0 twice: 0x6400|q == 1024+q
  static constexpr float kOffset = 1024.0f;
  static constexpr uint32_t kOnes = 0x3C003C00u;
  static __device__ __forceinline__ f32x4_t mfma(uint4 a, uint4 b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a),
                                                  __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t from_f32(float v) { return f32_to_f16_bits(v); }
  static __device__ __forceinline__ float to_f32(uint32_t h) { return f16_bits_to_f32(h); }
};

// 8 codes of one packed word -> MFMA operand, slot order k0,k4,k1,k5,k2,k6,k3,k7.
// `mask` (0x000F000F) and `magic` arrive in registers the compiler cannot see through, so
// that each pair of codes costs one v_and_or_b32 instead of an and plus an or with literals.
__device__ __forceinline__ uint4 unpack_codes(uint32_t w, uint32_t mask, uint32_t magic) {
  uint4 r;
  r.x = (w & mask) | magic;
  r.y = ((w >> 4) & mask) | magic;
  r.z = ((w >> 8) & mask) | magic;
  r.w = ((w >> 12) & mask) | magic;
  return r;
}

typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;

// 8 consecutive 16-bit activations (natural order) -> the same slot order.
__device__ __forceinline__ u32x4_t permute_x(u32x4_t v) {
  u32x4_t r;
  r.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);  // (x0, x4)
  r.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);  // (x1, x5)
  r.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);  // (x2, x6)
  r.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);  // (x3, x7)
  return r;
}

__device__ __forceinline__ uint4 as_uint4(u32x4_t v) { return make_uint4(v.x, v.y, v.z, v.w); }

typedef __attribute__((address_space(3))) void lds_void_t;
typedef __attribute__((address_space(1))) const void global_cvoid_t;

// Lane i of the wave lands at lds_base + 16*i (lds_base is wave-uniform).
__device__ __forceinline__ void load16_to_lds(const void* gptr, char* lds_base) {
  __builtin_amdgcn_global_load_lds((global_cvoid_t*)gptr, (lds_void_t*)lds_base, 16, 0, 0);
}

__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return (uint32_t)(uintptr_t)(const lds_void_t*)p;
}

// Preparation of one group of the next unit (waves 0-3): fragments j = 0, 1 of this lane
// are put into MFMA slot order in place, and the group's row sums of x land in `xs_addr`.
template <bool FP16>
__device__ __forceinline__ void prepare_group(uint32_t frag_addr, uint32_t xs_addr, uint4 ones) {
  u32x4_t f0, f1;
  asm volatile(
      "ds_read_b128 %0, %2\n"
      "ds_read_b128 %1, %2 offset:256\n"
      "s_waitcnt lgkmcnt(0)\n"
      : "=&v"(f0), "=&v"(f1)
      : "v"(frag_addr)
      : "memory");
  const u32x4_t a0 = permute_x(f0), a1 = permute_x(f1);
  f32x4_t xs = f32x4_t{0.f, 0.f, 0.f, 0.f};
  xs = Act<FP16>::mfma(as_uint4(a0), ones, xs);
  xs = Act<FP16>::mfma(as_uint4(a1), ones, xs);
  asm volatile(
      "ds_write_b128 %0, %2\n"
      "ds_write_b128 %0, %3 offset:256\n"
      "ds_write_b128 %1, %4\n"
      :
      : "v"(frag_addr), "v"(xs_addr), "v"(a0), "v"(a1), "v"(xs)
      : "memory");
}

// One unit's operands of a wave.  Completion of the unit is established by the caller.
//   af[2g+j] x fragment (slot order) feeding MFMA j of group g
//   xs[g]    row sums of x over group g, accumulator layout
//   wq[g]    packed codes of group g: .x feeds MFMA 0, .y MFMA 1
//   sc, bi   the four scales / biases of this lane's row, two 16-bit values per dword
__device__ __forceinline__ void read_unit_operands(uint32_t xaddr, uint32_t xsaddr,
                                                   const uint32_t (&waddr)[4], uint32_t saddr,
                                                   u32x4_t (&af)[8], f32x4_t (&xs)[4],
                                                   u32x2_t (&wq)[4], u32x2_t& sc, u32x2_t& bi) {
  asm volatile(
      "ds_read_b128 %0, %18\n"
      "ds_read_b128 %1, %18 offset:256\n"
      "ds_read_b128 %2, %18 offset:2048\n"
      "ds_read_b128 %3, %18 offset:2304\n"
      "ds_read_b128 %4, %18 offset:4096\n"
      "ds_read_b128 %5, %18 offset:4352\n"
      "ds_read_b128 %6, %18 offset:6144\n"
      "ds_read_b128 %7, %18 offset:6400\n"
      "ds_read_b64 %12, %20\n"
      "ds_read_b64 %13, %21\n"
      "ds_read_b64 %14, %22\n"
      "ds_read_b64 %15, %23\n"
      "ds_read_b64 %16, %24\n"
      "ds_read_b64 %17, %24 offset:4096\n"
      "ds_read_b128 %8, %19\n"
      "ds_read_b128 %9, %19 offset:1024\n"
      "ds_read_b128 %10, %19 offset:2048\n"
      "ds_read_b128 %11, %19 offset:3072\n"
      "s_waitcnt lgkmcnt(0)\n"
      : "=&v"(af[0]), "=&v"(af[1]), "=&v"(af[2]), "=&v"(af[3]), "=&v"(af[4]), "=&v"(af[5]),
        "=&v"(af[6]), "=&v"(af[7]), "=&v"(xs[0]), "=&v"(xs[1]), "=&v"(xs[2]), "=&v"(xs[3]),
        "=&v"(wq[0]), "=&v"(wq[1]), "=&v"(wq[2]), "=&v"(wq[3]), "=&v"(sc), "=&v"(bi)
      : "v"(xaddr), "v"(xsaddr), "v"(waddr[0]), "v"(waddr[1]), "v"(waddr[2]), "v"(waddr[3]),
        "v"(saddr)
      : "memory");
}

// Partial accumulator tiles cross XCDs: stored and loaded at agent scope (sc1).
__device__ __forceinline__ void store_partial(float* p, f32x4_t v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n" : : "v"(p), "v"(v) : "memory");
}
// four tiles at once, so that their latencies overlap
__device__ __forceinline__ void load_partials4(const float* p0, const float* p1, const float* p2,
                                               const float* p3, f32x4_t (&v)[4]) {
  asm volatile(
      "global_load_dwordx4 %0, %4, off sc1\n"
      "global_load_dwordx4 %1, %5, off sc1\n"
      "global_load_dwordx4 %2, %6, off sc1\n"
      "global_load_dwordx4 %3, %7, off sc1\n"
      "s_waitcnt vmcnt(0)\n"
      : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3])
      : "v"(p0), "v"(p1), "v"(p2), "v"(p3)
      : "memory");
}

struct Params {
  const uint16_t* x;
  const uint32_t* w;
  const uint16_t* scales;
  const uint16_t* biases;
  uint16_t* y;
  float* partials;     // [2 * grid][wave][lane][4] fp32
  uint32_t* counters;  // [row blocks]
  int K, N;
  int stages;          // K / 256
  int units;           // row blocks * stages
};

// Unit range of workgroup i out of n: [units*i/n, units*(i+1)/n)  (units*n < 2^31).
__device__ __forceinline__ int range_begin(int units, int i, int n) {
  return (int)(((unsigned)units * (unsigned)i) / (unsigned)n);
}

#define DFLASH_WAIT_CASE(n) \
  case n:                   \
    __builtin_amdgcn_s_waitcnt(0x0070 | ((n)&15) | (((n) >> 4) << 14)); \
    break;
// Wait until at most n of this wave's loads are outstanding and all its LDS traffic is done.
__device__ __forceinline__ void wait_loads(int n) {
  switch (n) {
    DFLASH_WAIT_CASE(0) DFLASH_WAIT_CASE(1) DFLASH_WAIT_CASE(2) DFLASH_WAIT_CASE(3)
    DFLASH_WAIT_CASE(4) DFLASH_WAIT_CASE(5) DFLASH_WAIT_CASE(6) DFLASH_WAIT_CASE(7)
    DFLASH_WAIT_CASE(8) DFLASH_WAIT_CASE(9) DFLASH_WAIT_CASE(10) DFLASH_WAIT_CASE(11)
    DFLASH_WAIT_CASE(12) DFLASH_WAIT_CASE(13) DFLASH_WAIT_CASE(14) DFLASH_WAIT_CASE(15)
    DFLASH_WAIT_CASE(16)
    default: __builtin_amdgcn_s_waitcnt(0x0070); break;
  }
}
#undef DFLASH_WAIT_CASE

template <bool ACT_FP16, bool SB_FP16>
__global__ __launch_bounds__(kThreads, 1) void qmm_stream_kernel(Params p) {
  using A = Act<ACT_FP16>;
  using SB = Act<SB_FP16>;
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  __shared__ int s_last;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int col = lane & 15;
  const int kblk = lane >> 4;
  const int G = p.K / kGS;
  const size_t row_bytes = (size_t)p.K >> 1;
  const int grid = gridDim.x;

  const int u0 = range_begin(p.units, blockIdx.x, grid);
  const int u1 = range_begin(p.units, blockIdx.x + 1, grid);
  if (u0 >= u1) return;

  // ---- producer state ---------------------------------------------------------------
  //  codes: 16 instructions cover 128 rows x 128 B; instruction q = wave + 8*i holds rows
  //         8q..8q+7; lane = 8*row_in_8 + slot, and slot holds granule slot ^ sw(row) with
  //         sw(row) = ((row >> 1) & 3) << 1  (swaps 32-byte pairs, i.e. whole groups)
  //  x:     wave w moves group w>>1, k-blocks 2*(w&1) and 2*(w&1)+1: lane = 16*(2*kbl + j) + m
  //         fetches x[m][64g + 16*(2*(w&1) + kbl) + 8j .. +7], 64 contiguous bytes per row
  //  scales/biases of a chunk: waves 0-3 scales, 4-7 biases, 32 rows per wave, two
  //         16-byte granules per row
  const int w_r = lane >> 3;
  const int w_c = (lane & 7) ^ (((w_r >> 1) & 3) << 1);
  const char* const xp0 = (const char*)(p.x + (size_t)(lane & 15) * p.K + (wave >> 1) * kGS +
                                        (2 * (wave & 1) + (lane >> 5)) * 16 + ((lane >> 4) & 1) * 8);
  const char* wp[2];   // codes of this lane's rows at stage 0 of the row block being issued
  const char* sbp;     // scales or biases of this lane's row, chunk 0
  auto set_row_block = [&](int rb) {
    const int row0 = rb * kRows;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      int row = row0 + 8 * (wave + kWaves * i) + w_r;
      row = row < p.N ? row : p.N - 1;
      wp[i] = (const char*)p.w + (size_t)row * row_bytes + w_c * 16;
    }
    int row = row0 + 32 * (wave & 3) + (lane >> 1);
    row = row < p.N ? row : p.N - 1;
    sbp = (const char*)(((wave & 4) ? p.biases : p.scales) + (size_t)row * G) + (lane & 1) * 16;
  };

  int rb_i = u0 / p.stages, st_i = u0 - rb_i * p.stages;  // next unit to issue
  int issued = u0;
  int slot_i = 0;     // ring slot of the next unit to issue
  int sb_slot_i = 0;  // scale/bias slot of the next chunk to issue
  set_row_block(rb_i);
  // Issues one unit (x first, so that x of unit u+1 can be awaited without its codes);
  // returns the number of loads this wave issued for it.
  auto issue_next = [&]() -> int {
    char* slot = lds + slot_i * kSlotBytes;
    int n = 3;
    load16_to_lds(xp0 + (size_t)st_i * (kUnitK * 2), slot + kXOffset + wave * 1024);
    if ((st_i % kChunk) == 0 || issued == u0) {
      load16_to_lds(sbp + (size_t)(st_i / kChunk) * (kChunk * kGroups * 2),
                    lds + kSbOffset + sb_slot_i * kSbSlotBytes + ((wave & 4) ? kSbArrayBytes : 0) +
                        (wave & 3) * 1024);
      if (++sb_slot_i == kSbDepth) sb_slot_i = 0;
      n = 4;
    }
    load16_to_lds(wp[0] + (size_t)st_i * (kUnitK / 2), slot + wave * 1024);
    load16_to_lds(wp[1] + (size_t)st_i * (kUnitK / 2), slot + (wave + kWaves) * 1024);
    ++issued;
    if (++slot_i == kDepth) slot_i = 0;
    if (++st_i == p.stages) {
      st_i = 0;
      ++rb_i;
      if (issued < u1) set_row_block(rb_i);
    }
    return n;
  };

  // ---- consumer state ---------------------------------------------------------------
  const uint4 ones = make_uint4(A::kOnes, A::kOnes, A::kOnes, A::kOnes);
  uint32_t mask = 0x000F000Fu, magic = A::kMagic;
  asm volatile("" : "+s"(mask), "+v"(magic));
  const uint32_t lds0 = lds_address(lds);
  //   x fragment (g, j) of lane (m = col, kb = kblk) inside a slot: + g*2048 + j*256
  const uint32_t xoff = kXOffset + (kblk >> 1) * 1024 + (16 * (2 * (kblk & 1)) + col) * 16;
  const uint32_t wrow = 16 * wave + col;
  uint32_t woff[4];
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    // group g of this row sits in the 32-byte pair g ^ ((row >> 1) & 3)
    woff[g] = wrow * 128 + ((g ^ ((wrow >> 1) & 3)) << 5) + (kblk >> 1) * 16 + (kblk & 1) * 8;
  }
  int rb = u0 / p.stages, st = u0 - rb * p.stages;  // unit being consumed
  const int rb_first = rb;
  int first_in_rb = u0;
  int slot_c = 0;      // ring slot of the unit being consumed
  int sb_slot_c = -1;  // scale/bias slot of the chunk being consumed
  int xs_c = 0;        // which row-sum buffer belongs to the unit being consumed
  f32x4_t acc = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // waves 0-3: prepare group `wave` of the unit in ring slot s, row sums into buffer b
  auto prepare = [&](int s, int b) {
    if (wave < 4) {
      prepare_group<ACT_FP16>(lds0 + s * kSlotBytes + xoff + wave * 2048,
                              lds0 + kXsOffset + b * kXsBytes + wave * 1024 + lane * 16, ones);
    }
  };

  // ---- prologue: fill the ring, prepare the first unit ------------------------------
  // y1..y3: loads this wave issued for the three units after the one being consumed
  int y1 = 0, y2 = 0, y3 = 0;
  const int n0 = issue_next();
  if (issued < u1) y1 = issue_next();
  if (issued < u1) y2 = issue_next();
  if (issued < u1) y3 = issue_next();
  wait_loads(n0 - 1 + y1 + y2 + y3);  // x of the first unit is the oldest load
  asm volatile("s_barrier" ::: "memory");
  prepare(0, 0);

#pragma unroll 1
  for (int u = u0; u < u1; ++u) {
    // unit u and the x slice of unit u+1 (the oldest load of that unit) must have landed
    wait_loads(y1 + y2 + y3 - (y1 ? 1 : 0));
    asm volatile("s_barrier" ::: "memory");  // ... for every wave; unit u-1 is consumed
    y1 = y2, y2 = y3, y3 = 0;
    if (issued < u1) y3 = issue_next();  // unit u+4 refills the slot of unit u-1
    if (u + 1 < u1) prepare(slot_c + 1 == kDepth ? 0 : slot_c + 1, xs_c ^ 1);
    if ((st % kChunk) == 0 || u == u0) {
      if (++sb_slot_c == kSbDepth) sb_slot_c = 0;
    }

    const uint32_t sbase = lds0 + slot_c * kSlotBytes;
    if (++slot_c == kDepth) slot_c = 0;
    // four scales of this lane's row for this unit; biases one array further
    const uint32_t saddr = lds0 + kSbOffset + sb_slot_c * kSbSlotBytes + wrow * 32 + (st % kChunk) * 8;
    const uint32_t xsaddr = lds0 + kXsOffset + xs_c * kXsBytes + lane * 16;
    xs_c ^= 1;
    u32x4_t af[8];
    f32x4_t xs[4];
    u32x2_t wq[4], sc, bi;
    const uint32_t waddr[4] = {sbase + woff[0], sbase + woff[1], sbase + woff[2], sbase + woff[3]};
    read_unit_operands(sbase + xoff, xsaddr, waddr, saddr, af, xs, wq, sc, bi);

#pragma unroll
    for (int g = 0; g < 4; ++g) {
      f32x4_t c = f32x4_t{0.f, 0.f, 0.f, 0.f};
      c = A::mfma(as_uint4(af[2 * g]), unpack_codes(wq[g].x, mask, magic), c);
      c = A::mfma(as_uint4(af[2 * g + 1]), unpack_codes(wq[g].y, mask, magic), c);
      const uint32_t sd = (g & 2) ? sc.y : sc.x;
      const uint32_t bd = (g & 2) ? bi.y : bi.x;
      const float s = SB::to_f32((g & 1) ? (sd >> 16) : (sd & 0xFFFFu));
      const float b = SB::to_f32((g & 1) ? (bd >> 16) : (bd & 0xFFFFu));
      const float bb = __builtin_fmaf(-A::kOffset, s, b);
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[r] = __builtin_fmaf(bb, xs[g][r], __builtin_fmaf(s, c[r], acc[r]));
    }

    // ---- advance; emit when this row block ends inside my range -------------------
    const int cur_rb = rb;
    const bool rb_ends = (u + 1 == u1) || (st + 1 == p.stages);
    if (++st == p.stages) {
      st = 0;
      ++rb;
    }
    if (!rb_ends) continue;

    const int lo = cur_rb * p.stages;
    const bool complete = (first_in_rb == lo) && (u + 1 == lo + p.stages);
    const int row0 = cur_rb * kRows;
    first_in_rb = u + 1;
    // accumulator r of lane l is output (m = 4*(l/16) + r, n = row0 + 16*wave + l%16)
    const int n_out = row0 + 16 * wave + col;
    if (!complete) {
      // a workgroup shares at most two row blocks with others: the one its range starts in
      // (slot 0) and the one it ends in (slot 1); tiles are kept in accumulator layout
      float* part = p.partials + ((size_t)blockIdx.x * 2 + (cur_rb == rb_first ? 0 : 1)) * kPartialFloats;
      store_partial(part + tid * 4, acc);
      // The barrier's own wait (vmcnt(0)) retires every thread's store before thread 0
      // bumps the counter; a release fence here would write back the whole L2.
      __syncthreads();
      // contributors: the workgroups whose ranges intersect [lo, lo+stages);
      // owner(v) = ceil((v+1)*grid/units) - 1 is the workgroup whose range holds unit v
      const int wg_first = (int)((((unsigned)lo + 1u) * (unsigned)grid + p.units - 1) / (unsigned)p.units) - 1;
      const int wg_last =
          (int)((((unsigned)(lo + p.stages)) * (unsigned)grid + p.units - 1) / (unsigned)p.units) - 1;
      if (tid == 0) {
        const uint32_t n_contrib = (uint32_t)(wg_last - wg_first + 1);
        // wrapping increment: the last arrival sees n-1 and leaves 0 behind for the next call
        const uint32_t prev = atomicInc(&p.counters[cur_rb], n_contrib - 1);
        s_last = (prev == n_contrib - 1);
      }
      __syncthreads();
      acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
      if (!s_last) continue;
      // only the first contributor can have started before this row block (then the block
      // is the one its range ends in); every later one starts inside it
      const int which_first = range_begin(p.units, wg_first, grid) < lo ? 1 : 0;
      for (int wg = wg_first; wg <= wg_last; wg += 4) {
        const float* src[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int w = wg + j <= wg_last ? wg + j : wg_last;  // surplus slots re-read the last tile
          src[j] = p.partials + ((size_t)w * 2 + (w == wg_first ? which_first : 0)) * kPartialFloats + tid * 4;
        }
        f32x4_t v[4];
        load_partials4(src[0], src[1], src[2], src[3], v);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (wg + j <= wg_last) {
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[r] += v[j][r];
          }
        }
      }
    }
    if (n_out < p.N) {
#pragma unroll
      for (int r = 0; r < 4; ++r) p.y[(size_t)(4 * kblk + r) * p.N + n_out] = (uint16_t)A::from_f32(acc[r]);
    }
    acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
}

}  // namespace stream
}  // namespace dflash

// ---------------------------------------------------------------------------------
// Host side of the streaming kernel (called from dflash_qmm_m16 for eligible shapes).
// ---------------------------------------------------------------------------------
namespace dflash {

int qmm_stream_grid() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 256;
    cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    if (cus > 1024) cus = 1024;
  }
  return cus;
}

bool qmm_stream_eligible(int K, int N, int group_size) {
  // whole scale/bias chunks: K must be a multiple of kChunk units
  if (group_size != 64 || K <= 0 || K % (stream::kUnitK * stream::kChunk) != 0 || N <= 0 || N % 16 != 0) return false;
  const long long row_blocks = (N + stream::kRows - 1) / stream::kRows;
  const long long units = row_blocks * (K / stream::kUnitK);
  return units * 1024 < (1ll << 31) && row_blocks <= (64 * 1024) / 4;
}

size_t qmm_stream_workspace_bytes(int N, int grid) {
  (void)N;
  return (size_t)64 * 1024 + (size_t)grid * 2 * stream::kPartialFloats * sizeof(float);
}

int qmm_stream_launch(const void* x, const uint32_t* w, const void* scales, const void* biases,
                      void* y, void* workspace, size_t workspace_bytes, int K, int N,
                      int act_dtype, int sb_dtype, hipStream_t stream) {
  using namespace stream;
  Params p;
  p.x = (const uint16_t*)x;
  p.w = w;
  p.scales = (const uint16_t*)scales;
  p.biases = (const uint16_t*)biases;
  p.y = (uint16_t*)y;
  p.K = K;
  p.N = N;
  p.stages = K / kUnitK;
  p.units = ((N + kRows - 1) / kRows) * p.stages;
  int grid = qmm_stream_grid();
  if (grid > p.units) grid = p.units;
  const size_t need = qmm_stream_workspace_bytes(N, grid);
  DFLASH_REQUIRE(workspace && workspace_bytes >= need, DFLASH_ERR_WORKSPACE,
                 "dflash_qmm_m16: workspace of %zu bytes needed, %zu given", need,
                 workspace ? workspace_bytes : (size_t)0);
  p.counters = (uint32_t*)workspace;
  p.partials = (float*)((char*)workspace + 64 * 1024);

  static bool attr_set[4] = {false, false, false, false};
  const bool a16 = act_dtype == DFLASH_FP16, s16 = sb_dtype == DFLASH_FP16;
  const int idx = (a16 ? 2 : 0) + (s16 ? 1 : 0);
  const void* fn = nullptr;
  if (!a16 && !s16) fn = (const void*)qmm_stream_kernel<false, false>;
  if (!a16 && s16) fn = (const void*)qmm_stream_kernel<false, true>;
  if (a16 && !s16) fn = (const void*)qmm_stream_kernel<true, false>;
  if (a16 && s16) fn = (const void*)qmm_stream_kernel<true, true>;
  if (!attr_set[idx]) {
    DFLASH_HIP_OK(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes));
    attr_set[idx] = true;
  }
  void* args[] = {&p};
  DFLASH_HIP_OK(hipLaunchKernel(fn, dim3(grid), dim3(kThreads), args, kLdsBytes, stream));
  return DFLASH_OK;
}

}  // namespace dflash
