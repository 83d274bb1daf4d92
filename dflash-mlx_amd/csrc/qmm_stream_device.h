// Device-side building blocks shared by the streaming qmm kernels (qmm_m16_stream.hip: one
// matrix per launch; qmm_m16_chain.hip: several matrices per launch): the unit and ring
// geometry in LDS, direct-to-LDS loads, the hand-written LDS reads of a unit's operands, the
// arithmetic of one unit, the cross-wave sum at the end of a row block and the agent-scope
// partial tiles of split K.
#pragma once

#include "dflash_common.h"

namespace dflash {
namespace stream {

constexpr int kWaves = 8;  // arithmetic waves
constexpr int kLoaders = 4;  // extra waves that only issue loads
constexpr int kThreads = (kWaves + kLoaders) * 64;
constexpr int kRows = 128;   // rows per unit (16 per wave)
constexpr int kUnitK = 256;  // k per unit (four groups of 64)
constexpr int kGS = 64;
constexpr int kGroups = kUnitK / kGS;
// packed weight images: codes of one unit, scales (or biases) of one chunk of four units
constexpr int kPackedUnitBytes = kRows * kUnitK / 2;      // 16 KiB
constexpr int kPackedChunkBytes = kRows * 4 * kGroups * 2;  // 4 KiB
constexpr int kDepth = 5;                      // ring slots of (codes + x)
// Units a loader keeps issued beyond the one being consumed.  A CU holds about 64 KiB of
// loads in flight (what HBM latency times its share of the bandwidth comes to); a loader
// that tries to issue more only sits in its issue stage and is late for the next barrier.
// Short ranges (fewer than four units per workgroup) keep two: most of such a launch is its
// start, where every request that is not for the first unit delays the first unit.
constexpr int kAhead = 3;
constexpr int kAheadShort = 2;
constexpr int kWBytes = kRows * (kUnitK / 2);  // 16 KiB: 128 B per row
constexpr int kXBytes = 16 * kUnitK * 2;       // 8 KiB
constexpr int kXOffset = kWBytes;
constexpr int kSlotBytes = kWBytes + kXBytes;  // 24 KiB
// Scales and biases are staged per chunk of CHUNK units (CHUNK = 4: 32 bytes per row and
// array; CHUNK = 2, for K that is a multiple of 512 only: 16 bytes): fetching them unit by
// unit would cost two 8-byte requests per row and unit, twice the number of memory requests
// the codes themselves need.
constexpr int kSbDepth = 3;
constexpr int kSbArrayBytes = kRows * 4 * kGroups * 2;  // 4 KiB, sized for CHUNK = 4
constexpr int kSbSlotBytes = 2 * kSbArrayBytes;         // scales then biases
constexpr int kSbOffset = kDepth * kSlotBytes;
constexpr int kLdsBytes = kSbOffset + kSbDepth * kSbSlotBytes;  // 144 KiB
constexpr int kPartialFloats = 16 * kRows;
// Gathered (per-expert) form: tables built in LDS by every workgroup at kernel start.
//   an "entry" is up to 16 rows of x that go through the same expert's weights
constexpr int kMaxEntries = 256;  // hence at most 256 rows of x
constexpr int kMaxExperts = 1024;
constexpr int kTabOffset = kLdsBytes;
constexpr int kTabCount = 0;                        // u32 [kMaxExperts]: rows << 16 | first entry
constexpr int kTabEntry = kTabCount + 4 * kMaxExperts;   // u32 [kMaxEntries]: rows << 16 | expert
constexpr int kTabRows = kTabEntry + 4 * kMaxEntries;    // u16 [kMaxEntries][16]: row of x, y
constexpr int kTabTotal = kTabRows + 2 * 16 * kMaxEntries;  // u32: number of entries
constexpr int kLdsBytesGather = kTabOffset + kTabTotal + 64;  // 157.1 KiB

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
// The same with the non-temporal cache policy (aux bit 1 = nt on gfx94x/gfx950): the codes
// are read exactly once, so they should not push x and the scale/bias lines, which are
// re-read, out of the L2.
__device__ __forceinline__ void load16_to_lds_stream(const void* gptr, char* lds_base) {
  __builtin_amdgcn_global_load_lds((global_cvoid_t*)gptr, (lds_void_t*)lds_base, 16, 0, 2);
}

__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return (uint32_t)(uintptr_t)(const lds_void_t*)p;
}

// One unit's operands of a worker wave (group g, rows 64h + 16j + col for tiles j = 0..3):
//   f0, f1  x fragments (natural order) feeding MFMA 0 / 1
//   wq[j]   packed codes of tile j: .x feeds MFMA 0, .y MFMA 1
//   sv, bv  scale / bias of this lane's row in tile j, 16 bits zero-extended
struct Operands {
  u32x4_t f0, f1;
  u32x2_t wq[4];
  uint32_t sv[4], bv[4];
};
// The LDS reads of a unit's operands are started in four pieces and return at once: the
// registers of `o` are written behind the compiler's back until operands_wait(o) has been
// executed, so nothing may touch `o` in between.  Piece j carries what tile j needs (piece 0
// also the x fragments).  An accumulator is threaded through every piece and through the
// wait, which pins piece j behind the arithmetic of tile j-1 of the previous unit's
// operands: issued in one go, the reads of eight waves queue up in the LDS pipeline and
// every wave sits in its issue stage instead of doing arithmetic.
// SBROW: bytes of scales per row and chunk in LDS (8 * CHUNK); tile j is 16 rows further.
template <int J, int SBROW>
__device__ __forceinline__ void operands_issue_piece(uint32_t xaddr, uint32_t waddr, uint32_t saddr,
                                                     Operands& o, f32x4_t& pin) {
  if (J == 0) {
    asm volatile(
        "ds_read_b128 %0, %6\n"
        "ds_read_b128 %1, %6 offset:256\n"
        "ds_read_b64 %2, %7\n"
        "ds_read_u16 %3, %8\n"
        "ds_read_u16 %4, %8 offset:4096\n"
        : "=&v"(o.f0), "=&v"(o.f1), "=&v"(o.wq[0]), "=&v"(o.sv[0]), "=&v"(o.bv[0]), "+v"(pin)
        : "v"(xaddr), "v"(waddr), "v"(saddr)
        : "memory");
  } else {
    asm volatile(
        "ds_read_b64 %0, %4 offset:%6\n"
        "ds_read_u16 %1, %5 offset:%7\n"
        "ds_read_u16 %2, %5 offset:%8\n"
        : "=&v"(o.wq[J]), "=&v"(o.sv[J]), "=&v"(o.bv[J]), "+v"(pin)
        : "v"(waddr), "v"(saddr), "n"(2048 * J), "n"(16 * SBROW * J), "n"(4096 + 16 * SBROW * J)
        : "memory");
  }
}
__device__ __forceinline__ void operands_wait(Operands& o, f32x4_t& acc0, f32x4_t& acc1,
                                              f32x4_t& acc2, f32x4_t& acc3) {
  asm volatile("s_waitcnt lgkmcnt(0)\n"
               : "+v"(o.f0), "+v"(o.f1), "+v"(o.wq[0]), "+v"(o.wq[1]), "+v"(o.wq[2]), "+v"(o.wq[3]),
                 "+v"(o.sv[0]), "+v"(o.sv[1]), "+v"(o.sv[2]), "+v"(o.sv[3]),
                 "+v"(o.bv[0]), "+v"(o.bv[1]), "+v"(o.bv[2]), "+v"(o.bv[3]),
                 "+v"(acc0), "+v"(acc1), "+v"(acc2), "+v"(acc3)
               :
               : "memory");
}

// The arithmetic of one unit: acc[j] += (scale, bias)-corrected x . codes^T of tile j, from
// the operands in `cur`.  With `fetch` set, the reads of the next unit's operands into `nxt`
// are started along the way (nothing else may touch `nxt` before operands_wait).
template <bool ACT_FP16, bool SB_FP16, int SBROW>
__device__ __forceinline__ void consume_unit(const Operands& cur, Operands& nxt, bool fetch,
                                             uint32_t xaddr, uint32_t waddr, uint32_t saddr,
                                             f32x4_t (&acc)[4], uint4 ones, uint32_t mask,
                                             uint32_t magic) {
  using A = Act<ACT_FP16>;
  using SB = Act<SB_FP16>;
  if (fetch) operands_issue_piece<0, SBROW>(xaddr, waddr, saddr, nxt, acc[3]);
  const uint4 a0 = as_uint4(permute_x(cur.f0)), a1 = as_uint4(permute_x(cur.f1));
  f32x4_t xs = f32x4_t{0.f, 0.f, 0.f, 0.f};  // row sums of x over this group
  xs = A::mfma(a0, ones, xs);
  xs = A::mfma(a1, ones, xs);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    f32x4_t c = f32x4_t{0.f, 0.f, 0.f, 0.f};
    c = A::mfma(a0, unpack_codes(cur.wq[j].x, mask, magic), c);
    c = A::mfma(a1, unpack_codes(cur.wq[j].y, mask, magic), c);
    const float s = SB::to_f32(cur.sv[j]);
    const float b = SB::to_f32(cur.bv[j]);
    const float bb = __builtin_fmaf(-A::kOffset, s, b);
#pragma unroll
    for (int r = 0; r < 4; ++r) acc[j][r] = __builtin_fmaf(bb, xs[r], __builtin_fmaf(s, c[r], acc[j][r]));
    if (fetch) {
      if (j == 0) operands_issue_piece<1, SBROW>(xaddr, waddr, saddr, nxt, acc[0]);
      if (j == 1) operands_issue_piece<2, SBROW>(xaddr, waddr, saddr, nxt, acc[1]);
      if (j == 2) operands_issue_piece<3, SBROW>(xaddr, waddr, saddr, nxt, acc[2]);
    }
  }
}

// Cross-wave sum at the end of a row block: every worker hands the three tiles it does
// not own to their owners through `base` (24 KiB: 8 owners x 3 tiles x 1 KiB), and after
// a barrier returns the sum of its own tile and the three it receives, in a fixed order.
__device__ __forceinline__ void reduce_groups_write(uint32_t base, const f32x4_t (&acc)[4], int wave,
                                                    int lane) {
  const int g = wave & 3, h = wave >> 2;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (j != g) {
      const int pos = (g - j - 1) & 3;  // 0..2
      const uint32_t addr = base + ((4 * h + j) * 3 + pos) * 1024 + lane * 16;
      asm volatile("ds_write_b128 %0, %1\n" : : "v"(addr), "v"(acc[j]) : "memory");
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
}
__device__ __forceinline__ f32x4_t reduce_groups_read(uint32_t base, const f32x4_t (&acc)[4], int wave,
                                                      int lane) {
  const int g = wave & 3;
  f32x4_t own = g == 0 ? acc[0] : g == 1 ? acc[1] : g == 2 ? acc[2] : acc[3];
  f32x4_t v0, v1, v2;
  const uint32_t addr = base + wave * 3 * 1024 + lane * 16;
  asm volatile(
      "ds_read_b128 %0, %3\n"
      "ds_read_b128 %1, %3 offset:1024\n"
      "ds_read_b128 %2, %3 offset:2048\n"
      "s_waitcnt lgkmcnt(0)\n"
      : "=&v"(v0), "=&v"(v1), "=&v"(v2)
      : "v"(addr)
      : "memory");
#pragma unroll
  for (int r = 0; r < 4; ++r) own[r] = ((own[r] + v0[r]) + v1[r]) + v2[r];
  return own;
}

// Word of the workspace's first 64 KiB that a workgroup sets when a bounded wait gives up
// (DFLASH_QMM_ERROR_OFFSET / 4 of the C interface).
constexpr int kErrorWord = 16384 - 64 + 1;
// Polls of a row block's partial tiles (about a microsecond each) before the adding workgroup
// gives up: seconds, so that other work that keeps a contributor off the device for a while
// (another stream's long kernel on a shared GPU) does not turn into an error.
constexpr int kSpinLimit = 1 << 22;

// A partial tile on its way through memory doubles as its own "ready" flag: +0.0 travels as
// -0.0 (the sum starts from +0.0, and +0.0 + -0.0 = +0.0, x + -0.0 = x: nothing changes), so
// no word of a stored tile is all zero bits, which is what an empty slot holds.
__device__ __forceinline__ f32x4_t nonzero_words(f32x4_t v) {
#pragma unroll
  for (int r = 0; r < 4; ++r) v[r] = v[r] == 0.0f ? -0.0f : v[r];
  return v;
}

// Partial accumulator tiles cross XCDs: stored and loaded at agent scope (sc1).
__device__ __forceinline__ void store_partial(float* p, f32x4_t v) {
  // A store of more than 64 bits reads the upper half of its data a cycle after it has been
  // issued, and the compiler, which inserts the wait states such hazards need, cannot see
  // inside this block: the next instruction it places may write those registers.
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n s_nop 1\n" : : "v"(p), "v"(v) : "memory");
}
// eight tiles at once, so that their latencies overlap
__device__ __forceinline__ void load_partials8(const float* const (&p)[8], f32x4_t (&v)[8]) {
  asm volatile(
      "global_load_dwordx4 %0, %8, off sc1\n"
      "global_load_dwordx4 %1, %9, off sc1\n"
      "global_load_dwordx4 %2, %10, off sc1\n"
      "global_load_dwordx4 %3, %11, off sc1\n"
      "global_load_dwordx4 %4, %12, off sc1\n"
      "global_load_dwordx4 %5, %13, off sc1\n"
      "global_load_dwordx4 %6, %14, off sc1\n"
      "global_load_dwordx4 %7, %15, off sc1\n"
      "s_waitcnt vmcnt(0)\n"
      : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]),
        "=&v"(v[7])
      : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]), "v"(p[7])
      : "memory");
}

// Unit range of workgroup i out of n: [units*i/n, units*(i+1)/n)  (units*n < 2^31).
__device__ __forceinline__ int range_begin(int units, int i, int n) {
  return (int)(((unsigned)units * (unsigned)i) / (unsigned)n);
}

#define DFLASH_WAIT_CASE(n) \
  case n:                   \
    __builtin_amdgcn_s_waitcnt(0x0F70 | ((n)&15) | (((n) >> 4) << 14)); \
    break;
// Wait until at most n of this wave's loads are outstanding (loads retire in issue order).
__device__ __forceinline__ void wait_loads(int n) {
  switch (n) {
    DFLASH_WAIT_CASE(0) DFLASH_WAIT_CASE(1) DFLASH_WAIT_CASE(2) DFLASH_WAIT_CASE(3)
    DFLASH_WAIT_CASE(4) DFLASH_WAIT_CASE(5) DFLASH_WAIT_CASE(6) DFLASH_WAIT_CASE(7)
    DFLASH_WAIT_CASE(8) DFLASH_WAIT_CASE(9) DFLASH_WAIT_CASE(10) DFLASH_WAIT_CASE(11)
    DFLASH_WAIT_CASE(12) DFLASH_WAIT_CASE(13) DFLASH_WAIT_CASE(14) DFLASH_WAIT_CASE(15)
    DFLASH_WAIT_CASE(16) DFLASH_WAIT_CASE(17) DFLASH_WAIT_CASE(18) DFLASH_WAIT_CASE(19)
    DFLASH_WAIT_CASE(20) DFLASH_WAIT_CASE(21) DFLASH_WAIT_CASE(22) DFLASH_WAIT_CASE(23)
    DFLASH_WAIT_CASE(24) DFLASH_WAIT_CASE(25) DFLASH_WAIT_CASE(26) DFLASH_WAIT_CASE(27)
    DFLASH_WAIT_CASE(28) DFLASH_WAIT_CASE(29) DFLASH_WAIT_CASE(30) DFLASH_WAIT_CASE(31)
    DFLASH_WAIT_CASE(32)
    default: __builtin_amdgcn_s_waitcnt(0x0F70); break;
  }
}
#undef DFLASH_WAIT_CASE

// Reads of the row tables by waves that have direct-to-LDS loads in flight: written out by
// hand for the same reason as the operand reads (the compiler would wait for all loads).
__device__ __forceinline__ uint32_t lds_read_u32(uint32_t addr) {
  uint32_t v;
  asm volatile("ds_read_b32 %0, %1\n s_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
  return v;
}
__device__ __forceinline__ uint32_t lds_read_u16(uint32_t addr) {
  uint32_t v;
  asm volatile("ds_read_u16 %0, %1\n s_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
  return v;
}
__device__ __forceinline__ u32x2_t lds_read_u64(uint32_t addr) {
  u32x2_t v;
  asm volatile("ds_read_b64 %0, %1\n s_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
  return v;
}

}  // namespace stream
}  // namespace dflash
