// (Shared by the per-format translation units vecq_flat_*.hip, which instantiate the kernels, and vecq_flat.hip, which
// holds the plans' host checks: each format compiles in its own unit so that the library builds in parallel.)
//
// llmp.vecq in the form the default launches take: one lane owns one whole unit of
// a weight row (a 144-byte Q4_K super-block, or four Q8_0 blocks: 136 bytes); every
// wave streams its own tiles through LDS with global-to-LDS loads and never waits
// for another wave.
//
// A tile is R consecutive rows of the weights (of both matrices with a GLU), at
// most 64 units: lane t of a wave owns unit t of the tile's flat list (the up
// rows' units, then the gate rows'). With packed rows a matrix's part of the list
// is one contiguous byte range; the wave fetches the list as 16-byte chunks with
// global_load_lds_dwordx4, chunk 64 j + lane by its j-th load, which lands at
// 16 * (64 j + lane) of the wave's LDS buffer: every cache line is requested once,
// by neighbouring lanes, and no register holds weights in flight. After s_waitcnt
// vmcnt(0) each lane reads its own unit (Q4_K: nine 16-byte reads 144 bytes apart,
// 36 dwords, so sixteen lanes' reads fall in distinct banks; Q8_0: seventeen 8-byte
// reads 136 bytes apart, 34 dwords, likewise for thirty-two lanes). A workgroup
// (8 wave64s, two a CU) stages its tokens' activations once (quantizing them to
// Q8_1 itself in the fused form) while the waves' first tiles are in flight; after
// that one barrier its waves are independent: wave w of the grid takes tiles w,
// w + waves, .... Sixteen waves a CU alternate between waiting for a tile and
// computing one, so a CU always has tiles in flight.
//
// Staged activations, Q4_K: per token and super-block a record of 336 bytes (84
// dwords, so that consecutive super-blocks start 20 banks apart and sixteen lanes'
// 16-byte reads of the same field never share a bank):
//   [0, 256)    the 256 int8 codes;
//   [256, 288)  the eight sub-blocks' scales d8 as floats;
//   [288, 320)  d8 * sum(codes) of each sub-block as floats (the minimum term);
//   [320, 336)  sum(codes) of each sub-block as int16 (read by the test dump).
// A lane's super-block sum is d * sum_g sc_g * d8_g * prod_g - dmin * sum_g m_g *
// d8_g * sum_g (tests/unit/dsv4_fast_test.cc:179-193), prod_g eight v_dot4_i32_i8.
//
// Staged activations, Q8_0: per token and unit a record of 152 bytes: an image of the
// unit's 136 bytes with the activation codes where the weight codes are and zeros
// where the four F16 scales are, then the four blocks' scales d8 as floats. A block's
// 32 weight codes start two bytes into a dword in every other block; against the image
// the 34 dwords of a unit multiply as they lie, v_dot4_i32_i8 by v_dot4_i32_i8 (the
// scale bytes meet zeros), and dwords 0-8, 9-16, 17-25 and 26-33 are the four blocks'
// sums (src/kernels/ggml/vecq.cu:398-418: sum w q times d times d8).
//
// Row sums: a suffix sum over the row's lanes by wave shuffles (a fixed tree), so
// a (token, row) value never depends on its neighbours or on which wave
// computed it.

#ifndef LLMP_AMD_CSRC_VECQ_FLAT_H_
#define LLMP_AMD_CSRC_VECQ_FLAT_H_

#include <hip/hip_runtime.h>

#include <type_traits>

#include "common.h"
#include "llmp_hip.h"
#include "vecq_common.h"

namespace llmp_hip {
namespace {

constexpr int kGroup = 512;      // threads a workgroup: eight waves, two workgroups a CU
constexpr int kWaves = kGroup / kWave;

// ---- the activations' first loads

// Staging is split in two so that a row's first loads can be queued before the wave's first
// tile: memory operations complete in order, and a load queued behind a tile would wait for it.
// A sweep of the workgroup covers blockDim.x / 8 blocks, eight lanes a block.
constexpr int kFront = 2;  // sweeps loaded ahead: rows up to 4096 values with eight waves

struct FrontX {
  float v[kFront][4];
};

template <int XT>
__device__ __forceinline__ FrontX LoadFrontX(const void* __restrict__ x, int k) {
  FrontX f;
  const int lane8 = threadIdx.x & 7;
  const bool wide = reinterpret_cast<uintptr_t>(x) % (XT == LLMP_X_F32 ? 16 : 8) == 0;
#pragma unroll
  for (int i = 0; i < kFront; ++i) {
    const int b = (threadIdx.x >> 3) + i * static_cast<int>(blockDim.x >> 3);
    if (b < k / 32) Load4Wide<XT>(x, static_cast<int64_t>(b) * 32 + lane8 * 4, k, wide, f.v[i]);
  }
  return f;
}

struct FrontQ8 {
  uint32_t w[9];
};

__device__ __forceinline__ FrontQ8 LoadFrontQ8(const uint8_t* __restrict__ y, int blocks) {
  FrontQ8 f;
  const int b = threadIdx.x;
  if (b < blocks) {
    const uint32_t* src = reinterpret_cast<const uint32_t*>(y + static_cast<int64_t>(b) * kQ8Block);
#pragma unroll
    for (int i = 0; i < 9; ++i) f.w[i] = src[i];
  }
  return f;
}

// The same loads written as instructions, always issued (a thread past the row's blocks reads the last block
// again): the compiler neither counts them nor waits for them, so the kernel's own wait, after the first tile's
// loads are queued, decides when they are read (AwaitFront). Loads the compiler knows of were waited for where
// they were issued, a trip to memory before the first tile's loads, and again with every tile load landed
// (their number is not known at compile time) before the staging that should run under them.
typedef uint32_t FrontWords __attribute__((ext_vector_type(4)));
struct FrontQ8Asm {
  FrontWords a, b;  // the block's first eight words
  uint32_t c;       // its ninth
};
__device__ __forceinline__ FrontQ8Asm LoadFrontQ8Asm(const uint8_t* __restrict__ y, int blocks) {
  FrontQ8Asm f;
  const int b = min(static_cast<int>(threadIdx.x), blocks - 1);
  const uint8_t* src = y + static_cast<int64_t>(b) * kQ8Block;
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(f.a) : "v"(src) : "memory");
  asm volatile("global_load_dwordx4 %0, %1, off offset:16" : "=v"(f.b) : "v"(src) : "memory");
  asm volatile("global_load_dword %0, %1, off offset:32" : "=v"(f.c) : "v"(src) : "memory");
  return f;
}
// The front loads have landed once no more than `later` memory operations issued after them are outstanding (a
// wave's memory operations complete in order); `later` must not exceed the number actually issued since.
__device__ __forceinline__ void AwaitFront(FrontQ8Asm& f, int later) {
  // One statement for every count: the registers go in and come out of it where they are. (A switch over ten
  // statements let the compiler copy the registers on its way into a case, ahead of the wait, while the loads were
  // still on their way.)
  const int n = __builtin_amdgcn_readfirstlane(later);
  asm volatile(
      "s_cmp_lt_u32 %3, 10\n\ts_cbranch_scc1 1f\n\ts_waitcnt vmcnt(10)\n\ts_branch 11f\n"
      "1:\ts_cmp_lt_u32 %3, 9\n\ts_cbranch_scc1 2f\n\ts_waitcnt vmcnt(9)\n\ts_branch 11f\n"
      "2:\ts_cmp_lt_u32 %3, 8\n\ts_cbranch_scc1 3f\n\ts_waitcnt vmcnt(8)\n\ts_branch 11f\n"
      "3:\ts_cmp_lt_u32 %3, 7\n\ts_cbranch_scc1 4f\n\ts_waitcnt vmcnt(7)\n\ts_branch 11f\n"
      "4:\ts_cmp_lt_u32 %3, 6\n\ts_cbranch_scc1 5f\n\ts_waitcnt vmcnt(6)\n\ts_branch 11f\n"
      "5:\ts_cmp_lt_u32 %3, 5\n\ts_cbranch_scc1 6f\n\ts_waitcnt vmcnt(5)\n\ts_branch 11f\n"
      "6:\ts_cmp_lt_u32 %3, 4\n\ts_cbranch_scc1 7f\n\ts_waitcnt vmcnt(4)\n\ts_branch 11f\n"
      "7:\ts_cmp_lt_u32 %3, 3\n\ts_cbranch_scc1 8f\n\ts_waitcnt vmcnt(3)\n\ts_branch 11f\n"
      "8:\ts_cmp_lt_u32 %3, 2\n\ts_cbranch_scc1 9f\n\ts_waitcnt vmcnt(2)\n\ts_branch 11f\n"
      "9:\ts_cmp_lt_u32 %3, 1\n\ts_cbranch_scc1 10f\n\ts_waitcnt vmcnt(1)\n\ts_branch 11f\n"
      "10:\ts_waitcnt vmcnt(0)\n"
      "11:"
      : "+v"(f.a), "+v"(f.b), "+v"(f.c)
      : "s"(n)
      : "scc", "memory");
}
// The unquantized activations' front pieces the same way: a lane's four values of a block as they lie in memory
// (sixteen bytes of F32, eight of BF16 or F16; the row aligned to that), always loaded (a lane past the row's blocks
// reads the last block's piece again), converted after the wait.
typedef uint32_t FrontPair __attribute__((ext_vector_type(2)));
template <int XT>
struct FrontXAsm {
  FrontWords w[kFront];  // F32
  FrontPair h[kFront];   // the 16-bit types
};
template <int XT>
__device__ __forceinline__ FrontXAsm<XT> LoadFrontXAsm(const void* __restrict__ x, int k) {
  FrontXAsm<XT> f;
  const int lane8 = threadIdx.x & 7;
#pragma unroll
  for (int i = 0; i < kFront; ++i) {
    const int b = min(static_cast<int>(threadIdx.x >> 3) + i * static_cast<int>(blockDim.x >> 3), k / 32 - 1);
    const int64_t at = static_cast<int64_t>(b) * 32 + lane8 * 4;
    if constexpr (XT == LLMP_X_F32) {
      const float* src = static_cast<const float*>(x) + at;
      asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(f.w[i]) : "v"(src) : "memory");
    } else {
      const uint16_t* src = static_cast<const uint16_t*>(x) + at;
      asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(f.h[i]) : "v"(src) : "memory");
    }
  }
  return f;
}
#define LLMP_WAIT_CHAIN                                                                            \
  "s_cmp_lt_u32 %2, 10\n\ts_cbranch_scc1 1f\n\ts_waitcnt vmcnt(10)\n\ts_branch 11f\n"               \
  "1:\ts_cmp_lt_u32 %2, 9\n\ts_cbranch_scc1 2f\n\ts_waitcnt vmcnt(9)\n\ts_branch 11f\n"             \
  "2:\ts_cmp_lt_u32 %2, 8\n\ts_cbranch_scc1 3f\n\ts_waitcnt vmcnt(8)\n\ts_branch 11f\n"             \
  "3:\ts_cmp_lt_u32 %2, 7\n\ts_cbranch_scc1 4f\n\ts_waitcnt vmcnt(7)\n\ts_branch 11f\n"             \
  "4:\ts_cmp_lt_u32 %2, 6\n\ts_cbranch_scc1 5f\n\ts_waitcnt vmcnt(6)\n\ts_branch 11f\n"             \
  "5:\ts_cmp_lt_u32 %2, 5\n\ts_cbranch_scc1 6f\n\ts_waitcnt vmcnt(5)\n\ts_branch 11f\n"             \
  "6:\ts_cmp_lt_u32 %2, 4\n\ts_cbranch_scc1 7f\n\ts_waitcnt vmcnt(4)\n\ts_branch 11f\n"             \
  "7:\ts_cmp_lt_u32 %2, 3\n\ts_cbranch_scc1 8f\n\ts_waitcnt vmcnt(3)\n\ts_branch 11f\n"             \
  "8:\ts_cmp_lt_u32 %2, 2\n\ts_cbranch_scc1 9f\n\ts_waitcnt vmcnt(2)\n\ts_branch 11f\n"             \
  "9:\ts_cmp_lt_u32 %2, 1\n\ts_cbranch_scc1 10f\n\ts_waitcnt vmcnt(1)\n\ts_branch 11f\n"            \
  "10:\ts_waitcnt vmcnt(0)\n"                                                                       \
  "11:"
template <int XT>
__device__ __forceinline__ void AwaitFrontX(FrontXAsm<XT>& f, int later) {
  static_assert(kFront == 2, "the registers this wait ties");
  const int n = __builtin_amdgcn_readfirstlane(later);
  if constexpr (XT == LLMP_X_F32) {
    asm volatile(LLMP_WAIT_CHAIN : "+v"(f.w[0]), "+v"(f.w[1]) : "s"(n) : "scc", "memory");
  } else {
    asm volatile(LLMP_WAIT_CHAIN : "+v"(f.h[0]), "+v"(f.h[1]) : "s"(n) : "scc", "memory");
  }
}
#undef LLMP_WAIT_CHAIN
template <int XT>
__device__ __forceinline__ void FrontValues(const FrontXAsm<XT>& f, int i, float (&v)[4]) {
  const FrontPair w = f.h[i];
  if constexpr (XT == LLMP_X_F32) {
    // (Through scalars: __builtin_bit_cast of a vector's component reads its first component with this compiler.)
    const uint32_t x0 = f.w[i].x, x1 = f.w[i].y, x2 = f.w[i].z, x3 = f.w[i].w;
    v[0] = __builtin_bit_cast(float, x0), v[1] = __builtin_bit_cast(float, x1);
    v[2] = __builtin_bit_cast(float, x2), v[3] = __builtin_bit_cast(float, x3);
  } else if constexpr (XT == LLMP_X_BF16) {
    v[0] = Bf16BitsToFloat(w.x & 0xFFFFu), v[1] = Bf16BitsToFloat(w.x >> 16);
    v[2] = Bf16BitsToFloat(w.y & 0xFFFFu), v[3] = Bf16BitsToFloat(w.y >> 16);
  } else {
    v[0] = HalfBitsToFloat(w.x & 0xFFFFu), v[1] = HalfBitsToFloat(w.x >> 16);
    v[2] = HalfBitsToFloat(w.y & 0xFFFFu), v[3] = HalfBitsToFloat(w.y >> 16);
  }
}
__device__ __forceinline__ uint32_t FlatLdsAddress(const void* p) { return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(p)); }
__device__ __forceinline__ void FlatLdsWrite16(uint32_t at, FrontWords v) { asm volatile("ds_write_b128 %0, %1" : : "v"(at), "v"(v) : "memory"); }
__device__ __forceinline__ void FlatLdsWrite4(uint32_t at, uint32_t v) { asm volatile("ds_write_b32 %0, %1" : : "v"(at), "v"(v) : "memory"); }
__device__ __forceinline__ void FlatLdsWrite2(uint32_t at, uint32_t v) { asm volatile("ds_write_b16 %0, %1" : : "v"(at), "v"(v) : "memory"); }

__device__ __forceinline__ float ByteToFloat(uint32_t word, int byte) {
  return static_cast<float>((word >> (8 * byte)) & 0xFFu);  // v_cvt_f32_ubyteN
}

// ---- Q4_K: a unit is a super-block

struct SuperBlock {
  U32x4 header;  // d, dmin, scales[12]
  U32x4 codes[8];
};

struct FormatQ4K {
  static constexpr int kUnitBytes = 144;    // of weights a lane
  static constexpr int kUnitValues = 256;
  static constexpr int kBlockBytes = 144;   // the descriptor's strides count these
  static constexpr int kBlockValues = 256;
  static constexpr int kRecord = 336;       // bytes a staged unit of activations
  static constexpr int kDumpInts = 16;      // block sums a unit
  using Unit = SuperBlock;

  static __device__ __forceinline__ Unit Read(const uint8_t* at) {
    SuperBlock b;
    const U32x4* mine = reinterpret_cast<const U32x4*>(at);
    b.header = mine[0];
#pragma unroll
    for (int i = 0; i < 8; ++i) b.codes[i] = mine[1 + i];
    return b;
  }

  // One block of 32 values, eight lanes: its codes, scale and sums into the record.
  static __device__ __forceinline__ void StageX(const float (&v)[4], int b, uint8_t* token) {
    const int lane8 = threadIdx.x & 7;
    const Q8Block q = QuantizeQ8Block(v[0], v[1], v[2], v[3]);
    uint8_t* record = token + (b >> 3) * kRecord;
    const int g = b & 7;
    *reinterpret_cast<uint32_t*>(record + g * 32 + lane8 * 4) = q.codes;
    int s = Dot4(0x01010101, static_cast<int>(q.codes), 0);
    s += ShflXor(s, 1);
    s += ShflXor(s, 2);
    s += ShflXor(s, 4);
    if (lane8 == 0) {
      // The products read the scale as a Q8_1 block stores it: rounded to F16.
      const float d8 = HalfBitsToFloat(FloatToHalfBits(q.d));
      reinterpret_cast<float*>(record + 256)[g] = d8;
      reinterpret_cast<float*>(record + 288)[g] = d8 * static_cast<float>(s);
      reinterpret_cast<int16_t*>(record + 320)[g] = static_cast<int16_t>(s);
    }
  }

  // StageX with the record written by instructions (see StageQ8Asm below).
  static __device__ __forceinline__ void StageXAsm(const float (&v)[4], int b, uint8_t* token) {
    const int lane8 = threadIdx.x & 7;
    const Q8Block q = QuantizeQ8Block(v[0], v[1], v[2], v[3]);
    const uint32_t record = FlatLdsAddress(token) + static_cast<uint32_t>((b >> 3) * kRecord);
    const int g = b & 7;
    FlatLdsWrite4(record + g * 32 + lane8 * 4, q.codes);
    int s = Dot4(0x01010101, static_cast<int>(q.codes), 0);
    s += ShflXor(s, 1);
    s += ShflXor(s, 2);
    s += ShflXor(s, 4);
    if (lane8 == 0) {
      const float d8 = HalfBitsToFloat(FloatToHalfBits(q.d));
      FlatLdsWrite4(record + 256 + g * 4, __builtin_bit_cast(uint32_t, d8));
      FlatLdsWrite4(record + 288 + g * 4, __builtin_bit_cast(uint32_t, d8 * static_cast<float>(s)));
      FlatLdsWrite2(record + 320 + g * 2, static_cast<uint32_t>(s));
    }
  }
  static constexpr bool kStagesXUnderLoads = true;

  // One Q8_1 block (nine dwords), one thread.
  static __device__ __forceinline__ void StageQ8(const uint32_t (&w)[9], int b, uint8_t* token) {
    uint8_t* record = token + (b >> 3) * kRecord;
    const int g = b & 7;
    uint4* dst = reinterpret_cast<uint4*>(record + g * 32);
    dst[0] = make_uint4(w[1], w[2], w[3], w[4]);
    dst[1] = make_uint4(w[5], w[6], w[7], w[8]);
    int s = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) s = Dot4(0x01010101, static_cast<int>(w[1 + i]), s);
    const float d8 = HalfBitsToFloat(w[0] & 0xFFFFu);
    reinterpret_cast<float*>(record + 256)[g] = d8;
    reinterpret_cast<float*>(record + 288)[g] = d8 * static_cast<float>(s);
    reinterpret_cast<int16_t*>(record + 320)[g] = static_cast<int16_t>(s);
  }

  // The same with the record written by instructions the compiler does not take for accesses of LDS: it would hold
  // them back until every load into LDS in flight has landed.
  static constexpr bool kStagesUnderLoads = true;
  static __device__ __forceinline__ void StageQ8Asm(const FrontQ8Asm& f, int b, uint8_t* token) {
    const uint32_t record = FlatLdsAddress(token) + static_cast<uint32_t>((b >> 3) * kRecord);
    const int g = b & 7;
    FlatLdsWrite16(record + g * 32, FrontWords{f.a.y, f.a.z, f.a.w, f.b.x});
    FlatLdsWrite16(record + g * 32 + 16, FrontWords{f.b.y, f.b.z, f.b.w, f.c});
    int s = Dot4(0x01010101, static_cast<int>(f.a.y), 0);
    s = Dot4(0x01010101, static_cast<int>(f.a.z), s);
    s = Dot4(0x01010101, static_cast<int>(f.a.w), s);
    s = Dot4(0x01010101, static_cast<int>(f.b.x), s);
    s = Dot4(0x01010101, static_cast<int>(f.b.y), s);
    s = Dot4(0x01010101, static_cast<int>(f.b.z), s);
    s = Dot4(0x01010101, static_cast<int>(f.b.w), s);
    s = Dot4(0x01010101, static_cast<int>(f.c), s);
    const float d8 = HalfBitsToFloat(f.a.x & 0xFFFFu);
    FlatLdsWrite4(record + 256 + g * 4, __builtin_bit_cast(uint32_t, d8));
    FlatLdsWrite4(record + 288 + g * 4, __builtin_bit_cast(uint32_t, d8 * static_cast<float>(s)));
    FlatLdsWrite2(record + 320 + g * 2, static_cast<uint32_t>(s));
  }

  // The super-block at `at` (LDS) times the staged tokens. With several tokens a pass the
  // codes are read a pair of sub-blocks at a time, each pair used by every token before the
  // next is read: the whole super-block and four tokens' operands do not fit the registers.
template <int P, bool kDump>
  static __device__ __forceinline__ void DotAt(const uint8_t* at, const uint8_t* records, int token_stride, int m,
                                                float (&out)[P], int32_t* dump) {
#pragma clang fp contract(off)
  const U32x4* mine = reinterpret_cast<const U32x4*>(at);
  const U32x4 header = mine[0];
  const uint32_t s0 = header.y, s1 = header.z, s2 = header.w;
  // Bytes g of sc[0], sc[1]: the scales of sub-blocks g and 4 + g; mn likewise.
  const uint32_t sc[2] = {s0 & 0x3F3F3F3Fu, (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u)};
  const uint32_t mn[2] = {s1 & 0x3F3F3F3Fu, ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u)};
  const float d = HalfBitsToFloat(header.x & 0xFFFFu);
  const float dmin = HalfBitsToFloat(header.x >> 16);
  float main[P];
#pragma unroll
  for (int t = 0; t < P; ++t) main[t] = 0.0f;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    // Pair p: 32 bytes, the low nibbles sub-block 2p, the high ones 2p + 1.
    if constexpr (P > 1) __builtin_amdgcn_sched_barrier(0);
    int lo[8], hi[8];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const U32x4 raw = mine[1 + 2 * p + i];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        lo[4 * i + c] = static_cast<int>(raw[c] & 0x0F0F0F0Fu);
        hi[4 * i + c] = static_cast<int>((raw[c] >> 4) & 0x0F0F0F0Fu);
      }
    }
    const float sc0 = ByteToFloat(sc[(2 * p) >> 2], (2 * p) & 3);
    const float sc1 = ByteToFloat(sc[(2 * p + 1) >> 2], (2 * p + 1) & 3);
#pragma unroll
    for (int t = 0; t < P; ++t) {
      if (t < m) {
        const uint8_t* record = records + t * token_stride;
        const uint4* a = reinterpret_cast<const uint4*>(record + p * 64);
        const uint4 a0 = a[0], a1 = a[1], a2 = a[2], a3 = a[3];
        const float2 d8 = *reinterpret_cast<const float2*>(record + 256 + p * 8);
        int prod0 = Dot4(lo[0], static_cast<int>(a0.x), 0);
        prod0 = Dot4(lo[1], static_cast<int>(a0.y), prod0);
        prod0 = Dot4(lo[2], static_cast<int>(a0.z), prod0);
        prod0 = Dot4(lo[3], static_cast<int>(a0.w), prod0);
        prod0 = Dot4(lo[4], static_cast<int>(a1.x), prod0);
        prod0 = Dot4(lo[5], static_cast<int>(a1.y), prod0);
        prod0 = Dot4(lo[6], static_cast<int>(a1.z), prod0);
        prod0 = Dot4(lo[7], static_cast<int>(a1.w), prod0);
        int prod1 = Dot4(hi[0], static_cast<int>(a2.x), 0);
        prod1 = Dot4(hi[1], static_cast<int>(a2.y), prod1);
        prod1 = Dot4(hi[2], static_cast<int>(a2.z), prod1);
        prod1 = Dot4(hi[3], static_cast<int>(a2.w), prod1);
        prod1 = Dot4(hi[4], static_cast<int>(a3.x), prod1);
        prod1 = Dot4(hi[5], static_cast<int>(a3.y), prod1);
        prod1 = Dot4(hi[6], static_cast<int>(a3.z), prod1);
        prod1 = Dot4(hi[7], static_cast<int>(a3.w), prod1);
        if (kDump && dump != nullptr) {
          dump[2 * p] = prod0;
          dump[2 * p + 1] = prod1;
          const int16_t* sums = reinterpret_cast<const int16_t*>(record + 320);
          dump[8 + 2 * p] = sums[2 * p];
          dump[8 + 2 * p + 1] = sums[2 * p + 1];
        }
        main[t] = fmaf(static_cast<float>(prod0), sc0 * d8.x, main[t]);
        main[t] = fmaf(static_cast<float>(prod1), sc1 * d8.y, main[t]);
      }
    }
  }
#pragma unroll
  for (int t = 0; t < P; ++t) {
    if (t < m) {
      const float4* ds = reinterpret_cast<const float4*>(records + t * token_stride + 288);
      const float4 lo4 = ds[0], hi4 = ds[1];
      float mins = ByteToFloat(mn[0], 0) * lo4.x;
      mins = fmaf(ByteToFloat(mn[0], 1), lo4.y, mins);
      mins = fmaf(ByteToFloat(mn[0], 2), lo4.z, mins);
      mins = fmaf(ByteToFloat(mn[0], 3), lo4.w, mins);
      mins = fmaf(ByteToFloat(mn[1], 0), hi4.x, mins);
      mins = fmaf(ByteToFloat(mn[1], 1), hi4.y, mins);
      mins = fmaf(ByteToFloat(mn[1], 2), hi4.z, mins);
      mins = fmaf(ByteToFloat(mn[1], 3), hi4.w, mins);
      out[t] = fmaf(d, main[t], -(dmin * mins));
    }
  }
}
};

// ---- Q5_K: Q4_K's header and nibbles with a fifth bit a value
//
// {f16 d; f16 dmin; u8 scales[12]; u8 qh[32]; u8 qs[128]} = 176 bytes (src/format/encoding.cc:116 of the
// reference; ggml's dequantize_row_q5_K): bit g of byte i of qh is the fifth bit of value i of sub-block g, so the
// eight dwords of qh line up with the eight dwords of every pair of sub-blocks, a bit of each byte moved to bit 4
// of the nibble's byte. The staged activations and the sums over them are Q4_K's.
struct FormatQ5K : FormatQ4K {
  static constexpr int kUnitBytes = 176;
  static constexpr int kBlockBytes = 176;

  template <int P, bool kDump>
  static __device__ __forceinline__ void DotAt(const uint8_t* at, const uint8_t* records, int token_stride, int m,
                                               float (&out)[P], int32_t* dump) {
#pragma clang fp contract(off)
    const U32x4* mine = reinterpret_cast<const U32x4*>(at);
    const U32x4 header = mine[0];
    const uint32_t s0 = header.y, s1 = header.z, s2 = header.w;
    const uint32_t sc[2] = {s0 & 0x3F3F3F3Fu, (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u)};
    const uint32_t mn[2] = {s1 & 0x3F3F3F3Fu, ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u)};
    const float d = HalfBitsToFloat(header.x & 0xFFFFu);
    const float dmin = HalfBitsToFloat(header.x >> 16);
    float main[P];
#pragma unroll
    for (int t = 0; t < P; ++t) main[t] = 0.0f;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      // Pair p: 32 bytes, the low nibbles sub-block 2p, the high ones 2p + 1; their fifth bits are bits 2p and
      // 2p + 1 of qh's bytes. With several tokens a pass qh is read again for every pair (the clobber keeps the
      // compiler from holding its eight dwords beside four tokens' operands).
      if constexpr (P > 1) {
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("" ::: "memory");
      }
      const U32x4 high0 = mine[1], high1 = mine[2];
      const uint32_t qh[8] = {high0.x, high0.y, high0.z, high0.w, high1.x, high1.y, high1.z, high1.w};
      int lo[8], hi[8];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const U32x4 raw = mine[3 + 2 * p + i];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          const uint32_t h = qh[4 * i + c];
          const uint32_t fifth_lo = (2 * p <= 4 ? h << (4 - 2 * p) : h >> (2 * p - 4)) & 0x10101010u;
          const uint32_t fifth_hi = (2 * p + 1 <= 4 ? h << (3 - 2 * p) : h >> (2 * p - 3)) & 0x10101010u;
          lo[4 * i + c] = static_cast<int>((raw[c] & 0x0F0F0F0Fu) | fifth_lo);
          hi[4 * i + c] = static_cast<int>(((raw[c] >> 4) & 0x0F0F0F0Fu) | fifth_hi);
        }
      }
      const float sc0 = ByteToFloat(sc[(2 * p) >> 2], (2 * p) & 3);
      const float sc1 = ByteToFloat(sc[(2 * p + 1) >> 2], (2 * p + 1) & 3);
#pragma unroll
      for (int t = 0; t < P; ++t) {
        if (t < m) {
          const uint8_t* record = records + t * token_stride;
          const uint4* a = reinterpret_cast<const uint4*>(record + p * 64);
          const uint4 a0 = a[0], a1 = a[1], a2 = a[2], a3 = a[3];
          const uint32_t first[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
          const uint32_t second[8] = {a2.x, a2.y, a2.z, a2.w, a3.x, a3.y, a3.z, a3.w};
          const float2 d8 = *reinterpret_cast<const float2*>(record + 256 + p * 8);
          int prod0 = 0, prod1 = 0;
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            prod0 = Dot4(lo[i], static_cast<int>(first[i]), prod0);
            prod1 = Dot4(hi[i], static_cast<int>(second[i]), prod1);
          }
          if constexpr (P > 1) asm volatile("" : "+v"(prod0), "+v"(prod1));  // taken here: the products stay with their pair
          if (kDump && dump != nullptr) {
            dump[2 * p] = prod0;
            dump[2 * p + 1] = prod1;
            const int16_t* sums = reinterpret_cast<const int16_t*>(record + 320);
            dump[8 + 2 * p] = sums[2 * p];
            dump[8 + 2 * p + 1] = sums[2 * p + 1];
          }
          main[t] = fmaf(static_cast<float>(prod0), sc0 * d8.x, main[t]);
          main[t] = fmaf(static_cast<float>(prod1), sc1 * d8.y, main[t]);
        }
      }
    }
#pragma unroll
    for (int t = 0; t < P; ++t) {
      if (t < m) {
        const float4* ds = reinterpret_cast<const float4*>(records + t * token_stride + 288);
        const float4 lo4 = ds[0], hi4 = ds[1];
        float mins = ByteToFloat(mn[0], 0) * lo4.x;
        mins = fmaf(ByteToFloat(mn[0], 1), lo4.y, mins);
        mins = fmaf(ByteToFloat(mn[0], 2), lo4.z, mins);
        mins = fmaf(ByteToFloat(mn[0], 3), lo4.w, mins);
        mins = fmaf(ByteToFloat(mn[1], 0), hi4.x, mins);
        mins = fmaf(ByteToFloat(mn[1], 1), hi4.y, mins);
        mins = fmaf(ByteToFloat(mn[1], 2), hi4.z, mins);
        mins = fmaf(ByteToFloat(mn[1], 3), hi4.w, mins);
        out[t] = fmaf(d, main[t], -(dmin * mins));
      }
    }
  }
};

// ---- Q6_K: {u8 ql[128]; u8 qh[64]; i8 scales[16]; f16 d} = 210 bytes, 256 values
//
// src/format/encoding.cc:117 of the reference; ggml's dequantize_row_q6_K: value 128 h + 32 t + l (h < 2, t < 4,
// l < 32) is the low (t < 2) or high nibble of ql[64 h + 32 (t & 1) + l] plus 16 times bits 2t, 2t + 1 of
// qh[32 h + l], minus 32, times scales[value / 16] times d. A block is not a whole number of dwords: a tile is
// fetched as 16-byte chunks from the boundary below its first byte, a lane's unit then starts 0 or 2 bytes into a
// dword and every dword it uses is put together from two (v_alignbyte). Codes
// become signed bytes without a subtraction a byte: x + 0x60 cannot carry for x < 64, and flipping bit 7 of that is
// x - 32. The staged activations are Q4_K's (the codes in order, d8 a block).
struct FormatQ6K : FormatQ4K {
  static constexpr int kUnitBytes = 210;
  static constexpr int kBlockBytes = 210;
  static constexpr int kDumpInts = 16;  // the sixteen sub-blocks' sums

  template <int P, bool kDump>
  static __device__ __forceinline__ void DotAt(const uint8_t* at, const uint8_t* records, int token_stride, int m,
                                               float (&out)[P], int32_t* dump) {
#pragma clang fp contract(off)
    const uint32_t shift = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(at)) & 3u;
    const uint32_t* base = reinterpret_cast<const uint32_t*>(at - shift);
    // Dwords first .. first + N - 1 of the unit.
    auto take = [&](int first, auto& dst) {
      constexpr int N = sizeof(dst) / sizeof(uint32_t);
      uint32_t raw[N + 1];
#pragma unroll
      for (int i = 0; i <= N; ++i) raw[i] = base[first + i];
#pragma unroll
      for (int i = 0; i < N; ++i) dst[i] = __builtin_amdgcn_alignbyte(raw[i + 1], raw[i], shift);
    };
    uint32_t tail[5];  // the sixteen scales, d
    take(48, tail);
    const float d = HalfBitsToFloat(tail[4] & 0xFFFFu);
    float v[P];
#pragma unroll
    for (int t = 0; t < P; ++t) v[t] = 0.0f;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      // One token a pass: the half's 96 bytes at once. Several: a block's 64 at a time, read again for every block
      // (the clobber keeps the compiler from holding them beside four tokens' operands).
      uint32_t ql[P > 1 ? 8 : 16], qh[8];
      if constexpr (P == 1) {
        take(16 * h, ql);
        take(32 + 8 * h, qh);
      }
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int block = 4 * h + g;  // of 32 values: two sub-blocks
        if constexpr (P > 1) {
          __builtin_amdgcn_sched_barrier(0);
          asm volatile("" ::: "memory");
          take(16 * h + 8 * (g & 1), ql);
          take(32 + 8 * h, qh);
        }
        int value[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const uint32_t low = ql[(P > 1 ? 0 : 8 * (g & 1)) + j];
          const uint32_t nibbles = (g >> 1) ? (low >> 4) & 0x0F0F0F0Fu : low & 0x0F0F0F0Fu;
          const uint32_t high = (2 * g <= 4 ? qh[j] << (4 - 2 * g) : qh[j] >> (2 * g - 4)) & 0x30303030u;
          value[j] = static_cast<int>(((nibbles | high) + 0x60606060u) ^ 0x80808080u);
        }
        const uint32_t both = tail[block >> 1] >> (16 * (block & 1));
        const int sc0 = static_cast<int8_t>(both & 0xFFu), sc1 = static_cast<int8_t>((both >> 8) & 0xFFu);
#pragma unroll
        for (int t = 0; t < P; ++t) {
          if (t < m) {
            const uint8_t* record = records + t * token_stride;
            const uint4* a = reinterpret_cast<const uint4*>(record + block * 32);
            const uint4 a0 = a[0], a1 = a[1];
            int first = Dot4(value[0], static_cast<int>(a0.x), 0);
            first = Dot4(value[1], static_cast<int>(a0.y), first);
            first = Dot4(value[2], static_cast<int>(a0.z), first);
            first = Dot4(value[3], static_cast<int>(a0.w), first);
            int second = Dot4(value[4], static_cast<int>(a1.x), 0);
            second = Dot4(value[5], static_cast<int>(a1.y), second);
            second = Dot4(value[6], static_cast<int>(a1.z), second);
            second = Dot4(value[7], static_cast<int>(a1.w), second);
            if constexpr (P > 1) asm volatile("" : "+v"(first), "+v"(second));  // taken here: the products stay with their block
            if (kDump && dump != nullptr) dump[2 * block] = first, dump[2 * block + 1] = second;
            const float d8 = reinterpret_cast<const float*>(record + 256)[block];
            v[t] = fmaf(d8, static_cast<float>(sc0 * first + sc1 * second), v[t]);
          }
        }
      }
    }
#pragma unroll
    for (int t = 0; t < P; ++t) {
      if (t < m) out[t] = d * v[t];
    }
  }
};

// ---- Q8_0: a unit is four blocks

struct FourBlocks {
  uint32_t w[34];  // {f16 d; i8 qs[32]} x 4, as they lie
};

struct FormatQ8 {
  static constexpr int kUnitBytes = 136;
  static constexpr int kUnitValues = 128;
  static constexpr int kBlockBytes = 34;
  static constexpr int kBlockValues = 32;
  static constexpr int kRecord = 152;
  static constexpr int kDumpInts = 4;
  using Unit = FourBlocks;

  static __device__ __forceinline__ Unit Read(const uint8_t* at) {
    FourBlocks u;
    const uint2* mine = reinterpret_cast<const uint2*>(at);
#pragma unroll
    for (int i = 0; i < 17; ++i) {
      const uint2 v = mine[i];
      u.w[2 * i] = v.x;
      u.w[2 * i + 1] = v.y;
    }
    return u;
  }

  // One block of 32 values, eight lanes: the lane's four codes go where the block's weight
  // codes 4 lane .. 4 lane + 3 lie in the unit, two bytes into it.
  static __device__ __forceinline__ void StageX(const float (&v)[4], int b, uint8_t* token) {
    const int lane8 = threadIdx.x & 7;
    const Q8Block q = QuantizeQ8Block(v[0], v[1], v[2], v[3]);
    uint8_t* record = token + (b >> 2) * kRecord;
    const int j = b & 3;
    uint16_t* at = reinterpret_cast<uint16_t*>(record + 34 * j + 2 + lane8 * 4);
    at[0] = static_cast<uint16_t>(q.codes & 0xFFFFu);
    at[1] = static_cast<uint16_t>(q.codes >> 16);
    if (lane8 == 0) {
      *reinterpret_cast<uint16_t*>(record + 34 * j) = 0;  // against the weight block's scale
      reinterpret_cast<float*>(record + 136)[j] = HalfBitsToFloat(FloatToHalfBits(q.d));
    }
  }

  // StageX with the record written by instructions (see FormatQ4K::StageQ8Asm).
  static constexpr bool kStagesXUnderLoads = true;
  static __device__ __forceinline__ void StageXAsm(const float (&v)[4], int b, uint8_t* token) {
    const int lane8 = threadIdx.x & 7;
    const Q8Block q = QuantizeQ8Block(v[0], v[1], v[2], v[3]);
    const uint32_t record = FlatLdsAddress(token) + static_cast<uint32_t>((b >> 2) * kRecord);
    const int j = b & 3;
    const uint32_t at = record + 34 * j + 2 + lane8 * 4;
    FlatLdsWrite2(at, q.codes & 0xFFFFu);
    FlatLdsWrite2(at + 2, q.codes >> 16);
    if (lane8 == 0) {
      FlatLdsWrite2(record + 34 * j, 0u);  // against the weight block's scale
      FlatLdsWrite4(record + 136 + 4 * j, __builtin_bit_cast(uint32_t, HalfBitsToFloat(FloatToHalfBits(q.d))));
    }
  }

  // One Q8_1 block (nine dwords), one thread. Blocks 1 and 3 of a unit have their codes on a
  // dword boundary (dwords 9-16 and 26-33); blocks 0 and 2 two bytes into dwords 0 and 17,
  // their nine dwords ending with the two bytes that face the next block's scale.
  static __device__ __forceinline__ void StageQ8(const uint32_t (&w)[9], int b, uint8_t* token) {
    uint8_t* record = token + (b >> 2) * kRecord;
    const int j = b & 3;
    uint32_t* image = reinterpret_cast<uint32_t*>(record);
    if (j & 1) {
      uint32_t* dst = image + (j == 1 ? 9 : 26);
#pragma unroll
      for (int i = 0; i < 8; ++i) dst[i] = w[1 + i];
    } else {
      uint32_t* dst = image + (j == 0 ? 0 : 17);
      dst[0] = w[1] << 16;
#pragma unroll
      for (int i = 1; i < 8; ++i) dst[i] = (w[i] >> 16) | (w[i + 1] << 16);
      dst[8] = w[8] >> 16;
    }
    reinterpret_cast<float*>(record + 136)[j] = HalfBitsToFloat(w[0] & 0xFFFFu);
  }

  // The same by instructions (see FormatQ4K::StageQ8Asm).
  static constexpr bool kStagesUnderLoads = true;
  static __device__ __forceinline__ void StageQ8Asm(const FrontQ8Asm& f, int b, uint8_t* token) {
    const uint32_t w[9] = {f.a.x, f.a.y, f.a.z, f.a.w, f.b.x, f.b.y, f.b.z, f.b.w, f.c};
    const uint32_t record = FlatLdsAddress(token) + static_cast<uint32_t>((b >> 2) * kRecord);
    const int j = b & 3;
    if (j & 1) {
      const uint32_t dst = record + 4 * (j == 1 ? 9 : 26);
#pragma unroll
      for (int i = 0; i < 8; ++i) FlatLdsWrite4(dst + 4 * i, w[1 + i]);
    } else {
      const uint32_t dst = record + 4 * (j == 0 ? 0 : 17);
      FlatLdsWrite4(dst, w[1] << 16);
#pragma unroll
      for (int i = 1; i < 8; ++i) FlatLdsWrite4(dst + 4 * i, (w[i] >> 16) | (w[i + 1] << 16));
      FlatLdsWrite4(dst + 32, w[8] >> 16);
    }
    FlatLdsWrite4(record + 136 + 4 * j, __builtin_bit_cast(uint32_t, HalfBitsToFloat(w[0] & 0xFFFFu)));
  }

  template <int P, bool kDump>
  static __device__ __forceinline__ void DotAt(const uint8_t* at, const uint8_t* records, int token_stride, int m,
                                               float (&out)[P], int32_t* dump) {
    Dot<P, kDump>(Read(at), records, token_stride, m, out, dump);
  }

  // Four blocks times the staged tokens.
  template <int P, bool kDump>
  static __device__ __forceinline__ void Dot(const Unit& u, const uint8_t* records, int token_stride, int m,
                                             float (&out)[P], int32_t* dump) {
#pragma clang fp contract(off)
    const float dw0 = HalfBitsToFloat(u.w[0] & 0xFFFFu);
    const float dw1 = HalfBitsToFloat(u.w[8] >> 16);
    const float dw2 = HalfBitsToFloat(u.w[17] & 0xFFFFu);
    const float dw3 = HalfBitsToFloat(u.w[25] >> 16);
#pragma unroll
    for (int t = 0; t < P; ++t) {
      if (t < m) {
        const uint8_t* record = records + t * token_stride;
        const uint2* image = reinterpret_cast<const uint2*>(record);
        int s[4] = {0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 17; ++i) {
          const uint2 x = image[i];
          constexpr int kOwner[34] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 1, 1, 1, 1, 1, 1, 1, 1,
                                      2, 2, 2, 2, 2, 2, 2, 2, 2, 3, 3, 3, 3, 3, 3, 3, 3};
          s[kOwner[2 * i]] = Dot4(static_cast<int>(u.w[2 * i]), static_cast<int>(x.x), s[kOwner[2 * i]]);
          s[kOwner[2 * i + 1]] = Dot4(static_cast<int>(u.w[2 * i + 1]), static_cast<int>(x.y), s[kOwner[2 * i + 1]]);
        }
        if constexpr (P > 1) asm volatile("" : "+v"(s[0]), "+v"(s[1]), "+v"(s[2]), "+v"(s[3]));  // a token's products together
        const float2 da = *reinterpret_cast<const float2*>(record + 136);
        const float2 db = *reinterpret_cast<const float2*>(record + 144);
        if (kDump && dump != nullptr) {
#pragma unroll
          for (int j = 0; j < 4; ++j) dump[j] = s[j];
        }
        float v = static_cast<float>(s[0]) * (dw0 * da.x);
        v = fmaf(static_cast<float>(s[1]), dw1 * da.y, v);
        v = fmaf(static_cast<float>(s[2]), dw2 * db.x, v);
        v = fmaf(static_cast<float>(s[3]), dw3 * db.y, v);
        out[t] = v;
      }
    }
  }
};

// ---- Q4_0: a unit is eight blocks of {f16 d; u8 nibbles[16]} (144 bytes, 256 values)
//
// Value i of a block is the low nibble of byte i (i < 16) or the high nibble of byte i - 16,
// minus 8; a block times a Q8_1 block is dw * (sum(code * q) * d8 - 8 * s8) with s8 the
// activation block's stored sum (tests/unit/dsv4_fast_test.cc:141-164 of the reference). A pair
// of blocks is 36 bytes, nine dwords: the even block's scale and first two code bytes, three
// dwords of codes, its last two code bytes and the odd block's scale, then the odd block's four
// dwords. The staged activations are two images of that layout, one for the low nibbles
// (values 0-15 of a block) and one for the high (16-31), with zeros where the weight scales lie:
// masked nibbles and images multiply dword by dword as they lie.
struct FormatQ40 {
  static constexpr int kUnitBytes = 144;
  static constexpr int kUnitValues = 256;
  static constexpr int kBlockBytes = 18;
  static constexpr int kBlockValues = 32;
  // Two images of 144 bytes, eight d8, eight s8, and eight bytes that put the records of a
  // row's first sixteen units in different LDS banks (90 dwords apart; read 4 or 8 bytes at a time).
  static constexpr int kRecord = 360;
  static constexpr int kDumpInts = 8;

  // The image byte of value v (0 .. 15) of block j of a unit.
  static __device__ __forceinline__ int ImageAt(int j, int v) { return 36 * (j >> 1) + ((j & 1) ? 20 : 2) + v; }

  // One block of 32 values, eight lanes, four values a lane: lanes 0-3 hold values 0-15 (the low
  // image), lanes 4-7 values 16-31 (the high image).
  static __device__ __forceinline__ void StageX(const float (&v)[4], int b, uint8_t* token) {
    const int lane8 = threadIdx.x & 7;
    const Q8Block q = QuantizeQ8Block(v[0], v[1], v[2], v[3]);
    uint8_t* record = token + (b >> 3) * kRecord;
    const int j = b & 7;
    uint8_t* image = record + (lane8 >> 2) * 144;
    uint16_t* at = reinterpret_cast<uint16_t*>(image + ImageAt(j, 4 * (lane8 & 3)));
    at[0] = static_cast<uint16_t>(q.codes & 0xFFFFu);
    at[1] = static_cast<uint16_t>(q.codes >> 16);
    if ((lane8 & 3) == 0) *reinterpret_cast<uint16_t*>(image + 36 * (j >> 1) + ((j & 1) ? 18 : 0)) = 0;  // against the scale
    if (lane8 == 0) {
      reinterpret_cast<float*>(record + 288)[j] = HalfBitsToFloat(FloatToHalfBits(q.d));
      reinterpret_cast<float*>(record + 320)[j] = HalfBitsToFloat(FloatToHalfBits(q.sum));
    }
  }

  // One Q8_1 block (nine dwords), one thread: both images' dwords of the block.
  static __device__ __forceinline__ void StageQ8(const uint32_t (&w)[9], int b, uint8_t* token) {
    uint8_t* record = token + (b >> 3) * kRecord;
    const int j = b & 7;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      uint32_t* pair = reinterpret_cast<uint32_t*>(record + half * 144) + 9 * (j >> 1);
      const uint32_t* c = w + 1 + 4 * half;  // the sixteen codes of this half
      if (j & 1) {
        // The dword shared with the even block holds only zeros of this block (its scale).
#pragma unroll
        for (int i = 0; i < 4; ++i) pair[5 + i] = c[i];
      } else {
        pair[0] = c[0] << 16;
#pragma unroll
        for (int i = 1; i < 4; ++i) pair[i] = (c[i - 1] >> 16) | (c[i] << 16);
        pair[4] = c[3] >> 16;
      }
    }
    reinterpret_cast<float*>(record + 288)[j] = HalfBitsToFloat(w[0] & 0xFFFFu);
    reinterpret_cast<float*>(record + 320)[j] = HalfBitsToFloat(w[0] >> 16);
  }

  // The unit at `at` (LDS) times the staged tokens.
  template <int P, bool kDump>
  static __device__ __forceinline__ void DotAt(const uint8_t* at, const uint8_t* records, int token_stride, int m,
                                               float (&out)[P], int32_t* dump) {
#pragma clang fp contract(off)
    if constexpr (P > 1) {
      // Several tokens a pass: a pair of blocks at a time, each pair used by every token before
      // the next is read (the whole unit's nibbles and the tokens' images do not fit the
      // registers); the same operations in the same order as below.
      float v[P];
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        __builtin_amdgcn_sched_barrier(0);
        const uint32_t* pair = reinterpret_cast<const uint32_t*>(at) + 9 * p;
        uint32_t lo_codes[9], hi_codes[9];
#pragma unroll
        for (int i = 0; i < 9; ++i) {
          const uint32_t word = pair[i];
          lo_codes[i] = word & 0x0F0F0F0Fu;
          hi_codes[i] = (word >> 4) & 0x0F0F0F0Fu;
        }
        const float dw_even = HalfBitsToFloat(pair[0] & 0xFFFFu), dw_odd = HalfBitsToFloat(pair[4] >> 16);
#pragma unroll
        for (int t = 0; t < P; ++t) {
          if (t < m) {
            const uint8_t* record = records + t * token_stride;
            const uint32_t* low = reinterpret_cast<const uint32_t*>(record) + 9 * p;
            const uint32_t* high = reinterpret_cast<const uint32_t*>(record + 144) + 9 * p;
            int even = 0, odd = 0;
#pragma unroll
            for (int i = 0; i < 9; ++i) {
              int& s = i >= 5 ? odd : even;
              s = Dot4(static_cast<int>(lo_codes[i]), static_cast<int>(low[i]), s);
              s = Dot4(static_cast<int>(hi_codes[i]), static_cast<int>(high[i]), s);
            }
            asm volatile("" : "+v"(even), "+v"(odd));  // taken here: the products stay with their pair
            const float2 d8 = *reinterpret_cast<const float2*>(record + 288 + 8 * p);
            const float2 s8 = *reinterpret_cast<const float2*>(record + 320 + 8 * p);
            const float term_even = dw_even * (static_cast<float>(even) * d8.x - 8.0f * s8.x);
            const float term_odd = dw_odd * (static_cast<float>(odd) * d8.y - 8.0f * s8.y);
            v[t] = p == 0 ? term_even : v[t] + term_even;
            v[t] = v[t] + term_odd;
          }
        }
      }
#pragma unroll
      for (int t = 0; t < P; ++t) {
        if (t < m) out[t] = v[t];
      }
      return;
    }
    const U32x4* mine = reinterpret_cast<const U32x4*>(at);
    uint32_t w[36];
#pragma unroll
    for (int i = 0; i < 9; ++i) {
      const U32x4 v = mine[i];
      w[4 * i] = v.x, w[4 * i + 1] = v.y, w[4 * i + 2] = v.z, w[4 * i + 3] = v.w;
    }
    float dw[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint32_t word = w[9 * (j >> 1) + ((j & 1) ? 4 : 0)];
      dw[j] = HalfBitsToFloat((j & 1) ? word >> 16 : word & 0xFFFFu);
    }
#pragma unroll
    for (int t = 0; t < P; ++t) {
      if (t < m) {
        const uint8_t* record = records + t * token_stride;
        const uint2* low = reinterpret_cast<const uint2*>(record);
        const uint2* high = reinterpret_cast<const uint2*>(record + 144);
        int s[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 18; ++i) {
          const uint2 lo = low[i], hi = high[i];
#pragma unroll
          for (int c = 0; c < 2; ++c) {
            const int index = 2 * i + c;
            const int owner = 2 * (index / 9) + (index % 9 >= 5 ? 1 : 0);  // the block the dword's codes belong to
            s[owner] = Dot4(static_cast<int>(w[index] & 0x0F0F0F0Fu), static_cast<int>(c ? lo.y : lo.x), s[owner]);
            s[owner] = Dot4(static_cast<int>((w[index] >> 4) & 0x0F0F0F0Fu), static_cast<int>(c ? hi.y : hi.x), s[owner]);
          }
        }
        if (kDump && dump != nullptr) {
#pragma unroll
          for (int j = 0; j < 8; ++j) dump[j] = s[j];
        }
        const float2* scales = reinterpret_cast<const float2*>(record + 288);
        float d8[8], s8[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float2 d = scales[j], sum = scales[4 + j];
          d8[2 * j] = d.x, d8[2 * j + 1] = d.y, s8[2 * j] = sum.x, s8[2 * j + 1] = sum.y;
        }
        float v = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float term = dw[j] * (static_cast<float>(s[j]) * d8[j] - 8.0f * s8[j]);
          v = j == 0 ? term : v + term;
        }
        out[t] = v;
      }
    }
  }
};

// ---- IQ4_NL: Q4_0's bytes {f16 d; u8 nibbles[16]}, each nibble an index into a codebook of sixteen int8
//
// src/kernels/ggml/vecq.cu:375-396 of the reference: a block times a Q8_1 block is (dw * d8) * sum(value[code] * q),
// the codebook being ggml's kvalues_iq4nl. Units, staged images and tiles are Q4_0's; a dword's eight nibbles
// become eight values by byte permutes: the code's low three bits pick from the lower and from the upper half
// of the codebook, its fourth bit between the two, byte by byte.
struct FormatIq4nl : FormatQ40 {
  static __device__ __forceinline__ uint32_t Merge(uint32_t mask, uint32_t a, uint32_t b) {
    uint32_t r;
    asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(r) : "s"(mask), "v"(a), "v"(b));  // (a & mask) | (b & ~mask)
    return r;
  }
  static __device__ __forceinline__ void Decode(uint32_t w, uint32_t& lo, uint32_t& hi) {
    // {-127, -104, -83, -65}, {-49, -35, -22, -10}, {1, 13, 25, 38}, {53, 69, 89, 113}
    constexpr uint32_t kLower0 = 0xBFAD9881u, kLower1 = 0xF6EADDCFu, kUpper0 = 0x26190D01u, kUpper1 = 0x71594535u;
    constexpr uint32_t kPlaces = 0x03020100u;  // byte k of the lower half's values; 4 + k, of the upper half's
    const uint32_t sel_lo = w & 0x07070707u;
    const uint32_t sel_hi = (w >> 4) & 0x07070707u;
    const uint32_t lower_lo = __builtin_amdgcn_perm(kLower1, kLower0, sel_lo);
    const uint32_t upper_lo = __builtin_amdgcn_perm(kUpper1, kUpper0, sel_lo);
    const uint32_t lower_hi = __builtin_amdgcn_perm(kLower1, kLower0, sel_hi);
    const uint32_t upper_hi = __builtin_amdgcn_perm(kUpper1, kUpper0, sel_hi);
    lo = __builtin_amdgcn_perm(upper_lo, lower_lo, Merge(0x04040404u, w >> 1, kPlaces));
    hi = __builtin_amdgcn_perm(upper_hi, lower_hi, Merge(0x04040404u, w >> 5, kPlaces));
  }

  // The unit at `at` (LDS) times the staged tokens: a pair of blocks (nine dwords) at a time, each pair used by
  // every token before the next is read. The dwords that hold a block's scale decode to values that meet the
  // images' zeros.
  template <int P, bool kDump>
  static __device__ __forceinline__ void DotAt(const uint8_t* at, const uint8_t* records, int token_stride, int m,
                                               float (&out)[P], int32_t* dump) {
#pragma clang fp contract(off)
    float v[P];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      __builtin_amdgcn_sched_barrier(0);
      const uint32_t* pair = reinterpret_cast<const uint32_t*>(at) + 9 * p;
      uint32_t word[9];
#pragma unroll
      for (int i = 0; i < 9; ++i) word[i] = pair[i];
      const float dw_even = HalfBitsToFloat(word[0] & 0xFFFFu), dw_odd = HalfBitsToFloat(word[4] >> 16);
      int even[P], odd[P];
#pragma unroll
      for (int t = 0; t < P; ++t) even[t] = 0, odd[t] = 0;
      // The low nibbles against the first image, then the high ones against the second: nine decoded dwords
      // live at a time, whatever the number of tokens.
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        uint32_t values[9];
#pragma unroll
        for (int i = 0; i < 9; ++i) {
          uint32_t lo, hi;
          Decode(word[i], lo, hi);
          values[i] = half ? hi : lo;
        }
#pragma unroll
        for (int t = 0; t < P; ++t) {
          if (t < m) {
            const uint32_t* image = reinterpret_cast<const uint32_t*>(records + t * token_stride + half * 144) + 9 * p;
#pragma unroll
            for (int i = 0; i < 9; ++i) {
              int& s = i >= 5 ? odd[t] : even[t];
              s = Dot4(static_cast<int>(values[i]), static_cast<int>(image[i]), s);
            }
            asm volatile("" : "+v"(even[t]), "+v"(odd[t]));  // taken here: the products stay with their pair
          }
        }
      }
#pragma unroll
      for (int t = 0; t < P; ++t) {
        if (t < m) {
          const uint8_t* record = records + t * token_stride;
          if (kDump && dump != nullptr) dump[2 * p] = even[t], dump[2 * p + 1] = odd[t];
          const float2 d8 = *reinterpret_cast<const float2*>(record + 288 + 8 * p);
          const float term_even = (dw_even * d8.x) * static_cast<float>(even[t]);
          const float term_odd = (dw_odd * d8.y) * static_cast<float>(odd[t]);
          v[t] = p == 0 ? term_even : v[t] + term_even;
          v[t] = v[t] + term_odd;
        }
      }
    }
#pragma unroll
    for (int t = 0; t < P; ++t) {
      if (t < m) out[t] = v[t];
    }
  }
};

// ---- Q4_1, Q5_0, Q5_1: a unit is eight blocks of {f16 d; [f16 m;] [u32 high bits;] u8 nibbles[16]}
//
// tests/unit/dsv4_fast_test.cc:141-164 of the reference: code i is the low (i < 16) or high
// nibble of byte i % 16, plus 16 where bit i of the high bits is set; a block times a Q8_1 block
// is dw * (sum * d8 - 16 * s8) (Q5_0), or sum * f16(dw * d8) + f16(m * s8) for the affine types.
// As for Q4_0 the staged activations are two images of the unit's byte layout with zeros
// wherever the unit holds something else than nibbles (no dword holds nibbles of two blocks:
// at least two header bytes lie between), and for the five-bit types the blocks' codes in
// plain order as well, against the expanded high bits.
template <int T>
struct FormatLegacy {
  static constexpr bool kAffine = T == 3 || T == 7;
  static constexpr bool kFive = T == 6 || T == 7;
  static constexpr int kPrefix = kAffine ? 4 : 2;
  static constexpr int kCodesAt = kPrefix + (kFive ? 4 : 0);
  static constexpr int kBlockBytes = kCodesAt + 16;
  static constexpr int kBlockValues = 32;
  static constexpr int kUnitBytes = 8 * kBlockBytes;
  static constexpr int kUnitValues = 256;
  static constexpr int kDwords = kUnitBytes / 4;
  static constexpr int kScalesAt = 2 * kUnitBytes;  // eight d8, eight s8
  // Eight more bytes put the records of a row's first sixteen units in different LDS banks
  // (98, 106 and 114 dwords apart; read 4 or 8 bytes at a time).
  static constexpr int kRecord = kScalesAt + 64 + 8;
  static constexpr int kDumpInts = 8;

  // The block whose nibbles dword i of a unit holds, or -1.
  static constexpr int Owner(int i) {
    for (int j = 0; j < 8; ++j) {
      const int first = j * kBlockBytes + kCodesAt;
      if (4 * i + 3 >= first && 4 * i < first + 16) return j;
    }
    return -1;
  }

  // One block of 32 values, eight lanes, four values a lane: lanes 0-3 hold values 0-15 (the low
  // image), lanes 4-7 values 16-31 (the high image); each image's first lane zeroes the header.
  static __device__ __forceinline__ void StageX(const float (&v)[4], int b, uint8_t* token) {
    const int lane8 = threadIdx.x & 7;
    const Q8Block q = QuantizeQ8Block(v[0], v[1], v[2], v[3]);
    uint8_t* record = token + (b >> 3) * kRecord;
    const int j = b & 7;
    uint8_t* image = record + (lane8 >> 2) * kUnitBytes + j * kBlockBytes;
    uint16_t* at = reinterpret_cast<uint16_t*>(image + kCodesAt + 4 * (lane8 & 3));
    at[0] = static_cast<uint16_t>(q.codes & 0xFFFFu);
    at[1] = static_cast<uint16_t>(q.codes >> 16);
    if ((lane8 & 3) == 0) {
#pragma unroll
      for (int i = 0; i < kCodesAt / 2; ++i) reinterpret_cast<uint16_t*>(image)[i] = 0;
    }
    if (lane8 == 0) {
      reinterpret_cast<float*>(record + kScalesAt)[j] = HalfBitsToFloat(FloatToHalfBits(q.d));
      reinterpret_cast<float*>(record + kScalesAt + 32)[j] = HalfBitsToFloat(FloatToHalfBits(q.sum));
    }
  }

  // One Q8_1 block (nine dwords), one thread: the dwords of both images that start within the
  // block's bytes (a dword that starts in the block before belongs to that block's thread).
  static __device__ __forceinline__ void StageQ8(const uint32_t (&w)[9], int b, uint8_t* token) {
    uint8_t* record = token + (b >> 3) * kRecord;
    const int j = b & 7;
    const int start = j * kBlockBytes;
    const int codes = start + kCodesAt;
    auto value = [&](int v) { return (w[1 + (v >> 2)] >> (8 * (v & 3))) & 0xFFu; };  // v 0 .. 31
#pragma unroll
    for (int i = 0; i < (kBlockBytes + 3) / 4 + 1; ++i) {
      const int at = ((start + 3) & ~3) + 4 * i;  // the dword's first byte
      if (at < start + kBlockBytes) {
        uint32_t lo = 0, hi = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int v = at + k - codes;
          if (v >= 0 && v < 16) {
            lo |= value(v) << (8 * k);
            hi |= value(16 + v) << (8 * k);
          }
        }
        *reinterpret_cast<uint32_t*>(record + at) = lo;
        *reinterpret_cast<uint32_t*>(record + kUnitBytes + at) = hi;
      }
    }
    reinterpret_cast<float*>(record + kScalesAt)[j] = HalfBitsToFloat(w[0] & 0xFFFFu);
    reinterpret_cast<float*>(record + kScalesAt + 32)[j] = HalfBitsToFloat(w[0] >> 16);
  }

  // Sixteen high bits (of values 0-15 or 16-31 of block j) as the bytes of 0 or 1 that face
  // dword i of the unit's image: value v sits at byte first + v of the unit, so the dword's four
  // bytes take bits 4 k - shift .. of them, k the dword's place among the block's code dwords.
  // Four bits spread to four bytes by a multiply: bit b of the nibble lands on bit 8 b.
  static __device__ __forceinline__ uint32_t RaisedMask(uint32_t sixteen, int j, int i) {
    const int first = j * kBlockBytes + kCodesAt;
    const int k = i - first / 4, shift = first % 4;
    return __umul24(((sixteen << shift) >> (4 * k)) & 15u, 0x204081u) & 0x01010101u;
  }

  // The 16 bits at byte `at` (even) of the unit's dwords.
  static __device__ __forceinline__ uint32_t HalfAt(const uint32_t (&w)[kDwords], int at) {
    return (at & 2) ? w[at >> 2] >> 16 : w[at >> 2] & 0xFFFFu;
  }

  // The unit at `at` (LDS) times the staged tokens.
  template <int P, bool kDump>
  static __device__ __forceinline__ void DotAt(const uint8_t* at, const uint8_t* records, int token_stride, int m,
                                               float (&out)[P], int32_t* dump) {
#pragma clang fp contract(off)
    if constexpr (P > 1 || T == 6) {
      // A block at a time, each used by every token before the next is read: the whole unit's
      // nibbles and several tokens' images do not fit the registers (nor one token's with
      // Q5_0's misaligned halves). The same operations in the same order as below.
      float v[P];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if constexpr (P > 1) __builtin_amdgcn_sched_barrier(0);
        constexpr int kSpan = (kBlockBytes + 3) / 4 + 1;  // dwords a block's bytes touch, at most
        const int first = j * kBlockBytes / 4;
        const int count = ((j + 1) * kBlockBytes + 3) / 4 - first;
        uint32_t bw[kSpan];
#pragma unroll
        for (int i = 0; i < kSpan; ++i) bw[i] = i < count ? reinterpret_cast<const uint32_t*>(at)[first + i] : 0u;
        auto half_at = [&](int byte) {  // the 16 bits at byte `byte` (even) of the unit
          const int local = byte - 4 * first;
          return (local & 2) ? bw[local >> 2] >> 16 : bw[local >> 2] & 0xFFFFu;
        };
        const float dw = HalfBitsToFloat(half_at(j * kBlockBytes));
        const float mw = kAffine ? HalfBitsToFloat(half_at(j * kBlockBytes + 2)) : 0.0f;
        uint32_t bits = 0;
        if constexpr (kFive) bits = half_at(j * kBlockBytes + kPrefix) | (half_at(j * kBlockBytes + kPrefix + 2) << 16);
#pragma unroll
        for (int t = 0; t < P; ++t) {
          if (t < m) {
            const uint8_t* record = records + t * token_stride;
            const uint32_t* low = reinterpret_cast<const uint32_t*>(record);
            const uint32_t* high = reinterpret_cast<const uint32_t*>(record + kUnitBytes);
            int sum = 0, raised = 0;
#pragma unroll
            for (int i = 0; i < kSpan; ++i) {
              if (i < count && Owner(first + i) == j) {
                const int lo = static_cast<int>(low[first + i]), hi = static_cast<int>(high[first + i]);
                sum = Dot4(static_cast<int>(bw[i] & 0x0F0F0F0Fu), lo, sum);
                sum = Dot4(static_cast<int>((bw[i] >> 4) & 0x0F0F0F0Fu), hi, sum);
                if constexpr (kFive) {
                  raised = Dot4(static_cast<int>(RaisedMask(bits & 0xFFFFu, j, first + i)), lo, raised);
                  raised = Dot4(static_cast<int>(RaisedMask(bits >> 16, j, first + i)), hi, raised);
                }
              }
            }
            sum += 16 * raised;
            asm volatile("" : "+v"(sum));  // taken here: the products stay with their block
            if (kDump && dump != nullptr) dump[j] = sum;
            const float d8 = reinterpret_cast<const float*>(record + kScalesAt)[j];
            const float s8 = reinterpret_cast<const float*>(record + kScalesAt + 32)[j];
            float term;
            if constexpr (kAffine) {
              const float scale = HalfBitsToFloat(FloatToHalfBits(dw * d8));
              const float minimum = HalfBitsToFloat(FloatToHalfBits(mw * s8));
              term = static_cast<float>(sum) * scale + minimum;
            } else {
              term = dw * (static_cast<float>(sum) * d8 - 16.0f * s8);
            }
            v[t] = j == 0 ? term : v[t] + term;
          }
        }
      }
#pragma unroll
      for (int t = 0; t < P; ++t) {
        if (t < m) out[t] = v[t];
      }
      return;
    }
    const U32x4* mine = reinterpret_cast<const U32x4*>(at);
    uint32_t w[kDwords];
#pragma unroll
    for (int i = 0; i < kDwords / 4; ++i) {
      const U32x4 v = mine[i];
      w[4 * i] = v.x, w[4 * i + 1] = v.y, w[4 * i + 2] = v.z, w[4 * i + 3] = v.w;
    }
#pragma unroll
    for (int t = 0; t < P; ++t) {
      if (t < m) {
        const uint8_t* record = records + t * token_stride;
        const uint2* low = reinterpret_cast<const uint2*>(record);
        const uint2* high = reinterpret_cast<const uint2*>(record + kUnitBytes);
        int s[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        int raised[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        uint2 low2 = {0, 0}, high2 = {0, 0};
#pragma unroll
        for (int i = 0; i < kDwords; ++i) {
          constexpr int kNone = -1;
          const int owner = Owner(i);
          if ((i & 1) == 0) low2 = low[i >> 1], high2 = high[i >> 1];
          if (owner != kNone) {
            const int lo = static_cast<int>((i & 1) ? low2.y : low2.x), hi = static_cast<int>((i & 1) ? high2.y : high2.x);
            s[owner] = Dot4(static_cast<int>(w[i] & 0x0F0F0F0Fu), lo, s[owner]);
            s[owner] = Dot4(static_cast<int>((w[i] >> 4) & 0x0F0F0F0Fu), hi, s[owner]);
            if constexpr (kFive) {
              const int at_bits = owner * kBlockBytes + kPrefix;
              raised[owner] = Dot4(static_cast<int>(RaisedMask(HalfAt(w, at_bits), owner, i)), lo, raised[owner]);
              raised[owner] = Dot4(static_cast<int>(RaisedMask(HalfAt(w, at_bits + 2), owner, i)), hi, raised[owner]);
            }
          }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) s[j] += 16 * raised[j];
        if (kDump && dump != nullptr) {
#pragma unroll
          for (int j = 0; j < 8; ++j) dump[j] = s[j];
        }
        const float* d8 = reinterpret_cast<const float*>(record + kScalesAt);
        const float* s8 = d8 + 8;
        float v = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float dw = HalfBitsToFloat(HalfAt(w, j * kBlockBytes));
          float term;
          if constexpr (kAffine) {
            const float mw = HalfBitsToFloat(HalfAt(w, j * kBlockBytes + 2));
            const float scale = HalfBitsToFloat(FloatToHalfBits(dw * d8[j]));
            const float minimum = HalfBitsToFloat(FloatToHalfBits(mw * s8[j]));
            term = static_cast<float>(s[j]) * scale + minimum;
          } else {
            term = dw * (static_cast<float>(s[j]) * d8[j] - 16.0f * s8[j]);
          }
          v = j == 0 ? term : v + term;
        }
        out[t] = v;
      }
    }
  }
};

using FormatQ41 = FormatLegacy<3>;
using FormatQ50 = FormatLegacy<6>;
using FormatQ51 = FormatLegacy<7>;

// ---- MXFP4: a unit is eight blocks of {e8m0 e; u8 nibbles[16]} (136 bytes, 256 values)
//
// src/kernels/reference/decode.cc:239-248 and 417-428 of the reference: value i of a block is
// the E2M1 value of the low (i < 16) or high nibble of byte 1 + i % 16, times 2^(e - 127), a
// scale byte of 0xFF making the block NaN; src/kernels/ggml/vecq.cu:421-437: a block times a
// Q8_1 block is (2^(e - 127) / 2 * d8) * sum(twice the E2M1 values * q). The staged activations
// are two images of the unit's bytes as for the other four-bit blocks, zeros where the scale
// bytes lie. A block is 17 bytes, so four of a unit's 34 dwords hold codes of two blocks: their
// decoded values go to either block's sum under a byte mask.
struct FormatMxfp4 {
  static constexpr int kUnitBytes = 136;
  static constexpr int kUnitValues = 256;
  static constexpr int kBlockBytes = 17;
  static constexpr int kBlockValues = 32;
  static constexpr int kDwords = 34;
  static constexpr int kImage = 144;  // the unit's 136 bytes, read sixteen at a time
  static constexpr int kScalesAt = 2 * kImage;
  // Two images, eight d8, and eight bytes so that the 16 records a 16-unit row's lanes read lie
  // in different LDS banks (82 dwords apart).
  static constexpr int kRecord = kScalesAt + 32 + 8;
  static constexpr int kDumpInts = 8;

  // The bytes of dword i that are codes of block j, as a mask.
  static constexpr uint32_t CodeMask(int i, int j) {
    uint32_t m = 0;
    for (int k = 0; k < 4; ++k) {
      const int at = 4 * i + k;
      if (at % 17 != 0 && at / 17 == j) m |= 0xFFu << (8 * k);
    }
    return m;
  }

  // Eight codes of a dword as twice their E2M1 values, int8: the low nibbles' four and the high
  // nibbles' four. Magnitudes {0, 1, 2, 3, 4, 6, 8, 12} by the code's low three bits, from the
  // positive and the negative table; the code's fourth bit picks between the two, byte by byte.
  // (a & mask) | (b & ~mask) in one instruction.
  static __device__ __forceinline__ uint32_t Merge(uint32_t mask, uint32_t a, uint32_t b) {
    uint32_t r;
    asm("v_bfi_b32 %0, %1, %2, %3" : "=v"(r) : "s"(mask), "v"(a), "v"(b));
    return r;
  }
  static __device__ __forceinline__ void Decode(uint32_t w, uint32_t& lo, uint32_t& hi) {
    constexpr uint32_t kPosLow = 0x03020100u, kPosHigh = 0x0C080604u;
    constexpr uint32_t kNegLow = 0xFDFEFF00u, kNegHigh = 0xF4F8FAFCu;
    constexpr uint32_t kPlaces = 0x03020100u;  // byte k of the positive values; 4 + k, of the negative
    const uint32_t sel_lo = w & 0x07070707u;
    const uint32_t sel_hi = (w >> 4) & 0x07070707u;
    const uint32_t pos_lo = __builtin_amdgcn_perm(kPosHigh, kPosLow, sel_lo);
    const uint32_t neg_lo = __builtin_amdgcn_perm(kNegHigh, kNegLow, sel_lo);
    const uint32_t pos_hi = __builtin_amdgcn_perm(kPosHigh, kPosLow, sel_hi);
    const uint32_t neg_hi = __builtin_amdgcn_perm(kNegHigh, kNegLow, sel_hi);
    lo = __builtin_amdgcn_perm(neg_lo, pos_lo, Merge(0x04040404u, w >> 1, kPlaces));
    hi = __builtin_amdgcn_perm(neg_hi, pos_hi, Merge(0x04040404u, w >> 5, kPlaces));
  }

  // Half the block's scale, 2^(e - 128): NaN for 0xFF, subnormal for 0 and 1.
  static __device__ __forceinline__ float HalfScale(uint32_t e) {
    const uint32_t bits = e == 0xFFu ? 0x7FC00000u : e < 2u ? 0x00200000u << e : (e - 1u) << 23;
    return __uint_as_float(bits);
  }

  // One block of 32 values, eight lanes, four values a lane: lanes 0-3 hold values 0-15 (the low
  // image), lanes 4-7 values 16-31 (the high image); each image's first lane zeroes the byte
  // that faces the scale.
  static __device__ __forceinline__ void StageX(const float (&v)[4], int b, uint8_t* token) {
    const int lane8 = threadIdx.x & 7;
    const Q8Block q = QuantizeQ8Block(v[0], v[1], v[2], v[3]);
    uint8_t* record = token + (b >> 3) * kRecord;
    const int j = b & 7;
    uint8_t* image = record + (lane8 >> 2) * kImage + 17 * j;
    uint8_t* at = image + 1 + 4 * (lane8 & 3);
#pragma unroll
    for (int i = 0; i < 4; ++i) at[i] = static_cast<uint8_t>(q.codes >> (8 * i));
    if ((lane8 & 3) == 0) image[0] = 0;
    if (lane8 == 0) reinterpret_cast<float*>(record + kScalesAt)[j] = HalfBitsToFloat(FloatToHalfBits(q.d));
  }

  // One Q8_1 block (nine dwords), one thread: sixteen codes into either image from byte
  // 17 j + 1 on. The three dwords that always lie within the block whole; its first three and
  // last four bytes one by one (the dwords there are shared with the neighbouring blocks'
  // threads), whichever of them the dwords covered already: no branches.
  static __device__ __forceinline__ void StageQ8(const uint32_t (&w)[9], int b, uint8_t* token) {
    uint8_t* record = token + (b >> 3) * kRecord;
    const int j = b & 7;
    const int first = 17 * j + 1;
    const int lead = (4 - (first & 3)) & 3;  // bytes before the first whole dword
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      uint8_t* image = record + half * kImage;
      const uint32_t* c = w + 1 + 4 * half;  // the sixteen codes of this half
      image[first - 1] = 0;
#pragma unroll
      for (int v = 0; v < 3; ++v) image[first + v] = static_cast<uint8_t>(c[0] >> (8 * v));
#pragma unroll
      for (int i = 0; i < 3; ++i)
        *reinterpret_cast<uint32_t*>(image + first + lead + 4 * i) = __builtin_amdgcn_alignbyte(c[i + 1], c[i], lead);
#pragma unroll
      for (int v = 0; v < 4; ++v) image[first + 12 + v] = static_cast<uint8_t>(c[3] >> (8 * v));
    }
    reinterpret_cast<float*>(record + kScalesAt)[j] = HalfBitsToFloat(w[0] & 0xFFFFu);
  }

  // Every code byte of dword i, whatever its block.
  static constexpr uint32_t Codes(int i) {
    uint32_t m = 0;
    for (int j = 0; j < 8; ++j) m |= CodeMask(i, j);
    return m;
  }

  // The unit at `at` (LDS) times the staged tokens: a pair of blocks (34 bytes, within nine
  // dwords) at a time, each pair decoded once and used by every token. A pair's first or last
  // dword also holds bytes of the pair beside it: the byte masks keep them apart.
  template <int P, bool kDump>
  static __device__ __forceinline__ void DotAt(const uint8_t* at, const uint8_t* records, int token_stride, int m,
                                               float (&out)[P], int32_t* dump) {
#pragma clang fp contract(off)
    float v[P];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      __builtin_amdgcn_sched_barrier(0);
      // The pair's nine dwords begin at dword `first`; they are read eight bytes at a time from
      // the even dword at or before it (conflict-free in LDS), units and images alike.
      const int first = 34 * p / 4, from = first & ~1, skip = first - from;
      const uint2* mine = reinterpret_cast<const uint2*>(at) + from / 2;
      uint32_t lo[9], hi[9];
      float scale[2] = {0.0f, 0.0f};
      {
        uint32_t w[10];
#pragma unroll
        for (int i = 0; i < 5; ++i) {
          const uint2 v = mine[i];
          w[2 * i] = v.x, w[2 * i + 1] = v.y;
        }
#pragma unroll
        for (int i = 0; i < 9; ++i) {
          Decode(w[skip + i], lo[i], hi[i]);
#pragma unroll
          for (int jj = 0; jj < 2; ++jj) {
            const int header = 17 * (2 * p + jj);
            if (header / 4 == first + i) scale[jj] = HalfScale((w[skip + i] >> (8 * (header % 4))) & 0xFFu);
          }
        }
      }
#pragma unroll
      for (int t = 0; t < P; ++t) {
        if (t < m) {
          const uint8_t* record = records + t * token_stride;
          const uint2* low2 = reinterpret_cast<const uint2*>(record) + from / 2;
          const uint2* high2 = reinterpret_cast<const uint2*>(record + kImage) + from / 2;
          uint32_t low[10], high[10];
#pragma unroll
          for (int i = 0; i < 5; ++i) {
            const uint2 a = low2[i], b = high2[i];
            low[2 * i] = a.x, low[2 * i + 1] = a.y, high[2 * i] = b.x, high[2 * i + 1] = b.y;
          }
          int s[2] = {0, 0};
#pragma unroll
          for (int i = 0; i < 9; ++i) {
            const int a = static_cast<int>(low[skip + i]), b = static_cast<int>(high[skip + i]);
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
              const uint32_t mask = CodeMask(first + i, 2 * p + jj);
              if (mask == 0) continue;
              const bool whole = mask == Codes(first + i);
              s[jj] = Dot4(static_cast<int>(whole ? lo[i] : lo[i] & mask), a, s[jj]);
              s[jj] = Dot4(static_cast<int>(whole ? hi[i] : hi[i] & mask), b, s[jj]);
            }
          }
          // The sums are taken here, not wherever they are first needed: otherwise the compiler
          // moves every pair's products to the end and keeps all their operands until then.
          asm volatile("" : "+v"(s[0]), "+v"(s[1]));
          if (kDump && dump != nullptr) dump[2 * p] = s[0], dump[2 * p + 1] = s[1];
          const float2 d8 = *reinterpret_cast<const float2*>(record + kScalesAt + 8 * p);
          const float even = (scale[0] * d8.x) * static_cast<float>(s[0]);
          const float odd = (scale[1] * d8.y) * static_cast<float>(s[1]);
          v[t] = p == 0 ? even : v[t] + even;
          v[t] = v[t] + odd;
        }
      }
    }
#pragma unroll
    for (int t = 0; t < P; ++t) {
      if (t < m) out[t] = v[t];
    }
  }
};

// ---- staging a token's row into records

template <class F, int XT>
__device__ __forceinline__ void StageRecordsX(const void* __restrict__ x, int k, const FrontX& front, uint8_t* token) {
  const int lane8 = threadIdx.x & 7;
  const int blocks = k / 32;
  const bool wide = reinterpret_cast<uintptr_t>(x) % (XT == LLMP_X_F32 ? 16 : 8) == 0;
  const int sweep = blockDim.x >> 3;
#pragma unroll
  for (int i = 0; i < kFront; ++i) {
    const int b = (threadIdx.x >> 3) + i * sweep;
    if (b < blocks) F::StageX(front.v[i], b, token);  // whole 8-lane groups together
  }
  for (int b = (threadIdx.x >> 3) + kFront * sweep; b < blocks; b += sweep) {
    float v[4];
    Load4Wide<XT>(x, static_cast<int64_t>(b) * 32 + lane8 * 4, k, wide, v);
    F::StageX(v, b, token);
  }
}

template <class F, class = void>
struct StagesXUnderLoads : std::false_type {};
template <class F>
struct StagesXUnderLoads<F, std::void_t<decltype(F::kStagesXUnderLoads)>> : std::bool_constant<F::kStagesXUnderLoads> {};

// The front pieces quantized and their records written by instructions; every block of the row is a front block
// (the launcher sees to it).
template <class F, int XT>
__device__ __forceinline__ void StageRecordsXAsm(const FrontXAsm<XT>& front, int k, uint8_t* token) {
  const int blocks = k / 32;
  const int sweep = blockDim.x >> 3;
#pragma unroll
  for (int i = 0; i < kFront; ++i) {
    const int b = (threadIdx.x >> 3) + i * sweep;
    if (b < blocks) {  // whole 8-lane groups together
      float v[4];
      FrontValues<XT>(front, i, v);
      F::StageXAsm(v, b, token);
    }
  }
}

// Formats whose records of Q8_1 activations are staged by instructions, under the first tile's loads.
template <class F, class = void>
struct StagesUnderLoads : std::false_type {};
template <class F>
struct StagesUnderLoads<F, std::void_t<decltype(F::kStagesUnderLoads)>> : std::bool_constant<F::kStagesUnderLoads> {};

// The front block by instructions; the row's further blocks (rows of more blocks than the workgroup has threads)
// as the compiler orders them.
template <class F>
__device__ __forceinline__ void StageRecordsQ8Asm(const uint8_t* __restrict__ y, int blocks, const FrontQ8Asm& front,
                                                  uint8_t* token) {
  if (static_cast<int>(threadIdx.x) < blocks) F::StageQ8Asm(front, threadIdx.x, token);
  for (int b = threadIdx.x + blockDim.x; b < blocks; b += blockDim.x) {
    const uint32_t* src = reinterpret_cast<const uint32_t*>(y + static_cast<int64_t>(b) * kQ8Block);
    uint32_t w[9];
#pragma unroll
    for (int i = 0; i < 9; ++i) w[i] = src[i];
    F::StageQ8(w, b, token);
  }
}

template <class F>
__device__ __forceinline__ void StageRecordsQ8(const uint8_t* __restrict__ y, int blocks, const FrontQ8& front,
                                               uint8_t* token) {
  if (static_cast<int>(threadIdx.x) < blocks) F::StageQ8(front.w, threadIdx.x, token);
  for (int b = threadIdx.x + blockDim.x; b < blocks; b += blockDim.x) {
    const uint32_t* src = reinterpret_cast<const uint32_t*>(y + static_cast<int64_t>(b) * kQ8Block);
    uint32_t w[9];
#pragma unroll
    for (int i = 0; i < 9; ++i) w[i] = src[i];
    F::StageQ8(w, b, token);
  }
}

typedef __attribute__((address_space(3))) void* LdsPointer;
typedef const __attribute__((address_space(1))) void* GlobalPointer;

// Queues one matrix's part of a tile into the wave's buffer at `ring`: chunk c = 64 j + lane
// of `chunks` lands at byte 16 c. `base` and `ring` are the same in every lane.
// kPacked: rows follow each other without a gap, so the part is one byte range; else a row's
// bytes (a whole number of chunks) are `row_bytes` of every `stride_bytes`.
// The same value in every lane, and known to the compiler as such: a pointer that came
// through LDS or a per-lane load otherwise costs two vector registers wherever it is used.
__device__ __forceinline__ const uint8_t* Uniform(const uint8_t* p) {
  const uint64_t bits = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bits));
  const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bits >> 32));
  return reinterpret_cast<const uint8_t*>((static_cast<uint64_t>(hi) << 32) | lo);
}

template <int kLoads, bool kPacked>
__device__ __forceinline__ void FetchPart(const uint8_t* base, int chunks, int64_t stride_bytes, int row_bytes,
                                          uint8_t* ring, int lane) {
  base = Uniform(base);
#pragma unroll
  for (int j = 0; j < kLoads; ++j) {
    const int c = j * kWave + lane;
    if (j * kWave < chunks && lane < chunks - j * kWave) {  // a load is issued exactly when some lane has a chunk
      const uint8_t* from;
      if constexpr (kPacked) {
        // The load's base in scalar registers, the lane's sixteen bytes the same register for
        // every load (hidden from the compiler here, or it keeps an address a load alive
        // across the whole tile loop).
        uint32_t mine = static_cast<uint32_t>(lane) * 16u;
        asm volatile("" : "+v"(mine));
        from = base + j * (kWave * 16) + mine;
      } else {
        const int byte = c * 16;
        const int row = byte / row_bytes;
        from = base + row * stride_bytes + (byte - row * row_bytes);
      }
      __builtin_amdgcn_global_load_lds((GlobalPointer)from, (LdsPointer)(ring + j * kWave * 16), 16, 0, 0);
    }
  }
}

// Where a tile's first byte lies in its buffer: 0 unless the format's units are not whole 16-byte chunks.
template <class F>
__device__ __forceinline__ int TileShift(const llmp_vecq_desc& d, int64_t expert_block, int row0) {
  if constexpr (F::kUnitBytes % 16 != 0) {
    return static_cast<int>(((expert_block + static_cast<int64_t>(row0) * d.stride_row) * F::kBlockBytes) & 15);
  } else {
    return 0;
  }
}

// The tile of `rows` rows from `row0`. A matrix's part always starts where a full tile's
// would (`gate_at` bytes into the buffer), so a lane's place in a tile never changes.
template <class F, bool kGlu, bool kPacked>
__device__ __forceinline__ void FetchTile(const llmp_vecq_desc& d, int64_t expert_block, int row0, int rows, int units,
                                          int gate_at, uint8_t* ring, int lane) {
  int64_t first = (expert_block + static_cast<int64_t>(row0) * d.stride_row) * F::kBlockBytes;
  const int row_bytes = units * F::kUnitBytes;
  // Units that are not whole chunks (packed rows): the tile is fetched from the 16-byte boundary below its first
  // byte and lies that many bytes into the buffer (TileShift); its last chunk ends within the matrix, whose rows'
  // blocks are a multiple of eight.
  int shift = 0;
  if constexpr (F::kUnitBytes % 16 != 0) {
    shift = static_cast<int>(first & 15);
    first -= shift;
  }
  const int chunks = (shift + rows * row_bytes + 15) / 16;
  const int64_t stride_bytes = static_cast<int64_t>(d.stride_row) * F::kBlockBytes;
  // The loads (1 KB a wave each) of a part: at most 32 units a matrix with a GLU, else 64.
  constexpr int kLoads = ((kGlu ? kWave / 2 : kWave) * F::kUnitBytes + 1023) / 1024;
  if constexpr (kGlu) {
    FetchPart<kLoads, kPacked>(static_cast<const uint8_t*>(d.w) + first, chunks, stride_bytes, row_bytes, ring, lane);
    FetchPart<kLoads, kPacked>(static_cast<const uint8_t*>(d.g) + first, chunks, stride_bytes, row_bytes,
                               ring + gate_at, lane);
  } else {
    FetchPart<kLoads, kPacked>(static_cast<const uint8_t*>(d.w) + first, chunks, stride_bytes, row_bytes, ring, lane);
  }
}

// The tile has landed: all of this wave's memory operations are complete.
__device__ __forceinline__ void AwaitTile() {
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
  __builtin_amdgcn_wave_barrier();
  asm volatile("" ::: "memory");
}

// The loads FetchTile issues for a tile of `rows` rows: one for every 64 chunks of a part.
template <class F, bool kGlu>
__device__ __forceinline__ int TileLoads(int rows, int units) {
  const int chunks = rows * units * F::kUnitBytes / 16;
  constexpr int kLoads = ((kGlu ? kWave / 2 : kWave) * F::kUnitBytes + 1023) / 1024;
  const int part = min((chunks + kWave - 1) / kWave, kLoads);
  return kGlu ? 2 * part : part;
}

// All but this wave's `left` latest memory operations are complete (0 to 10; the same in
// every lane).
__device__ __forceinline__ void AwaitAllBut(int left) {
  switch (left) {
    case 0: __builtin_amdgcn_s_waitcnt(0x0F70); break;
    case 1: __builtin_amdgcn_s_waitcnt(0x0F71); break;
    case 2: __builtin_amdgcn_s_waitcnt(0x0F72); break;
    case 3: __builtin_amdgcn_s_waitcnt(0x0F73); break;
    case 4: __builtin_amdgcn_s_waitcnt(0x0F74); break;
    case 5: __builtin_amdgcn_s_waitcnt(0x0F75); break;
    case 6: __builtin_amdgcn_s_waitcnt(0x0F76); break;
    case 7: __builtin_amdgcn_s_waitcnt(0x0F77); break;
    case 8: __builtin_amdgcn_s_waitcnt(0x0F78); break;
    case 9: __builtin_amdgcn_s_waitcnt(0x0F79); break;
    default: __builtin_amdgcn_s_waitcnt(0x0F7A); break;
  }
  __builtin_amdgcn_wave_barrier();
  asm volatile("" ::: "memory");
}

// grid (workgroups, slots); LDS: P tokens' records, then a tile buffer a wave.
// kUnder (1 or 2): the activations' records are staged under the first tile's loads: the activations loaded and
// the records written by instructions, and with 1 a barrier for LDS alone. Over Q8_1 activations it is for launches
// whose waves take one tile each: the launch is then one trip to memory, and the trip for the activations and their
// staging no longer stand in front of it and behind it; with two tiles a wave it measured slower (the gate/up pair
// 14.7 to 15.2 us against 14.2: there the waves do better entering the first products together). Over unquantized
// activations the staging is their quantization, some four hundred vector instructions a wave, and running it under
// the loads pays whatever the tiles a wave (the gate/up pair 16.5 -> 14.6-14.9 us; 2 keeps the full barrier).
template <class F, int P, bool kGlu, int XT, bool kDump, bool kPacked, bool kDeep, int kUnder = 0>
__global__ __launch_bounds__(kDeep ? kGroup : 2 * kGroup, kDeep ? 2 : 4) void VecQFlat(const VecQArgs a, const int rows_per_tile) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  __shared__ int pairs[kMaxPairs];
  __shared__ int count;

  const llmp_vecq_desc& d = a.d;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int nsb = d.ncols_x / F::kUnitValues;  // units a row
  const int token_stride = nsb * F::kRecord;
  const int tiles = (d.nrows + rows_per_tile - 1) / rows_per_tile;
  // kDeep: two tile buffers a wave (one workgroup a CU), the next tile in flight while this one
  // is multiplied.
  // (Units that are not whole chunks: room for the tile's shift, the gate part's own boundary and a lane's reads
  // past its unit.)
  constexpr bool kOdd = F::kUnitBytes % 16 != 0;
  constexpr int kTileBytes = kWave * F::kUnitBytes + (kOdd ? 80 : 0);
  // The tile buffers take 16-byte chunks: they start at the next 16-byte boundary after the records.
  // (A dense product of fewer tokens than a pass takes stages only those: more room for waves.)
  const int staged = a.offsets == nullptr && a.d.ids == nullptr && a.d.tokens < P ? a.d.tokens : P;
  uint8_t* ring = lds + ((staged * token_stride + 15) & ~15) + wave * ((kDeep ? 2 : 1) * kTileBytes);

  // A lane's place in every tile: its matrix, row and unit of the row.
  const int half = rows_per_tile * nsb;
  const bool gate_lane = kGlu && lane >= half;
  const int f = gate_lane ? lane - half : lane;
  const int row = f / nsb;
  const int sb = f - row * nsb;
  const bool placed = lane < (kGlu ? 2 * half : half);
  const int gate_at = kOdd ? ((half * F::kUnitBytes + 15) & ~15) + 32 : half * F::kUnitBytes;
  const uint8_t* my_block = ring + (gate_lane ? gate_at + f * F::kUnitBytes : lane * F::kUnitBytes);
  const uint8_t* my_records = lds + sb * F::kRecord;

  // A routed product's workgroup first learns whether it owns its expert; one over sorted
  // rows takes its expert's row range.
  int expert = blockIdx.y;
  int sorted_first = 0;
  int rank = 0, sharers = 1, routed_pairs = 0;
  if (a.offsets != nullptr) {
    sorted_first = a.offsets[expert];
    if (tid == 0) count = a.offsets[expert + 1] - sorted_first;
    __syncthreads();
    if (count == 0) return;  // uniform over the workgroup
  } else if (d.ids != nullptr) {
    // The pairs that name this pair's expert share its tiles: `count` pairs' workgroups, this pair's at `rank`.
    expert = SharePairs(d, blockIdx.y, pairs, &sharers, &rank);
    routed_pairs = sharers;
  }
  const int64_t expert_block = static_cast<int64_t>(expert) * d.stride_expert;
  const int waves = blockDim.x / kWave;  // eight, fewer where a long row's records leave less room
  const int first_tile = (rank * gridDim.x + blockIdx.x) * waves + wave;
  const int tile_step = sharers * gridDim.x * waves;
  // A dense or grouped product's pairs are its tokens on the workgroup's matrix: no list.
  const bool listed = d.ids != nullptr && a.offsets == nullptr;
  const int n = a.offsets != nullptr ? count : d.ids != nullptr ? routed_pairs : d.tokens;
  auto pair_at = [&](int i) {
    return a.offsets != nullptr ? (sorted_first + i) << 8 : listed ? pairs[i] : (i << 8) | expert;
  };

  for (int p0 = 0; p0 < n; p0 += P) {
    const int m = min(P, n - p0);
    if (p0 > 0) __syncthreads();  // the last pass's readers of the records
    // The activations' first loads, then the wave's first tile, then the staging.
    constexpr bool kAsmFront = kUnder != 0 && XT < 0;
    constexpr bool kAsmX = kUnder != 0 && XT >= 0;
    const void* rows_x[P];
    FrontX front_x[XT < 0 || kAsmX ? 1 : P];
    FrontXAsm<XT < 0 ? 0 : XT> front_xa[kAsmX ? P : 1];
    FrontQ8 front_q[XT < 0 && !kAsmFront ? P : 1];
    FrontQ8Asm front_a[kAsmFront ? P : 1];
#pragma unroll
    for (int j = 0; j < P; ++j) {
      if (j < m) {
        const int pr = pair_at(p0 + j);
        const int token = pr >> 8;
        const int slot = pr & 0xFF;
        if constexpr (XT < 0) {
          rows_x[j] = static_cast<const uint8_t*>(d.y) +
                      (static_cast<int64_t>(token) * d.y_token + static_cast<int64_t>(slot) * d.y_slot) * kQ8Block;
          if constexpr (kAsmFront) {
            front_a[j] = LoadFrontQ8Asm(static_cast<const uint8_t*>(rows_x[j]), d.ncols_x / 32);
          } else {
            front_q[j] = LoadFrontQ8(static_cast<const uint8_t*>(rows_x[j]), d.ncols_x / 32);
          }
        } else {
          const int64_t at = token * a.x_token + slot * a.x_slot;
          rows_x[j] = XT == LLMP_X_F32 ? static_cast<const void*>(static_cast<const float*>(a.x) + at)
                                       : static_cast<const void*>(static_cast<const uint16_t*>(a.x) + at);
          if constexpr (kAsmX) {
            front_xa[j] = LoadFrontXAsm<XT>(rows_x[j], d.ncols_x);
          } else {
            front_x[j] = LoadFrontX<XT>(rows_x[j], d.ncols_x);
          }
        }
      }
    }
    int index = first_tile;
    int tile_loads = 0;  // no more than the loads the first tile's fetch issues
    if (index < tiles) {
      const int row0 = index * rows_per_tile;
      FetchTile<F, kGlu, kPacked>(d, expert_block, row0, min(rows_per_tile, d.nrows - row0), nsb, gate_at, ring, lane);
      tile_loads = TileLoads<F, kGlu>(min(rows_per_tile, d.nrows - row0), nsb);
    }
    if constexpr (kAsmFront) {
      // The activations' blocks have landed once only the tile's loads, issued after them, are outstanding.
#pragma unroll
      for (int j = 0; j < P; ++j) {
        if (j < m) AwaitFront(front_a[j], tile_loads);
      }
    }
    if constexpr (kAsmX) {
#pragma unroll
      for (int j = 0; j < P; ++j) {
        if (j < m) AwaitFrontX(front_xa[j], tile_loads);
      }
    }
#pragma unroll
    for (int j = 0; j < P; ++j) {
      if (j < m) {
        uint8_t* records = lds + j * token_stride;
        if constexpr (kAsmFront) {
          StageRecordsQ8Asm<F>(static_cast<const uint8_t*>(rows_x[j]), d.ncols_x / 32, front_a[j], records);
        } else if constexpr (XT < 0) {
          StageRecordsQ8<F>(static_cast<const uint8_t*>(rows_x[j]), d.ncols_x / 32, front_q[j], records);
        } else if constexpr (kAsmX) {
          StageRecordsXAsm<F, XT>(front_xa[j], d.ncols_x, records);
        } else {
          StageRecordsX<F, XT>(rows_x[j], d.ncols_x, front_x[j], records);
        }
      }
    }
    // The records are staged; from here the waves run alone. (A barrier for LDS alone where the staging ran under
    // the tile's loads: __syncthreads would wait for those to land as well.)
    if constexpr (kUnder == 1) {
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_s_barrier();
    } else {
      __syncthreads();
    }

    int buffer = 0;  // kDeep: the tile buffer the tile `index` is in
    while (index < tiles) {
      const int row0 = index * rows_per_tile;
      const bool live = placed && row0 + row < d.nrows;
      const int next = index + tile_step;
      if constexpr (kDeep) {
        // The next tile into the other buffer, whose readers finished an iteration ago; then
        // wait for everything older than its loads: this tile, and the last one's stores.
        if (next < tiles) {
          const int next0 = next * rows_per_tile;
          const int rows = min(rows_per_tile, d.nrows - next0);
          FetchTile<F, kGlu, kPacked>(d, expert_block, next0, rows, nsb, gate_at, ring + (buffer ^ 1) * kTileBytes, lane);
          AwaitAllBut(TileLoads<F, kGlu>(rows, nsb));
        } else {
          AwaitTile();
        }
      } else {
        AwaitTile();
      }
      float out[P];
      if (live) {
        int32_t* dump = kDump ? a.dump + (static_cast<int64_t>(row0 + row) * nsb + sb) * F::kDumpInts : nullptr;
        F::template DotAt<P, kDump>(my_block + (kDeep ? buffer * kTileBytes : 0) + TileShift<F>(d, expert_block, row0),
                                    my_records, token_stride, m, out, dump);
      }
      // Row sums: a suffix sum over each row's lanes (a fixed tree), the total in the row's
      // first lane; a gate row's total then moves to its up row's lane.
#pragma unroll
      for (int t = 0; t < P; ++t) {
        if (t < m) {
          float v = live ? out[t] : 0.0f;
          for (int off = 1; off < nsb; off <<= 1) {
            const float other = __shfl_down(v, off, kWave);
            if (sb + off < nsb) v += other;
          }
          float gate = 0.0f;
          if constexpr (kGlu) gate = __shfl_down(v, half, kWave);
          if (live && !gate_lane && sb == 0) {
            const int pr = pair_at(p0 + t);
            float* dst =
                d.dst + static_cast<int64_t>(pr >> 8) * d.dst_token + static_cast<int64_t>(pr & 0xFF) * d.dst_slot;
            dst[row0 + row] = kGlu ? Glu(d.glu, gate, v, d.limit) : v;
          }
        }
      }
      index = next;
      if constexpr (kDeep) {
        buffer ^= 1;
        __builtin_amdgcn_wave_barrier();  // every lane has read its unit before the buffer is refilled
      } else if (index < tiles) {
        // The next tile may overwrite the buffer: every lane's reads of it were consumed above.
        // (Queueing these loads before the row sums measured slower.)
        const int next0 = index * rows_per_tile;
        FetchTile<F, kGlu, kPacked>(d, expert_block, next0, min(rows_per_tile, d.nrows - next0), nsb, gate_at, ring,
                                    lane);
      }
    }
  }
}

// Rows longer than a wave's 64 units: a row is cut into `split` pieces of `piece` units (the
// last may be shorter), a wave takes whole rows, a piece a tile, and each lane adds up its
// units' products over the pieces before the lanes are summed. One token a pass, no GLU.
// grid (workgroups, slots); LDS: the token's records, then a tile buffer a wave.
template <class F, int XT>
__global__ __launch_bounds__(kGroup, 4) void VecQFlatSplit(const VecQArgs a, const int split, const int piece) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  __shared__ int pairs[kMaxPairs];
  __shared__ int count;

  const llmp_vecq_desc& d = a.d;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int units = d.ncols_x / F::kUnitValues;
  const int token_stride = units * F::kRecord;
  uint8_t* ring = lds + ((token_stride + 15) & ~15) + wave * (kWave * F::kUnitBytes);
  const uint8_t* my_block = ring + lane * F::kUnitBytes;

  int expert = blockIdx.y;
  int sorted_first = 0;
  if (a.offsets != nullptr) {
    sorted_first = a.offsets[expert];
    if (tid == 0) count = a.offsets[expert + 1] - sorted_first;
    __syncthreads();
    if (count == 0) return;  // uniform over the workgroup
  } else if (d.ids != nullptr) {
    expert = ResolvePairs(d, blockIdx.y, pairs, &count);
    if (count == 0) return;  // uniform over the workgroup
  }
  const bool listed = d.ids != nullptr && a.offsets == nullptr;
  const int n = a.offsets == nullptr && d.ids == nullptr ? d.tokens : count;
  const uint8_t* matrix = Uniform(static_cast<const uint8_t*>(d.w) +
                                  static_cast<int64_t>(expert) * d.stride_expert * F::kBlockBytes);
  const int64_t row_bytes = static_cast<int64_t>(d.stride_row) * F::kBlockBytes;
  const int waves = blockDim.x / kWave;
  const int first_row = blockIdx.x * waves + wave;
  const int row_step = gridDim.x * waves;
  auto fetch = [&](int row, int c) {
    const int here = min(piece, units - c * piece);
    FetchPart<(kWave * F::kUnitBytes / 16 + kWave - 1) / kWave, true>(
        matrix + row * row_bytes + c * piece * F::kUnitBytes, here * F::kUnitBytes / 16, 0, 0, ring, lane);
  };

  for (int p0 = 0; p0 < n; ++p0) {
    if (p0 > 0) __syncthreads();  // the last pass's readers of the records
    const int pr = a.offsets != nullptr ? (sorted_first + p0) << 8 : listed ? pairs[p0] : (p0 << 8) | expert;
    const int token = pr >> 8;
    const int slot = pr & 0xFF;
    const void* row_x;
    FrontX front_x;
    FrontQ8 front_q;
    if constexpr (XT < 0) {
      row_x = static_cast<const uint8_t*>(d.y) +
              (static_cast<int64_t>(token) * d.y_token + static_cast<int64_t>(slot) * d.y_slot) * kQ8Block;
      front_q = LoadFrontQ8(static_cast<const uint8_t*>(row_x), d.ncols_x / 32);
    } else {
      const int64_t at = token * a.x_token + slot * a.x_slot;
      row_x = XT == LLMP_X_F32 ? static_cast<const void*>(static_cast<const float*>(a.x) + at)
                               : static_cast<const void*>(static_cast<const uint16_t*>(a.x) + at);
      front_x = LoadFrontX<XT>(row_x, d.ncols_x);
    }
    if (first_row < d.nrows) fetch(first_row, 0);
    if constexpr (XT < 0) {
      StageRecordsQ8<F>(static_cast<const uint8_t*>(row_x), d.ncols_x / 32, front_q, lds);
    } else {
      StageRecordsX<F, XT>(row_x, d.ncols_x, front_x, lds);
    }
    __syncthreads();  // the records are staged; from here the waves run alone

    float* dst = d.dst + static_cast<int64_t>(token) * d.dst_token + static_cast<int64_t>(slot) * d.dst_slot;
    for (int row = first_row; row < d.nrows; row += row_step) {
      float total = 0.0f;
      for (int c = 0; c < split; ++c) {
        AwaitTile();
        if (lane < min(piece, units - c * piece)) {
          float out[1];
          F::template DotAt<1, false>(my_block, lds + (c * piece + lane) * F::kRecord, token_stride, 1, out, nullptr);
          total += out[0];
        }
        // The next tile may overwrite the buffer: every lane's reads of it were consumed above.
        if (c + 1 < split) {
          fetch(row, c + 1);
        } else if (row + row_step < d.nrows) {
          fetch(row + row_step, 0);
        }
      }
      // A suffix sum over the wave's lanes (a fixed tree), the total in lane 0.
#pragma unroll
      for (int off = 1; off < kWave; off <<= 1) {
        const float other = __shfl_down(total, off, kWave);
        if (lane + off < kWave) total += other;
      }
      if (lane == 0) dst[row] = total;
    }
  }
}

// The rows of a tile: as many as a wave's 64 lanes hold (half of them a matrix with a GLU).
struct FlatPlan {
  int rows;
  int waves;
  size_t lds;
  bool wide = false;  // one workgroup of up to sixteen waves a CU instead of two of up to eight
};

constexpr size_t kFlatLdsLimit = 80 * 1024;  // two workgroups share a CU's 160 KB
constexpr size_t kWideLdsLimit = 160 * 1024 - 1024;  // one workgroup, beside the kernel's own few words
constexpr int kFewestWaves = 3;

// Eight waves a workgroup, fewer (down to kFewestWaves) where a long row's records would
// otherwise push the workgroup past half a CU's LDS.
template <class F>
FlatPlan PlanFlat(int pass, int units, bool glu, bool deep = false) {
  FlatPlan p;
  p.rows = (glu ? kWave / 2 : kWave) / units;
  // Units that are not whole 16-byte chunks: a wave's buffer has room for the tile's shift, the gate part's own
  // boundary and a lane's reads past its unit.
  constexpr bool kOdd = F::kUnitBytes % 16 != 0;
  p.waves = kWaves;
  for (;;) {
    p.lds = ((static_cast<size_t>(pass) * units * F::kRecord + 15) & ~static_cast<size_t>(15)) +
            static_cast<size_t>(deep ? 2 : 1) * p.waves * (kWave * F::kUnitBytes + (kOdd ? 80 : 0));
    if (deep || p.lds <= kFlatLdsLimit || p.waves == kFewestWaves) break;
    --p.waves;
  }
  if (deep || p.waves == kWaves) return p;
  // A long row's records are staged once a workgroup: two workgroups a CU hold them twice and have room for fewer
  // than sixteen tiles between them. One workgroup of up to sixteen waves holds them once: more tiles in flight a
  // CU (15360 values: 15 tiles against 12, and the 3840 rows of a down projection are then one tile a wave).
  const size_t records = (static_cast<size_t>(pass) * units * F::kRecord + 15) & ~static_cast<size_t>(15);
  const size_t tile = kWave * F::kUnitBytes + (kOdd ? 80 : 0);
  if (records >= kWideLdsLimit) return p;
  int wide = static_cast<int>((kWideLdsLimit - records) / tile);
  if (wide > 2 * kWaves) wide = 2 * kWaves;
  if (wide > 2 * p.waves) {
    p.waves = wide;
    p.lds = records + wide * tile;
    p.wide = true;
  }
  return p;
}
inline bool PlanFits(const FlatPlan& p) { return p.lds <= (p.wide ? kWideLdsLimit : kFlatLdsLimit); }
constexpr size_t kDeepLdsLimit = 160 * 1024 - 1024;  // one workgroup, beside the kernel's own few words
int g_compute_units = 0;

template <class F, int P, bool kGlu, int XT, bool kDump, bool kPacked, bool kDeep = false, int kUnder = 0>
void LaunchK(const VecQArgs& a, dim3 grid, const FlatPlan& plan, hipStream_t stream) {
  static bool sized = false;  // more than 64 KB of dynamic LDS must be asked for once
  if (!AllowLds(reinterpret_cast<const void*>(&VecQFlat<F, P, kGlu, XT, kDump, kPacked, kDeep, kUnder>), static_cast<int>(kDeepLdsLimit), &sized)) return;
  hipLaunchKernelGGL((VecQFlat<F, P, kGlu, XT, kDump, kPacked, kDeep, kUnder>), grid, dim3(plan.waves * kWave), plan.lds, stream, a,
                     plan.rows);
}

template <class F, int P, bool kGlu, int XT>
void LaunchT(const VecQArgs& a, dim3 grid, const FlatPlan& plan, bool deep, hipStream_t stream) {
  const bool packed = a.d.stride_row == a.d.ncols_x / F::kBlockValues;
  if (a.dump != nullptr) {
    if constexpr (P == 1 && !kGlu && XT < 0) LaunchK<F, P, kGlu, XT, true, false>(a, grid, plan, stream);
    return;
  }
  if (deep) {
    if constexpr (P == 1) LaunchK<F, P, kGlu, XT, false, true, true>(a, grid, plan, stream);
    return;
  }
  if constexpr (P == 1 && XT < 0 && StagesUnderLoads<F>::value) {
    // One tile a wave at most: the records staged under its loads.
    const int tiles = (a.d.nrows + plan.rows - 1) / plan.rows;
    if (packed && tiles <= static_cast<int>(grid.x) * plan.waves) {
      LaunchK<F, P, kGlu, XT, false, true, false, 1>(a, grid, plan, stream);
      return;
    }
  }
  if constexpr (P == 1 && XT >= 0 && StagesXUnderLoads<F>::value) {
    // Unquantized activations quantized under the first tile's loads: rows whose blocks are all front blocks,
    // aligned for the pieces' loads.
    const int tiles = (a.d.nrows + plan.rows - 1) / plan.rows;
    const int64_t align = XT == LLMP_X_F32 ? 16 : 8, width = XT == LLMP_X_F32 ? 4 : 2;
    const bool aligned = reinterpret_cast<uintptr_t>(a.x) % align == 0 && (a.x_token * width) % align == 0 &&
                         (a.x_slot * width) % align == 0;
    const bool front = a.d.ncols_x / 32 <= kFront * (plan.waves * kWave / 8);
    if (packed && aligned && front && a.d.ncols_x >= 32) {
      // One tile a wave: the barrier for LDS alone; more: the full barrier, which keeps the waves together.
      if (tiles <= static_cast<int>(grid.x) * plan.waves) {
        LaunchK<F, P, kGlu, XT, false, true, false, 1>(a, grid, plan, stream);
      } else {
        LaunchK<F, P, kGlu, XT, false, true, false, 2>(a, grid, plan, stream);
      }
      return;
    }
  }
  if (packed) {
    LaunchK<F, P, kGlu, XT, false, true>(a, grid, plan, stream);
  } else {
    LaunchK<F, P, kGlu, XT, false, false>(a, grid, plan, stream);
  }
}

template <class F, int P>
void LaunchP(const VecQArgs& a, int x_type, dim3 grid, const FlatPlan& plan, bool deep, hipStream_t stream) {
  const bool glu = a.d.g != nullptr;
  switch (x_type) {
    case -1:
      glu ? LaunchT<F, P, true, -1>(a, grid, plan, deep, stream) : LaunchT<F, P, false, -1>(a, grid, plan, deep, stream);
      break;
    case LLMP_X_F32:
      glu ? LaunchT<F, P, true, LLMP_X_F32>(a, grid, plan, deep, stream)
          : LaunchT<F, P, false, LLMP_X_F32>(a, grid, plan, deep, stream);
      break;
    default:
      glu ? LaunchT<F, P, true, LLMP_X_BF16>(a, grid, plan, deep, stream)
          : LaunchT<F, P, false, LLMP_X_BF16>(a, grid, plan, deep, stream);
      break;
  }
}

// The slots of a routed product whose workgroups own an expert, as far as the host can tell:
// one token's picks are distinct; several tokens' picks repeat, and about five in eight slots
// own an expert when they are many.
inline int LiveSlots(const llmp_vecq_desc& d, int slots) {
  if (d.tokens == 1) return slots;
  const int guess = slots * 5 / 8;
  return guess > d.used ? guess : d.used;
}

// A row of more than 64 units in pieces: the fewest pieces, of even length (a Q8_0 unit is 136
// bytes and a tile is fetched in 16-byte chunks).
struct SplitPlan {
  int split;
  int piece;
  int waves;
  size_t lds;
};

template <class F>
SplitPlan PlanSplit(int units) {
  SplitPlan p;
  p.split = (units + kWave - 1) / kWave;
  p.piece = ((units + p.split - 1) / p.split + 1) & ~1;
  p.waves = kWaves;
  for (;;) {
    p.lds = ((static_cast<size_t>(units) * F::kRecord + 15) & ~static_cast<size_t>(15)) +
            static_cast<size_t>(p.waves) * kWave * F::kUnitBytes;
    if (p.lds <= kFlatLdsLimit || p.waves == kFewestWaves) return p;
    --p.waves;
  }
}

template <class F, int XT>
void LaunchS(const VecQArgs& a, dim3 grid, const SplitPlan& plan, hipStream_t stream) {
  static bool sized = false;  // more than 64 KB of dynamic LDS must be asked for once
  if (!AllowLds(reinterpret_cast<const void*>(&VecQFlatSplit<F, XT>), static_cast<int>(kFlatLdsLimit), &sized)) return;
  hipLaunchKernelGGL((VecQFlatSplit<F, XT>), grid, dim3(plan.waves * kWave), plan.lds, stream, a, plan.split,
                     plan.piece);
}

template <class F>
void LaunchF(const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream) {
  const llmp_vecq_desc& d = a.d;
  const int units = d.ncols_x / F::kUnitValues;
  const bool glu = d.g != nullptr;
  if (units > kWave) {
    const SplitPlan plan = PlanSplit<F>(units);
    if (g_compute_units == 0) {
      const int cus = llmp_hip_compute_units();
      g_compute_units = cus > 0 ? cus : 256;
    }
    const int slots = a.offsets != nullptr ? d.used : d.ids != nullptr ? d.used * d.tokens : d.used;
    const int live_slots = a.offsets == nullptr && d.ids != nullptr ? LiveSlots(d, slots) : slots;
    int groups = 2 * g_compute_units / (live_slots > 0 ? live_slots : 1);
    if (groups < 1) groups = 1;
    if (groups > (d.nrows + plan.waves - 1) / plan.waves) groups = (d.nrows + plan.waves - 1) / plan.waves;
    const dim3 grid(static_cast<unsigned>(groups), static_cast<unsigned>(slots));
    switch (x_type) {
      case -1: LaunchS<F, -1>(a, grid, plan, stream); break;
      case LLMP_X_F32: LaunchS<F, LLMP_X_F32>(a, grid, plan, stream); break;
      default: LaunchS<F, LLMP_X_BF16>(a, grid, plan, stream); break;
    }
    return;
  }
  // The records a pass stages: four tokens', or a dense product's fewer.
  const int staged = a.offsets == nullptr && d.ids == nullptr && d.tokens < 4 ? d.tokens : 4;
  if (pass > 1 && !PlanFits(PlanFlat<F>(staged, units, glu))) pass = 1;
  // Two tile buffers a wave: one token a pass, packed rows, one workgroup a CU.
  deep = deep && F::kUnitBytes <= 144 && pass == 1 && a.dump == nullptr && d.stride_row == d.ncols_x / F::kBlockValues &&
         PlanFlat<F>(1, units, glu, true).lds <= kDeepLdsLimit;
  const FlatPlan plan = PlanFlat<F>(pass > 1 ? staged : 1, units, glu, deep);
  if (g_compute_units == 0) {
    const int cus = llmp_hip_compute_units();
    g_compute_units = cus > 0 ? cus : 256;
  }
  const int slots = a.offsets != nullptr ? d.used : d.ids != nullptr ? d.used * d.tokens : d.used;
  const int tiles = (d.nrows + plan.rows - 1) / plan.rows;
  // What is resident at once: two workgroups a CU, shared by the slots (every pair of a routed product has work:
  // the pairs that name an expert share it).
  int groups = (deep || plan.wide ? 1 : 2) * g_compute_units / (slots > 0 ? slots : 1);
  if (groups < 1) groups = 1;
  if (groups > (tiles + plan.waves - 1) / plan.waves) groups = (tiles + plan.waves - 1) / plan.waves;
  const dim3 grid(static_cast<unsigned>(groups), static_cast<unsigned>(slots));
  if (pass > 1) {
    LaunchP<F, 4>(a, x_type, grid, plan, deep, stream);
  } else {
    LaunchP<F, 1>(a, x_type, grid, plan, deep, stream);
  }
}

}  // namespace
}  // namespace llmp_hip

#endif  // LLMP_AMD_CSRC_VECQ_FLAT_H_
