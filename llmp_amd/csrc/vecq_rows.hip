// llmp.vecq over Q4_K weights for 2 to 8 tokens of a dense or grouped product: a lane a weight row,
// the dot products on the 4 x 4 x 4 int8 matrix instruction.
//
// v_mfma_i32_4x4x4_16B_i8 multiplies, in each of sixteen blocks of four lanes, a 4 x 4 matrix A by a
// 4 x 4 matrix B over four int8 values: lane 4 b + j supplies column j of B (four values of its own),
// and A can be one block's, broadcast to all sixteen. With a lane's weight row as its column of B
// and four tokens' codes as A, one instruction adds four values' products to a 4-token x 64-row
// tile of int32 sums; eight of them make a sub-block's exact sums for four tokens, with every lane
// of the result holding its own row. What is left in floats is what the one-token kernel does,
//   main = float(P_g) * (sc_g * d8_g), then fma over g;  out = fma(main, d, out),
// but four tokens a lane where the 16 x 16 instructions give sixteen tokens to sixteen rows: at
// four and eight tokens that is a quarter and a half of their vector work a weight byte. The
// minimums' part, (dmin * m_g) * (d8_g * sum of the codes), is an outer product a sub-block:
// v_mfma_f32_4x4x1_16B_f32 into an accumulator of its own.
//
// A workgroup is four waves and takes 64 rows at a time, each wave a quarter of K, meeting in LDS.
// A wave's weights come by global_load_lds_dwordx4 into a ring of its own in LDS, a 64-row
// super-block (9216 bytes, row after row) a stage, two or three stages deep; a lane then reads
// its row's 144 bytes (lanes 36 dwords apart: no two on a bank). The tokens' Q8_1 blocks are
// staged once a workgroup:
//   codes  [block][half][token] 16 bytes: the block's codes 16 half .. 16 half + 15 (lane t reads
//          token t's; the instruction broadcasts block t / 4's to all);
//   d8     [block][token] F32 (read four tokens at a time, the same for every lane);
//   ds8    [super-block][token] 8 floats, d8 * sum(codes) of sub-block g at g.
// A (token, row) value depends on its own token and row alone.

#include <hip/hip_runtime.h>

#include "common.h"
#include "llmp_hip.h"
#include "vecq_common.h"

namespace llmp_hip {
namespace {

constexpr int kRowsGroup = 256;
constexpr int kRowsWaves = kRowsGroup / kWave;
constexpr int kTileRows = 64;
constexpr int kPieceBytes = kTileRows * 144;  // one super-block of a tile's rows
constexpr int kPieceLoads = kPieceBytes / (kWave * 16);
constexpr size_t kRowsLdsLimit = 160 * 1024 - 1024;

typedef int V4i __attribute__((ext_vector_type(4)));
typedef float V4f __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* LdsPointer;
typedef const __attribute__((address_space(1))) void* GlobalPointer;

template <int LEFT>
__device__ __forceinline__ void AwaitLoads() {
  __builtin_amdgcn_s_waitcnt(0x0F70 | (LEFT & 15) | ((LEFT >> 4) << 14));
  asm volatile("" ::: "memory");  // what the loads wrote into LDS is read after this
}

// While a global_load_lds is in flight the compiler makes every wait it inserts a wait for everything: a read or
// a write of LDS it knows of waits until every load into LDS has landed (it cannot tell which of them the access
// could alias), and a wait for an ordinary load's register is taken to zero as well (the instruction counts as
// one that may touch both memories, whose returns are not ordered). The ring would never hold a load in flight
// while the wave computes. So between the first such load and the drain at a tile's end this kernel touches LDS
// and global memory only through the instructions written out below, and orders them itself: a wait, then Tie on
// every register the waited-for instructions wrote (which keeps the compiler from using one earlier).
typedef uint32_t U32v4 __attribute__((ext_vector_type(4)));
#define LLMP_TIE(x) asm volatile("" : "+v"(x))
// (By value: __builtin_bit_cast straight on an element of a vector reads element 0 whatever the index.)
__device__ __forceinline__ float AsFloat(uint32_t bits) { return __builtin_bit_cast(float, bits); }

template <int OFFSET>
__device__ __forceinline__ U32v4 LdsRead16(uint32_t at) {
  U32v4 v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(at), "n"(OFFSET));
  return v;
}
__device__ __forceinline__ void LdsWaited() { asm volatile("s_waitcnt lgkmcnt(0)"); }
__device__ __forceinline__ void LdsWrite16(uint32_t at, U32v4 value) { asm volatile("ds_write_b128 %0, %1" : : "v"(at), "v"(value)); }
__device__ __forceinline__ void LdsWrite4(uint32_t at, float value) { asm volatile("ds_write_b32 %0, %1" : : "v"(at), "v"(value)); }
__device__ __forceinline__ U32v4 GlobalLoad16(const void* from) {
  U32v4 v;
  asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(v) : "v"(from));
  return v;
}
__device__ __forceinline__ uint32_t GlobalLoad4(const void* from) {
  uint32_t v;
  asm volatile("global_load_dword %0, %1, off" : "=v"(v) : "v"(from));
  return v;
}
// A workgroup barrier for LDS alone: what the waves wrote to LDS is there, loads from global memory stay in flight
// (__syncthreads waits for those too).
__device__ __forceinline__ void LdsBarrier() {
  asm volatile("s_waitcnt lgkmcnt(0)");
  __builtin_amdgcn_s_barrier();
}

template <int NT>
struct Tokens {
  static constexpr int kCodesBlock = 2 * NT * 16;  // bytes of codes a block
  static constexpr int kScalesBlock = NT * 4;      // of d8
  static constexpr int kSumsSb = NT * 32;          // of ds8 a super-block
  static constexpr size_t Bytes(int blocks) {
    return static_cast<size_t>(blocks) * (kCodesBlock + kScalesBlock) + static_cast<size_t>(blocks / 8) * kSumsSb;
  }
};

// One super-block of one matrix for this lane's row (`row`: the LDS address of its 144 bytes) times the staged
// tokens. `codes`, `d8`: the LDS addresses of the super-block's, `codes` at this lane's token; `sums`: of this
// lane's token's eight ds8. Every LDS read is a RingRead (see there): a pair of sub-blocks' token operands are
// asked for while the pair before is multiplied.
// CBSZ: the matrix instructions' broadcast of the tokens, 4 from the wave's first lanes to all of it, 3 or 2 from the
// first lanes of every half or quarter of the wave to that half or quarter (whose lanes then stand at a super-block
// of their own: `codes`, `d8`, `sums` are this lane's); `live`: 1, or 0 for a lane whose super-block does not count.
template <int NT, int CBSZ = 4>
__device__ __forceinline__ void PieceDot(uint32_t row, uint32_t codes, uint32_t d8, uint32_t sums, float (&out)[NT],
                                         V4f (&mins)[NT / 4], float live = 1.0f) {
#pragma clang fp contract(off)
  using T = Tokens<NT>;
  constexpr int kQuads = NT / 4;
  U32v4 header = LdsRead16<0>(row);
  U32v4 qs[8] = {LdsRead16<16>(row), LdsRead16<32>(row), LdsRead16<48>(row), LdsRead16<64>(row),
                 LdsRead16<80>(row), LdsRead16<96>(row), LdsRead16<112>(row), LdsRead16<128>(row)};
  U32v4 s_lo = LdsRead16<0>(sums), s_hi = LdsRead16<16>(sums);
  // Pair p's token operands: the codes of sub-blocks 2 p and 2 p + 1 (two reads each) and their d8 (a read a quad).
  U32v4 c[2][4], scale[2][2 * kQuads];
  auto ask = [&](int p, U32v4 (&cs)[4], U32v4 (&ds)[2 * kQuads]) {
    const uint32_t at = codes + static_cast<uint32_t>(2 * p * T::kCodesBlock);
    cs[0] = LdsRead16<0>(at), cs[1] = LdsRead16<NT * 16>(at);
    cs[2] = LdsRead16<T::kCodesBlock>(at), cs[3] = LdsRead16<T::kCodesBlock + NT * 16>(at);
    const uint32_t dat = d8 + static_cast<uint32_t>(2 * p * T::kScalesBlock);
    ds[0] = LdsRead16<0>(dat), ds[kQuads] = LdsRead16<T::kScalesBlock>(dat);
    if constexpr (kQuads >= 2) ds[1] = LdsRead16<16>(dat), ds[kQuads + 1] = LdsRead16<T::kScalesBlock + 16>(dat);
  };
  auto landed = [&](U32v4 (&cs)[4], U32v4 (&ds)[2 * kQuads]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) LLMP_TIE(cs[i]);
#pragma unroll
    for (int i = 0; i < 2 * kQuads; ++i) LLMP_TIE(ds[i]);
  };
  ask(0, c[0], scale[0]);
  LdsWaited();
  LLMP_TIE(header);
#pragma unroll
  for (int i = 0; i < 8; ++i) LLMP_TIE(qs[i]);
  LLMP_TIE(s_lo);
  LLMP_TIE(s_hi);
  landed(c[0], scale[0]);
  U32x4 header4;
  header4.x = header[0], header4.y = header[1], header4.z = header[2], header4.w = header[3];
  Q4KHeader h = DecodeQ4KHeader(header4);
  if constexpr (CBSZ != 4) h.d *= live, h.dmin *= live;
  const float ds8[8] = {AsFloat(s_lo[0]), AsFloat(s_lo[1]), AsFloat(s_lo[2]),
                        AsFloat(s_lo[3]), AsFloat(s_hi[0]), AsFloat(s_hi[1]),
                        AsFloat(s_hi[2]), AsFloat(s_hi[3])};
  uint32_t w[32];
#pragma unroll
  for (int i = 0; i < 8; ++i) w[4 * i] = qs[i][0], w[4 * i + 1] = qs[i][1], w[4 * i + 2] = qs[i][2], w[4 * i + 3] = qs[i][3];
  float main[NT];
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const U32v4 (&cs)[4] = c[p & 1];
    const U32v4 (&ds)[2 * kQuads] = scale[p & 1];
    if (p < 3) ask(p + 1, c[(p + 1) & 1], scale[(p + 1) & 1]);
    const uint32_t code[2][8] = {{cs[0][0], cs[0][1], cs[0][2], cs[0][3], cs[1][0], cs[1][1], cs[1][2], cs[1][3]},
                                 {cs[2][0], cs[2][1], cs[2][2], cs[2][3], cs[3][0], cs[3][1], cs[3][2], cs[3][3]}};
    // The pair's two (four with eight tokens) chains of products interleaved: a wave is alone on its SIMD, and
    // a chain alone would wait out every instruction's latency.
    V4i sum[2][kQuads];
#pragma unroll
    for (int upper = 0; upper < 2; ++upper)
#pragma unroll
      for (int tq = 0; tq < kQuads; ++tq) sum[upper][tq] = V4i{0, 0, 0, 0};
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int low = static_cast<int>(w[8 * p + s] & 0x0F0F0F0Fu), high = static_cast<int>((w[8 * p + s] >> 4) & 0x0F0F0F0Fu);
      if constexpr (kQuads >= 1) {
        sum[0][0] = __builtin_amdgcn_mfma_i32_4x4x4i8(static_cast<int>(code[0][s]), low, sum[0][0], CBSZ, 0, 0);
        sum[1][0] = __builtin_amdgcn_mfma_i32_4x4x4i8(static_cast<int>(code[1][s]), high, sum[1][0], CBSZ, 0, 0);
      }
      if constexpr (kQuads >= 2) {
        sum[0][1] = __builtin_amdgcn_mfma_i32_4x4x4i8(static_cast<int>(code[0][s]), low, sum[0][1], CBSZ, 1, 0);
        sum[1][1] = __builtin_amdgcn_mfma_i32_4x4x4i8(static_cast<int>(code[1][s]), high, sum[1][1], CBSZ, 1, 0);
      }
    }
#pragma unroll
    for (int upper = 0; upper < 2; ++upper) {
      const int g = 2 * p + upper;
      const float sc = static_cast<float>((h.sc[g >> 2] >> (8 * (g & 3))) & 0xFFu);
      const float dm = h.dmin * static_cast<float>((h.mn[g >> 2] >> (8 * (g & 3))) & 0xFFu);
      if constexpr (kQuads >= 1) mins[0] = __builtin_amdgcn_mfma_f32_4x4x1f32(ds8[g], dm, mins[0], CBSZ, 0, 0);
      if constexpr (kQuads >= 2) mins[1] = __builtin_amdgcn_mfma_f32_4x4x1f32(ds8[g], dm, mins[1], CBSZ, 1, 0);
#pragma unroll
      for (int tq = 0; tq < kQuads; ++tq) {
        const U32v4 d4 = ds[upper * kQuads + tq];
        const float token_scale[4] = {AsFloat(d4[0]), AsFloat(d4[1]),
                                      AsFloat(d4[2]), AsFloat(d4[3])};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float by = sc * token_scale[q];
          const float product = static_cast<float>(sum[upper][tq][q]);
          main[4 * tq + q] = g == 0 ? product * by : fmaf(product, by, main[4 * tq + q]);
        }
      }
    }
    if (p < 3) {
      LdsWaited();
      landed(c[(p + 1) & 1], scale[(p + 1) & 1]);
    }
  }
#pragma unroll
  for (int t = 0; t < NT; ++t) out[t] = fmaf(main[t], h.d, out[t]);
}

// Q8_0 over weights relaid out into 64-row tiles (llmp_hip_relayout_q8_0_tiles64): a piece is four blocks of each
// of 64 rows, the codes first (row r's 128 at 128 r, its 16-byte chunk c at place c ^ (r % 8): eight lanes' 16-byte
// reads of one chunk then cover all 32 banks), then the rows' four F16 scales, 8 bytes a row from byte 8192. The
// codes are whole dwords as they lie (no 34-byte blocks to realign), and a dword goes into the instruction as it is.
// `stage`: the LDS address of the piece; `swizzle[c]`: this lane's 128 r + 16 (c ^ (r % 8)); `codes`, `d8`: as PieceDot's.
//   out[t] = fma(float(sum of block b's products with token t), dw_b * d8_b[t], out[t]), b = 0 .. 3.
template <int NT>
__device__ __forceinline__ void PieceDotQ8(uint32_t stage, const uint32_t (&swizzle)[8], uint32_t scales_at, uint32_t codes, uint32_t d8,
                                           float (&out)[NT]) {
#pragma clang fp contract(off)
  using T = Tokens<NT>;
  constexpr int kQuads = NT / 4;
  U32v4 w[8];
#pragma unroll
  for (int c = 0; c < 8; ++c) w[c] = LdsRead16<0>(stage + swizzle[c]);
  uint2 row_scales;
  asm volatile("ds_read_b64 %0, %1" : "=v"(row_scales) : "v"(stage + scales_at));
  U32v4 cs[2][2], ds[2][kQuads];
  auto ask = [&](int b, U32v4 (&c2)[2], U32v4 (&d2)[kQuads]) {
    const uint32_t at = codes + static_cast<uint32_t>(b * T::kCodesBlock);
    c2[0] = LdsRead16<0>(at), c2[1] = LdsRead16<NT * 16>(at);
    const uint32_t dat = d8 + static_cast<uint32_t>(b * T::kScalesBlock);
    d2[0] = LdsRead16<0>(dat);
    if constexpr (kQuads >= 2) d2[1] = LdsRead16<16>(dat);
  };
  auto landed = [&](U32v4 (&c2)[2], U32v4 (&d2)[kQuads]) {
    LLMP_TIE(c2[0]);
    LLMP_TIE(c2[1]);
#pragma unroll
    for (int i = 0; i < kQuads; ++i) LLMP_TIE(d2[i]);
  };
  ask(0, cs[0], ds[0]);
  LdsWaited();
#pragma unroll
  for (int c = 0; c < 8; ++c) LLMP_TIE(w[c]);
  LLMP_TIE(row_scales.x);
  LLMP_TIE(row_scales.y);
  landed(cs[0], ds[0]);
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const U32v4 (&c2)[2] = cs[b & 1];
    const U32v4 (&d2)[kQuads] = ds[b & 1];
    if (b < 3) ask(b + 1, cs[(b + 1) & 1], ds[(b + 1) & 1]);
    V4i sum[kQuads];
#pragma unroll
    for (int tq = 0; tq < kQuads; ++tq) sum[tq] = V4i{0, 0, 0, 0};
#pragma unroll
    for (int half = 0; half < 2; ++half) {
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const int code = static_cast<int>(c2[half][s]), weight = static_cast<int>(w[2 * b + half][s]);
        if constexpr (kQuads >= 1) sum[0] = __builtin_amdgcn_mfma_i32_4x4x4i8(code, weight, sum[0], 4, 0, 0);
        if constexpr (kQuads >= 2) sum[1] = __builtin_amdgcn_mfma_i32_4x4x4i8(code, weight, sum[1], 4, 1, 0);
      }
    }
    const uint32_t pair = b < 2 ? row_scales.x : row_scales.y;
    const float dw = HalfBitsToFloat((b & 1) != 0 ? pair >> 16 : pair & 0xFFFFu);
#pragma unroll
    for (int tq = 0; tq < kQuads; ++tq) {
      const U32v4 d4 = d2[tq];
      const float token_scale[4] = {AsFloat(d4[0]), AsFloat(d4[1]), AsFloat(d4[2]), AsFloat(d4[3])};
#pragma unroll
      for (int q = 0; q < 4; ++q) out[4 * tq + q] = fmaf(static_cast<float>(sum[tq][q]), dw * token_scale[q], out[4 * tq + q]);
    }
    if (b < 3) {
      LdsWaited();
      landed(cs[(b + 1) & 1], ds[(b + 1) & 1]);
    }
  }
}

// Q8_0 in the file's layout: a lane's row of a piece is 144 bytes fetched from the 16-byte boundary at or below its
// unit of four 34-byte blocks, which begins `shift` bytes (0 or 8, the same for every row: rows are whole 16-byte
// chunks apart) into it. Blocks 1 and 3 of a unit have their codes on dword boundaries; blocks 0 and 2 have them two
// bytes off, and every dword of theirs is put together from two (v_alignbyte).
// CBSZ, `live`: as PieceDot's.
template <int NT, int CBSZ = 4>
__device__ __forceinline__ void PieceDotQ8Native(uint32_t row, uint32_t codes, uint32_t d8, float (&out)[NT], float live = 1.0f) {
#pragma clang fp contract(off)
  using T = Tokens<NT>;
  constexpr int kQuads = NT / 4;
  uint2 raw[17];
#pragma unroll
  for (int i = 0; i < 17; ++i) asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(raw[i]) : "v"(row), "n"(8 * i));
  U32v4 cs[2][2], ds[2][kQuads];
  auto ask = [&](int b, U32v4 (&c2)[2], U32v4 (&d2)[kQuads]) {
    const uint32_t at = codes + static_cast<uint32_t>(b * T::kCodesBlock);
    c2[0] = LdsRead16<0>(at), c2[1] = LdsRead16<NT * 16>(at);
    const uint32_t dat = d8 + static_cast<uint32_t>(b * T::kScalesBlock);
    d2[0] = LdsRead16<0>(dat);
    if constexpr (kQuads >= 2) d2[1] = LdsRead16<16>(dat);
  };
  auto landed = [&](U32v4 (&c2)[2], U32v4 (&d2)[kQuads]) {
    LLMP_TIE(c2[0]);
    LLMP_TIE(c2[1]);
#pragma unroll
    for (int i = 0; i < kQuads; ++i) LLMP_TIE(d2[i]);
  };
  ask(0, cs[0], ds[0]);
  LdsWaited();
  uint32_t d[34];
#pragma unroll
  for (int i = 0; i < 17; ++i) {
    LLMP_TIE(raw[i].x);
    LLMP_TIE(raw[i].y);
    d[2 * i] = raw[i].x, d[2 * i + 1] = raw[i].y;
  }
  landed(cs[0], ds[0]);
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const U32v4 (&c2)[2] = cs[b & 1];
    const U32v4 (&d2)[kQuads] = ds[b & 1];
    if (b < 3) ask(b + 1, cs[(b + 1) & 1], ds[(b + 1) & 1]);
    // Block b begins at byte 34 b: dword 8 b + b / 2, on its boundary (b even) or two bytes past it (b odd); its
    // codes follow its two bytes of scale.
    const int first = 8 * b + b / 2;
    uint32_t weight[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      weight[s] = (b & 1) != 0 ? d[first + 1 + s] : __builtin_amdgcn_alignbyte(d[first + 1 + s], d[first + s], 2);
    }
    float dw = HalfBitsToFloat((b & 1) != 0 ? d[first] >> 16 : d[first] & 0xFFFFu);
    if constexpr (CBSZ != 4) dw *= live;
    V4i sum[kQuads];
#pragma unroll
    for (int tq = 0; tq < kQuads; ++tq) sum[tq] = V4i{0, 0, 0, 0};
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const int code = static_cast<int>(c2[s >> 2][s & 3]);
      if constexpr (kQuads >= 1) sum[0] = __builtin_amdgcn_mfma_i32_4x4x4i8(code, static_cast<int>(weight[s]), sum[0], CBSZ, 0, 0);
      if constexpr (kQuads >= 2) sum[1] = __builtin_amdgcn_mfma_i32_4x4x4i8(code, static_cast<int>(weight[s]), sum[1], CBSZ, 1, 0);
    }
#pragma unroll
    for (int tq = 0; tq < kQuads; ++tq) {
      const U32v4 d4 = d2[tq];
      const float token_scale[4] = {AsFloat(d4[0]), AsFloat(d4[1]), AsFloat(d4[2]), AsFloat(d4[3])};
#pragma unroll
      for (int q = 0; q < 4; ++q) out[4 * tq + q] = fmaf(static_cast<float>(sum[tq][q]), dw * token_scale[q], out[4 * tq + q]);
    }
    if (b < 3) {
      LdsWaited();
      landed(cs[(b + 1) & 1], ds[(b + 1) & 1]);
    }
  }
}

constexpr int kQ8PieceBytes = kTileRows * 136;  // a relaid-out Q8_0 piece in device memory: 8192 bytes of codes, 512 of scales

// grid (workgroups, slots); LDS: the tokens, then the waves' rings (whose first bytes also carry the
// waves' sums to their meeting). FMT 0: Q4_K (a unit a super-block); 1: Q8_0 relaid out (a unit four blocks); 2: Q8_0
// in the file's layout; 3, 4: Q4_K, and 5, 6: Q8_0 in the file's layout, in tiles of 32 and 16 rows (for matrices of
// few rows, whose 64-row tiles would leave most of the device idle): a piece is two or four consecutive units of each
// row, a half or a quarter of the wave's lanes at each, the lanes' sums meeting at the tile's end.
// kSpans: the tokens staged a span of the row at a time (below).
template <bool kGlu, int NT, int STAGES, int FMT = 0, bool kSpans = false>
__global__ __launch_bounds__(kRowsGroup, 2) void VecQRows(const VecQArgs a) {
  using T = Tokens<NT>;
  constexpr int kMatrices = kGlu ? 2 : 1;
  constexpr bool kQ4K = FMT == 0 || FMT == 3 || FMT == 4;
  constexpr bool kNative8 = FMT == 2 || FMT >= 5;
  constexpr int kParts = FMT == 3 || FMT == 5 ? 2 : FMT == 4 || FMT == 6 ? 4 : 1;  // units of a row that a piece holds
  constexpr int kRows = kTileRows / kParts;                // rows a tile
  constexpr int kUnitBlocks = kQ4K ? 8 : 4;
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

  const llmp_vecq_desc& d = a.d;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int nsb = d.ncols_x / 32 / kUnitBlocks;  // units a row
  // Rows whose tokens do not fit LDS beside the rings are taken in spans, the span's tokens staged anew (for every
  // tile: long rows are the down projections' few tiles), the sums carried in registers. A span is `a.span` units of
  // every wave's own quarter of the row, so a wave adds its units in the row's order whatever the spans: the same
  // bits as one span gives.
  const int spans = kSpans ? ((nsb + kRowsWaves - 1) / kRowsWaves + a.span - 1) / a.span : 1;
  const int staged_blocks = (kSpans ? kRowsWaves * a.span : nsb) * kUnitBlocks;  // the room for tokens
  const int slot = blockIdx.y;
  uint8_t* codes = lds;
  uint8_t* d8 = codes + staged_blocks * T::kCodesBlock;
  uint8_t* sums = d8 + staged_blocks * T::kScalesBlock;
  uint8_t* rings = lds + ((T::Bytes(staged_blocks) + 1023) & ~static_cast<size_t>(1023));
  uint8_t* ring = rings + wave * (STAGES * kPieceBytes);

  auto lds_address = [](const uint8_t* p) { return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(p)); };  // the pointer's low half
  // The tokens: a thread a block. Their loads are asked for first and held in registers while the first
  // tile's weights are asked for (loads return in order: the tokens are there while the weights still
  // come), then staged. No branch around a load or a store: past the last block a thread repeats it, the
  // same bytes to the same place.
  const int tokens = d.tokens;
  constexpr int kHeld = 4;
  struct HeldBlock {
    U32v4 lower, upper;  // the codes
    uint32_t scale;      // d8 and the block's sum as F16
  };
  HeldBlock held[kHeld];
  // The span at hand: how far into the quarters it starts, this wave's units of it, and the unit that the first
  // staged one of this wave is (the staged tokens of a wave's units follow those of the wave before).
  const int blocks = staged_blocks, last_block = NT * blocks - 1;
  const int quarter_first = wave * nsb / kRowsWaves, quarter_end = (wave + 1) * nsb / kRowsWaves;
  int span_at = 0, sb_first = quarter_first, sb_end = quarter_end, staged_from = 0;
  int pieces = (sb_end - sb_first + kParts - 1) / kParts * kMatrices;
  auto set_span = [&](int span) {
    span_at = span * a.span;
    sb_first = quarter_first + span_at;
    sb_end = min(sb_first + a.span, quarter_end);
    staged_from = sb_first - wave * a.span;
    pieces = (sb_end - sb_first + kParts - 1) / kParts * kMatrices;
  };
  if constexpr (kSpans) set_span(0);
  auto token_block = [&](int index) {
    const int t = index / blocks;
    int b = index - t * blocks;
    if constexpr (kSpans) {  // the staged unit's place in the row: its wave's quarter, the span's start, its own
      const int unit = b / kUnitBlocks, of_wave = unit / a.span;
      const int in_row = min(of_wave * nsb / kRowsWaves + span_at + (unit - of_wave * a.span), nsb - 1);
      b = in_row * kUnitBlocks + (b - unit * kUnitBlocks);
    }
    const int from = min(t, tokens - 1);  // the tokens a group lacks repeat its last: computed and dropped
    return static_cast<const uint8_t*>(d.y) +
           (static_cast<int64_t>(from) * d.y_token + static_cast<int64_t>(slot) * d.y_slot + b) * kQ8Block;
  };
  auto ask_block = [&](int index, HeldBlock& block) {
    const uint8_t* src = token_block(min(index, last_block));
    block.scale = GlobalLoad4(src);
    block.lower = GlobalLoad16(src + 4);
    block.upper = GlobalLoad16(src + 20);
  };
  auto stage_block = [&](HeldBlock& block, int index) {
    LLMP_TIE(block.lower);
    LLMP_TIE(block.upper);
    LLMP_TIE(block.scale);
    index = min(index, last_block);
    const int t = index / blocks, b = index - t * blocks;
    LdsWrite16(lds_address(codes) + static_cast<uint32_t>(b * T::kCodesBlock + t * 16), block.lower);
    LdsWrite16(lds_address(codes) + static_cast<uint32_t>(b * T::kCodesBlock + (NT + t) * 16), block.upper);
    int sum = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) sum = Dot4(0x01010101, static_cast<int>(block.lower[i]), sum);
#pragma unroll
    for (int i = 0; i < 4; ++i) sum = Dot4(0x01010101, static_cast<int>(block.upper[i]), sum);
    const float scale = HalfBitsToFloat(block.scale & 0xFFFFu);
    LdsWrite4(lds_address(d8) + static_cast<uint32_t>(b * T::kScalesBlock + t * 4), scale);
    LdsWrite4(lds_address(sums) + static_cast<uint32_t>((b >> 3) * T::kSumsSb + t * 32 + (b & 7) * 4), scale * static_cast<float>(sum));
  };

  // This wave's quarter of K, and this lane's sixteen bytes of each of a piece's nine loads: byte
  // 1024 j + 16 lane of the 64 rows x 144 bytes lies in row (that / 144), rows past the matrix's end
  // repeating its last.
  const int tiles = (d.nrows + kRows - 1) / kRows;
  const int64_t matrix_block = static_cast<int64_t>(slot) * d.stride_expert;
  const int part = lane / kRows;  // which of a piece's super-blocks of its row this lane multiplies
  const int token_lane = min(lane & (kRows - 1), NT - 1);
  const uint32_t ring_at = lds_address(ring) + (FMT != 1 ? static_cast<uint32_t>(lane) * 144u : 0u);  // this lane's row of a stage (Q8_0 relaid out: the stage)
  uint32_t swizzle[8];
#pragma unroll
  for (int c = 0; c < 8; ++c) swizzle[c] = static_cast<uint32_t>(lane * 128 + ((c ^ (lane & 7)) << 4));
  const uint32_t scales_at = 8192u + static_cast<uint32_t>(lane) * 8u;
  const uint32_t codes_at = lds_address(codes) + static_cast<uint32_t>(token_lane) * 16u;
  const uint32_t d8_at = lds_address(d8);
  const uint32_t sums_at = lds_address(sums) + static_cast<uint32_t>(token_lane) * 32u;

  uint32_t offsets[kPieceLoads];
  [[maybe_unused]] uint32_t odd_first[kPieceLoads];  // (narrow Q8_0 tiles: what a piece whose first unit is an odd one adds)
  const uint8_t* up_tile = nullptr;
  const uint8_t* gate_tile = nullptr;
  auto aim = [&](int tile) {
    const int row0 = tile * kRows;
#pragma unroll
    for (int j = 0; j < kPieceLoads; ++j) {
      const int byte = j * (kWave * 16) + lane * 16;
      const int row = byte / 144;  // the lane that reads these 144 bytes of the stage
      // (Relaid-out weights: a piece is 9216 consecutive bytes, every 64-byte unit of HBM asked for once.)
      if constexpr (kNative8) {
        // A row's 144 bytes from the 16-byte boundary at or below its unit (issue adds the place of the piece's first
        // unit). Narrow tiles: unit u of the piece lies 136 u bytes on, its boundary 0, 128, 272, 400 on where the
        // first unit begins at a boundary (an even unit), 0, 144, 272, 416 where it begins 8 bytes past one.
        const int u = row / kRows;
        offsets[j] = static_cast<uint32_t>(min(row0 + (row & (kRows - 1)), d.nrows - 1) - row0) * static_cast<uint32_t>(d.stride_row) * 34u +
                     static_cast<uint32_t>((u * 136 & ~15) + (byte - row * 144));
        odd_first[j] = static_cast<uint32_t>((u & 1) * 16);
      } else if constexpr (FMT == 1) {
        // The piece's last 512 bytes (the scales) by the lower half of the wave, the upper half the same again
        // (into the stage's spare 512 bytes).
        offsets[j] = j < 8 ? static_cast<uint32_t>(byte) : 8192u + static_cast<uint32_t>(lane & 31) * 16u;
      } else if constexpr (kQ4K && kParts > 1) {
        offsets[j] = static_cast<uint32_t>(min(row0 + (row & (kRows - 1)), d.nrows - 1) - row0) * static_cast<uint32_t>(d.stride_row) * 144u +
                     static_cast<uint32_t>(row / kRows * 144 + (byte - row * 144));
      } else {
        offsets[j] = a.tiled != 0 ? static_cast<uint32_t>(byte)
                                  : static_cast<uint32_t>(min(row0 + row, d.nrows - 1) - row0) * static_cast<uint32_t>(d.stride_row) * 144u +
                                        static_cast<uint32_t>(byte - row * 144);
      }
    }
    const int64_t at = (matrix_block + static_cast<int64_t>(row0) * d.stride_row) * (kQ4K ? 144 : 34);
    up_tile = static_cast<const uint8_t*>(d.w) + at;
    if constexpr (kGlu) gate_tile = static_cast<const uint8_t*>(d.g) + at;
  };
  // Piece i, in the order the loop below multiplies them: two super-blocks of the up matrix, the same two of the
  // gate matrix, the next two (an odd one out last, up then gate). Past the
  // wave's last piece its last again (a load is never skipped: the waits count loads).
  auto issue = [&](int i) {
    const int piece = min(i, pieces - 1);
    const int count = (sb_end - sb_first + kParts - 1) / kParts;
    int gate = 0, sb = piece;
    if constexpr (kGlu) {
      const int paired = count / 2 * 4;  // pieces of whole pairs of super-blocks
      gate = piece < paired ? (piece & 3) >> 1 : piece - paired;
      sb = piece < paired ? (piece >> 2) * 2 + (piece & 1) : count - 1;
    }
    // (Narrow tiles: the last piece of a quarter that is no whole number of pieces starts early, see piece_dot.)
    sb = sb_first + (kParts == 1 ? sb : min(kParts * sb, sb_end - sb_first - kParts));
    const uint8_t* from = (gate != 0 ? gate_tile : up_tile) +
                          (kNative8 ? static_cast<int64_t>(sb) * 136 & ~int64_t{15}
                                    : static_cast<int64_t>(sb) * (FMT == 1 ? kQ8PieceBytes : a.tiled != 0 ? kPieceBytes : 144));
    uint8_t* to = ring + (i % STAGES) * kPieceBytes;
    [[maybe_unused]] const uint32_t odd = (sb & 1) != 0 ? ~0u : 0u;
#pragma unroll
    for (int j = 0; j < kPieceLoads; ++j) {
      const uint32_t offset = kNative8 && kParts > 1 ? offsets[j] + (odd_first[j] & odd) : offsets[j];
      __builtin_amdgcn_global_load_lds((GlobalPointer)(from + offset), (LdsPointer)(to + j * (kWave * 16)), 16, 0, 0);
    }
  };
  // Before piece i is multiplied: the piece STAGES - 1 ahead is asked for, and all but the STAGES - 1 youngest
  // pieces have landed. At the tile's end nothing is asked for (a repeat of the last piece would be read from HBM
  // again: the copies of the weights are rotated) and the wait is for what is left.
  auto next_piece = [&](int i) {
    const int left = pieces - 1 - i;  // pieces after this one
    if (left >= STAGES - 1) {
      issue(i + STAGES - 1);
      AwaitLoads<kPieceLoads*(STAGES - 1)>();
    } else {
      static_assert(STAGES <= 4, "a wait for each count of pieces left");
      if (STAGES > 3 && left == 2) {
        AwaitLoads<kPieceLoads * 2>();
      } else if (STAGES > 2 && left == 1) {
        AwaitLoads<kPieceLoads>();
      } else {
        AwaitLoads<0>();
      }
    }
  };
  // (Every wave has pieces: rows of at least four super-blocks; and every workgroup a tile: the grid is no larger.)
  auto prologue = [&](int tile) {
    aim(tile);
#pragma unroll
    for (int i = 0; i < STAGES - 1; ++i) issue(i);
  };
  // The tokens are asked for before anything else, the ring's first pieces after them: when no more than those
  // pieces' loads are outstanding (loads return in order) the tokens are there, and they are staged, and the
  // workgroup past its barrier, while the first piece is still on its way. (With the first piece asked for ahead of
  // the tokens the staging and the barrier stood between its landing and its products: the down projection 15360 ->
  // 3840 took 12.4 us at 4 tokens and 20.0 at 8 where it takes 11.4 and 18.2.)
  aim(blockIdx.x);
#pragma unroll
  for (int it = 0; it < kHeld; ++it) ask_block(tid + it * kRowsGroup, held[it]);
#pragma unroll
  for (int i = 0; i < STAGES - 1; ++i) issue(i);
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(kPieceLoads * (STAGES - 1)));
#pragma unroll
  for (int it = 0; it < kHeld; ++it) stage_block(held[it], tid + it * kRowsGroup);
  for (int index = tid + kHeld * kRowsGroup; index <= last_block; index += kHeld * kRowsGroup) {  // rows too long for that
#pragma unroll
    for (int it = 0; it < kHeld; ++it) ask_block(index + it * kRowsGroup, held[it]);
    asm volatile("s_waitcnt vmcnt(0)");
#pragma unroll
    for (int it = 0; it < kHeld; ++it) stage_block(held[it], index + it * kRowsGroup);
  }

  for (int tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    const int row0 = tile * kRows;
    float up_out[NT], gate_out[NT];
    V4f up_mins[NT / 4], gate_mins[NT / 4];
#pragma unroll
    for (int t = 0; t < NT; ++t) up_out[t] = 0.0f, gate_out[t] = 0.0f;
#pragma unroll
    for (int tq = 0; tq < NT / 4; ++tq) up_mins[tq] = V4f{0.0f, 0.0f, 0.0f, 0.0f}, gate_mins[tq] = up_mins[tq];
    for (int span = 0; span < spans; ++span) {
    if (tile != static_cast<int>(blockIdx.x) || span != 0) {
      if constexpr (kSpans) {
        __syncthreads();  // the tokens' readers are done with the span before
        set_span(span);
        for (int index = tid; index <= last_block; index += kHeld * kRowsGroup) {
#pragma unroll
          for (int it = 0; it < kHeld; ++it) ask_block(index + it * kRowsGroup, held[it]);
          asm volatile("s_waitcnt vmcnt(0)");
#pragma unroll
          for (int it = 0; it < kHeld; ++it) stage_block(held[it], index + it * kRowsGroup);
        }
      }
      prologue(tile);
    }
    LdsBarrier();  // the tokens are staged
    {
      // Two super-blocks of the up matrix, then the same two of the gate matrix: neighbours in a row share a 64-byte
      // unit of HBM more often than not, and the sooner the second asks for it the likelier L2 still has it.
      const int count = (sb_end - sb_first + kParts - 1) / kParts;
      int i = 0;
      auto piece_dot = [&](int step, float (&out)[NT], V4f (&mins)[NT / 4]) {
        // Narrow tiles: the piece starts kParts super-blocks a step on, the last one kParts before the quarter's end,
        // where the lanes at super-blocks that the step before had do not count.
        const int start = kParts == 1 ? step : min(kParts * step, sb_end - sb_first - kParts);
        const int sb = sb_first + start + part;
        [[maybe_unused]] const float live = start + part >= kParts * step ? 1.0f : 0.0f;
        const int staged_unit = sb - staged_from;
        const uint32_t sb_codes = codes_at + static_cast<uint32_t>(staged_unit * kUnitBlocks * T::kCodesBlock);
        const uint32_t sb_d8 = d8_at + static_cast<uint32_t>(staged_unit * kUnitBlocks * T::kScalesBlock);
        const uint32_t sb_sums = sums_at + static_cast<uint32_t>(staged_unit * T::kSumsSb);
        next_piece(i);
        if constexpr (FMT == 0) {
          PieceDot<NT>(ring_at + (i % STAGES) * kPieceBytes, sb_codes, sb_d8, sb_sums, out, mins);
        } else if constexpr (kQ4K && kParts > 1) {
          PieceDot<NT, kParts == 2 ? 3 : 2>(ring_at + (i % STAGES) * kPieceBytes, sb_codes, sb_d8, sb_sums, out, mins, live);
        } else if constexpr (kNative8 && kParts > 1) {
          PieceDotQ8Native<NT, kParts == 2 ? 3 : 2>(ring_at + (i % STAGES) * kPieceBytes + static_cast<uint32_t>((sb & 1) * 8), sb_codes, sb_d8, out, live);
        } else if constexpr (FMT == 2) {
          PieceDotQ8Native<NT>(ring_at + (i % STAGES) * kPieceBytes + static_cast<uint32_t>((sb & 1) * 8), sb_codes, sb_d8, out);
        } else {
          PieceDotQ8<NT>(ring_at + (i % STAGES) * kPieceBytes, swizzle, scales_at, sb_codes, sb_d8, out);
        }
        ++i;
        __builtin_amdgcn_s_waitcnt(0xC07F);  // the stage about to be refilled has been read
      };
      for (int n = 0; n < count; n += kMatrices) {
        const int width = min(kMatrices, count - n);
        for (int w = 0; w < width; ++w) piece_dot(n + w, up_out, up_mins);
        if constexpr (kGlu) {
          for (int w = 0; w < width; ++w) piece_dot(n + w, gate_out, gate_mins);
        }
      }
    }
    }
    // The four quarters of K meet: [wave][matrix][token][row] floats at the head of each wave's ring.
    // (Narrow tiles: the lanes of a row first, halves of the wave then quarters; every lane of a row ends with the sum.)
    float* mine = reinterpret_cast<float*>(ring);
    auto of_row = [&](float mine_alone) {
#pragma clang fp contract(off)
      if constexpr (kParts >= 2) mine_alone += __shfl_xor(mine_alone, 32);
      if constexpr (kParts >= 4) mine_alone += __shfl_xor(mine_alone, 16);
      return mine_alone;
    };
#pragma unroll
    for (int t = 0; t < NT; ++t) {
#pragma clang fp contract(off)
      mine[t * kRows + (lane & (kRows - 1))] = of_row(up_out[t] - up_mins[t / 4][t % 4]);
      if constexpr (kGlu) mine[(NT + t) * kRows + (lane & (kRows - 1))] = of_row(gate_out[t] - gate_mins[t / 4][t % 4]);
    }
    __syncthreads();
    for (int index = tid; index < tokens * kRows; index += kRowsGroup) {
#pragma clang fp contract(off)
      const int t = index / kRows, r = index - t * kRows;
      auto total = [&](int matrix) {
        const float* at = reinterpret_cast<const float*>(rings) + (matrix * NT + t) * kRows + r;
        constexpr int kRing = STAGES * kPieceBytes / 4;
        return (at[0] + at[kRing]) + (at[2 * kRing] + at[3 * kRing]);
      };
      const float up = total(0);
      if (row0 + r < d.nrows) {
        float* dst = d.dst + static_cast<int64_t>(t) * d.dst_token + static_cast<int64_t>(slot) * d.dst_slot;
        dst[row0 + r] = kGlu ? Glu(d.glu, total(1), up, d.limit) : up;
      }
    }
    __syncthreads();  // the next tile's first loads land where the sums were
  }
}

int g_rows_compute_units = 0;


template <int NT>
int StagesFor(int blocks) {
  const size_t tokens = (Tokens<NT>::Bytes(blocks) + 1023) & ~static_cast<size_t>(1023);
  for (int stages = 3; stages >= 2; --stages)
    if (tokens + static_cast<size_t>(kRowsWaves) * stages * kPieceBytes <= kRowsLdsLimit) return stages;
  return 0;
}

// The units of a wave's quarter that a span takes, for rows of `units` units of `unit_blocks` blocks: 0 where the whole
// row's tokens fit beside the rings, else those of the fewest spans that do (every wave with a unit or more in every
// span), -1 if none.
// `parts`: the units that a wave's share of a span is at least (a piece's units in narrow tiles), and that a span is a
// multiple of: a unit then meets the same lane whatever the spans, and the sums the same order.
template <int NT>
int SpanFor(int units, int unit_blocks, int parts = 1) {
  const int shortest = units / kRowsWaves, longest = (units + kRowsWaves - 1) / kRowsWaves;
  if (shortest < parts) return -1;
  if (StagesFor<NT>(units * unit_blocks) != 0) return 0;
  for (int spans = 2; spans <= shortest; ++spans) {
    const int span = ((longest + spans - 1) / spans + parts - 1) / parts * parts;  // whole pieces in all but the last
    if (shortest - (spans - 1) * span < parts) continue;
    if (StagesFor<NT>(kRowsWaves * span * unit_blocks) != 0) return span;
  }
  return -1;
}

// Tiles of 64 rows, or of 32 or 16 (the file's layouts) where that many more workgroups still find a compute
// unit each and the rows are long enough for a piece of two or four units a wave and span. Measured at 4 tokens of
// Q4_K rows of 4096 values, tiles of 64 / 32 / 16 rows: 80 tiles 10.6 / 7.9 / 10.1 us, 128 tiles 10.9 / 8.6 / 10.9,
// 160 tiles 11.2 / 12.8 / 14.1, 256 tiles 13.3 / 13.9 / 18.3.
int RowsParts(const VecQArgs& a, int cus) {
  const llmp_vecq_desc& d = a.d;
  if (a.tiled != 0 && a.tiled != 3) return 1;
  const int64_t tiles = static_cast<int64_t>((d.nrows + kTileRows - 1) / kTileRows) * d.used;
  const int unit_blocks = a.tiled == 3 ? 4 : 8, units = d.ncols_x / 32 / unit_blocks;
  auto takes = [&](int parts) { return (d.tokens <= 4 ? SpanFor<4>(units, unit_blocks, parts) : SpanFor<8>(units, unit_blocks, parts)) >= 0; };
  for (int parts = 4; parts > 1; parts /= 2) {
    if (tiles * parts <= cus && takes(parts)) return parts;
  }
  // More tiles than compute units: the workgroups go through them in rounds, and half tiles end the last round
  // sooner where that saves a fifth of the rounds (320 tiles on 256 units: three rounds of half tiles for two of
  // whole ones, 18.6 us against 20.4 at 4096 x 20480).
  const int64_t rounds = (tiles + cus - 1) / cus, half_rounds = (2 * tiles + cus - 1) / cus;
  if (5 * half_rounds <= 8 * rounds && takes(2)) return 2;
  return 1;
}

template <bool kGlu, int NT, int STAGES, int FMT, bool kSpans = false>
void LaunchRowsKernel(const VecQArgs& a, int staged_blocks, dim3 grid, hipStream_t stream) {
  static bool sized = false;  // more than 64 KB of dynamic LDS must be asked for once
  if (!AllowLds(reinterpret_cast<const void*>(&VecQRows<kGlu, NT, STAGES, FMT, kSpans>), static_cast<int>(kRowsLdsLimit), &sized)) return;
  const size_t lds = ((Tokens<NT>::Bytes(staged_blocks) + 1023) & ~static_cast<size_t>(1023)) +
                     static_cast<size_t>(kRowsWaves) * STAGES * kPieceBytes;
  hipLaunchKernelGGL((VecQRows<kGlu, NT, STAGES, FMT, kSpans>), grid, dim3(kRowsGroup), lds, stream, a);
}

// Three stages a wave where they fit beside the whole row's tokens, else two; two with spans.
template <bool kGlu, int NT, int FMT>
void LaunchRowsFormat(const VecQArgs& a, int staged_blocks, dim3 grid, hipStream_t stream) {
  if (a.span > 0) {
    LaunchRowsKernel<kGlu, NT, 2, FMT, true>(a, staged_blocks, grid, stream);
  } else if (StagesFor<NT>(staged_blocks) == 3) {
    LaunchRowsKernel<kGlu, NT, 3, FMT>(a, staged_blocks, grid, stream);
  } else {
    LaunchRowsKernel<kGlu, NT, 2, FMT>(a, staged_blocks, grid, stream);
  }
}

template <bool kGlu, int NT>
void LaunchRowsStages(const VecQArgs& whole, dim3 grid, hipStream_t stream) {
  VecQArgs a = whole;
  const int unit_blocks = a.tiled >= 2 ? 4 : 8;
  const int units = a.d.ncols_x / 32 / unit_blocks;
  a.span = SpanFor<NT>(units, unit_blocks, a.parts);
  const int staged_blocks = (a.span > 0 ? kRowsWaves * a.span : units) * unit_blocks;
  const int format = a.tiled == 2 ? 1 : a.tiled == 3 ? (a.parts == 2 ? 5 : a.parts == 4 ? 6 : 2) : a.tiled == 0 ? (a.parts == 2 ? 3 : a.parts == 4 ? 4 : 0) : 0;
  switch (format) {
    case 1:
      return LaunchRowsFormat<kGlu, NT, 1>(a, staged_blocks, grid, stream);
    case 2:
      return LaunchRowsFormat<kGlu, NT, 2>(a, staged_blocks, grid, stream);
    case 3:
      return LaunchRowsFormat<kGlu, NT, 3>(a, staged_blocks, grid, stream);
    case 4:
      return LaunchRowsFormat<kGlu, NT, 4>(a, staged_blocks, grid, stream);
    case 5:
      return LaunchRowsFormat<kGlu, NT, 5>(a, staged_blocks, grid, stream);
    case 6:
      return LaunchRowsFormat<kGlu, NT, 6>(a, staged_blocks, grid, stream);
    default:
      return LaunchRowsFormat<kGlu, NT, 0>(a, staged_blocks, grid, stream);
  }
}

// A thread a row's unit of four blocks (136 bytes): into its tile's piece (see PieceDotQ8), or back.
__global__ void RelayoutQ8Tiles64Kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst, int64_t units_all, int units, int inverse) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= units_all) return;
  const int64_t row = i / units;
  const int unit = static_cast<int>(i - row * units);
  const int r = static_cast<int>(row % kTileRows);
  const uint16_t* native = src + (inverse != 0 ? 0 : i * 68);
  uint16_t* native_to = dst + (inverse != 0 ? i * 68 : 0);
  const int64_t piece = ((row / kTileRows) * units + unit) * (kQ8PieceBytes / 2);  // in halfwords
  for (int b = 0; b < 4; ++b) {
    const int64_t scale_at = piece + 4096 + r * 4 + b;
    if (inverse != 0) {
      native_to[17 * b] = src[scale_at];
    } else {
      dst[scale_at] = native[17 * b];
    }
    for (int h = 0; h < 16; ++h) {  // the block's codes, two a halfword: chunk 2 b + h / 8, halfword h % 8 of it
      const int c = 2 * b + (h >> 3);
      const int64_t code_at = piece + r * 64 + ((c ^ (r & 7)) << 3) + (h & 7);
      if (inverse != 0) {
        native_to[17 * b + 1 + h] = src[code_at];
      } else {
        dst[code_at] = native[17 * b + 1 + h];
      }
    }
  }
}

// 16 bytes a thread: block (row, sb) of the row-major matrix is block (sb, row % 64) of its 64-row tile.
__global__ void RelayoutTiles64Kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, int64_t chunks, int nsb, int inverse) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= chunks) return;
  const int64_t block = i / 9;
  const int part = static_cast<int>(i - block * 9);
  const int64_t row = block / nsb;
  const int sb = static_cast<int>(block - row * nsb);
  const int64_t tiled = ((row / kTileRows) * nsb + sb) * kTileRows + row % kTileRows;
  if (inverse != 0) {
    dst[block * 9 + part] = src[tiled * 9 + part];
  } else {
    dst[tiled * 9 + part] = src[block * 9 + part];
  }
}

}  // namespace

// Q4_K, 2 to 8 tokens of a dense or grouped product (no routing ids) over Q8_1 activations, rows of at
// least four super-blocks (a wave a quarter of K) whose staged tokens leave room for two stages a wave. Q8_0: rows of
// whole 256 values (an even number of four-block units, so that a row's last 16-byte chunk ends inside the row), at
// least four units, every row and matrix at a 16-byte boundary.
bool RowsTakes(int type, const llmp_vecq_desc& whole, int parts) {
  // Nine to kRowsTokensMost tokens are launches of eight or fewer each.
  llmp_vecq_desc d = whole;
  if (d.tokens > 8 && d.tokens <= kRowsTokensMost) d.tokens = 8;
  if (type == LLMP_TYPE_Q8_0) {
    if (d.ids != nullptr || d.tokens < 2 || d.tokens > 8 || d.ncols_x % 256 != 0 || d.ncols_x / 128 < kRowsWaves) return false;
    if (d.stride_row % 8 != 0 || d.stride_expert % 8 != 0 || reinterpret_cast<uintptr_t>(d.w) % 16 != 0 ||
        (d.g != nullptr && reinterpret_cast<uintptr_t>(d.g) % 16 != 0))
      return false;
    return (d.tokens <= 4 ? SpanFor<4>(d.ncols_x / 128, 4, parts) : SpanFor<8>(d.ncols_x / 128, 4, parts)) >= 0;
  }
  if (type != LLMP_TYPE_Q4_K || d.ids != nullptr || d.tokens < 2 || d.tokens > 8) return false;
  const int nsb = d.ncols_x / 256;
  if (nsb < kRowsWaves) return false;
  return (d.tokens <= 4 ? SpanFor<4>(nsb, 8, parts) : SpanFor<8>(nsb, 8, parts)) >= 0;
}

// The same over relaid-out weights: whole tiles of packed rows. Q8_0 has this form alone (rows of whole units of four
// blocks, at least four of them).
bool RowsTiledTakes(int type, const llmp_vecq_desc& d) {
  if (type == LLMP_TYPE_Q8_0) {
    if (d.ids != nullptr || d.tokens < 2 || d.tokens > 8 || d.ncols_x % 128 != 0 || d.ncols_x / 128 < kRowsWaves) return false;
    if ((d.tokens <= 4 ? SpanFor<4>(d.ncols_x / 128, 4) : SpanFor<8>(d.ncols_x / 128, 4)) < 0) return false;
    return d.nrows % kTileRows == 0 && d.stride_row == d.ncols_x / 32 && d.stride_expert % (kTileRows * (d.ncols_x / 32)) == 0;
  }
  return type == LLMP_TYPE_Q4_K && RowsTakes(type, d, 1) && d.nrows % kTileRows == 0 && d.stride_row == d.ncols_x / 256 &&
         d.stride_expert % (kTileRows * (d.ncols_x / 256)) == 0;
}

void LaunchRows(const VecQArgs& whole, hipStream_t stream) {
  VecQArgs a = whole;
  const llmp_vecq_desc& d = a.d;
  if (g_rows_compute_units == 0) {
    const int cus = llmp_hip_compute_units();
    g_rows_compute_units = cus > 0 ? cus : 256;
  }
  if (a.parts == 0) a.parts = RowsParts(a, g_rows_compute_units);
  if (d.tokens > 8) {
    // Equal shares of eight tokens or fewer, a launch each (the weights read once a launch): for rows too long for the
    // 16 x 16 form, whose other choice is a pass for every four tokens.
    const int launches = (d.tokens + 7) / 8, share = (d.tokens + launches - 1) / launches;
    for (int first = 0; first < d.tokens; first += share) {
      VecQArgs some = a;
      some.d.tokens = min(share, d.tokens - first);
      some.d.y = static_cast<const uint8_t*>(d.y) + static_cast<int64_t>(first) * d.y_token * kQ8Block;
      some.d.dst = d.dst + static_cast<int64_t>(first) * d.dst_token;
      LaunchRows(some, stream);
    }
    return;
  }
  const int tile_rows = kTileRows / a.parts;
  const int tiles = (d.nrows + tile_rows - 1) / tile_rows;
  int groups = g_rows_compute_units / d.used;
  if (groups < 1) groups = 1;
  if (groups > tiles) groups = tiles;
  const dim3 grid(static_cast<unsigned>(groups), static_cast<unsigned>(d.used));
  const bool glu = d.g != nullptr;
  if (d.tokens <= 4) {
    glu ? LaunchRowsStages<true, 4>(a, grid, stream) : LaunchRowsStages<false, 4>(a, grid, stream);
  } else {
    glu ? LaunchRowsStages<true, 8>(a, grid, stream) : LaunchRowsStages<false, 8>(a, grid, stream);
  }
}

}  // namespace llmp_hip

extern "C" int llmp_hip_relayout_q4_k_tiles64(const void* src, void* dst, int64_t nrows, int64_t blocks_per_row, int inverse, void* stream) {
  using namespace llmp_hip;
  BeginLaunches();
  if (src == nullptr || dst == nullptr || src == dst) return Refuse(1, "relayout: null operands, or in place");
  if (nrows < 1 || nrows % kTileRows != 0 || blocks_per_row < 1 || blocks_per_row > INT32_MAX)
    return Refuse(1, "relayout: rows in whole tiles of %d and at least a block a row, not %lld x %lld", kTileRows, (long long)nrows, (long long)blocks_per_row);
  if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) % 16 != 0) return Refuse(1, "relayout: operands at 16-byte boundaries");
  const uintptr_t a = reinterpret_cast<uintptr_t>(src), b = reinterpret_cast<uintptr_t>(dst);
  const uint64_t bytes = static_cast<uint64_t>(nrows) * static_cast<uint64_t>(blocks_per_row) * 144u;
  if (a < b + bytes && b < a + bytes) return Refuse(1, "relayout: the source and the destination overlap");
  const int64_t chunks = static_cast<int64_t>(bytes / 16);
  hipLaunchKernelGGL(RelayoutTiles64Kernel, dim3(static_cast<unsigned>((chunks + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint4*>(src), static_cast<uint4*>(dst), chunks, static_cast<int>(blocks_per_row), inverse);
  return LaunchStatus("relayout");
}

extern "C" int llmp_hip_relayout_q8_0_tiles64(const void* src, void* dst, int64_t nrows, int64_t blocks_per_row, int inverse, void* stream) {
  using namespace llmp_hip;
  BeginLaunches();
  if (src == nullptr || dst == nullptr || src == dst) return Refuse(1, "relayout: null operands, or in place");
  if (nrows < 1 || nrows % kTileRows != 0 || blocks_per_row < 4 || blocks_per_row % 4 != 0 || blocks_per_row > INT32_MAX)
    return Refuse(1, "relayout: rows in whole tiles of %d and of whole units of four blocks, not %lld x %lld", kTileRows, (long long)nrows,
                  (long long)blocks_per_row);
  // The native rows at 2-byte boundaries (their blocks are 34 bytes), the tiles at 16-byte ones (their chunks are read whole).
  if (reinterpret_cast<uintptr_t>(inverse != 0 ? dst : src) % 2 != 0 || reinterpret_cast<uintptr_t>(inverse != 0 ? src : dst) % 16 != 0)
    return Refuse(1, "relayout: the rows at 2-byte, the tiles at 16-byte boundaries");
  const uintptr_t a = reinterpret_cast<uintptr_t>(src), b = reinterpret_cast<uintptr_t>(dst);
  const uint64_t bytes = static_cast<uint64_t>(nrows) * static_cast<uint64_t>(blocks_per_row) * 34u;
  if (a < b + bytes && b < a + bytes) return Refuse(1, "relayout: the source and the destination overlap");
  const int64_t units_all = nrows * (blocks_per_row / 4);
  hipLaunchKernelGGL(RelayoutQ8Tiles64Kernel, dim3(static_cast<unsigned>((units_all + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint16_t*>(src), static_cast<uint16_t*>(dst), units_all, static_cast<int>(blocks_per_row / 4), inverse);
  return LaunchStatus("relayout");
}
