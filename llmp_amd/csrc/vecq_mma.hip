// llmp.vecq over Q4_K and Q8_0 weights for several tokens a pass: the dot products of the
// 32-value sub-blocks on the matrix cores.
//
// Q4_K (the first half of this file). A weight of sub-block g of a super-block is
// d * sc_g * q - dmin * m_g with q in 0 .. 15 and sc_g, m_g in 0 .. 63. sc_g * q is an integer
// below 1024 and a Q8_1 code an integer of 8 bits: both are exact in F16, their products and
// the sum of a sub-block's 32 products are integers below 2^24, exact in the F32 accumulator
// of v_mfma_f32_16x16x32_f16 in whatever order it adds. So one instruction gives, for 16 weight
// rows and 16 tokens, the sub-block's int32 sum already multiplied by the row's 6-bit scale
// and already a float; what is left a (token, row, sub-block) is one fma by the token's block
// scale d8:
//   main = P_0 * d8_0, then fma(P_g, d8_g, main), g = 1 .. 7;  out = fma(main, d, out)
// over a row's super-blocks in order. The minimums' part, sum over g of (dmin * m_g) *
// (d8_g * sum of the token's codes), is a plain product of a 16 x 8 by an 8 x 16 matrix a
// super-block: two v_mfma_f32_16x16x4_f32, with -dmin * m as the operand, into the same
// accumulator. A (token, row) value depends on nothing but its own token and row (a column of the
// instruction's result only on its own column of the operand), whatever else the pass holds.
//
// The weights are the instruction's first operand (a lane holds row lane % 16 and eight
// consecutive values, K group lane / 16, of the sub-block), the tokens its second; a lane of the
// result holds token lane % 16 and rows 4 (lane / 16) + q. A lane reads its row's header and
// the 32 bytes of one pair of sub-blocks straight from global memory, three super-blocks deep,
// and the row's four lanes exchange them into K groups (Transpose); a nibble becomes F16 by
// or-ing it under 0x6400 (1024 + q, or 1024 + 16 q for a high nibble in place) and one packed
// fma by the sub-block's scale takes the 1024 off and multiplies: (1024 + q) * sc - 1024 * sc,
// exact. The row scales d reach the result's layout by one more small product (the column d
// times a row of ones).
//
// The tokens' Q8_1 blocks are staged in LDS once a pass and workgroup, in operand layout:
//   codes  [super-block][sub-block][token group][K group][token] 16 bytes: eight codes as F16;
//   d8     [super-block][token group][token] 8 floats, sub-block g at g;
//   ds8    the same, d8_g * sum(codes) of sub-block g at 2 (g % 4) + g / 4 (a lane reads the
//          pair of its K group for the two small products).
// A pass takes up to TG groups of MT tokens (MT 16, in one, two or, without a GLU and for rows of
// up to four super-blocks, four groups; 8 or 4 with one group, for rows so long that sixteen
// tokens do not fit), the weights prepared once for all of them. A wave owns 16 rows (of both
// matrices with a GLU) and all of K (rows of up to eight super-blocks) or one half of it (two
// waves a tile, meeting in LDS).
//
// On this chip the vector unit and the matrix cores of a SIMD do not run at the same time (448
// fma and 32 of these products a wave take the sum of their separate times at one, two and four
// waves a SIMD): a step costs its vector instructions at 4 cycles plus its matrix instructions at
// 16 (F16) and 32 (F32) cycles, and most of it is preparing the weight operand, which is why a
// pass takes as many tokens as LDS holds. Sorted rows (an expert's rows, any number) are shared
// among the workgroups by cost, not by expert: see the kernel.

#include <hip/hip_runtime.h>

#include "common.h"
#include "llmp_hip.h"
#include "vecq_common.h"

namespace llmp_hip {
namespace {

constexpr int kMmaGroup = 512;
constexpr int kMmaWaves = kMmaGroup / kWave;
constexpr int kMmaTokens = 16;                       // a token group: the instruction's columns
constexpr int kTilesGroup = kMmaWaves / 2;           // row tiles a workgroup: two waves a tile
constexpr int kWholeRow = 8;                         // super-blocks a row up to which a wave takes all of K
constexpr int kPartialBytes = kMmaWaves * 2 * kWave * 16;  // a wave's four floats a lane and matrix
constexpr size_t kMmaLdsLimit = 160 * 1024 - 2048;

typedef int V4i __attribute__((ext_vector_type(4)));
typedef float V4f __attribute__((ext_vector_type(4)));
typedef _Float16 H2 __attribute__((ext_vector_type(2)));
typedef _Float16 H8 __attribute__((ext_vector_type(8)));

// A lane's part of one super-block of its weight row: the header and, for each pair of
// sub-blocks, the eight code bytes of its K group (low nibbles sub-block 2 p, high 2 p + 1).
// As loaded, lane (row, j) holds the whole 32 bytes of pair j instead (two 16-byte loads
// where four 8-byte ones would be needed: these scattered reads cost by the instruction), K
// group g's eight bytes in q[g]; Transpose exchanges them among the row's four lanes.
struct RowPart {
  U32x4 header;  // d, dmin, scales[12]
  uint2 q[4];
};

typedef unsigned Swapped __attribute__((ext_vector_type(2)));

__device__ __forceinline__ RowPart LoadRowPart(const uint8_t* row, int sb, int kg) {
  RowPart part;
  const uint8_t* at = row + static_cast<int64_t>(sb) * 144;
  part.header = *reinterpret_cast<const U32x4*>(at);
  const U32x4 lo = *reinterpret_cast<const U32x4*>(at + 16 + 32 * kg);
  const U32x4 hi = *reinterpret_cast<const U32x4*>(at + 32 + 32 * kg);
  part.q[0] = make_uint2(lo.x, lo.y);
  part.q[1] = make_uint2(lo.z, lo.w);
  part.q[2] = make_uint2(hi.x, hi.y);
  part.q[3] = make_uint2(hi.z, hi.w);
  return part;
}

// q[g] of the row's lane j becomes q[j] of its lane g (the lanes of a row are 16 apart): a
// 4 x 4 transpose in two rounds of row swaps, lanes 32 apart then lanes 16 apart. Every lane
// of the wave takes part.
__device__ __forceinline__ void Transpose(RowPart& part) {
  uint32_t* w = reinterpret_cast<uint32_t*>(part.q);  // q[g] = w[2 g], w[2 g + 1]
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    uint32_t x0 = w[half], x1 = w[2 + half], x2 = w[4 + half], x3 = w[6 + half];
    const Swapped a = __builtin_amdgcn_permlane32_swap(x0, x2, false, false);
    const Swapped b = __builtin_amdgcn_permlane32_swap(x1, x3, false, false);
    x0 = a.x, x2 = a.y, x1 = b.x, x3 = b.y;
    const Swapped c = __builtin_amdgcn_permlane16_swap(x0, x1, false, false);
    const Swapped e = __builtin_amdgcn_permlane16_swap(x2, x3, false, false);
    w[half] = c.x, w[2 + half] = c.y, w[4 + half] = e.x, w[6 + half] = e.y;
  }
}

__device__ __forceinline__ int64_t Pack(uint32_t lo, uint32_t hi) {
  return static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo);
}

// Two F16 from two bytes of `word` (each below 0x64's reach: the bytes go under 0x64, which
// makes 1024 + byte): `places` names the byte of the low and of the high half.
constexpr uint32_t kHalfHigh = 0x64646464u;
__device__ __forceinline__ H2 Biased(uint32_t word, uint32_t places) {
  return __builtin_bit_cast(H2, __builtin_amdgcn_perm(kHalfHigh, word, places));
}
constexpr uint32_t kBytes01 = 0x04010400u, kBytes23 = 0x04030402u;

__device__ __forceinline__ H2 Both(float v) {
  const _Float16 h = static_cast<_Float16>(v);
  return H2{h, h};
}

// The layout of a pass's staged tokens.
template <int TG, int MT>
struct Staged {
  static constexpr int kCodesSb = 8 * TG * 4 * MT * 16;  // bytes of codes a super-block
  static constexpr int kCodesBlock = TG * 4 * MT * 16;   // a sub-block of it
  static constexpr int kCodesGroup = 4 * MT * 16;        // a token group of that
  static constexpr int kScalesSb = TG * MT * 32;         // bytes of d8 (and of ds8) a super-block
  static constexpr size_t Bytes(int nsb) { return static_cast<size_t>(nsb) * (kCodesSb + 2 * kScalesSb); }
};

// What a lane keeps of one super-block of its row between the pairs of sub-blocks.
struct Prepared {
  RowPart part;  // exchanged into K groups
  uint32_t sc[2];
  float d;
};

// The first part of a super-block's step for one matrix: the exchange among the row's lanes, the header, and
// the product that does not depend on the codes: the minimums' part, subtracted from `out` as it is formed
// (the operand is -dmin * m).
template <int TG, int MT, int LIVE>
__device__ __forceinline__ void Begin(const RowPart& loaded, int kg, const uint8_t* ds8, Prepared& prepared, V4f (&out)[TG]) {
  prepared.part = loaded;
  Transpose(prepared.part);
  const Q4KHeader h = DecodeQ4KHeader(prepared.part.header);
  prepared.sc[0] = h.sc[0], prepared.sc[1] = h.sc[1];
  prepared.d = h.d;
  // The minimums of sub-blocks kg and 4 + kg.
  const float m0 = -h.dmin * static_cast<float>((h.mn[0] >> (8 * kg)) & 0xFFu);
  const float m1 = -h.dmin * static_cast<float>((h.mn[1] >> (8 * kg)) & 0xFFu);
#pragma unroll
  for (int tg = 0; tg < LIVE; ++tg) {
    const float2 s = *reinterpret_cast<const float2*>(ds8 + tg * MT * 32);
    out[tg] = __builtin_amdgcn_mfma_f32_16x16x4f32(m0, s.x, out[tg], 0, 0, 0);
    out[tg] = __builtin_amdgcn_mfma_f32_16x16x4f32(m1, s.y, out[tg], 0, 0, 0);
  }
}

// The F16 operands of pair p of a super-block: sub-block 2 p (the low nibbles) and 2 p + 1.
__device__ __forceinline__ void Operands(const Prepared& prepared, int p, H8& w_lo, H8& w_hi) {
  // 1024 + sc in both halves, less 1024: the scale of sub-block 2 p, then of 2 p + 1.
  const uint32_t word = prepared.sc[p >> 1];
  const uint32_t place_lo = 2 * (p & 1), place_hi = 2 * (p & 1) + 1;
  const H2 sc_lo = Biased(word, 0x04000400u | place_lo | (place_lo << 16)) - Both(1024.0f);
  const H2 sc_hi = Biased(word, 0x04000400u | place_hi | (place_hi << 16)) - Both(1024.0f);
  const H2 off_lo = sc_lo * Both(-1024.0f);
  const H2 by_hi = sc_hi * Both(0.0625f);  // a high nibble in place is 16 q
  const H2 off_hi = sc_hi * Both(-64.0f);
  H2 lo[4], hi[4];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const uint32_t w = i == 0 ? prepared.part.q[p].x : prepared.part.q[p].y;
    const uint32_t low = w & 0x0F0F0F0Fu, high = w & 0xF0F0F0F0u;
    lo[2 * i] = __builtin_elementwise_fma(Biased(low, kBytes01), sc_lo, off_lo);
    lo[2 * i + 1] = __builtin_elementwise_fma(Biased(low, kBytes23), sc_lo, off_lo);
    hi[2 * i] = __builtin_elementwise_fma(Biased(high, kBytes01), by_hi, off_hi);
    hi[2 * i + 1] = __builtin_elementwise_fma(Biased(high, kBytes23), by_hi, off_hi);
  }
  w_lo = __builtin_shufflevector(__builtin_shufflevector(lo[0], lo[1], 0, 1, 2, 3),
                                 __builtin_shufflevector(lo[2], lo[3], 0, 1, 2, 3), 0, 1, 2, 3, 4, 5, 6, 7);
  w_hi = __builtin_shufflevector(__builtin_shufflevector(hi[0], hi[1], 0, 1, 2, 3),
                                 __builtin_shufflevector(hi[2], hi[3], 0, 1, 2, 3), 0, 1, 2, 3, 4, 5, 6, 7);
}

// Pair p of one matrix against the token operands: two products a live group, each an fma by the token's
// block scale into `main`.
template <int LIVE>
__device__ __forceinline__ void Pair(const Prepared& prepared, int p, const H8 (&t_lo)[LIVE], const H8 (&t_hi)[LIVE],
                                     const float2 (&s)[LIVE], float (&main)[LIVE][4]) {
  const V4f zero = {0.0f, 0.0f, 0.0f, 0.0f};
  H8 w_lo, w_hi;
  Operands(prepared, p, w_lo, w_hi);
#pragma unroll
  for (int tg = 0; tg < LIVE; ++tg) {
    const V4f a_lo = __builtin_amdgcn_mfma_f32_16x16x32_f16(w_lo, t_lo[tg], zero, 0, 0, 0);
    const V4f a_hi = __builtin_amdgcn_mfma_f32_16x16x32_f16(w_hi, t_hi[tg], zero, 0, 0, 0);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      main[tg][q] = p == 0 ? a_lo[q] * s[tg].x : fmaf(a_lo[q], s[tg].x, main[tg][q]);
      main[tg][q] = fmaf(a_hi[q], s[tg].y, main[tg][q]);
    }
  }
}

// The last part: the super-block's sums times the row scales, which reach the result's layout (rows
// 4 (lane / 16) + q) by a small product of their own: the column d times a row of ones.
template <int TG, int LIVE>
__device__ __forceinline__ void End(const Prepared& prepared, int kg, const float (&main)[LIVE][4], V4f (&out)[TG]) {
  const V4f zero = {0.0f, 0.0f, 0.0f, 0.0f};
  const V4f rows = __builtin_amdgcn_mfma_f32_16x16x4f32(kg == 0 ? prepared.d : 0.0f, 1.0f, zero, 0, 0, 0);
#pragma unroll
  for (int tg = 0; tg < LIVE; ++tg) {
    const V4f before = out[tg];
    out[tg] = V4f{fmaf(main[tg][0], rows[0], before[0]), fmaf(main[tg][1], rows[1], before[1]),
                  fmaf(main[tg][2], rows[2], before[2]), fmaf(main[tg][3], rows[3], before[3])};
  }
}

// One super-block of the up (and gate) matrix times the staged tokens: this lane's token of every live group, rows
// 4 (lane / 16) + q. `codes`, `d8`, `ds8`: this lane's places in the super-block's staged tokens; LIVE: the token
// groups the pass holds (a constant: a branch a group would cut the step into pieces). A pair of sub-blocks at a
// time, both matrices against the same token operands (read from LDS once), one matrix after the other, the
// compiler kept from moving work between them: the matrix cores and the vector unit do not run at the same
// time on this chip, so there is nothing to gain from interleaving further, and holding more operands and
// results at once costs registers the kernel does not have.
template <bool kGlu, int TG, int MT, int LIVE>
__device__ __forceinline__ void DotStep(const RowPart& up, const RowPart& gate, int kg, const uint8_t* codes, const uint8_t* d8,
                                        const uint8_t* ds8, V4f (&up_out)[TG], V4f (&gate_out)[TG]) {
  using L = Staged<TG, MT>;
  Prepared pu, pg;
  Begin<TG, MT, LIVE>(up, kg, ds8, pu, up_out);
  if constexpr (kGlu) Begin<TG, MT, LIVE>(gate, kg, ds8, pg, gate_out);
  float up_main[LIVE][4], gate_main[LIVE][4];
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    H8 t_lo[LIVE], t_hi[LIVE];
    float2 s[LIVE];
#pragma unroll
    for (int tg = 0; tg < LIVE; ++tg) {
      t_lo[tg] = *reinterpret_cast<const H8*>(codes + (2 * p) * L::kCodesBlock + tg * L::kCodesGroup);
      t_hi[tg] = *reinterpret_cast<const H8*>(codes + (2 * p + 1) * L::kCodesBlock + tg * L::kCodesGroup);
      s[tg] = *reinterpret_cast<const float2*>(d8 + tg * MT * 32 + p * 8);
    }
    Pair<LIVE>(pu, p, t_lo, t_hi, s, up_main);
    if constexpr (kGlu) {
      __builtin_amdgcn_sched_barrier(0);
      Pair<LIVE>(pg, p, t_lo, t_hi, s, gate_main);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  End<TG, LIVE>(pu, kg, up_main, up_out);
  if constexpr (kGlu) End<TG, LIVE>(pg, kg, gate_main, gate_out);
}

// One Q8_1 block of a token into the operand layout.
template <int TG, int MT>
__device__ __forceinline__ void StageBlock(const uint32_t (&w)[9], int t, int b, uint8_t* codes, uint8_t* d8, uint8_t* ds8) {
  using L = Staged<TG, MT>;
  const int tg = t / MT, token = t - tg * MT;
  const int sb = b >> 3, g = b & 7;
  uint8_t* to = codes + sb * L::kCodesSb + g * L::kCodesBlock + tg * L::kCodesGroup + token * 16;
#pragma unroll
  for (int kg = 0; kg < 4; ++kg) {
    // A code plus 128 is a byte: 1024 + 128 + code under 0x64, less 1152.
    const uint32_t a = w[1 + 2 * kg] ^ 0x80808080u, c = w[2 + 2 * kg] ^ 0x80808080u;
    const H2 h0 = Biased(a, kBytes01) - Both(1152.0f), h1 = Biased(a, kBytes23) - Both(1152.0f);
    const H2 h2 = Biased(c, kBytes01) - Both(1152.0f), h3 = Biased(c, kBytes23) - Both(1152.0f);
    U32x4 packed;
    packed.x = __builtin_bit_cast(uint32_t, h0), packed.y = __builtin_bit_cast(uint32_t, h1);
    packed.z = __builtin_bit_cast(uint32_t, h2), packed.w = __builtin_bit_cast(uint32_t, h3);
    *reinterpret_cast<U32x4*>(to + kg * MT * 16) = packed;
  }
  int sum = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) sum = Dot4(0x01010101, static_cast<int>(w[1 + i]), sum);
  const float scale = HalfBitsToFloat(w[0] & 0xFFFFu);
  const int at = sb * L::kScalesSb + (tg * MT + token) * 32;
  *reinterpret_cast<float*>(d8 + at + g * 4) = scale;
  *reinterpret_cast<float*>(ds8 + at + (2 * (g & 3) + (g >> 2)) * 4) = scale * static_cast<float>(sum);
}

constexpr int kStageAhead = 4;  // blocks a thread holds in registers between their loads and their staging

// The work of a workgroup between two stagings of tokens: tokens first .. first + m - 1 of the rows
// listed for `expert` against its row tiles' groups group_first, group_first + group_step, ...
// (group_count of them).
struct Segment {
  int expert, first, m, group_first, group_step, group_count;
};

// grid (workgroups, slots), or (workgroups) with `balanced` (sorted rows: the workgroups share the
// passes of all experts evenly, whatever the experts' row counts); LDS: codes, d8, ds8, the waves'
// partial sums.
template <bool kGlu, int TG, int MT>
__global__ __launch_bounds__(kMmaGroup, 1) void VecQMma(const VecQArgs a, int balanced) {
  using L = Staged<TG, MT>;
  constexpr int kDepth = TG == 1 ? 3 : TG == 2 ? 3 : 2;  // weight buffers: the fetches run kDepth - 1 steps ahead
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  __shared__ int pairs[kMaxPairs];
  __shared__ int count;
  __shared__ int scan[kMmaGroup / kWave];

  const llmp_vecq_desc& d = a.d;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int nsb = d.ncols_x / 256;
  const int blocks = d.ncols_x / 32;
  uint8_t* codes = lds;
  uint8_t* d8 = lds + nsb * L::kCodesSb;
  uint8_t* ds8 = d8 + nsb * L::kScalesSb;
  float4* partial = reinterpret_cast<float4*>(ds8 + nsb * L::kScalesSb);

  // This wave's part of K. Rows of up to eight super-blocks: all of it, a tile a wave (too few
  // steps to be worth two waves and their meeting). Longer rows: a half.
  const bool whole = nsb <= kWholeRow;
  const int half = whole ? 0 : wave & 1;
  const int first = half == 0 ? 0 : (nsb + 1) / 2;
  const int last = whole || half == 1 ? nsb : (nsb + 1) / 2;
  const int row_in_tile = lane & 15, kg = lane >> 4;
  const int token_in_group = lane & (MT - 1);
  const int tiles = (d.nrows + 15) / 16;
  const int tiles_group = whole ? kMmaWaves : kTilesGroup;
  const int tile_in_group = whole ? wave : wave >> 1;
  const int groups = (tiles + tiles_group - 1) / tiles_group;

  const uint8_t* my_codes = codes + (kg * MT + token_in_group) * 16;
  const uint8_t* my_d8 = d8 + token_in_group * 32;
  const uint8_t* my_ds8 = ds8 + token_in_group * 32 + kg * 8;

  int sorted_first = 0;
  auto pair_at = [&](int i) { return a.offsets != nullptr ? (sorted_first + i) << 8 : pairs[i]; };

  bool staged_before = false;
  auto run = [&](const Segment& seg) {
    const int64_t expert_block = static_cast<int64_t>(seg.expert) * d.stride_expert;
    const int p0 = seg.first, m = seg.m;
    const int steps = seg.group_count * (last - first);
    // The live token groups rounded up to a power of two: one compiled step each.
    const int token_groups = (m + MT - 1) / MT;
    const int live = token_groups <= 1 ? 1 : token_groups <= 2 ? 2 : 4;

    // The tokens' blocks are asked for before the weights (loads return in order, and the tokens are
    // needed whole before the first step), staged after the first weights are.
    if (staged_before) __syncthreads();  // the last segment's readers of the staged tokens
    staged_before = true;
    const int staged = min(live, TG) * MT * blocks;
    auto row_of = [&](int j) {
      const int pr = pair_at(p0 + min(j, m - 1));  // tokens past m repeat the last: computed and dropped
      return static_cast<const uint8_t*>(d.y) +
             (static_cast<int64_t>(pr >> 8) * d.y_token + static_cast<int64_t>(pr & 0xFF) * d.y_slot) * kQ8Block;
    };
    uint32_t held[kStageAhead][9];
#pragma unroll
    for (int it = 0; it < kStageAhead; ++it) {
      const int index = tid + it * kMmaGroup;
      if (index < staged) {
        const int t = index / blocks, b = index - t * blocks;
        const uint32_t* src = reinterpret_cast<const uint32_t*>(row_of(t) + static_cast<int64_t>(b) * kQ8Block);
#pragma unroll
        for (int i = 0; i < 9; ++i) held[it][i] = src[i];
      }
    }
    __builtin_amdgcn_sched_barrier(0);

    // The fetches run kDepth - 1 steps ahead of the products, through the segment's tiles in order.
    const uint8_t* up_row = nullptr;
    const uint8_t* gate_row = nullptr;
    int fetch_group = seg.group_first, fetch_sb = first, fetched = 0;
    auto aim = [&]() {
      const int row = min((fetch_group * tiles_group + tile_in_group) * 16 + row_in_tile, d.nrows - 1);
      const int64_t at = (expert_block + static_cast<int64_t>(row) * d.stride_row) * 144;
      up_row = static_cast<const uint8_t*>(d.w) + at;
      if constexpr (kGlu) gate_row = static_cast<const uint8_t*>(d.g) + at;
    };
    // The loads are queued here and no later: the compiler would otherwise sink them to their
    // first use, steps on, and the wave would wait out the whole memory latency there. Past the
    // segment's end its last part again: a load under a branch would make every wait for loads a wait for
    // all of them (the count of loads in flight is not known where branches join).
    auto fetch = [&](RowPart& u, RowPart& g) {
      u = LoadRowPart(up_row, fetch_sb, kg);
      if constexpr (kGlu) g = LoadRowPart(gate_row, fetch_sb, kg);
      __builtin_amdgcn_sched_barrier(0);
      if (++fetched < steps && ++fetch_sb == last) {
        fetch_sb = first;
        fetch_group += seg.group_step;
        aim();
      }
    };
    RowPart ub[kDepth], gb[kDepth];
    aim();
#pragma unroll
    for (int j = 0; j < kDepth - 1; ++j) fetch(ub[j], gb[j]);

#pragma unroll
    for (int it = 0; it < kStageAhead; ++it) {
      const int index = tid + it * kMmaGroup;
      if (index < staged) {
        const int t = index / blocks, b = index - t * blocks;
        StageBlock<TG, MT>(held[it], t, b, codes, d8, ds8);
      }
    }
    for (int index = tid + kStageAhead * kMmaGroup; index < staged; index += kMmaGroup) {
      const int t = index / blocks, b = index - t * blocks;
      const uint32_t* src = reinterpret_cast<const uint32_t*>(row_of(t) + static_cast<int64_t>(b) * kQ8Block);
      uint32_t w[9];
#pragma unroll
      for (int i = 0; i < 9; ++i) w[i] = src[i];
      StageBlock<TG, MT>(w, t, b, codes, d8, ds8);
    }
    __syncthreads();

    V4f up_out[TG], gate_out[TG];
    auto clear = [&]() {
#pragma unroll
      for (int tg = 0; tg < TG; ++tg) up_out[tg] = V4f{0.0f, 0.0f, 0.0f, 0.0f}, gate_out[tg] = up_out[tg];
    };
    clear();
    int group = seg.group_first, sb = first;
    // A tile's rows are done: the two halves of K meet (the upper half's sums through LDS),
    // and the lower half's wave stores.
    auto finish = [&]() {
#pragma clang fp contract(off)
      const int tile = group * tiles_group + tile_in_group;
      float4* slot = partial + ((wave >> 1) * 2 * TG) * kWave + lane;  // a tile's
      if (half == 1) {
#pragma unroll
        for (int tg = 0; tg < TG; ++tg) {
          const V4f u = up_out[tg];
          slot[(2 * tg) * kWave] = make_float4(u[0], u[1], u[2], u[3]);
          if constexpr (kGlu) {
            const V4f g = gate_out[tg];
            slot[(2 * tg + 1) * kWave] = make_float4(g[0], g[1], g[2], g[3]);
          }
        }
      }
      if (!whole) __syncthreads();
      if (half == 0 && tile < tiles) {
#pragma unroll
        for (int tg = 0; tg < TG; ++tg) {
          V4f u = up_out[tg], g = gate_out[tg];
          if (!whole) {
            const float4 x = slot[(2 * tg) * kWave];
            u[0] += x.x, u[1] += x.y, u[2] += x.z, u[3] += x.w;
            if constexpr (kGlu) {
              const float4 y = slot[(2 * tg + 1) * kWave];
              g[0] += y.x, g[1] += y.y, g[2] += y.z, g[3] += y.w;
            }
          }
          const int t = tg * MT + row_in_tile;  // this lane's token of the group, when the group has it
          if (row_in_tile < MT && t < m) {
            const int pr = pair_at(p0 + t);
            float* dst = d.dst + static_cast<int64_t>(pr >> 8) * d.dst_token + static_cast<int64_t>(pr & 0xFF) * d.dst_slot;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int row = tile * 16 + 4 * kg + q;
              if (row < d.nrows) dst[row] = kGlu ? Glu(d.glu, g[q], u[q], d.limit) : u[q];
            }
          }
        }
      }
      if (!whole) __syncthreads();  // the partial sums may be overwritten
      clear();
    };
    auto step = [&](const RowPart& u, const RowPart& g) {
      const uint8_t* c = my_codes + sb * L::kCodesSb;
      const uint8_t* s8 = my_d8 + sb * L::kScalesSb;
      const uint8_t* ds = my_ds8 + sb * L::kScalesSb;
      if (TG == 1 || live >= TG) {
        DotStep<kGlu, TG, MT, TG>(u, g, kg, c, s8, ds, up_out, gate_out);
      } else if (TG == 4 && live == 2) {
        DotStep<kGlu, TG, MT, TG == 4 ? 2 : 1>(u, g, kg, c, s8, ds, up_out, gate_out);
      } else {
        DotStep<kGlu, TG, MT, 1>(u, g, kg, c, s8, ds, up_out, gate_out);
      }
      if (++sb == last) {
        finish();
        sb = first;
        group += seg.group_step;
      }
    };
    for (int s = 0; s < steps; s += kDepth) {
#pragma unroll
      for (int j = 0; j < kDepth; ++j) {
        if (j == 0 || s + j < steps) {
          fetch(ub[(j + kDepth - 1) % kDepth], gb[(j + kDepth - 1) % kDepth]);
          step(ub[j], gb[j]);
        }
      }
    }
  };

  if (balanced == 0) {
    int expert = blockIdx.y;
    if (a.offsets != nullptr) {
      sorted_first = a.offsets[expert];
      if (tid == 0) count = a.offsets[expert + 1] - sorted_first;
      __syncthreads();
    } else {
      expert = ResolvePairs(d, blockIdx.y, pairs, &count);
    }
    const int n = count;
    const int mine = (groups - static_cast<int>(blockIdx.x) + static_cast<int>(gridDim.x) - 1) / static_cast<int>(gridDim.x);
    for (int p0 = 0; p0 < n; p0 += TG * MT)
      run(Segment{expert, p0, min(TG * MT, n - p0), static_cast<int>(blockIdx.x), static_cast<int>(gridDim.x), mine});
  } else {
    // Sorted rows, shared evenly: expert e brings ceil(rows / (TG MT)) passes, a pass `groups` groups of
    // tiles, and a group of a pass costs by the pass's live token groups (Cost). The groups of all passes in
    // expert order lie end to end on a line of cost, and workgroup w takes the groups that start within its
    // W-th of the line: a few segments of consecutive groups.
    const int experts = d.used;
    constexpr int kPass = TG * MT;
    auto live_of = [](int m) {
      const int token_groups = (m + MT - 1) / MT;
      return token_groups <= 1 ? 1 : token_groups <= 2 ? 2 : 4;
    };
    // A step's instructions: about 12 parts for the weights and 7 a live token group.
    auto cost_of = [](int live) { return 12 + 7 * min(live, TG); };
    auto expert_cost = [&](int rows) {
      if (rows <= 0) return 0;
      const int passes = (rows + kPass - 1) / kPass;
      return (passes - 1) * cost_of(TG) + cost_of(live_of(rows - (passes - 1) * kPass));
    };
    int* walk = pairs;  // [0] all experts' cost, [1] the first expert with groups of this workgroup, [2] the cost
                        // before it, [3] the last such expert
    if (tid == 0) walk[0] = 0, walk[1] = experts, walk[2] = 0, walk[3] = -1;
    __syncthreads();
    for (int base = 0; base < experts; base += kMmaGroup) {
      const int e = base + tid;
      int cost = e < experts ? expert_cost(a.offsets[e + 1] - a.offsets[e]) : 0;
#pragma unroll
      for (int delta = kWave / 2; delta >= 1; delta /= 2) cost += ShflXor(cost, delta);
      if (lane == 0 && cost != 0) atomicAdd(&walk[0], cost);
    }
    __syncthreads();
    const int64_t line = static_cast<int64_t>(walk[0]) * groups;
    const int64_t from = line * blockIdx.x / gridDim.x, to = line * (blockIdx.x + 1) / gridDim.x;
    int carried = 0;  // cost of the experts before this round of kMmaGroup
    for (int base = 0; base < experts; base += kMmaGroup) {
      const int e = base + tid;
      const int cost = e < experts ? expert_cost(a.offsets[e + 1] - a.offsets[e]) : 0;
      int inclusive = cost;  // over the wave, then over the workgroup
#pragma unroll
      for (int delta = 1; delta < kWave; delta *= 2) {
        const int other = __shfl_up(inclusive, delta, kWave);
        if (lane >= delta) inclusive += other;
      }
      __syncthreads();  // the last round's readers of scan
      if (lane == kWave - 1) scan[wave] = inclusive;
      __syncthreads();
      int before = carried;
      for (int w = 0; w < kMmaGroup / kWave; ++w) {
        if (w < wave) before += scan[w];
        carried += scan[w];
      }
      const int exclusive = before + inclusive - cost;
      const bool mine = cost != 0 && max(from, static_cast<int64_t>(exclusive) * groups) <
                                         min(to, static_cast<int64_t>(exclusive + cost) * groups);
      if (mine) {
        atomicMin(&walk[1], e);
        atomicMax(&walk[3], e);
      }
      __syncthreads();
      if (mine && walk[1] == e) walk[2] = exclusive;
    }
    __syncthreads();
    const int e_first = walk[1], e_last = walk[3];
    int before = walk[2];
    __syncthreads();  // pairs is free again
    for (int e = e_first; e <= e_last; ++e) {
      sorted_first = a.offsets[e];
      const int rows = a.offsets[e + 1] - sorted_first;
      for (int p0 = 0; p0 < rows; p0 += kPass) {
        const int m = min(kPass, rows - p0);
        const int cost = cost_of(live_of(m));
        // The pass's groups start at start, start + cost, ...: those within [from, to).
        const int64_t start = static_cast<int64_t>(before) * groups;
        const int g_first = from <= start ? 0 : static_cast<int>((from - start + cost - 1) / cost);
        const int g_end = to <= start ? 0 : static_cast<int>(min<int64_t>((to - start + cost - 1) / cost, groups));
        if (g_first < g_end) run(Segment{e, p0, m, g_first, 1, g_end - g_first});
        before += cost;
      }
    }
  }
}

// ------------------------------------------------------------------ Q8_0
//
// The same instruction over Q8_0 blocks: its K is a block, a product the block's int32 sum.
// The float operations are the one-token kernel's: over a unit of four blocks
//   v = float(s_0) * (dw_0 * d8_0), then v = fma(float(s_j), dw_j * d8_j, v), j = 1 .. 3,
// and a row's units are added in that kernel's tree. A tile of 16 rows is taken by four waves,
// each a quarter of the tree's leaves (the next power of two at or above the row's units, cut in
// four aligned runs of up to sixteen units), which meet in LDS.
//
// A lane reads its row's weights straight into the operand layout: of every pair of blocks
// (68 bytes, so 4-byte aligned in a row of whole pairs) the eight codes of its K group in the
// even block lie two bytes into three dwords, those of the odd block in two dwords. The tokens
// are staged once a workgroup:
//   codes   [block][K group][token] 8 bytes (a wave's read is a contiguous 512 bytes);
//   scales  [block][token] F32, a lane reading its four tokens' 16 bytes.

// Sums of a row's units in the order of the one-token kernel's shuffle tree: aligned
// pairs first, then pairs of pairs, .... The kernel adds each aligned group of four itself;
// the groups of four then go through a binary counter's carries, which builds the
// rest of the same tree: l2 holds a finished group of four waiting for its neighbour, l3 one
// of eight, l4 one of sixteen. Everything is selects on values the same in every lane, so
// that the levels stay in registers.
struct TreeSum {
  float l2[4], l3[4], l4[4];
};

__device__ __forceinline__ void Sum4(const float (&a)[4], const float (&b)[4], float (&out)[4]) {
#pragma clang fp contract(off)
#pragma unroll
  for (int q = 0; q < 4; ++q) out[q] = a[q] + b[q];
}

// `index`: the group's place counted from the first pushed.
__device__ __forceinline__ void Push(TreeSum& t, const float (&v)[4], int index) {
#pragma unroll
  for (int q = 0; q < 4; ++q) {
#pragma clang fp contract(off)
    const float c2 = v[q];
    const float c3 = t.l2[q] + c2;
    const float c4 = t.l3[q] + c3;
    t.l2[q] = (index & 1) == 0 ? c2 : t.l2[q];
    t.l3[q] = (index & 3) == 1 ? c3 : t.l3[q];
    t.l4[q] = (index & 3) == 3 ? c4 : t.l4[q];
  }
}

// The total of `count` pushed groups (1 to 4): the unfinished ones from the smallest up.
__device__ __forceinline__ void Total(const TreeSum& t, int count, float (&out)[4]) {
#pragma unroll
  for (int q = 0; q < 4; ++q) {
#pragma clang fp contract(off)
    float v = 0.0f;
    bool any = false;
    if (count & 1) v = t.l2[q], any = true;
    if (count & 2) v = any ? t.l3[q] + v : t.l3[q], any = true;
    if (count & 4) v = t.l4[q];  // four groups: nothing else is pending
    out[q] = v;
  }
}

constexpr int kQ8CodesBlock = 4 * kMmaTokens * 8;  // 512 bytes of codes a block
constexpr int kQ8ScalesBlock = kMmaTokens * 4;     // 64 bytes of scales a block
constexpr int kQ8Chunks = 4;                       // waves a tile
constexpr int kQ8Tiles = kMmaWaves / kQ8Chunks;    // tiles a workgroup at a time

struct __attribute__((packed, aligned(4))) Dwords3 {
  uint32_t a, b, c;
};

// A lane's part of one unit (four blocks, 136 bytes) of its weight row. The blocks' F16 scales
// lie in what the row's first and last K group read anyway (bytes 0-1 of a pair in the first's
// even dwords, bytes 34-35 in the last's) and reach the row's other lanes by a lane exchange:
// fewer memory requests, which bound this access pattern.
struct UnitPart {
  Dwords3 even[2];  // bytes 8 kg .. 8 kg + 11 of each pair: the even block's codes from byte 2
  uint2 odd[2];     // bytes 36 + 8 kg .. of each pair: the odd block's codes
};

__device__ __forceinline__ UnitPart LoadUnitPart(const uint8_t* row, int unit, int kg) {
  UnitPart part;
  const uint8_t* at = row + static_cast<int64_t>(unit) * 136;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    part.even[i] = *reinterpret_cast<const Dwords3*>(at + 68 * i + 8 * kg);
    part.odd[i] = *reinterpret_cast<const uint2*>(at + 68 * i + 36 + 8 * kg);
  }
  return part;
}

// One unit of one matrix times the staged tokens: four tokens of this lane's row.
__device__ __forceinline__ void DotUnit(const UnitPart& part, const uint8_t* codes, const uint8_t* scales, int unit,
                                        int lane, float (&out)[4]) {
#pragma clang fp contract(off)
  const int kg = lane >> 4;
  // The even blocks' scales from the row's lane of K group 0, the odd blocks' from K group 3's.
  const uint32_t evens = __shfl((part.even[0].a & 0xFFFFu) | (part.even[1].a << 16), lane & 15, kWave);
  const uint32_t odds = __shfl((part.even[0].c >> 16) | (part.even[1].c & 0xFFFF0000u), (lane & 15) + 48, kWave);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    int64_t weights;
    const uint32_t both = (j & 1) == 0 ? evens : odds;
    const float dw = HalfBitsToFloat((j >> 1) == 0 ? both & 0xFFFFu : both >> 16);
    if ((j & 1) == 0) {
      const Dwords3& e = part.even[j >> 1];
      weights = Pack(__builtin_amdgcn_alignbit(e.b, e.a, 16), __builtin_amdgcn_alignbit(e.c, e.b, 16));
    } else {
      weights = Pack(part.odd[j >> 1].x, part.odd[j >> 1].y);
    }
    const int block = 4 * unit + j;
    const int64_t tokens = *reinterpret_cast<const int64_t*>(codes + block * kQ8CodesBlock + lane * 8);
    const float4 d8 = *reinterpret_cast<const float4*>(scales + block * kQ8ScalesBlock + kg * 16);
    const V4i zero = {0, 0, 0, 0};
    const V4i prod = __builtin_amdgcn_mfma_i32_16x16x32_i8(tokens, weights, zero, 0, 0, 0);
    const float d[4] = {d8.x, d8.y, d8.z, d8.w};
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      out[q] = j == 0 ? static_cast<float>(prod[q]) * (dw * d[q]) : fmaf(static_cast<float>(prod[q]), dw * d[q], out[q]);
    }
  }
}

template <class RowOf>
__device__ __forceinline__ void StageTokensQ8(RowOf row_of, int m, int blocks, uint8_t* codes, uint8_t* scales) {
  for (int index = threadIdx.x; index < m * blocks; index += kMmaGroup) {
    const int j = index / blocks, b = index - j * blocks;
    const uint32_t* src = reinterpret_cast<const uint32_t*>(row_of(j) + static_cast<int64_t>(b) * kQ8Block);
    uint32_t w[9];
#pragma unroll
    for (int i = 0; i < 9; ++i) w[i] = src[i];
#pragma unroll
    for (int kg = 0; kg < 4; ++kg) {
      *reinterpret_cast<uint2*>(codes + b * kQ8CodesBlock + (kg * kMmaTokens + j) * 8) =
          make_uint2(w[1 + 2 * kg], w[2 + 2 * kg]);
    }
    *reinterpret_cast<float*>(scales + b * kQ8ScalesBlock + j * 4) = HalfBitsToFloat(w[0] & 0xFFFFu);
  }
}

// grid (workgroups, slots); LDS: codes, scales, the waves' partial sums.
template <bool kGlu>
__global__ __launch_bounds__(kMmaGroup, 1) void VecQMmaQ8(const VecQArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  __shared__ int pairs[kMaxPairs];
  __shared__ int count;

  const llmp_vecq_desc& d = a.d;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int blocks = d.ncols_x / 32;
  const int units = blocks / 4;
  uint8_t* codes = lds;
  uint8_t* scales = lds + blocks * kQ8CodesBlock;
  float4* partial = reinterpret_cast<float4*>(lds + blocks * (kQ8CodesBlock + kQ8ScalesBlock));

  int expert = blockIdx.y;
  int sorted_first = 0;
  if (a.offsets != nullptr) {
    sorted_first = a.offsets[expert];
    if (tid == 0) count = a.offsets[expert + 1] - sorted_first;
    __syncthreads();
  } else if (d.ids != nullptr) {
    expert = ResolvePairs(d, blockIdx.y, pairs, &count);
  }
  const bool listed = d.ids != nullptr && a.offsets == nullptr;
  const int n = a.offsets == nullptr && d.ids == nullptr ? d.tokens : count;
  if (n == 0) return;  // uniform over the workgroup
  auto pair_at = [&](int i) {
    return a.offsets != nullptr ? (sorted_first + i) << 8 : listed ? pairs[i] : (i << 8) | expert;
  };
  const int64_t expert_block = static_cast<int64_t>(expert) * d.stride_expert;

  // This wave's run of the row's units.
  int leaves = 1;
  while (leaves < units) leaves *= 2;
  const int run = max(leaves / kQ8Chunks, 1);
  const int chunk = wave & (kQ8Chunks - 1);
  const int first = min(chunk * run, units);
  const int last = min(first + run, units);
  const int tile_in_group = wave / kQ8Chunks;
  const int row_in_tile = lane & 15, kg = lane >> 4;
  const int tiles = (d.nrows + 15) / 16;
  const int groups = (tiles + kQ8Tiles - 1) / kQ8Tiles;

  const uint8_t* up_row = nullptr;
  const uint8_t* gate_row = nullptr;
  auto aim = [&](int group) {
    const int row = min((group * kQ8Tiles + tile_in_group) * 16 + row_in_tile, d.nrows - 1);
    const int64_t at = (expert_block + static_cast<int64_t>(row) * d.stride_row) * 34;
    up_row = static_cast<const uint8_t*>(d.w) + at;
    if constexpr (kGlu) gate_row = static_cast<const uint8_t*>(d.g) + at;
  };
  // Four units a matrix in flight; the loads are queued where they are written (past the run's
  // end the last unit again: no branch).
  UnitPart u0, u1, u2, u3, g0, g1, g2, g3;
  auto fetch = [&](int unit, UnitPart& u, UnitPart& g) {
    const int at = max(min(unit, last - 1), 0);
    u = LoadUnitPart(up_row, at, kg);
    if constexpr (kGlu) g = LoadUnitPart(gate_row, at, kg);
    __builtin_amdgcn_sched_barrier(0);
  };
  aim(blockIdx.x);
  fetch(first, u0, g0);
  fetch(first + 1, u1, g1);
  fetch(first + 2, u2, g2);
  fetch(first + 3, u3, g3);

  for (int p0 = 0; p0 < n; p0 += kMmaTokens) {
    const int m = min(kMmaTokens, n - p0);
    __syncthreads();  // the last pass's readers of the staged tokens
    auto row_of = [&](int j) {
      const int pr = pair_at(p0 + j);
      return static_cast<const uint8_t*>(d.y) +
             (static_cast<int64_t>(pr >> 8) * d.y_token + static_cast<int64_t>(pr & 0xFF) * d.y_slot) * kQ8Block;
    };
    StageTokensQ8(row_of, m, blocks, codes, scales);
    __syncthreads();

    for (int group = blockIdx.x; group < groups; group += gridDim.x) {
      const int tile = group * kQ8Tiles + tile_in_group;
      TreeSum up_sum{}, gate_sum{};
      int quads = 0;
      auto step = [&](int unit, const UnitPart& u, const UnitPart& g, float (&up_out)[4], float (&gate_out)[4]) {
        DotUnit(u, codes, scales, unit, lane, up_out);
        if constexpr (kGlu) DotUnit(g, codes, scales, unit, lane, gate_out);
      };
      if (tile < tiles) {
        for (int unit = first; unit < last; unit += 4, ++quads) {
          const int here = min(4, last - unit);
          // The quad's sum as its values come: (x0 + x1) + (x2 + x3), absent ones left out.
          float up_quad[4], gate_quad[4], up_next[4], gate_next[4];
          step(unit, u0, g0, up_quad, gate_quad);
          fetch(unit + 4, u0, g0);
          if (here >= 2) {
            step(unit + 1, u1, g1, up_next, gate_next);
            Sum4(up_quad, up_next, up_quad);
            if constexpr (kGlu) Sum4(gate_quad, gate_next, gate_quad);
          }
          fetch(unit + 5, u1, g1);
          if (here >= 3) {
            float up_rest[4], gate_rest[4];
            step(unit + 2, u2, g2, up_rest, gate_rest);
            if (here >= 4) {
              step(unit + 3, u3, g3, up_next, gate_next);
              Sum4(up_rest, up_next, up_rest);
              if constexpr (kGlu) Sum4(gate_rest, gate_next, gate_rest);
            }
            Sum4(up_quad, up_rest, up_quad);
            if constexpr (kGlu) Sum4(gate_quad, gate_rest, gate_quad);
          }
          fetch(unit + 6, u2, g2);
          fetch(unit + 7, u3, g3);
          Push(up_sum, up_quad, quads);
          if constexpr (kGlu) Push(gate_sum, gate_quad, quads);
        }
      }
      // The next group's (or the next pass's first group's) first loads.
      {
        int next = group + static_cast<int>(gridDim.x);
        if (next >= groups) next = blockIdx.x;
        aim(next);
        fetch(first, u0, g0);
        fetch(first + 1, u1, g1);
        fetch(first + 2, u2, g2);
        fetch(first + 3, u3, g3);
      }
      // The four runs meet: (r0 + r1) + (r2 + r3), absent ones left out, through LDS.
      float up_total[4] = {0.0f, 0.0f, 0.0f, 0.0f}, gate_total[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      if (tile < tiles && last > first) {
        Total(up_sum, quads, up_total);
        if constexpr (kGlu) Total(gate_sum, quads, gate_total);
      }
      float4* slot = partial + (wave * 2) * kWave + lane;
      if (chunk != 0) {
        slot[0] = make_float4(up_total[0], up_total[1], up_total[2], up_total[3]);
        if constexpr (kGlu) slot[kWave] = make_float4(gate_total[0], gate_total[1], gate_total[2], gate_total[3]);
      }
      __syncthreads();
      if (chunk == 0 && tile < tiles) {
#pragma clang fp contract(off)
        auto merge = [&](int matrix, float (&total)[4]) {
          const float4* other = partial + (wave * 2 + matrix) * kWave + lane;  // this tile's runs follow this wave
          float rest[4];
          const bool has1 = run < units, has2 = 2 * run < units, has3 = 3 * run < units;
          if (has1) {
            const float4 r1 = other[2 * kWave];
            total[0] += r1.x, total[1] += r1.y, total[2] += r1.z, total[3] += r1.w;
          }
          if (has2) {
            const float4 r2 = other[4 * kWave];
            rest[0] = r2.x, rest[1] = r2.y, rest[2] = r2.z, rest[3] = r2.w;
            if (has3) {
              const float4 r3 = other[6 * kWave];
              rest[0] += r3.x, rest[1] += r3.y, rest[2] += r3.z, rest[3] += r3.w;
            }
            total[0] += rest[0], total[1] += rest[1], total[2] += rest[2], total[3] += rest[3];
          }
        };
        merge(0, up_total);
        if constexpr (kGlu) merge(1, gate_total);
        if (tile * 16 + row_in_tile < d.nrows) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int t = 4 * kg + q;
            if (t < m) {
              const int pr = pair_at(p0 + t);
              float* dst = d.dst + static_cast<int64_t>(pr >> 8) * d.dst_token + static_cast<int64_t>(pr & 0xFF) * d.dst_slot;
              dst[tile * 16 + row_in_tile] = kGlu ? Glu(d.glu, gate_total[q], up_total[q], d.limit) : up_total[q];
            }
          }
        }
      }
      __syncthreads();  // the partial sums may be overwritten
    }
  }
}

size_t MmaLdsQ8(int blocks) {
  return static_cast<size_t>(blocks) * (kQ8CodesBlock + kQ8ScalesBlock) + kPartialBytes;
}

// The Q4_K kernel's token groups a pass (TG) and tokens a group (MT) for rows of `nsb`
// super-blocks when a slot brings up to `tokens` tokens: two groups of sixteen where more than
// sixteen may come and fit, else the smallest group that holds them all, else the largest that
// fits. 0 groups: not even four tokens fit.
struct MmaShape {
  int groups, tokens;
  size_t lds;
};

template <int TG, int MT>
bool Fits(int nsb, MmaShape* shape) {
  const size_t partial = nsb <= kWholeRow ? 0 : static_cast<size_t>(kTilesGroup) * 2 * TG * kWave * 16;
  const size_t lds = Staged<TG, MT>::Bytes(nsb) + partial;
  if (lds > kMmaLdsLimit) return false;
  *shape = MmaShape{TG, MT, lds};
  return true;
}

MmaShape ShapeFor(int nsb, int tokens, bool glu) {
  MmaShape shape{0, 0, 0};
  if (tokens > 32 && !glu && Fits<4, 16>(nsb, &shape)) return shape;  // (with a GLU: more registers than a wave has)
  if (tokens > 16 && Fits<2, 16>(nsb, &shape)) return shape;
  if (tokens <= 4 && Fits<1, 4>(nsb, &shape)) return shape;
  if (tokens <= 8 && Fits<1, 8>(nsb, &shape)) return shape;
  if (Fits<1, 16>(nsb, &shape) || Fits<1, 8>(nsb, &shape) || Fits<1, 4>(nsb, &shape)) return shape;
  return shape;
}

int g_mma_compute_units = 0;

}  // namespace


// Q4_K rows of which at least eight staged tokens fit LDS (k up to 8448; sixteen up to 4096, two
// groups of sixteen up to 2048). Q8_0 rows of whole units of 128 values, up to 64 units (8192
// values) as far as they fit LDS, whose rows, matrices and experts start on 4-byte boundaries (a
// lane reads dwords).
bool MmaTakes(int type, const llmp_vecq_desc& d) {
  if (type == LLMP_TYPE_Q4_K) {
    const int nsb = d.ncols_x / 256;
    return nsb >= 1 && ShapeFor(nsb, 8, true).tokens >= 8;
  }
  if (type != LLMP_TYPE_Q8_0 || d.ncols_x < 128 || d.ncols_x % 128 != 0 || d.ncols_x > 8192) return false;
  const uintptr_t at = reinterpret_cast<uintptr_t>(d.w) | reinterpret_cast<uintptr_t>(d.g);
  return d.stride_row % 2 == 0 && d.stride_expert % 2 == 0 && at % 4 == 0 && MmaLdsQ8(d.ncols_x / 32) <= kMmaLdsLimit;
}

namespace {

template <bool kGlu>
void LaunchMmaQ8(const VecQArgs& a, dim3 grid, size_t lds, hipStream_t stream) {
  static bool sized = false;  // more than 64 KB of dynamic LDS must be asked for once
  if (!AllowLds(reinterpret_cast<const void*>(&VecQMmaQ8<kGlu>), static_cast<int>(kMmaLdsLimit), &sized)) return;
  hipLaunchKernelGGL((VecQMmaQ8<kGlu>), grid, dim3(kMmaGroup), lds, stream, a);
}

template <bool kGlu, int TG, int MT>
void LaunchMmaQ4K(const VecQArgs& a, dim3 grid, size_t lds, int balanced, hipStream_t stream) {
  static bool sized = false;
  if (!AllowLds(reinterpret_cast<const void*>(&VecQMma<kGlu, TG, MT>), static_cast<int>(kMmaLdsLimit), &sized)) return;
  hipLaunchKernelGGL((VecQMma<kGlu, TG, MT>), grid, dim3(kMmaGroup), lds, stream, a, balanced);
}

template <bool kGlu>
void LaunchMmaQ4KShape(const MmaShape& shape, const VecQArgs& a, dim3 grid, int balanced, hipStream_t stream) {
  if constexpr (!kGlu) {
    if (shape.groups == 4) return LaunchMmaQ4K<kGlu, 4, 16>(a, grid, shape.lds, balanced, stream);
  }
  if (shape.groups == 2) return LaunchMmaQ4K<kGlu, 2, 16>(a, grid, shape.lds, balanced, stream);
  if (shape.tokens == 16) return LaunchMmaQ4K<kGlu, 1, 16>(a, grid, shape.lds, balanced, stream);
  if (shape.tokens == 8) return LaunchMmaQ4K<kGlu, 1, 8>(a, grid, shape.lds, balanced, stream);
  return LaunchMmaQ4K<kGlu, 1, 4>(a, grid, shape.lds, balanced, stream);
}

}  // namespace

void LaunchMma(int type, const VecQArgs& a, hipStream_t stream) {
  const llmp_vecq_desc& d = a.d;
  const bool q8 = type == LLMP_TYPE_Q8_0;
  const int nsb = d.ncols_x / 256;
  if (g_mma_compute_units == 0) {
    const int cus = llmp_hip_compute_units();
    g_mma_compute_units = cus > 0 ? cus : 256;
  }
  const int slots = a.offsets != nullptr ? d.used : d.ids != nullptr ? d.used * d.tokens : d.used;
  const int tiles = (d.nrows + 15) / 16;
  const int tiles_group = q8 ? kQ8Tiles : nsb <= kWholeRow ? kMmaWaves : kTilesGroup;
  const int tile_groups = (tiles + tiles_group - 1) / tiles_group;
  const int live_slots = a.offsets == nullptr && d.ids != nullptr ? (d.used < slots ? d.used : slots) : slots;
  int groups = g_mma_compute_units / (live_slots > 0 ? live_slots : 1);
  if (groups < 1) groups = 1;
  if (groups > tile_groups) groups = tile_groups;
  const dim3 grid(static_cast<unsigned>(groups), static_cast<unsigned>(slots));
  const bool glu = d.g != nullptr;
  if (q8) {
    const size_t lds = MmaLdsQ8(d.ncols_x / 32);
    glu ? LaunchMmaQ8<true>(a, grid, lds, stream) : LaunchMmaQ8<false>(a, grid, lds, stream);
    return;
  }
  // A slot's tokens: a dense or grouped product's own; sorted rows bring any number an expert, a
  // routed product up to all its pairs.
  const int tokens = a.offsets != nullptr ? 64 : d.ids != nullptr ? d.used * d.tokens : d.tokens;
  const MmaShape shape = ShapeFor(nsb, tokens, glu);
  // Sorted rows: one workgroup a compute unit, the passes of all experts shared among them evenly.
  const int balanced = a.offsets != nullptr ? 1 : 0;
  const dim3 shared_grid(static_cast<unsigned>(g_mma_compute_units), 1);
  glu ? LaunchMmaQ4KShape<true>(shape, a, balanced ? shared_grid : grid, balanced, stream)
      : LaunchMmaQ4KShape<false>(shape, a, balanced ? shared_grid : grid, balanced, stream);
}

}  // namespace llmp_hip
