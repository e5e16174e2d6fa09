// llmp.vecq over Q4_K weights for 2 to 16 tokens a pass: the sub-block dot products on the
// int8 matrix cores.
//
// v_mfma_i32_16x16x32_i8 multiplies one 32-value sub-block of 16 weight rows with the same
// sub-block of 16 tokens: the instruction's K is a Q4_K sub-block, so every product comes out
// as the int32 sum the scalar kernel's eight v_dot4 give, for 256 (token, row) pairs at once.
// What is left per sub-block is the scaling, in floats, and it is done with exactly the
// operations of the one-token kernel (vecq_flat.hip) in exactly its order: per super-block
//   main = fma(float(prod_g), sc_g * d8_g, main), g = 0 .. 7;  mins = m_0 * ds8_0, then
//   fma(m_g, ds8_g, mins);  out = fma(d, main, -(dmin * mins))
// and the super-blocks of a row are added in the tree that kernel's wave shuffles form
// (aligned pairs, then pairs of pairs, ...), so a (token, row) value is bit for bit the
// one-token product's (src/kernels/ggml/vecq.cu:1150-1166 of the reference asks for that).
//
// A lane of the instruction's result holds one weight row (lane % 16) and four tokens
// (4 (lane / 16) + q): the weights are the second operand. A wave owns 16 rows (of both
// matrices with a GLU) and half of K; the two waves of a tile split K at the largest power of
// two below the row's super-blocks, which is the top node of the tree, and meet in LDS. A
// workgroup is eight waves, four tiles (rows of up to eight super-blocks: eight tiles, a wave
// all of K). Weights come straight from global memory into the
// operand layout (a lane reads its row's header and, per pair of sub-blocks, the eight code
// bytes of its K group), three super-blocks deep; the tokens' Q8_1 codes and scales are staged
// in LDS once a workgroup, in the first operand's layout:
//   codes   [super-block][pair of sub-blocks][K group][token] 16 bytes: the eight codes of
//           the K group in sub-block 2 p, then in 2 p + 1 (a lane's read is its 16 bytes of a
//           contiguous 1 KB);
//   scales  [super-block][token][pair] 4 floats: d8 of 2 p and 2 p + 1, d8 * sum(codes) of
//           2 p and 2 p + 1.

#include <hip/hip_runtime.h>

#include "common.h"
#include "llmp_hip.h"
#include "vecq_common.h"

namespace llmp_hip {
namespace {

constexpr int kMmaGroup = 512;
constexpr int kMmaWaves = kMmaGroup / kWave;
constexpr int kMmaTokens = 16;                       // a pass
constexpr int kTilesGroup = kMmaWaves / 2;           // row tiles a workgroup: two waves a tile
constexpr int kWholeRow = 8;                         // super-blocks a row up to which a wave takes all of K
constexpr int kCodesSb = 4 * kMmaTokens * 4 * 16;    // 4096 bytes of codes a super-block
constexpr int kScalesSb = kMmaTokens * 4 * 16;       // 1024 bytes of scales a super-block
constexpr int kPartialBytes = kMmaWaves * 2 * kWave * 16;  // a wave's four floats a lane and matrix
constexpr size_t kMmaLdsLimit = 160 * 1024 - 2048;

typedef int V4i __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float ByteOf(uint32_t word, int byte) {
  return static_cast<float>((word >> (8 * byte)) & 0xFFu);  // v_cvt_f32_ubyteN
}

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

// The decoded header of a super-block: 6-bit scales and minimums as bytes g of sc[g / 4],
// mn[g / 4] (the packing of tests/unit/dsv4_fast_test.cc:180-183 of the reference).
struct Header {
  uint32_t sc[2], mn[2];
  float d, dmin;
};

__device__ __forceinline__ Header Decode(const U32x4& h) {
  Header out;
  const uint32_t s0 = h.y, s1 = h.z, s2 = h.w;
  out.sc[0] = s0 & 0x3F3F3F3Fu;
  out.sc[1] = (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u);
  out.mn[0] = s1 & 0x3F3F3F3Fu;
  out.mn[1] = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
  out.d = HalfBitsToFloat(h.x & 0xFFFFu);
  out.dmin = HalfBitsToFloat(h.x >> 16);
  return out;
}

__device__ __forceinline__ int64_t Pack(uint32_t lo, uint32_t hi) {
  return static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo);
}

// Sums of a row's super-blocks in the order of the one-token kernel's shuffle tree: aligned
// pairs first, then pairs of pairs, .... The kernel adds each aligned group of four itself
// (Quad); the groups of four then go through a binary counter's carries, which builds the
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

// One super-block of one matrix times the staged tokens: four tokens of this lane's row.
// `a`: the tokens' codes as first operands, sub-block by sub-block; `entries[4 q + p]`: token
// q's four scale floats of pair p (in LDS, read a pair at a time).
__device__ __forceinline__ void DotPart(const RowPart& loaded, const int64_t (&a)[8], const float4* entries,
                                        float (&out)[4]) {
#pragma clang fp contract(off)
  RowPart part = loaded;
  Transpose(part);
  const Header h = Decode(part.header);
  float main[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  float mins[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const uint32_t q0 = part.q[p].x, q1 = part.q[p].y;
    const int64_t lo = Pack(q0 & 0x0F0F0F0Fu, q1 & 0x0F0F0F0Fu);
    const int64_t hi = Pack((q0 >> 4) & 0x0F0F0F0Fu, (q1 >> 4) & 0x0F0F0F0Fu);
    const V4i zero = {0, 0, 0, 0};
    const V4i prod0 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a[2 * p], lo, zero, 0, 0, 0);
    const V4i prod1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(a[2 * p + 1], hi, zero, 0, 0, 0);
    const float sc0 = ByteOf(h.sc[(2 * p) >> 2], (2 * p) & 3);
    const float sc1 = ByteOf(h.sc[(2 * p + 1) >> 2], (2 * p + 1) & 3);
    const float m0 = ByteOf(h.mn[(2 * p) >> 2], (2 * p) & 3);
    const float m1 = ByteOf(h.mn[(2 * p + 1) >> 2], (2 * p + 1) & 3);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float4 s = entries[4 * q + p];
      main[q] = fmaf(static_cast<float>(prod0[q]), sc0 * s.x, main[q]);
      main[q] = fmaf(static_cast<float>(prod1[q]), sc1 * s.y, main[q]);
      mins[q] = p == 0 ? m0 * s.z : fmaf(m0, s.z, mins[q]);
      mins[q] = fmaf(m1, s.w, mins[q]);
    }
  }
#pragma unroll
  for (int q = 0; q < 4; ++q) out[q] = fmaf(h.d, main[q], -(h.dmin * mins[q]));
}

// Stages `m` tokens' Q8_1 rows (one thread a block) into the operand layout. `row_of(j)`: token
// j's row of Q8_1 blocks.
template <class RowOf>
__device__ __forceinline__ void StageTokens(RowOf row_of, int m, int blocks, uint8_t* codes, uint8_t* scales) {
  for (int index = threadIdx.x; index < m * blocks; index += kMmaGroup) {
    const int j = index / blocks, b = index - j * blocks;
    const uint32_t* src = reinterpret_cast<const uint32_t*>(row_of(j) + static_cast<int64_t>(b) * kQ8Block);
    uint32_t w[9];
#pragma unroll
    for (int i = 0; i < 9; ++i) w[i] = src[i];
    const int sb = b >> 3, g = b & 7;
    uint8_t* to = codes + sb * kCodesSb + ((g >> 1) * 4 * kMmaTokens + j) * 16 + (g & 1) * 8;
#pragma unroll
    for (int kg = 0; kg < 4; ++kg)
      *reinterpret_cast<uint2*>(to + kg * kMmaTokens * 16) = make_uint2(w[1 + 2 * kg], w[2 + 2 * kg]);
    int sum = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) sum = Dot4(0x01010101, static_cast<int>(w[1 + i]), sum);
    const float d8 = HalfBitsToFloat(w[0] & 0xFFFFu);
    float* entry = reinterpret_cast<float*>(scales + sb * kScalesSb + (j * 4 + (g >> 1)) * 16);
    entry[g & 1] = d8;
    entry[2 + (g & 1)] = d8 * static_cast<float>(sum);
  }
}

// grid (workgroups, slots); LDS: codes, scales, the waves' partial sums.
template <bool kGlu>
__global__ __launch_bounds__(kMmaGroup, 1) void VecQMma(const VecQArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  __shared__ int pairs[kMaxPairs];
  __shared__ int count;

  const llmp_vecq_desc& d = a.d;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int nsb = d.ncols_x / 256;
  uint8_t* codes = lds;
  uint8_t* scales = lds + nsb * kCodesSb;
  float* partial = reinterpret_cast<float*>(lds + nsb * (kCodesSb + kScalesSb));

  int expert = blockIdx.y;
  int sorted_first = 0;
  if (a.offsets != nullptr) {
    sorted_first = a.offsets[expert];
    if (tid == 0) count = a.offsets[expert + 1] - sorted_first;
    __syncthreads();
  } else {
    expert = ResolvePairs(d, blockIdx.y, pairs, &count);
  }
  const int n = count;
  if (n == 0) return;  // uniform over the workgroup
  const int64_t expert_block = static_cast<int64_t>(expert) * d.stride_expert;

  // This wave's part of K. Rows of up to eight super-blocks: all of it, a tile a wave (too few
  // steps to be worth two waves and their meeting). Longer rows: a half, split at the top node
  // of the row's summation tree.
  const bool whole = nsb <= kWholeRow;
  int split = 1;
  while (split * 2 < nsb) split *= 2;
  const int half = whole ? 0 : wave & 1;
  const int first = half == 0 ? 0 : split;
  const int last = whole ? nsb : half == 0 ? min(split, nsb) : nsb;
  const int row_in_tile = lane & 15, kg = lane >> 4;
  const int tiles = (d.nrows + 15) / 16;
  const int tiles_group = whole ? kMmaWaves : kTilesGroup;
  const int tile_in_group = whole ? wave : wave >> 1;
  const int groups = (tiles + tiles_group - 1) / tiles_group;

  // This lane's weight rows of the tile its wave takes in a group of tiles (rows past the end
  // repeat the last, unstored).
  const uint8_t* up_row = nullptr;
  const uint8_t* gate_row = nullptr;
  auto aim = [&](int group) {
    const int row = min((group * tiles_group + tile_in_group) * 16 + row_in_tile, d.nrows - 1);
    const int64_t at = (expert_block + static_cast<int64_t>(row) * d.stride_row) * 144;
    up_row = static_cast<const uint8_t*>(d.w) + at;
    if constexpr (kGlu) gate_row = static_cast<const uint8_t*>(d.g) + at;
  };
  RowPart u0, u1, u2, u3, g0, g1, g2, g3;  // three are live at a time
  // The loads of super-block sb, queued here and no later: the compiler would otherwise sink
  // them to their first use, two steps on, and the wave would wait out the whole memory latency
  // there. (Past the end the last super-block again: no branch, no copies of what was loaded.)
  auto fetch = [&](int sb, RowPart& u, RowPart& g) {
    const int at = min(sb, last - 1);
    u = LoadRowPart(up_row, at, kg);
    if constexpr (kGlu) g = LoadRowPart(gate_row, at, kg);
    __builtin_amdgcn_sched_barrier(0);
  };
  // A group's first two super-blocks are asked for while the group before it finishes (the
  // first group's before the tokens are staged).
  aim(blockIdx.x);
  fetch(first, u0, g0);
  fetch(first + 1, u1, g1);

  for (int p0 = 0; p0 < n; p0 += kMmaTokens) {
    const int m = min(kMmaTokens, n - p0);
    __syncthreads();  // the last pass's readers of the staged tokens
    auto row_of = [&](int j) {
      const int pr = a.offsets != nullptr ? (sorted_first + p0 + j) << 8 : pairs[p0 + j];
      return static_cast<const uint8_t*>(d.y) +
             (static_cast<int64_t>(pr >> 8) * d.y_token + static_cast<int64_t>(pr & 0xFF) * d.y_slot) * kQ8Block;
    };
    StageTokens(row_of, m, d.ncols_x / 32, codes, scales);
    __syncthreads();

    for (int group = blockIdx.x; group < groups; group += gridDim.x) {
      const int tile = group * tiles_group + tile_in_group;
      TreeSum up_sum{}, gate_sum{};
      auto step = [&](int sb, const RowPart& u, const RowPart& g, float (&up_out)[4], float (&gate_out)[4]) {
        int64_t acts[8];
        const uint8_t* mine = codes + sb * kCodesSb + lane * 16;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          const U32x4 c = *reinterpret_cast<const U32x4*>(mine + p * (kMmaTokens * 4 * 16));
          acts[2 * p] = Pack(c.x, c.y);
          acts[2 * p + 1] = Pack(c.z, c.w);
        }
        const float4* entries = reinterpret_cast<const float4*>(scales + sb * kScalesSb) + (4 * kg) * 4;
        DotPart(u, acts, entries, up_out);
        if constexpr (kGlu) DotPart(g, acts, entries, gate_out);
      };
      int quads = 0;
      if (tile < tiles) {
        for (int sb = first; sb < last; sb += 4, ++quads) {
          const int n = min(4, last - sb);
          // The group's sum as its values come: (x0 + x1) + (x2 + x3), absent ones left out.
          float up_quad[4], gate_quad[4], up_next[4], gate_next[4];
          fetch(sb + 2, u2, g2);
          step(sb, u0, g0, up_quad, gate_quad);
          if (n >= 2) {
            fetch(sb + 3, u3, g3);
            step(sb + 1, u1, g1, up_next, gate_next);
            Sum4(up_quad, up_next, up_quad);
            if constexpr (kGlu) Sum4(gate_quad, gate_next, gate_quad);
          }
          if (n >= 3) {
            float up_rest[4], gate_rest[4];
            fetch(sb + 4, u0, g0);
            step(sb + 2, u2, g2, up_rest, gate_rest);
            if (n >= 4) {
              fetch(sb + 5, u1, g1);
              step(sb + 3, u3, g3, up_next, gate_next);
              Sum4(up_rest, up_next, up_rest);
              if constexpr (kGlu) Sum4(gate_rest, gate_next, gate_rest);
            }
            Sum4(up_quad, up_rest, up_quad);
            if constexpr (kGlu) Sum4(gate_quad, gate_rest, gate_quad);
          }
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
      }
      // The two halves of K meet: the upper half's totals through LDS.
      float up_total[4] = {0.0f, 0.0f, 0.0f, 0.0f}, gate_total[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      const bool has = tile < tiles && last > first;
      if (has) {
        Total(up_sum, quads, up_total);
        if constexpr (kGlu) Total(gate_sum, quads, gate_total);
      }
      float4* slot = reinterpret_cast<float4*>(partial) + (wave * 2) * kWave + lane;
      if (half == 1) {
        slot[0] = make_float4(up_total[0], up_total[1], up_total[2], up_total[3]);
        if constexpr (kGlu) slot[kWave] = make_float4(gate_total[0], gate_total[1], gate_total[2], gate_total[3]);
      }
      if (!whole) __syncthreads();
      if (half == 0 && tile < tiles) {
#pragma clang fp contract(off)
        if (!whole && split < nsb) {
          const float4* other = reinterpret_cast<const float4*>(partial) + ((wave + 1) * 2) * kWave + lane;
          const float4 u = other[0];
          up_total[0] += u.x, up_total[1] += u.y, up_total[2] += u.z, up_total[3] += u.w;
          if constexpr (kGlu) {
            const float4 g = other[kWave];
            gate_total[0] += g.x, gate_total[1] += g.y, gate_total[2] += g.z, gate_total[3] += g.w;
          }
        }
        if (tile * 16 + row_in_tile < d.nrows) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int t = 4 * kg + q;
            if (t < m) {
              const int pr = a.offsets != nullptr ? (sorted_first + p0 + t) << 8 : pairs[p0 + t];
              float* dst = d.dst + static_cast<int64_t>(pr >> 8) * d.dst_token + static_cast<int64_t>(pr & 0xFF) * d.dst_slot;
              dst[tile * 16 + row_in_tile] = kGlu ? Glu(d.glu, gate_total[q], up_total[q], d.limit) : up_total[q];
            }
          }
        }
      }
      if (!whole) __syncthreads();  // the partial sums may be overwritten
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

size_t MmaLds(int nsb) { return static_cast<size_t>(nsb) * (kCodesSb + kScalesSb) + kPartialBytes; }

int g_mma_compute_units = 0;

}  // namespace

// Q4_K rows whose sixteen staged tokens fit LDS (k up to 7168). Q8_0 rows of whole units of
// 128 values, up to 64 units (8192 values) as far as they fit LDS, whose rows, matrices and
// experts start on 4-byte boundaries (a lane reads dwords).
bool MmaTakes(int type, const llmp_vecq_desc& d) {
  if (type == LLMP_TYPE_Q4_K) {
    const int nsb = d.ncols_x / 256;
    return nsb >= 1 && MmaLds(nsb) <= kMmaLdsLimit;
  }
  if (type != LLMP_TYPE_Q8_0 || d.ncols_x < 128 || d.ncols_x % 128 != 0 || d.ncols_x > 8192) return false;
  const uintptr_t at = reinterpret_cast<uintptr_t>(d.w) | reinterpret_cast<uintptr_t>(d.g);
  return d.stride_row % 2 == 0 && d.stride_expert % 2 == 0 && at % 4 == 0 && MmaLdsQ8(d.ncols_x / 32) <= kMmaLdsLimit;
}

namespace {

template <bool kQ8, bool kGlu>
void LaunchMmaKernel(const VecQArgs& a, dim3 grid, size_t lds, hipStream_t stream) {
  static bool sized = false;  // more than 64 KB of dynamic LDS must be asked for once
  if constexpr (kQ8) {
    if (!AllowLds(reinterpret_cast<const void*>(&VecQMmaQ8<kGlu>), static_cast<int>(kMmaLdsLimit), &sized)) return;
    hipLaunchKernelGGL((VecQMmaQ8<kGlu>), grid, dim3(kMmaGroup), lds, stream, a);
  } else {
    if (!AllowLds(reinterpret_cast<const void*>(&VecQMma<kGlu>), static_cast<int>(kMmaLdsLimit), &sized)) return;
    hipLaunchKernelGGL((VecQMma<kGlu>), grid, dim3(kMmaGroup), lds, stream, a);
  }
}

}  // namespace

void LaunchMma(int type, const VecQArgs& a, hipStream_t stream) {
  const llmp_vecq_desc& d = a.d;
  const bool q8 = type == LLMP_TYPE_Q8_0;
  const int nsb = d.ncols_x / 256;
  const size_t lds = q8 ? MmaLdsQ8(d.ncols_x / 32) : MmaLds(nsb);
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
    glu ? LaunchMmaKernel<true, true>(a, grid, lds, stream) : LaunchMmaKernel<true, false>(a, grid, lds, stream);
  } else {
    glu ? LaunchMmaKernel<false, true>(a, grid, lds, stream) : LaunchMmaKernel<false, false>(a, grid, lds, stream);
  }
}

}  // namespace llmp_hip
