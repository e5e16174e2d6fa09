// The EXL3 trellis-coded linear (QTIP-style) for gfx950: codebook decode, weight
// reconstruction, the 128-point Hadamard transforms and the packed product for up to 16 rows.
//
// Format (src/kernels/reference/decode_exl3.cc of the reference): the weights are
// [K / 16][N / 16] tiles of 16 x 16 values at K bits a value; a tile's 256 K bits are a
// circular stream of uint32 words, most significant bit first, and the value at position t is
// the codebook value of the 16-bit state ending at bit (t + 1) K. Position 8 L + i (L below 32
// without bit 2) lands at row (L % 4) * 2 + {0, 1, 8, 9}[i % 4], column 2 (L / 8 + 4 (i / 4)),
// and lane L + 4's same position one column right. W = diag(suh) H W^ H diag(svh) / 128 with
// H block diagonal over 128, so y = H(H(x * suh) / sqrt(128) -> f16, times W^) / sqrt(128) * svh.
//
// Lane mapping, wave64: that placement is a bijection between a tile's 64 groups of four
// consecutive positions and the 64 lanes of a 16 x 16 x 16 MFMA's second operand. Lane
// l = (n = l % 16, g = l / 16) takes positions 8 L + 4 (n / 8) + [0, 4) with
// L = g + 4 (n % 2) + 8 ((n % 8) / 2): the values of column n at rows 2 g, 2 g + 1, 2 g + 8,
// 2 g + 9, which is column n of the operand with its four k slots in that row order; the other
// operand (the transformed activations, a row a token) is loaded with the same row order. So a
// wave decodes a tile with four states a lane and multiplies it by one MFMA, whatever the
// token count up to 16. A wave takes the eight tiles of one 128-column block (1 KB, contiguous)
// per 16 rows of K, fetched with global_load_lds_dwordx4 into a small ring, and a slice of K;
// the slices' partial sums are added in slice order by the output transform (no atomics).
//
// Reference behaviour restated here: src/kernels/reference/decode_exl3.cc:25-66 (codebooks),
// :82-127 (state and placement), :173-265 (transforms); src/kernels/exl3/validate.h:61-131
// (scale constant, operand structs), launch.cc:430-481 (reconstruct and Hadamard launches).

#include <hip/hip_runtime.h>

#include <initializer_list>
#include <mutex>

#include <type_traits>

#include "common.h"
#include "llmp_hip.h"

// The partial sums of llmp_hip_exl3_linear_static: one array a device, held until the process ends. In host code
// this name is only a handle for hipGetSymbolAddress; kernels and copies take the address that call returns.
constexpr size_t kStaticScratchBytes = LLMP_EXL3_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace llmp_hip {
namespace {

constexpr float kHadamardScale = 0.088388347648f;  // validate.h:64

typedef __attribute__((address_space(3))) void* LdsPointer;
typedef const __attribute__((address_space(1))) void* GlobalPointer;
typedef _Float16 Half4 __attribute__((ext_vector_type(4)));
typedef float V4f __attribute__((ext_vector_type(4)));

// ------------------------------------------------------------------ codebooks

// s * m + add mod 2^32 for a 16-bit s, as two 24-bit multiplies (full rate; a 32-bit multiply
// runs at a quarter of it). Written as instructions: the compiler folds the pair back into one
// 32-bit multiply otherwise.
template <uint32_t kMultiplier>
__device__ __forceinline__ uint32_t MulState(uint32_t s, uint32_t add) {
  constexpr uint32_t lo = kMultiplier & 0xFFFFFFu;
  constexpr uint32_t hi = kMultiplier >> 24;
  uint32_t x;
  asm("v_mad_u32_u24 %0, %1, %2, %3" : "=v"(x) : "v"(s), "s"(lo), "v"(add));  // the product's low 32 bits
  if constexpr (hi == 0) return x;
  uint32_t top;
  asm("v_mul_u32_u24 %0, %1, %2" : "=v"(top) : "v"(s), "s"(hi));
  return x + (top << 24);
}

// decode_exl3.cc:28-37: each half keeps its sign and low 12 bits under exponent 0b011xx, then
// the halves are added as one F16 addition.
__device__ __forceinline__ _Float16 SumHalves(uint32_t x) {
  const uint32_t y = __builtin_amdgcn_bitop3_b32(x, 0x8FFF8FFFu, 0x3B603B60u, 0x6A);  // (x & mask) ^ bias
  const _Float16 lo = __builtin_bit_cast(_Float16, static_cast<uint16_t>(y & 0xFFFFu));
  const _Float16 hi = __builtin_bit_cast(_Float16, static_cast<uint16_t>(y >> 16));
  return lo + hi;
}

// Two 3INST or MCG values at once: each one's halves added (the same F16 addition as SumHalves) straight into a
// half of one dword, by the instruction's operand selects: an instruction a value, and none to pack the results
// (left to itself the compiler permutes the four halves into two dwords and adds those: three for two values).
template <int CB>
__device__ __forceinline__ uint32_t CodebookPair(uint32_t state0, uint32_t state1) {
  static_assert(CB == LLMP_EXL3_3INST || CB == LLMP_EXL3_MCG, "MUL1 values are not sums of halves");
  const uint32_t x0 = CB == LLMP_EXL3_3INST ? MulState<89226354u>(state0, 64248484u) : MulState<0xCBAC1FEDu>(state0, 0u);
  const uint32_t x1 = CB == LLMP_EXL3_3INST ? MulState<89226354u>(state1, 64248484u) : MulState<0xCBAC1FEDu>(state1, 0u);
  const uint32_t y0 = __builtin_amdgcn_bitop3_b32(x0, 0x8FFF8FFFu, 0x3B603B60u, 0x6A);  // (x & mask) ^ bias
  const uint32_t y1 = __builtin_amdgcn_bitop3_b32(x1, 0x8FFF8FFFu, 0x3B603B60u, 0x6A);
  uint32_t pair;
  // (A wait state after each: the result of an instruction that writes half a register may not be read by the
  // next one, and inside these statements the compiler does not see that it is.)
  asm("v_add_f16_sdwa %0, %1, %1 dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:WORD_0 src1_sel:WORD_1\n\ts_nop 0"
      : "=v"(pair)
      : "v"(y0));
  asm("v_add_f16_sdwa %0, %1, %1 dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_0 src1_sel:WORD_1\n\ts_nop 0"
      : "+v"(pair)
      : "v"(y1));
  return pair;
}

// decode_exl3.cc:41-66
template <int CB>
__device__ __forceinline__ _Float16 Codebook(uint32_t state) {
  if constexpr (CB == LLMP_EXL3_3INST) {
    return SumHalves(MulState<89226354u>(state, 64248484u));
  } else if constexpr (CB == LLMP_EXL3_MCG) {
    return SumHalves(MulState<0xCBAC1FEDu>(state, 0u));
  } else {
    const uint32_t x = MulState<0x83DCD12Du>(state, 0u);
    const uint32_t sum = (x & 0xFFu) + ((x >> 8) & 0xFFu) + ((x >> 16) & 0xFFu) + (x >> 24) + 0x6400u;
    const _Float16 h = __builtin_bit_cast(_Float16, static_cast<uint16_t>(sum & 0xFFFFu));
    const _Float16 m = __builtin_bit_cast(_Float16, static_cast<uint16_t>(0x1EEEu));
    const _Float16 a = __builtin_bit_cast(_Float16, static_cast<uint16_t>(0xC931u));
    return __builtin_fmaf16(h, m, a);  // one rounding
  }
}

// The state of position `t` of a tile of `words` uint32 (decode_exl3.cc:82-96); Word(i) reads
// word i of the tile.
template <int BITS, typename WordFn>
__device__ __forceinline__ uint32_t State(int t, WordFn word) {
  constexpr int words = BITS * 8;
  const int end = (t + 1) * BITS + 256 * BITS;  // past the state's last bit, a period ahead
  const int i1 = (end - 1) >> 5;
  const int i0 = (end - 16) >> 5;  // may be i1
  const int shift = ((i1 + 1) << 5) - end;
  const uint64_t merged = (static_cast<uint64_t>(word(i0 % words)) << 32) | word(i1 % words);
  // When both indices agree the high word is shifted out of the 16 bits kept.
  return static_cast<uint32_t>(merged >> shift) & 0xFFFFu;
}

// A lane's place in a tile: column n, row group g, and its first position.
struct Place {
  int n, g, first;
};
__device__ __forceinline__ Place PlaceOf(int lane) {
  Place p;
  p.n = lane & 15;
  p.g = lane >> 4;
  const int l32 = p.g + 4 * (p.n & 1) + 8 * ((p.n & 7) >> 1);
  p.first = 8 * l32 + 4 * (p.n >> 3);
  return p;
}
// The rows of a lane's four values, in position order.
__device__ __forceinline__ int RowOf(int g, int j) { return 2 * g + (j & 1) + 8 * (j >> 1); }

// The codebook values of positions first .. first + 3 (first a multiple of four). Up to five
// bits a value the four states lie within 31 bits of the stream, so within the two words from
// the first state's first bit: one 64-bit shift brings the last state to bit 0 and the others
// sit at fixed offsets above it.
template <int CB, int BITS, typename WordFn>
__device__ __forceinline__ Half4 DecodeFour(int first, WordFn word) {
  Half4 v;
  if constexpr (BITS <= 5) {
    constexpr int words = BITS * 8;
    const int end0 = (first + 1) * BITS + 256 * BITS;  // past the first state's last bit, a period ahead
    const int ia = (end0 - 16) >> 5;
    const int shift = 32 * ia + 64 - (end0 + 3 * BITS);  // 2 .. 45
    const uint64_t merged = (static_cast<uint64_t>(word(ia % words)) << 32) | word((ia + 1) % words);
    const uint32_t window = static_cast<uint32_t>(merged >> shift);
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = Codebook<CB>((window >> ((3 - j) * BITS)) & 0xFFFFu);
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = Codebook<CB>(State<BITS>(first + j, word));
  }
  return v;
}

// ---------------------------------------------------------------- reconstruct

// Columns [column, column + columns) of the rotated-basis weights into w[k][columns] F16: a
// wave a tile; grid (columns / 16, k / 16 / 4), 4 waves a workgroup.
template <int CB, int BITS>
__global__ __launch_bounds__(256) void ReconstructKernel(const uint32_t* __restrict__ trellis,
                                                        uint16_t* __restrict__ w, int n, int k, int column,
                                                        int columns) {
  const int lane = threadIdx.x & 63;
  const int kt = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (kt >= k / 16) return;  // whole waves
  const int nt = column / 16 + blockIdx.x;
  const uint32_t* tile = trellis + (static_cast<int64_t>(kt) * (n / 16) + nt) * (BITS * 8);
  const Place p = PlaceOf(lane);
  const Half4 v = DecodeFour<CB, BITS>(p.first, [&](int i) { return tile[i]; });
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = kt * 16 + RowOf(p.g, j);
    const _Float16 value = v[j];  // (a bit cast straight from a vector's element reads element 0)
    w[static_cast<int64_t>(row) * columns + blockIdx.x * 16 + p.n] = __builtin_bit_cast(uint16_t, value);
  }
}

// ------------------------------------------------------------------ Hadamard

// The 128-point Walsh-Hadamard transform of a wave's 128 values, lane l holding values 2 l and
// 2 l + 1, natural order (H[i][j] = (-1)^popcount(i & j)), unscaled, in F32.
__device__ __forceinline__ void Hadamard128(float& a, float& b, int lane) {
#pragma clang fp contract(off)
  const float s = a + b;
  b = a - b;
  a = s;
#pragma unroll
  for (int mask = 1; mask < 64; mask <<= 1) {
    const float pa = ShflXor(a, mask);
    const float pb = ShflXor(b, mask);
    // The partner's value plus or minus this lane's: one fused operation with a sign of one, which rounds as the
    // addition or subtraction does (the product is exact), where a choice between the two takes three.
    const float sign = (lane & mask) != 0 ? -1.0f : 1.0f;
    a = __builtin_fmaf(a, sign, pa);
    b = __builtin_fmaf(b, sign, pb);
  }
}

// The same transform of four vectors a wave, one a row of sixteen lanes: lane l of a row holds elements l + 16 e,
// e = 0 .. 7. (The transform does not change when the bits of its index are permuted on both sides.) The three index
// bits that e holds are butterflies within the lane, the four that l holds exchanges within the row, which are
// data-parallel moves: nothing passes through LDS, and a value costs twelve operations where the wave-wide form
// takes over twenty. `sign[b]`: -1 where bit b of l is set, else 1.
__device__ __forceinline__ void Hadamard128Rows(float (&x)[8], const float (&sign)[4]) {
#pragma clang fp contract(off)
#pragma unroll
  for (int bit = 1; bit < 8; bit <<= 1) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if ((e & bit) == 0) {
        const float sum = x[e] + x[e | bit];
        x[e | bit] = x[e] - x[e | bit];
        x[e] = sum;
      }
    }
  }
#pragma unroll
  for (int b = 0; b < 4; ++b) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float other = ShflXor(x[e], 1 << b);
      x[e] = __builtin_fmaf(x[e], sign[b], other);
    }
  }
}

// y = f(H(x * in_scale)) * r * out_scale over each 128 block of each row; grid (rows, columns
// / 128), a wave a block. X / Y: 0 F16, 1 F32. `slices` partial inputs are added in order first.
// One or two transforms a launch (grid z): a linear's, or the two of a gate/up pair.
struct HadamardSides {
  const void* x[2];
  void* y[2];
  const uint16_t* in_scale[2];
  const uint16_t* out_scale[2];
};
inline HadamardSides OneSide(const void* x, void* y, const uint16_t* in_scale, const uint16_t* out_scale) {
  return HadamardSides{{x, x}, {y, y}, {in_scale, in_scale}, {out_scale, out_scale}};
}

template <int X, int Y>
__global__ __launch_bounds__(64) void HadamardKernel(const HadamardSides sides, int columns, int slices,
                                                    int64_t slice_stride) {
  // No fused multiply-adds: the transform inside the product kernel rounds every step the same way, so that a
  // row's transformed input, and with it its output, is the same bits whichever launch computed it.
#pragma clang fp contract(off)
  const void* __restrict__ x = sides.x[blockIdx.z];
  void* __restrict__ y = sides.y[blockIdx.z];
  const uint16_t* __restrict__ in_scale = sides.in_scale[blockIdx.z];
  const uint16_t* __restrict__ out_scale = sides.out_scale[blockIdx.z];
  const int lane = threadIdx.x;
  const int64_t at = static_cast<int64_t>(blockIdx.x) * columns + blockIdx.y * 128 + 2 * lane;
  float a = 0.0f, b = 0.0f;
  // Added in slice order; unrolled so that eight slices' loads are in flight at a time.
#pragma unroll 8
  for (int s = 0; s < slices; ++s) {
    if constexpr (X == 0) {
      const uint32_t v = *reinterpret_cast<const uint32_t*>(static_cast<const uint16_t*>(x) + s * slice_stride + at);
      a += HalfBitsToFloat(v & 0xFFFFu);
      b += HalfBitsToFloat(v >> 16);
    } else {
      const float2 v = *reinterpret_cast<const float2*>(static_cast<const float*>(x) + s * slice_stride + at);
      a += v.x;
      b += v.y;
    }
  }
  const int c = blockIdx.y * 128 + 2 * lane;
  if (in_scale != nullptr) {
    const uint32_t s = *reinterpret_cast<const uint32_t*>(in_scale + c);
    a *= HalfBitsToFloat(s & 0xFFFFu);
    b *= HalfBitsToFloat(s >> 16);
  }
  Hadamard128(a, b, lane);
  a *= kHadamardScale;
  b *= kHadamardScale;
  if (out_scale != nullptr) {
    const uint32_t s = *reinterpret_cast<const uint32_t*>(out_scale + c);
    a *= HalfBitsToFloat(s & 0xFFFFu);
    b *= HalfBitsToFloat(s >> 16);
  }
  if constexpr (Y == 0) {
    *reinterpret_cast<uint32_t*>(static_cast<uint16_t*>(y) + at) = FloatToHalfBits(a) | (FloatToHalfBits(b) << 16);
  } else {
    *reinterpret_cast<float2*>(static_cast<float*>(y) + at) = make_float2(a, b);
  }
}

// ------------------------------------------------------- reconstruct, transformed

// Columns [column, column + columns) of the weights themselves, W = diag(suh) H What H diag(svh) / 128 with H the
// 128-point transform over each block of 128 inputs and of 128 outputs, into w[k][columns] F16 (the reference's
// reconstruct_had_kernel, launch.cc:440-448; the definition decode.h:37-43). A workgroup of four waves a block of 128
// inputs by 128 outputs; LDS 128 x 129 floats. The rotated values are decoded into
// LDS (exact), every column is transformed along the inputs and every row along the outputs in F32 (four vectors a
// wave at a time, Hadamard128Rows), and the block is rounded to F16 once, after the scales: the reference's kernel
// rounds every butterfly to F16.
constexpr int kHadBlockPitch = 129;
constexpr int kHadBlockLds = 128 * kHadBlockPitch * 4;

// kTransform false: the rotated values as they are (the reconstruction without the transforms, through the same
// block). kTransposed: w[columns][k] instead, a column's inputs together, which is how the product below reads its
// second operand (both operands' rows along K).
template <int CB, int BITS, bool kTransform, bool kTransposed>
__global__ __launch_bounds__(256) void ReconstructHadKernel(const uint32_t* __restrict__ trellis,
                                                           const uint16_t* __restrict__ suh,
                                                           const uint16_t* __restrict__ svh,
                                                           uint16_t* __restrict__ w, int n, int k, int column, int columns) {
#pragma clang fp contract(off)
  extern __shared__ __attribute__((aligned(16))) float had_block[];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const Place p = PlaceOf(lane);
  const int l16 = lane & 15, row4 = lane >> 4;
  float sign[4];
#pragma unroll
  for (int b = 0; b < 4; ++b) sign[b] = (l16 >> b) & 1 ? -1.0f : 1.0f;
  // Sixteen of a block's 64 tiles a wave. A lane's four states lie within three consecutive words of a tile's
  // stream, the same three in every tile: they are asked for from all sixteen tiles before the first is decoded (a
  // tile after the other, each decode would wait for its own loads), and a workgroup goes through its blocks (every
  // gridDim.x-th, columns fastest) with the next block's words asked for ahead of this block's transforms.
  constexpr int kWords = BITS * 8;
  const int word0 = (((p.first + 1) * BITS + 256 * BITS - 16) >> 5) % kWords;
  const int blocks_n = columns / 128;
  const int blocks = blocks_n * (k / 128);
  uint32_t words[16][3];
  auto ask = [&](int block) {
    const int k_at = (block / blocks_n) * 128, c_at = (block % blocks_n) * 128;
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int t = wave * 16 + u;
      const int kt = t >> 3, nt = t & 7;
      const uint32_t* tile =
          trellis + (static_cast<int64_t>(k_at / 16 + kt) * (n / 16) + (column + c_at) / 16 + nt) * kWords;
#pragma unroll
      for (int i = 0; i < 3; ++i) words[u][i] = tile[(word0 + i) % kWords];
    }
  };
  if (static_cast<int>(blockIdx.x) < blocks) ask(blockIdx.x);
  for (int block = blockIdx.x; block < blocks; block += gridDim.x) {
  const int k0 = (block / blocks_n) * 128;
  const int c0 = (block % blocks_n) * 128;  // within the slice
#pragma unroll
  for (int u = 0; u < 16; ++u) {
    const int t = wave * 16 + u;
    const int kt = t >> 3, nt = t & 7;
    const Half4 v = DecodeFour<CB, BITS>(p.first, [&](int i) {
      const int d = (i - word0 + kWords) % kWords;
      return d == 0 ? words[u][0] : d == 1 ? words[u][1] : words[u][2];
    });
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const _Float16 value = v[j];
      had_block[(kt * 16 + RowOf(p.g, j)) * kHadBlockPitch + nt * 16 + p.n] = static_cast<float>(value);
    }
  }
  // (A block past the last is the last again: no load under a branch.)
  ask(min(block + static_cast<int>(gridDim.x), blocks - 1));
  __syncthreads();
  if constexpr (kTransform) {
    // Along the inputs: a wave 32 columns, four at a time, one a row of sixteen lanes (Hadamard128Rows).
    for (int j = wave * 32 + row4; j < wave * 32 + 32; j += 4) {
      float x[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = had_block[(l16 + 16 * e) * kHadBlockPitch + j];
      Hadamard128Rows(x, sign);
#pragma unroll
      for (int e = 0; e < 8; ++e) had_block[(l16 + 16 * e) * kHadBlockPitch + j] = x[e];
    }
    __syncthreads();
    // Along the outputs, then the scales: a wave 32 rows.
    float sv[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) sv[e] = HalfBitsToFloat(svh[column + c0 + l16 + 16 * e]) * (1.0f / 128.0f);
    for (int i = wave * 32 + row4; i < wave * 32 + 32; i += 4) {
      float x[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = had_block[i * kHadBlockPitch + l16 + 16 * e];
      Hadamard128Rows(x, sign);
      const float su = HalfBitsToFloat(suh[k0 + i]);
#pragma unroll
      for (int e = 0; e < 8; ++e) had_block[i * kHadBlockPitch + l16 + 16 * e] = x[e] * (su * sv[e]);
    }
    __syncthreads();
  }
  // Sixteen bytes a thread: a row (a column, transposed) is sixteen threads' worth.
  const int part = threadIdx.x & 15;
  for (int i = threadIdx.x >> 4; i < 128; i += 16) {
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      v[e] = kTransposed ? had_block[(part * 8 + e) * kHadBlockPitch + i] : had_block[i * kHadBlockPitch + part * 8 + e];
    }
    U32x4 out;
    out.x = FloatToHalfBits(v[0]) | (FloatToHalfBits(v[1]) << 16);
    out.y = FloatToHalfBits(v[2]) | (FloatToHalfBits(v[3]) << 16);
    out.z = FloatToHalfBits(v[4]) | (FloatToHalfBits(v[5]) << 16);
    out.w = FloatToHalfBits(v[6]) | (FloatToHalfBits(v[7]) << 16);
    if constexpr (kTransposed) {
      *reinterpret_cast<U32x4*>(w + static_cast<int64_t>(c0 + i) * k + k0 + part * 8) = out;
    } else {
      *reinterpret_cast<U32x4*>(w + static_cast<int64_t>(k0 + i) * columns + c0 + part * 8) = out;
    }
  }
  __syncthreads();  // the block's readers, before the next is decoded into it
  }
}

// ------------------------------------------------------------------- product

constexpr int kRingDepth = 4;  // K steps of a 128-column block in flight a wave
constexpr int kFusedRows = 4;  // up to here the product transforms its input itself
constexpr int kProductWaves = 8;
constexpr int kOperandBytes = 16 * 128 * 2;  // a wave's transformed activations of one 128 block of K
constexpr int kReduceBytes = kProductWaves * 32 * 64 * 4;

// partial[blockIdx.y][m][n] = sum over a K range of xh[m][k] W^[k][n] with xh = H(x * suh) /
// sqrt(128) as F16; grid (n / 128, outer slices), m <= 16. A workgroup a 128-column block, its
// eight waves `blocks_per_wave` 128-blocks of K each: a wave transforms its own activations a
// block at a time (the workgroups of the first column block also write them to a_had), decodes
// eight tiles per 16 rows of K, and the waves' sums are added in wave order through LDS.
// Every column block repeats the transform, which is cheap for a few tokens only: without
// kFused, x is the transformed input already and a_had is not written.
struct ProductSides {  // one or two linears a launch (grid z)
  const uint8_t* trellis[2];
  const uint16_t* x[2];
  const uint16_t* suh[2];
  uint16_t* a_had[2];
  float* partial[2];
};

// LDS accesses written as instructions, for the product's loop: while a global_load_lds is in flight the
// compiler makes every access of LDS it knows of wait until all of them have landed (it cannot tell which the
// access could alias), the ring's newest fetch included, and the ring would never overlap a fetch with a decode.
// The loop orders its reads and the loads itself: LdsWaited, then Tie on every register read.
#define LLMP_TIE(x) asm volatile("" : "+v"(x))
template <int OFFSET>
__device__ __forceinline__ uint32_t LdsRead4(uint32_t at) {
  uint32_t v;
  asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v) : "v"(at), "n"(OFFSET));
  return v;
}
__device__ __forceinline__ void LdsWrite4(uint32_t at, uint32_t value) { asm volatile("ds_write_b32 %0, %1" : : "v"(at), "v"(value)); }
__device__ __forceinline__ void LdsWaited() { asm volatile("s_waitcnt lgkmcnt(0)"); }
// The same for the few loads from global memory into registers inside that loop: the compiler's own wait for one
// is a wait for every load in flight, the ring's included.
__device__ __forceinline__ uint32_t GlobalLoad4(const void* from) {
  uint32_t v;
  asm volatile("global_load_dword %0, %1, off" : "=v"(v) : "v"(from));
  return v;
}
template <int LEFT>
__device__ __forceinline__ void LoadsWaited() {
  __builtin_amdgcn_s_waitcnt(0x0F70 | (LEFT & 0xF) | ((LEFT >> 4) << 14));
  asm volatile("" ::: "memory");
}
__device__ __forceinline__ uint32_t LdsAddress(const void* p) { return static_cast<uint32_t>(reinterpret_cast<uintptr_t>(p)); }

// Where a lane finds the 32 bits of a tile's stream that end at bit `end` (counted a period ahead, so never
// negative): the word holding the last bit, the word before it (circular), and the shift that brings bit `end`
// down to bit 0 of the pair.
template <int BITS>
struct Window {
  uint32_t high, low;  // byte offsets in the tile
  uint32_t shift;
};
template <int BITS>
__device__ __forceinline__ Window<BITS> WindowAt(int end) {
  constexpr int words = BITS * 8;
  const int i1 = ((end - 1) >> 5) % words;
  Window<BITS> w;
  w.low = static_cast<uint32_t>(i1) * 4u;
  w.high = static_cast<uint32_t>((i1 + words - 1) % words) * 4u;
  w.shift = static_cast<uint32_t>((32 - (end & 31)) & 31);
  return w;
}

// The windows of a lane's four positions first .. first + 3: one of 16 + 3 BITS bits up to five bits a value
// (within 32), else one a pair of positions (16 + BITS bits each).
template <int BITS>
struct Windows {
  static constexpr int kCount = BITS <= 5 ? 1 : 2;
  Window<BITS> w[kCount];
};
template <int BITS>
__device__ __forceinline__ Windows<BITS> WindowsOf(int first) {
  Windows<BITS> out;
  if constexpr (BITS <= 5) {
    out.w[0] = WindowAt<BITS>((first + 4) * BITS + 256 * BITS);
  } else {
    out.w[0] = WindowAt<BITS>((first + 2) * BITS + 256 * BITS);
    out.w[1] = WindowAt<BITS>((first + 4) * BITS + 256 * BITS);
  }
  return out;
}

// The codebook values of a lane's four positions from the words of its windows (high, low a window).
template <int CB, int BITS>
__device__ __forceinline__ Half4 DecodeWindows(const Windows<BITS>& at, const uint32_t (&words)[2 * Windows<BITS>::kCount]) {
  Half4 v;
  if constexpr (BITS <= 5 && CB != LLMP_EXL3_MUL1) {
    const uint32_t window = __builtin_amdgcn_alignbit(words[0], words[1], at.w[0].shift);
    uint2 pairs;
    pairs.x = CodebookPair<CB>((window >> (3 * BITS)) & 0xFFFFu, (window >> (2 * BITS)) & 0xFFFFu);
    pairs.y = CodebookPair<CB>((window >> BITS) & 0xFFFFu, window & 0xFFFFu);
    return __builtin_bit_cast(Half4, pairs);
  } else if constexpr (BITS <= 5) {
    const uint32_t window = __builtin_amdgcn_alignbit(words[0], words[1], at.w[0].shift);
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = Codebook<CB>((window >> ((3 - j) * BITS)) & 0xFFFFu);
  } else if constexpr (CB != LLMP_EXL3_MUL1) {
    uint2 pairs;
    const uint32_t first = __builtin_amdgcn_alignbit(words[0], words[1], at.w[0].shift);
    const uint32_t second = __builtin_amdgcn_alignbit(words[2], words[3], at.w[1].shift);
    pairs.x = CodebookPair<CB>((first >> BITS) & 0xFFFFu, first & 0xFFFFu);
    pairs.y = CodebookPair<CB>((second >> BITS) & 0xFFFFu, second & 0xFFFFu);
    return __builtin_bit_cast(Half4, pairs);
  } else {
#pragma unroll
    for (int pair = 0; pair < 2; ++pair) {
      const uint32_t window = __builtin_amdgcn_alignbit(words[2 * pair], words[2 * pair + 1], at.w[pair].shift);
      v[2 * pair] = Codebook<CB>((window >> BITS) & 0xFFFFu);
      v[2 * pair + 1] = Codebook<CB>(window & 0xFFFFu);
    }
  }
  return v;
}

template <int CB, int BITS, bool kFused>
__global__ __launch_bounds__(kProductWaves * 64) void ProductKernel(const ProductSides sides, int m, int n, int k,
                                                                   int blocks_per_wave) {
#pragma clang fp contract(off)
  const uint8_t* __restrict__ trellis = sides.trellis[blockIdx.z];
  const uint16_t* __restrict__ x = sides.x[blockIdx.z];
  const uint16_t* __restrict__ suh = sides.suh[blockIdx.z];
  uint16_t* __restrict__ a_had = sides.a_had[blockIdx.z];
  float* __restrict__ partial = sides.partial[blockIdx.z];
  constexpr int kTileBytes = BITS * 32;
  constexpr int kStepBytes = 8 * kTileBytes;  // a 128-column block's tiles of one K step
  constexpr int kLoads = (kStepBytes + 1023) / 1024;
  constexpr int kStageBytes = kLoads * 1024;
  constexpr int kRingBytes = kRingDepth * kStageBytes;
  constexpr int kWords = 2 * Windows<BITS>::kCount;  // a lane reads of a tile
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int block = blockIdx.x;  // of 128 columns
  uint8_t* ring = lds + wave * (kRingBytes + kOperandBytes);
  uint8_t* operand = ring + kRingBytes;  // [token][128] F16
  const int slice = blockIdx.y * kProductWaves + wave;
  const int first = min(slice * blocks_per_wave, k / 128) * 8;  // in K steps of 16
  const int last = min((slice + 1) * blocks_per_wave, k / 128) * 8;
  const Place p = PlaceOf(lane);
  const Windows<BITS> windows = WindowsOf<BITS>(p.first);
  const int64_t row_bytes = static_cast<int64_t>(n / 16) * kTileBytes;
  const uint8_t* source = trellis + static_cast<int64_t>(block) * kStepBytes;
  const uint32_t ring_at = LdsAddress(ring);

  // Step `step`'s tiles into its stage of the ring; past the wave's last step the last again (a load is never
  // skipped: the waits count loads).
  auto fetch = [&](int step) {
    const uint8_t* from = source + min(step, last - 1) * row_bytes;
    uint8_t* to = ring + (step % kRingDepth) * kStageBytes;
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      if (i * 1024 + lane * 16 < kStepBytes) {
        __builtin_amdgcn_global_load_lds((GlobalPointer)(from + i * 1024 + lane * 16), (LdsPointer)(to + i * 1024), 16,
                                         0, 0);
      }
    }
  };
  // Step `step`'s words of this lane's windows of the eight tiles, asked for (they are there after LdsWaited).
  auto ask = [&](int step, uint32_t (&words)[8][kWords]) {
    const uint32_t stage = ring_at + static_cast<uint32_t>((step % kRingDepth) * kStageBytes);
#pragma unroll
    for (int w = 0; w < Windows<BITS>::kCount; ++w) {
      const uint32_t high = stage + windows.w[w].high, low = stage + windows.w[w].low;
      words[0][2 * w] = LdsRead4<0 * kTileBytes>(high), words[0][2 * w + 1] = LdsRead4<0 * kTileBytes>(low);
      words[1][2 * w] = LdsRead4<1 * kTileBytes>(high), words[1][2 * w + 1] = LdsRead4<1 * kTileBytes>(low);
      words[2][2 * w] = LdsRead4<2 * kTileBytes>(high), words[2][2 * w + 1] = LdsRead4<2 * kTileBytes>(low);
      words[3][2 * w] = LdsRead4<3 * kTileBytes>(high), words[3][2 * w + 1] = LdsRead4<3 * kTileBytes>(low);
      words[4][2 * w] = LdsRead4<4 * kTileBytes>(high), words[4][2 * w + 1] = LdsRead4<4 * kTileBytes>(low);
      words[5][2 * w] = LdsRead4<5 * kTileBytes>(high), words[5][2 * w + 1] = LdsRead4<5 * kTileBytes>(low);
      words[6][2 * w] = LdsRead4<6 * kTileBytes>(high), words[6][2 * w + 1] = LdsRead4<6 * kTileBytes>(low);
      words[7][2 * w] = LdsRead4<7 * kTileBytes>(high), words[7][2 * w + 1] = LdsRead4<7 * kTileBytes>(low);
    }
  };
  auto landed = [&](uint32_t (&words)[8][kWords]) {
#pragma unroll
    for (int t = 0; t < 8; ++t)
#pragma unroll
      for (int w = 0; w < kWords; ++w) LLMP_TIE(words[t][w]);
  };

  V4f acc[8];
#pragma unroll
  for (int t = 0; t < 8; ++t) acc[t] = V4f{0.0f, 0.0f, 0.0f, 0.0f};
  // The activations' operand: token l % 16, k slots in the lane group's row order.
  const uint32_t my_operand = LdsAddress(operand) + static_cast<uint32_t>(min(p.n, m - 1) * 256 + 4 * p.g);
  const uint16_t* my_row = x + static_cast<int64_t>(min(p.n, m - 1)) * k + 2 * p.g;

  if (first < last) {
    // The ring runs kRingDepth - 1 steps ahead of the words read, the words one step ahead of the decode. Every
    // step asks for the same loads in the same order (the next step's two activation words, then a stage of the
    // ring; with kFused the next block's activations in place of the words), so that a wait can count them.
    uint32_t words[2][8][kWords];
    uint32_t xa[2] = {0, 0}, xb[2] = {0, 0};  // a step's activation words (unfused: from global memory)
    uint32_t held[kFusedRows + 1];             // the next block's scales and activations (fused)
    auto ask_block = [&](int step) {           // of K step `step`'s 128 block
      const int at = min(step >> 3, k / 128 - 1) * 128 + 2 * lane;
      held[0] = GlobalLoad4(suh + at);
#pragma unroll
      for (int t = 0; t < kFusedRows; ++t) held[1 + t] = GlobalLoad4(x + static_cast<int64_t>(min(t, m - 1)) * k + at);
    };
    if constexpr (kFused) {
      ask_block(first);
    } else {
      xa[0] = GlobalLoad4(my_row + first * 16);
      xb[0] = GlobalLoad4(my_row + first * 16 + 8);
    }
#pragma unroll
    for (int s = 0; s < kRingDepth - 1; ++s) fetch(first + s);
    LoadsWaited<kLoads*(kRingDepth - 2)>();
    ask(first, words[0]);
    auto one = [&](int step, int parity) {
      uint32_t (&mine)[8][kWords] = words[parity];
      uint32_t (&next)[8][kWords] = words[parity ^ 1];
      if (kFused && ((step & 7) == 0 || step == first)) {
        // The wave's 128 values of every token for this block of K, transformed as the input transform does
        // (asked for a block ago), and the next block's asked for.
        const int at = (step >> 3) * 128 + 2 * lane;
        // (They were asked for before the ring stages the waits have since counted in: they are there.)
#pragma unroll
        for (int i = 0; i <= kFusedRows; ++i) LLMP_TIE(held[i]);
        const float sa = HalfBitsToFloat(held[0] & 0xFFFFu), sb = HalfBitsToFloat(held[0] >> 16);
        LdsWaited();  // the last block's operand has been read
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int t = 0; t < kFusedRows; ++t) {
          if (t < m) {
            const uint32_t v = held[1 + t];
            float a = HalfBitsToFloat(v & 0xFFFFu) * sa;
            float b = HalfBitsToFloat(v >> 16) * sb;
            Hadamard128(a, b, lane);
            a *= kHadamardScale;
            b *= kHadamardScale;
            const uint32_t packed = FloatToHalfBits(a) | (FloatToHalfBits(b) << 16);
            LdsWrite4(LdsAddress(operand) + static_cast<uint32_t>(t * 256 + 4 * lane), packed);
            if (block == 0) *reinterpret_cast<uint32_t*>(a_had + static_cast<int64_t>(t) * k + at) = packed;
          }
        }
        ask_block(step + 8);
        LdsWaited();
        __builtin_amdgcn_wave_barrier();
      }
      uint32_t x01, x89;
      if constexpr (kFused) {
        const uint32_t at = my_operand + static_cast<uint32_t>((step & 7) * 32);
        x01 = LdsRead4<0>(at);
        x89 = LdsRead4<16>(at);
      } else {
        xa[parity ^ 1] = GlobalLoad4(my_row + min(step + 1, last - 1) * 16);
        xb[parity ^ 1] = GlobalLoad4(my_row + min(step + 1, last - 1) * 16 + 8);
      }
      // The ring's next stage asked for; the stage after this step's has landed (and this step's activation
      // words): its words asked for, and this step's words (asked for a step ago) decoded while those come.
      fetch(step + kRingDepth - 1);
      LoadsWaited<kLoads*(kRingDepth - 2) + (kFused ? 0 : 2)>();
      LdsWaited();
      landed(mine);
      if constexpr (kFused) {
        LLMP_TIE(x01);
        LLMP_TIE(x89);
      } else {
        LLMP_TIE(xa[parity]);
        LLMP_TIE(xb[parity]);
        x01 = xa[parity], x89 = xb[parity];
      }
      ask(step + 1, next);
      if (p.n >= m) x01 = 0, x89 = 0;
      Half4 xv;
      xv[0] = __builtin_bit_cast(_Float16, static_cast<uint16_t>(x01 & 0xFFFFu));
      xv[1] = __builtin_bit_cast(_Float16, static_cast<uint16_t>(x01 >> 16));
      xv[2] = __builtin_bit_cast(_Float16, static_cast<uint16_t>(x89 & 0xFFFFu));
      xv[3] = __builtin_bit_cast(_Float16, static_cast<uint16_t>(x89 >> 16));
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const Half4 wv = DecodeWindows<CB, BITS>(windows, mine[t]);
        // D[token][n] += sum_j xv[token][j] wv[j][n]: first operand rows are tokens.
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x16f16(xv, wv, acc[t], 0, 0, 0);
      }
    };
    for (int step = first; step < last; step += 2) {
      one(step, 0);
      if (step + 1 < last) one(step + 1, 1);
    }
    LdsWaited();  // the words asked for past the end
    LoadsWaited<0>();
  }

  // The waves' sums through LDS (over the rings, which every wave has left), added in wave
  // order. acc[t][q] = D[token 4 g + q][column 16 t + n].
  __syncthreads();
  float* sums = reinterpret_cast<float*>(lds);  // [wave][8 t + q][lane]
#pragma unroll
  for (int t = 0; t < 8; ++t) {
#pragma unroll
    for (int q = 0; q < 4; ++q) sums[(wave * 32 + t * 4 + q) * 64 + lane] = acc[t][q];
  }
  __syncthreads();
  float* out = partial + static_cast<int64_t>(blockIdx.y) * m * n + block * 128;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int e = tid + j * (kProductWaves * 64);  // of 32 x 64
    float total = sums[e];
#pragma unroll
    for (int w = 1; w < kProductWaves; ++w) total += sums[w * 2048 + e];
    const int tq = e >> 6, l = e & 63;
    const int row = 4 * (l >> 4) + (tq & 3);
    if (row < m) out[static_cast<int64_t>(row) * n + (tq >> 2) * 16 + (l & 15)] = total;
  }
}

// Outer slices of K: enough workgroups for about 4096 waves, each wave at least one 128 block.
int SlicesFor(int n, int k) {
  const int blocks = k / 128;
  const int column_blocks = n / 128;
  int want = (4096 / kProductWaves + column_blocks - 1) / column_blocks;
  const int most = (blocks + kProductWaves - 1) / kProductWaves;
  if (want > most) want = most;
  return want < 1 ? 1 : want;
}

int CheckWeights(const llmp_exl3_weights& w) {
  if (w.trellis == nullptr || w.suh == nullptr || w.svh == nullptr) return Refuse(1, "exl3: null weights");
  if (w.k <= 0 || w.n <= 0 || w.k % 128 != 0 || w.n % 128 != 0)
    return Refuse(1, "exl3: dimensions %d x %d are not multiples of 128", w.k, w.n);
  if (w.k > (1 << 19) || w.n > (1 << 19)) return Refuse(1, "exl3: a dimension exceeds 2^19");
  if (w.bits < 1 || w.bits > 8) return Refuse(1, "exl3: rate %d outside 1..8", w.bits);
  if (w.codebook < LLMP_EXL3_3INST || w.codebook > LLMP_EXL3_MUL1) return Refuse(1, "exl3: no codebook %d", w.codebook);
  if (reinterpret_cast<uintptr_t>(w.trellis) % 16 != 0) return Refuse(1, "exl3: trellis not 16-byte aligned");
  if ((reinterpret_cast<uintptr_t>(w.suh) | reinterpret_cast<uintptr_t>(w.svh)) % 8 != 0)
    return Refuse(1, "exl3: side vectors not 8-byte aligned");
  return 0;
}

// Byte ranges of operands, and the reference's refusal of a written range that meets another
// (src/kernels/exl3/validate.cc:32-62: "{} overlaps {}"), before anything is queued.
struct Range {
  const char* name;
  uintptr_t base;
  size_t bytes;
};
bool Overlap(const Range& a, const Range& b) {
  return a.bytes > 0 && b.bytes > 0 && a.base < b.base + b.bytes && b.base < a.base + a.bytes;
}
int Disjoint(const char* what, const Range& written, std::initializer_list<Range> others) {
  for (const Range& other : others) {
    if (Overlap(written, other)) return Refuse(1, "%s: %s overlaps %s", what, written.name, other.name);
  }
  return 0;
}
Range TrellisRange(const llmp_exl3_weights& w) {
  return {"the trellis", reinterpret_cast<uintptr_t>(w.trellis), static_cast<size_t>(w.k) * w.n * w.bits / 8};
}
Range SuhRange(const llmp_exl3_weights& w) { return {"suh", reinterpret_cast<uintptr_t>(w.suh), static_cast<size_t>(w.k) * 2}; }
Range SvhRange(const llmp_exl3_weights& w) { return {"svh", reinterpret_cast<uintptr_t>(w.svh), static_cast<size_t>(w.n) * 2}; }

template <int CB, int BITS>
void LaunchReconstruct(const llmp_exl3_weights& w, void* out, int column, int columns, hipStream_t stream) {
  const dim3 grid(static_cast<unsigned>(columns / 16), static_cast<unsigned>((w.k / 16 + 3) / 4));
  hipLaunchKernelGGL((ReconstructKernel<CB, BITS>), grid, dim3(256), 0, stream,
                     static_cast<const uint32_t*>(w.trellis), static_cast<uint16_t*>(out), w.n, w.k, column, columns);
}

template <int CB, int BITS, bool kTransform, bool kTransposed>
bool g_reconstruct_had_sized = false;
template <int CB, int BITS, bool kTransform, bool kTransposed>
void LaunchReconstructHad(const llmp_exl3_weights& w, void* out, int column, int columns, hipStream_t stream) {
  if (!AllowLds(reinterpret_cast<const void*>(&ReconstructHadKernel<CB, BITS, kTransform, kTransposed>), kHadBlockLds,
                &g_reconstruct_had_sized<CB, BITS, kTransform, kTransposed>))
    return;
  // Two workgroups a compute unit are resident (LDS): that many go through the blocks.
  const int blocks = (columns / 128) * (w.k / 128);
  const int cus = llmp_hip_compute_units() > 0 ? llmp_hip_compute_units() : 256;
  const dim3 grid(static_cast<unsigned>(blocks < 2 * cus ? blocks : 2 * cus));
  hipLaunchKernelGGL((ReconstructHadKernel<CB, BITS, kTransform, kTransposed>), grid, dim3(256), kHadBlockLds, stream,
                     static_cast<const uint32_t*>(w.trellis), static_cast<const uint16_t*>(w.suh),
                     static_cast<const uint16_t*>(w.svh), static_cast<uint16_t*>(out), w.n, w.k, column, columns);
}

template <int BITS>
constexpr int ProductLds() {
  constexpr int kLoads = (BITS * 32 * 8 + 1023) / 1024;
  constexpr int kWork = kProductWaves * (kRingDepth * kLoads * 1024 + kOperandBytes);
  return kWork > kReduceBytes ? kWork : kReduceBytes;
}
// More than 64 KB of dynamic LDS must be asked for once a kernel instance: a runtime call that is no launch, so a
// caller that captures makes it beforehand (llmp_hip_exl3_linear_static_prepare).
template <int CB, int BITS, bool kFused>
bool g_product_sized = false;
template <int CB, int BITS, bool kFused>
bool SizeProduct() {
  return AllowLds(reinterpret_cast<const void*>(&ProductKernel<CB, BITS, kFused>), ProductLds<BITS>(), &g_product_sized<CB, BITS, kFused>);
}

template <int CB, int BITS, bool kFused>
void LaunchProduct(const llmp_exl3_weights& w, const ProductSides& sides, int count, int m, int slices,
                   hipStream_t stream) {
  constexpr int kLds = ProductLds<BITS>();
  if (!SizeProduct<CB, BITS, kFused>()) return;
  const int blocks = w.k / 128;
  const int per = (blocks + slices * kProductWaves - 1) / (slices * kProductWaves);
  const dim3 grid(static_cast<unsigned>(w.n / 128), static_cast<unsigned>(slices), static_cast<unsigned>(count));
  hipLaunchKernelGGL((ProductKernel<CB, BITS, kFused>), grid, dim3(kProductWaves * 64), kLds, stream, sides, m, w.n, w.k,
                     per);
}

template <typename F>
bool DispatchBits(int bits, F&& f) {
  switch (bits) {
    case 1: f(std::integral_constant<int, 1>{}); return true;
    case 2: f(std::integral_constant<int, 2>{}); return true;
    case 3: f(std::integral_constant<int, 3>{}); return true;
    case 4: f(std::integral_constant<int, 4>{}); return true;
    case 5: f(std::integral_constant<int, 5>{}); return true;
    case 6: f(std::integral_constant<int, 6>{}); return true;
    case 7: f(std::integral_constant<int, 7>{}); return true;
    case 8: f(std::integral_constant<int, 8>{}); return true;
    default: return false;
  }
}

template <typename F>
void Dispatch(int codebook, int bits, F&& f) {
  DispatchBits(bits, [&](auto b) {
    constexpr int kBits = decltype(b)::value;
    if (codebook == LLMP_EXL3_3INST) {
      f(std::integral_constant<int, LLMP_EXL3_3INST>{}, std::integral_constant<int, kBits>{});
    } else if (codebook == LLMP_EXL3_MCG) {
      f(std::integral_constant<int, LLMP_EXL3_MCG>{}, std::integral_constant<int, kBits>{});
    } else {
      f(std::integral_constant<int, LLMP_EXL3_MUL1>{}, std::integral_constant<int, kBits>{});
    }
  });
}

}  // namespace
}  // namespace llmp_hip

using namespace llmp_hip;

extern "C" int llmp_hip_exl3_reconstruct(const llmp_exl3_weights* weights, void* w, int column, int columns,
                                         void* stream) {
  BeginLaunches();
  if (weights == nullptr || w == nullptr) return Refuse(1, "exl3.reconstruct: null operand");
  if (const int bad = CheckWeights(*weights); bad != 0) return bad;
  if (column < 0 || columns <= 0 || column % 16 != 0 || columns % 16 != 0 || column + columns > weights->n)
    return Refuse(1, "exl3.reconstruct: columns [%d, %d) are not whole tiles of the weights", column, column + columns);
  // validate.cc:379-382: the reconstructed matrix meets none of the weights' tensors.
  if (const int bad = Disjoint("exl3.reconstruct", {"w", reinterpret_cast<uintptr_t>(w), static_cast<size_t>(weights->k) * columns * 2},
                               {TrellisRange(*weights), SuhRange(*weights), SvhRange(*weights)});
      bad != 0)
    return bad;
  Dispatch(weights->codebook, weights->bits, [&](auto cb, auto bits) {
    LaunchReconstruct<decltype(cb)::value, decltype(bits)::value>(*weights, w, column, columns,
                                                                  static_cast<hipStream_t>(stream));
  });
  return LaunchStatus("exl3.reconstruct");
}

extern "C" int llmp_hip_exl3_reconstruct_fused(const llmp_exl3_weights* weights, void* w, int column, int columns,
                                               void* stream) {
  BeginLaunches();
  if (weights == nullptr || w == nullptr) return Refuse(1, "exl3.reconstruct_fused: null operand");
  if (const int bad = CheckWeights(*weights); bad != 0) return bad;
  // validate.cc:367-372: 128-column blocks inside the matrix.
  if (column < 0 || columns < 128 || column % 128 != 0 || columns % 128 != 0 || column > weights->n - columns)
    return Refuse(1, "exl3.reconstruct_fused: columns [%d, %lld) of %d: 128-column blocks inside the matrix", column,
                  static_cast<long long>(column) + columns, weights->n);
  if (reinterpret_cast<uintptr_t>(w) % 16 != 0) return Refuse(1, "exl3.reconstruct_fused: w at a 16-byte boundary");
  if (const int bad = Disjoint("exl3.reconstruct_fused", {"w", reinterpret_cast<uintptr_t>(w), static_cast<size_t>(weights->k) * columns * 2},
                               {TrellisRange(*weights), SuhRange(*weights), SvhRange(*weights)});
      bad != 0)
    return bad;
  Dispatch(weights->codebook, weights->bits, [&](auto cb, auto bits) {
    LaunchReconstructHad<decltype(cb)::value, decltype(bits)::value, true, false>(*weights, w, column, columns,
                                                                                  static_cast<hipStream_t>(stream));
  });
  return LaunchStatus("exl3.reconstruct_fused");
}

extern "C" int llmp_hip_exl3_hadamard(const void* x, void* y, const void* scale, int rows, int columns, int f32,
                                      int input_scale, void* stream) {
  BeginLaunches();
  if (x == nullptr || y == nullptr || scale == nullptr) return Refuse(1, "exl3.hadamard: null operand");
  if (rows <= 0 || rows > 65535 || columns <= 0 || columns % 128 != 0)
    return Refuse(1, "exl3.hadamard: 1 to 65535 rows of whole 128-value blocks");
  if (input_scale && f32) return Refuse(1, "exl3.hadamard: the input scale's transform is F16");
  {
    // validate.cc:411-416: in place (y == x, F16 only: a lane reads its values before it writes them) or disjoint.
    const size_t cells = static_cast<size_t>(rows) * columns;
    const Range xr{"x", reinterpret_cast<uintptr_t>(x), cells * 2};
    const Range yr{"y", reinterpret_cast<uintptr_t>(y), cells * (f32 ? 4 : 2)};
    if (x == y && f32) return Refuse(1, "exl3.hadamard: an F32 output cannot be the F16 input");
    if (x != y) {
      if (const int bad = Disjoint("exl3.hadamard", yr, {xr}); bad != 0) return bad;
    }
    if (const int bad = Disjoint("exl3.hadamard", yr, {{"the scale", reinterpret_cast<uintptr_t>(scale), static_cast<size_t>(columns) * 2}});
        bad != 0)
      return bad;
  }
  const dim3 grid(static_cast<unsigned>(rows), static_cast<unsigned>(columns / 128));
  const auto s = static_cast<hipStream_t>(stream);
  const auto* sc = static_cast<const uint16_t*>(scale);
  if (f32) {
    hipLaunchKernelGGL((HadamardKernel<1, 1>), grid, dim3(64), 0, s, OneSide(x, y, nullptr, sc), columns, 1, int64_t{0});
  } else if (input_scale) {
    hipLaunchKernelGGL((HadamardKernel<0, 0>), grid, dim3(64), 0, s, OneSide(x, y, sc, nullptr), columns, 1, int64_t{0});
  } else {
    hipLaunchKernelGGL((HadamardKernel<0, 0>), grid, dim3(64), 0, s, OneSide(x, y, nullptr, sc), columns, 1, int64_t{0});
  }
  return LaunchStatus("exl3.hadamard");
}

namespace llmp_hip {
namespace {

// `count` linears of the same shape, rate and codebook over one input: the transformed input
// (a launch of its own above a few rows), the products in slices of K, the slices' sums
// transformed. Linear i writes a_had[i], scratch[i] and y[i].
int LaunchLinears(const llmp_exl3_weights* const (&w)[2], int count, const void* x, void* const (&a_had)[2],
                  void* const (&y)[2], float* const (&scratch)[2], bool f32, int m, const char* what, hipStream_t s) {
  const llmp_exl3_weights& w0 = *w[0];
  const int slices = SlicesFor(w0.n, w0.k);
  const bool fused = m <= kFusedRows;
  const auto* suh0 = static_cast<const uint16_t*>(w[0]->suh);
  const auto* suh1 = static_cast<const uint16_t*>(w[1]->suh);
  if (!fused) {
    const HadamardSides in{{x, x}, {a_had[0], a_had[1]}, {suh0, suh1}, {nullptr, nullptr}};
    hipLaunchKernelGGL((HadamardKernel<0, 0>),
                       dim3(static_cast<unsigned>(m), static_cast<unsigned>(w0.k / 128), static_cast<unsigned>(count)),
                       dim3(64), 0, s, in, w0.k, 1, int64_t{0});
    if (const int bad = LaunchStatus(what); bad != 0) return bad;
  }
  ProductSides sides;
  for (int i = 0; i < 2; ++i) {
    sides.trellis[i] = static_cast<const uint8_t*>(w[i]->trellis);
    sides.x[i] = static_cast<const uint16_t*>(fused ? x : a_had[i]);
    sides.suh[i] = static_cast<const uint16_t*>(w[i]->suh);
    sides.a_had[i] = fused ? static_cast<uint16_t*>(a_had[i]) : nullptr;
    sides.partial[i] = scratch[i];
  }
  Dispatch(w0.codebook, w0.bits, [&](auto cb, auto bits) {
    constexpr int kCb = decltype(cb)::value, kBits = decltype(bits)::value;
    if (fused) {
      LaunchProduct<kCb, kBits, true>(w0, sides, count, m, slices, s);
    } else {
      LaunchProduct<kCb, kBits, false>(w0, sides, count, m, slices, s);
    }
  });
  if (const int bad = LaunchStatus(what); bad != 0) return bad;
  const dim3 grid(static_cast<unsigned>(m), static_cast<unsigned>(w0.n / 128), static_cast<unsigned>(count));
  const int64_t stride = static_cast<int64_t>(m) * w0.n;
  const HadamardSides out{{scratch[0], scratch[1]},
                          {y[0], y[1]},
                          {nullptr, nullptr},
                          {static_cast<const uint16_t*>(w[0]->svh), static_cast<const uint16_t*>(w[1]->svh)}};
  if (f32) {
    hipLaunchKernelGGL((HadamardKernel<1, 1>), grid, dim3(64), 0, s, out, w0.n, slices, stride);
  } else {
    hipLaunchKernelGGL((HadamardKernel<1, 0>), grid, dim3(64), 0, s, out, w0.n, slices, stride);
  }
  // A failure here follows queued launches: a fault, not a refusal.
  const int status = LaunchStatus(what);
  return status > 0 ? -status : status;
}

}  // namespace
}  // namespace llmp_hip

// The rows of one pass of the packed product (the matrix instruction's sixteen); more rows take more passes,
// each streaming the weights again (src/kernels/exl3/validate.h:76: a launch takes 1 to 65536 rows).
constexpr int kPassRows = 16;
constexpr int kMostRows = 1 << 16;

extern "C" size_t llmp_hip_exl3_linear_scratch(const llmp_exl3_linear* op) {
  if (op == nullptr || op->m <= 0 || op->weights.k <= 0 || op->weights.n <= 0) return 0;
  const int pass = op->m < kPassRows ? op->m : kPassRows;  // the passes share the area
  return static_cast<size_t>(SlicesFor(op->weights.n, op->weights.k)) * pass * op->weights.n * sizeof(float);
}

namespace llmp_hip {
namespace {

// The checks and launches of the packed linear over `area` (area_bytes of partial sums: the caller's, or this
// device's static array).
int LinearOver(const llmp_exl3_linear* op, void* area, size_t area_bytes, hipStream_t stream) {
  if (op == nullptr) return Refuse(1, "exl3.linear: null operands");
  if (const int bad = CheckWeights(op->weights); bad != 0) return bad;
  if (op->x == nullptr || op->a_had == nullptr || op->y == nullptr || area == nullptr)
    return Refuse(1, "exl3.linear: null operand");
  if (op->m < 1 || op->m > kMostRows) return Refuse(1, "exl3.linear: the packed product takes 1 to %d rows, not %d", kMostRows, op->m);
  if (area_bytes < llmp_hip_exl3_linear_scratch(op))
    return Refuse(1, "exl3.linear: scratch too small: %zu bytes of partial sums, %zu given", llmp_hip_exl3_linear_scratch(op), area_bytes);
  if ((reinterpret_cast<uintptr_t>(op->x) | reinterpret_cast<uintptr_t>(op->a_had) |
       reinterpret_cast<uintptr_t>(op->y) | reinterpret_cast<uintptr_t>(area)) % 8 != 0)
    return Refuse(1, "exl3.linear: operands not 8-byte aligned");
  {
    // validate.cc:120-126: what the launches write (a_had, y, the partial sums in place of the lock area) meets
    // nothing they read and not one another.
    const size_t m = static_cast<size_t>(op->m);
    const Range x{"x", reinterpret_cast<uintptr_t>(op->x), m * op->weights.k * 2};
    const Range a_had{"a_had", reinterpret_cast<uintptr_t>(op->a_had), m * op->weights.k * 2};
    const Range y{"y", reinterpret_cast<uintptr_t>(op->y), m * op->weights.n * (op->f32 ? 4 : 2)};
    const Range partials{"the scratch", reinterpret_cast<uintptr_t>(area), llmp_hip_exl3_linear_scratch(op)};
    const llmp_exl3_weights& w = op->weights;
    if (const int bad = Disjoint("exl3.linear", a_had, {x, y, TrellisRange(w), SuhRange(w), SvhRange(w), partials}); bad != 0) return bad;
    if (const int bad = Disjoint("exl3.linear", y, {x, TrellisRange(w), SuhRange(w), SvhRange(w), partials}); bad != 0) return bad;
    if (const int bad = Disjoint("exl3.linear", partials, {x, TrellisRange(w), SuhRange(w), SvhRange(w)}); bad != 0) return bad;
  }
  const llmp_exl3_weights* const w[2] = {&op->weights, &op->weights};
  float* const partial[2] = {static_cast<float*>(area), static_cast<float*>(area)};
  // Sixteen rows a pass, the passes in stream order over the one area of partial sums.
  for (int row = 0; row < op->m; row += kPassRows) {
    const int rows = op->m - row < kPassRows ? op->m - row : kPassRows;
    const size_t in = static_cast<size_t>(row) * op->weights.k * 2;
    const size_t out = static_cast<size_t>(row) * op->weights.n * (op->f32 ? 4 : 2);
    void* const a_had[2] = {static_cast<uint8_t*>(op->a_had) + in, static_cast<uint8_t*>(op->a_had) + in};
    void* const y[2] = {static_cast<uint8_t*>(op->y) + out, static_cast<uint8_t*>(op->y) + out};
    const int status = LaunchLinears(w, 1, static_cast<const uint8_t*>(op->x) + in, a_had, y, partial, op->f32 != 0, rows,
                                     "exl3.linear", stream);
    if (status != 0) return row == 0 ? status : (status > 0 ? -status : status);  // after a queued pass: a fault
  }
  return 0;
}

// This device's copy of the static array: its address is asked for once a device, with that device current.
constexpr int kMostDevices = 64;
std::mutex g_static_lock;
void* g_static_area[kMostDevices] = {};

int StaticArea(void** area) {
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) {
    SetError("exl3.linear_static: %s", hipGetErrorString(e));
    return -static_cast<int>(e);
  }
  if (device < 0 || device >= kMostDevices) return Refuse(1, "exl3.linear_static: device %d beyond the %d this library keeps an area for", device, kMostDevices);
  std::lock_guard<std::mutex> hold(g_static_lock);
  if (g_static_area[device] == nullptr) {
    void* at = nullptr;
    e = hipGetSymbolAddress(&at, HIP_SYMBOL(scratch));
    if (e != hipSuccess || at == nullptr) {
      (void)hipGetLastError();
      SetError("exl3.linear_static: the static area's address: %s", hipGetErrorString(e));
      return e != hipSuccess ? -static_cast<int>(e) : -1;
    }
    g_static_area[device] = at;
  }
  *area = g_static_area[device];
  return 0;
}

}  // namespace
}  // namespace llmp_hip

extern "C" int llmp_hip_exl3_linear(const llmp_exl3_linear* op, void* scratch, size_t scratch_bytes, void* stream) {
  BeginLaunches();
  return LinearOver(op, scratch, scratch_bytes, static_cast<hipStream_t>(stream));
}

extern "C" int llmp_hip_exl3_linear_static(const llmp_exl3_linear* op, void* stream) {
  BeginLaunches();
  if (op == nullptr) return Refuse(1, "exl3.linear_static: null operands");
  // The size first: a linear whose partial sums do not fit the static area is refused whatever else holds.
  const size_t needs = llmp_hip_exl3_linear_scratch(op);
  if (needs > kStaticScratchBytes)
    return Refuse(1, "exl3.linear_static: %zu bytes of partial sums exceed the static area's %zu; use llmp_hip_exl3_linear with "
                     "scratch of the caller's", needs, kStaticScratchBytes);
  void* area = nullptr;
  if (const int bad = StaticArea(&area); bad != 0) return bad;
  return LinearOver(op, area, kStaticScratchBytes, static_cast<hipStream_t>(stream));
}

extern "C" int llmp_hip_exl3_linear_static_prepare(const llmp_exl3_linear* op) {
  BeginLaunches();
  if (op == nullptr) return Refuse(1, "exl3.linear_static_prepare: null operands");
  if (const int bad = llmp_hip::CheckWeights(op->weights); bad != 0) return bad;
  void* area = nullptr;
  if (const int bad = StaticArea(&area); bad != 0) return bad;
  llmp_hip::Dispatch(op->weights.codebook, op->weights.bits, [&](auto cb, auto bits) {
    (void)llmp_hip::SizeProduct<decltype(cb)::value, decltype(bits)::value, true>();
    (void)llmp_hip::SizeProduct<decltype(cb)::value, decltype(bits)::value, false>();
  });
  return LaunchStatus("exl3.linear_static_prepare");
}

namespace llmp_hip {
// mxfp8.hip: D[m][n] = A[m][k] B[n][k]^T over F16 operands, F32 sums.
int LaunchHalfGemm(const void* a_rows, const void* b_rows, void* d, int m, int n, int k, int64_t ldd, bool f16_out,
                   int compute_units, hipStream_t stream);
}  // namespace llmp_hip

constexpr int kReconstructSlice = 32768;  // validate.h:257-261: columns a slice of the reconstruction

extern "C" size_t llmp_hip_exl3_reconstructed_scratch(const llmp_exl3_weights* weights) {
  if (weights == nullptr || weights->k <= 0 || weights->n <= 0) return 0;
  const int columns = weights->n < kReconstructSlice ? weights->n : kReconstructSlice;
  return static_cast<size_t>(weights->k) * columns * 2;
}

extern "C" int llmp_hip_exl3_linear_reconstructed(const llmp_exl3_linear* op, void* w, size_t w_bytes, int fused,
                                                  int compute_units, void* stream) {
  BeginLaunches();
  if (op == nullptr || w == nullptr) return Refuse(1, "exl3.linear_reconstructed: null operands");
  const llmp_exl3_weights& weights = op->weights;
  if (const int bad = llmp_hip::CheckWeights(weights); bad != 0) return bad;
  if (op->x == nullptr || op->y == nullptr || (!fused && op->a_had == nullptr)) return Refuse(1, "exl3.linear_reconstructed: null operand");
  if (op->m < 1 || op->m > 65536) return Refuse(1, "exl3.linear_reconstructed: 1 to 65536 rows, not %d", op->m);
  if (static_cast<int64_t>(op->m) * weights.k * 2 >= (int64_t{1} << 32)) return Refuse(1, "exl3.linear_reconstructed: an input of 4 GiB or more");
  const size_t needs = llmp_hip_exl3_reconstructed_scratch(&weights);
  if (w_bytes < needs) return Refuse(1, "exl3.linear_reconstructed: %zu bytes of weight scratch, %zu needed", w_bytes, needs);
  const uintptr_t aligned = reinterpret_cast<uintptr_t>(op->x) | reinterpret_cast<uintptr_t>(op->y) | reinterpret_cast<uintptr_t>(w) |
                            (fused ? 0 : reinterpret_cast<uintptr_t>(op->a_had));
  if (aligned % 16 != 0) return Refuse(1, "exl3.linear_reconstructed: operands not 16-byte aligned");
  {
    // validate.cc:508-539: the scratch the path writes meets nothing it later reads or writes, and nothing it writes
    // holds the weights.
    const size_t cells = static_cast<size_t>(op->m) * weights.k;
    const llmp_hip::Range x{"x", reinterpret_cast<uintptr_t>(op->x), cells * 2};
    const llmp_hip::Range xh{"xh", fused ? 0 : reinterpret_cast<uintptr_t>(op->a_had), fused ? 0 : cells * 2};
    const llmp_hip::Range wr{"w", reinterpret_cast<uintptr_t>(w), needs};
    const llmp_hip::Range y{"y", reinterpret_cast<uintptr_t>(op->y), static_cast<size_t>(op->m) * weights.n * (op->f32 ? 4 : 2)};
    if (const int bad = llmp_hip::Disjoint("exl3.linear_reconstructed", wr, {x, xh, y}); bad != 0) return bad;
    if (const int bad = llmp_hip::Disjoint("exl3.linear_reconstructed", xh, {x, y}); bad != 0) return bad;
    if (const int bad = llmp_hip::Disjoint("exl3.linear_reconstructed", y, {x}); bad != 0) return bad;
    for (const llmp_hip::Range& written : {xh, wr, y}) {
      if (const int bad = llmp_hip::Disjoint("exl3.linear_reconstructed", written,
                                             {llmp_hip::TrellisRange(weights), llmp_hip::SuhRange(weights), llmp_hip::SvhRange(weights)});
          bad != 0)
        return bad;
    }
  }
  const auto s = static_cast<hipStream_t>(stream);
  const auto* suh = static_cast<const uint16_t*>(weights.suh);
  const auto* svh = static_cast<const uint16_t*>(weights.svh);
  const void* product_input = op->x;
  if (!fused) {
    // The input's transform, y = H(x * suh) / sqrt(128), as the packed path's.
    hipLaunchKernelGGL((llmp_hip::HadamardKernel<0, 0>), dim3(static_cast<unsigned>(op->m), static_cast<unsigned>(weights.k / 128)), dim3(64),
                       0, s, llmp_hip::OneSide(op->x, op->a_had, suh, nullptr), weights.k, 1, int64_t{0});
    product_input = op->a_had;
  }
  for (int column = 0; column < weights.n; column += kReconstructSlice) {
    const int columns = weights.n - column < kReconstructSlice ? weights.n - column : kReconstructSlice;
    // The slice's weights, a column's inputs together (the product reads both operands along K).
    llmp_hip::Dispatch(weights.codebook, weights.bits, [&](auto cb, auto bits) {
      if (fused) {
        llmp_hip::LaunchReconstructHad<decltype(cb)::value, decltype(bits)::value, true, true>(weights, w, column, columns, s);
      } else {
        llmp_hip::LaunchReconstructHad<decltype(cb)::value, decltype(bits)::value, false, true>(weights, w, column, columns, s);
      }
    });
    void* y_at = op->f32 ? static_cast<void*>(static_cast<float*>(op->y) + column) : static_cast<void*>(static_cast<uint16_t*>(op->y) + column);
    if (const int bad = llmp_hip::LaunchHalfGemm(product_input, w, y_at, op->m, columns, weights.k, weights.n, !op->f32, compute_units, s); bad != 0)
      return bad;
  }
  if (!fused) {
    // The output's transform in place, y = H(y) / sqrt(128) * svh.
    const dim3 grid(static_cast<unsigned>(op->m), static_cast<unsigned>(weights.n / 128));
    if (op->f32) {
      hipLaunchKernelGGL((llmp_hip::HadamardKernel<1, 1>), grid, dim3(64), 0, s, llmp_hip::OneSide(op->y, op->y, nullptr, svh), weights.n, 1, int64_t{0});
    } else {
      hipLaunchKernelGGL((llmp_hip::HadamardKernel<0, 0>), grid, dim3(64), 0, s, llmp_hip::OneSide(op->y, op->y, nullptr, svh), weights.n, 1, int64_t{0});
    }
  }
  return LaunchStatus("exl3.linear_reconstructed");
}

extern "C" size_t llmp_hip_exl3_multi_linear_scratch(const llmp_exl3_multi_linear* op) {
  if (op == nullptr || op->m <= 0 || op->first.k <= 0 || op->first.n <= 0) return 0;
  const int pass = op->m < kPassRows ? op->m : kPassRows;  // the passes share the area
  return 2 * static_cast<size_t>(SlicesFor(op->first.n, op->first.k)) * pass * op->first.n * sizeof(float);
}

extern "C" int llmp_hip_exl3_multi_linear(const llmp_exl3_multi_linear* op, void* scratch, size_t scratch_bytes,
                                          void* stream) {
  BeginLaunches();
  if (op == nullptr) return Refuse(1, "exl3.multi_linear: null operands");
  if (const int bad = CheckWeights(op->first); bad != 0) return bad;
  if (const int bad = CheckWeights(op->second); bad != 0) return bad;
  if (op->first.k != op->second.k || op->first.n != op->second.n || op->first.bits != op->second.bits)
    return Refuse(1, "exl3.multi_linear: the two linears of a multi-GEMM share k, n and K");
  if (op->x == nullptr || op->a_had == nullptr || op->y == nullptr || scratch == nullptr)
    return Refuse(1, "exl3.multi_linear: null operand");
  if (op->m < 1 || op->m > kMostRows)
    return Refuse(1, "exl3.multi_linear: the packed product takes 1 to %d rows, not %d", kMostRows, op->m);
  if (scratch_bytes < llmp_hip_exl3_multi_linear_scratch(op)) return Refuse(1, "exl3.multi_linear: scratch too small");
  if ((reinterpret_cast<uintptr_t>(op->x) | reinterpret_cast<uintptr_t>(op->a_had) |
       reinterpret_cast<uintptr_t>(op->y) | reinterpret_cast<uintptr_t>(scratch)) % 8 != 0)
    return Refuse(1, "exl3.multi_linear: operands not 8-byte aligned");
  {
    // validate.cc:310-323: a_had, y and the partial sums meet nothing the launches read and not one another.
    const size_t rows = static_cast<size_t>(op->m);
    const Range x{"x", reinterpret_cast<uintptr_t>(op->x), rows * op->first.k * 2};
    const Range a_had{"a_had", reinterpret_cast<uintptr_t>(op->a_had), 2 * rows * op->first.k * 2};
    const Range y{"y", reinterpret_cast<uintptr_t>(op->y), 2 * rows * op->first.n * (op->f32 ? 4 : 2)};
    const Range area{"the scratch", reinterpret_cast<uintptr_t>(scratch), llmp_hip_exl3_multi_linear_scratch(op)};
    for (const llmp_exl3_weights* w : {&op->first, &op->second}) {
      for (const Range& written : {a_had, y, area}) {
        if (const int bad = Disjoint("exl3.multi_linear", written, {TrellisRange(*w), SuhRange(*w), SvhRange(*w)}); bad != 0)
          return bad;
      }
    }
    if (const int bad = Disjoint("exl3.multi_linear", a_had, {x, y, area}); bad != 0) return bad;
    if (const int bad = Disjoint("exl3.multi_linear", y, {x, area}); bad != 0) return bad;
    if (const int bad = Disjoint("exl3.multi_linear", area, {x}); bad != 0) return bad;
  }
  const auto s = static_cast<hipStream_t>(stream);
  const int m = op->m, k = op->first.k, n = op->first.n;
  const size_t element = op->f32 ? 4 : 2;
  float* const part = static_cast<float*>(scratch);
  const size_t part_floats = static_cast<size_t>(SlicesFor(n, k)) * (m < kPassRows ? m : kPassRows) * n;
  const llmp_exl3_weights* const w[2] = {&op->first, &op->second};
  float* const partial[2] = {part, part + part_floats};
  bool queued = false;
  // Sixteen rows a pass, the passes in stream order over the one area of partial sums.
  for (int row = 0; row < m; row += kPassRows) {
    const int rows = m - row < kPassRows ? m - row : kPassRows;
    const uint8_t* x = static_cast<const uint8_t*>(op->x) + static_cast<size_t>(row) * k * 2;
    void* const a_had[2] = {static_cast<uint16_t*>(op->a_had) + static_cast<size_t>(row) * k,
                            static_cast<uint16_t*>(op->a_had) + (static_cast<size_t>(m) + row) * k};
    void* const y[2] = {static_cast<uint8_t*>(op->y) + static_cast<size_t>(row) * n * element,
                        static_cast<uint8_t*>(op->y) + (static_cast<size_t>(m) + row) * n * element};
    if (op->first.codebook == op->second.codebook) {
      const int status = LaunchLinears(w, 2, x, a_had, y, partial, op->f32 != 0, rows, "exl3.multi_linear", s);
      if (status != 0) return !queued ? status : (status > 0 ? -status : status);
      queued = true;
      continue;
    }
    // Different codebooks decode differently: one linear after the other.
    for (int i = 0; i < 2; ++i) {
      const llmp_exl3_weights* const one[2] = {w[i], w[i]};
      void* const a[2] = {a_had[i], a_had[i]};
      void* const out[2] = {y[i], y[i]};
      float* const p[2] = {partial[i], partial[i]};
      const int status = LaunchLinears(one, 1, x, a, out, p, op->f32 != 0, rows, "exl3.multi_linear", s);
      if (status != 0) return !queued ? status : (status > 0 ? -status : status);
      queued = true;
    }
  }
  return 0;
}
