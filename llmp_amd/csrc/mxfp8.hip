// MXFP8 (E4M3 codes, one E8M0 scale per 32 values along K) for gfx950: the activation
// quantizer, the weight-scale swizzle, the decode-shaped vector product and the prefill GEMM
// on CDNA4's block-scaled MFMA.
//
// Scale interchange layout ("atoms", src/format/layout.h:108-113 of the reference): atoms of
// 128 rows by 4 scales, 512 bytes, along K first; in an atom row r's four scales sit together
// at (r mod 32) * 16 + (r mod 128) / 32 * 4. A 128-row tile's scales of one 128-value K step
// are therefore one atom, and a row's four scales one aligned dword, which is what the GEMM
// loads per lane.
//
// GEMM: D[m, n] = sum_k A[m, k] B[n, k], both operands K-major. A workgroup (4 wave64s, 2 x 2)
// computes a 128 x 128 tile in K steps of 128; a wave 64 x 64 as 4 x 4
// v_mfma_scale_f32_16x16x128_f8f6f4, the weights as the instruction's first operand so that
// a lane's four results are four consecutive n of one m (one 8-byte bf16 store). For that
// instruction lane l holds, of row l % 16, the 32 codes k = 16 (l / 16) + [0, 16) and
// 64 + 16 (l / 16) + [0, 16), and supplies the scale of its row's 32-block l / 16. Tiles come
// into LDS by global_load_lds_dwordx4, double buffered; a row's eight 16-byte chunks are
// stored xor-swizzled by (row / 2) % 8 so that a fragment's sixteen rows read distinct banks.
//
// Reference behaviour restated here: src/kernels/ggml/mxfp8_quant.cuh:19-46 (scale code,
// inverse scale, saturating E4M3), llmp_ops.cu:610-663 (quantize and swizzle kernels),
// :145-224 (vector product), mxfp8_cutlass.h:12-79 (the GEMM's operands and status codes).

#include <hip/hip_runtime.h>

#include <type_traits>
#include <utility>

#include "common.h"
#include "llmp_hip.h"

namespace llmp_hip {
namespace {

__host__ __device__ __forceinline__ uint64_t AtomOffset(uint64_t row, uint64_t block, uint64_t blocks) {
  return (((row / 128) * (blocks / 4) + (block / 4)) * 512) + ((row % 32) * 16) + (((row % 128) / 32) * 4) + (block % 4);
}

// mxfp8_quant.cuh:22-29
__device__ __forceinline__ uint32_t ScaleCode(float amax) {
#pragma clang fp contract(off)
  const uint32_t bits = __builtin_bit_cast(uint32_t, amax * (1.0f / 448.0f));
  uint32_t e = (bits >> 23) & 0xFFu;
  if ((bits & 0x7FFFFFu) != 0u) ++e;
  return e > 253u ? 253u : e;
}
// mxfp8_quant.cuh:33-35: 2^(127 - e), exactly. e = 254 cannot occur.
__device__ __forceinline__ float InverseScale(uint32_t e) { return __builtin_bit_cast(float, (254u - e) << 23); }

// OCP E4M3 of a float: nearest even, saturating to +-448, NaN to 0x7F.
__device__ __forceinline__ uint32_t ToE4m3(float x) {
  const uint32_t bits = __builtin_bit_cast(uint32_t, x);
  const uint32_t sign = (bits >> 24) & 0x80u;
  const uint32_t mag = bits & 0x7FFFFFFFu;
  if (mag > 0x7F800000u) return sign | 0x7Fu;
  uint32_t code;
  if (mag >= 0x43E00000u) {  // 448 and beyond
    code = 0x7Eu;
  } else if (mag < 0x3C800000u) {  // below 2^-6: units of 2^-9
    code = static_cast<uint32_t>(__builtin_rintf(__builtin_bit_cast(float, mag) * 512.0f));
  } else {
    const uint32_t rounded = mag + 0x7FFFFu + ((mag >> 20) & 1u);  // to 3 mantissa bits
    code = (rounded >> 20) - (120u << 3);
    if (code > 0x7Eu) code = 0x7Eu;
  }
  return sign | code;
}

template <typename T>
__device__ __forceinline__ void Load32(const T* p, float (&v)[32]);
template <>
__device__ __forceinline__ void Load32<float>(const float* p, float (&v)[32]) {
#pragma unroll
  for (int i = 0; i < 32; ++i) v[i] = p[i];
}
template <>
__device__ __forceinline__ void Load32<uint16_t>(const uint16_t* p, float (&v)[32]) {  // bf16
#pragma unroll
  for (int i = 0; i < 32; ++i) v[i] = Bf16BitsToFloat(p[i]);
}

// One 32-value block a thread; rows past `rows`, up to the atoms' padding, write a zero scale.
template <typename T>
__global__ void QuantizeKernel(const T* __restrict__ x, int64_t x_stride, uint8_t* __restrict__ codes,
                               uint8_t* __restrict__ scales, int k, int rows, int64_t items) {
#pragma clang fp contract(off)
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= items) return;
  const int blocks = k / 32;
  const int r = static_cast<int>(i / blocks);
  const int b = static_cast<int>(i % blocks);
  const uint64_t at = AtomOffset(r, b, blocks);
  if (r >= rows) {
    scales[at] = 0;
    return;
  }
  float v[32];
  Load32<T>(x + static_cast<int64_t>(r) * x_stride + b * 32, v);
  float amax = 0.0f;
#pragma unroll
  for (int j = 0; j < 32; ++j) amax = fmaxf(amax, fabsf(v[j]));
  const uint32_t e = ScaleCode(amax);
  const float inverse = InverseScale(e);
  uint32_t packed[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    packed[j] = ToE4m3(v[4 * j] * inverse) | (ToE4m3(v[4 * j + 1] * inverse) << 8) |
                (ToE4m3(v[4 * j + 2] * inverse) << 16) | (ToE4m3(v[4 * j + 3] * inverse) << 24);
  }
  uint4* out = reinterpret_cast<uint4*>(codes + static_cast<int64_t>(r) * k + b * 32);
  out[0] = make_uint4(packed[0], packed[1], packed[2], packed[3]);
  out[1] = make_uint4(packed[4], packed[5], packed[6], packed[7]);
  scales[at] = static_cast<uint8_t>(e);
}

// The same quantizer for rows that allow 16-byte loads: eight values a lane, four lanes a block, sixteen lanes
// the four blocks whose scales are one dword of an atom. Loads and stores are coalesced (a wave reads 512
// consecutive values and writes their 512 bytes of codes), the block's largest magnitude crosses its quad by
// data-parallel moves, and the codes come from the hardware's conversion (OCP E4M3, nearest even) after a clamp
// to +-448, with a NaN's code put in by hand: bit for bit ToE4m3's.
template <typename T>
__global__ __launch_bounds__(256) void QuantizeWideKernel(const T* __restrict__ x, int64_t x_stride, uint8_t* __restrict__ codes,
                                                          uint8_t* __restrict__ scales, int k, int rows, int64_t items) {
#pragma clang fp contract(off)
  // One piece of eight values a lane (two, half of the rows apart, with both loads queued first, measured
  // slower: 7.3 us against 6.7 for 2048 rows of 4096). Whole groups of sixteen lanes share a row: k / 8 is a
  // multiple of sixteen.
  constexpr int kPieces = 1;
  const int64_t first = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t half = items / kPieces;
  if (first >= half) return;
  const int per_row = k / 8;
  const int blocks = k / 32;
  const int lane = threadIdx.x & 63;
  int r[kPieces], c[kPieces];
  float v[kPieces][8];
#pragma unroll
  for (int p = 0; p < kPieces; ++p) {
    const int64_t i = first + p * half;
    r[p] = static_cast<int>(i / per_row);
    c[p] = static_cast<int>(i % per_row) * 8;
    if (r[p] >= rows) continue;
    const T* from = x + static_cast<int64_t>(r[p]) * x_stride + c[p];
    if constexpr (sizeof(T) == 4) {
      const float4 a = reinterpret_cast<const float4*>(from)[0], b = reinterpret_cast<const float4*>(from)[1];
      v[p][0] = a.x, v[p][1] = a.y, v[p][2] = a.z, v[p][3] = a.w, v[p][4] = b.x, v[p][5] = b.y, v[p][6] = b.z, v[p][7] = b.w;
    } else {
      const uint4 raw = *reinterpret_cast<const uint4*>(from);
      const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) v[p][2 * j] = Bf16BitsToFloat(w[j] & 0xFFFFu), v[p][2 * j + 1] = Bf16BitsToFloat(w[j] >> 16);
    }
  }
#pragma unroll
  for (int p = 0; p < kPieces; ++p) {
    if (r[p] >= rows) {  // the atoms' padding rows: zero scales, no codes (whole rows: uniform over the group)
      if ((lane & 15) == 0) *reinterpret_cast<uint32_t*>(scales + AtomOffset(r[p], c[p] / 32, blocks)) = 0;
      continue;
    }
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[p][j]));
    amax = fmaxf(amax, ShflXor(amax, 1));
    amax = fmaxf(amax, ShflXor(amax, 2));
    const uint32_t e = ScaleCode(amax);
    const float inverse = InverseScale(e);
    uint32_t word[2] = {0, 0};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float a = v[p][2 * j] * inverse, b = v[p][2 * j + 1] * inverse;
      const float ca = __builtin_amdgcn_fmed3f(a, -448.0f, 448.0f), cb = __builtin_amdgcn_fmed3f(b, -448.0f, 448.0f);
      word[j >> 1] = (j & 1) != 0 ? static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(ca, cb, static_cast<int>(word[j >> 1]), true))
                                  : static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(ca, cb, static_cast<int>(word[j >> 1]), false));
      // A NaN keeps its sign and takes the format's NaN, whatever the clamp and the conversion made of it.
      const int at = 16 * (j & 1);
      if (a != a) word[j >> 1] = (word[j >> 1] & ~(0xFFu << at)) | ((((__builtin_bit_cast(uint32_t, a) >> 24) & 0x80u) | 0x7Fu) << at);
      if (b != b) word[j >> 1] = (word[j >> 1] & ~(0xFF00u << at)) | ((((__builtin_bit_cast(uint32_t, b) >> 24) & 0x80u) | 0x7Fu) << (at + 8));
    }
    *reinterpret_cast<uint2*>(codes + static_cast<int64_t>(r[p]) * k + c[p]) = make_uint2(word[0], word[1]);
    // The four blocks' scales of these sixteen lanes into one dword: block (lane / 4) % 4 in byte (lane / 4) % 4.
    uint32_t four = e << (8 * ((lane >> 2) & 3));
    four |= ShflXor(four, 4);
    four |= ShflXor(four, 8);
    if ((lane & 15) == 0) *reinterpret_cast<uint32_t*>(scales + AtomOffset(r[p], c[p] / 32, blocks)) = four;
  }
}

// One scale a thread: row r's block b to its place in the atoms (zero for the padding rows).
__global__ void SwizzleKernel(const uint8_t* __restrict__ in, uint8_t* __restrict__ out, int n, int blocks,
                              int64_t items) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= items) return;
  const int r = static_cast<int>(i / blocks);
  const int b = static_cast<int>(i % blocks);
  out[AtomOffset(r, b, blocks)] = r < n ? in[i] : 0;
}

// y[t][r] = sum_blocks (sum_32 E4M3(code) * x) * 2^(s - 127): a wave a row, lane l the 16-code
// vectors l, l + 64, ..., up to 16 tokens (llmp_ops.cu:145-224). Scales: plain [n][k / 32].
template <int kTokens>
__global__ __launch_bounds__(256) void GemvKernel(const uint8_t* __restrict__ codes, const uint8_t* __restrict__ scales,
                                                 const float* __restrict__ x, float* __restrict__ y, int n, int k) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= n) return;  // whole waves
  float acc[kTokens];
#pragma unroll
  for (int t = 0; t < kTokens; ++t) acc[t] = 0.0f;
  const uint8_t* w = codes + static_cast<int64_t>(row) * k;
  for (int v = lane; v < k / 16; v += 64) {
    const U32x4 c = __builtin_nontemporal_load(reinterpret_cast<const U32x4*>(w + v * 16));
    const float s = E8m0ToFloat(scales[static_cast<int64_t>(row) * (k / 32) + v / 2]);
    float wv[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) wv[i] = E4m3ToFloat((c[i / 4] >> (8 * (i % 4))) & 0xFFu);
#pragma unroll
    for (int t = 0; t < kTokens; ++t) {
      const float4* xv = reinterpret_cast<const float4*>(x + static_cast<int64_t>(t) * k + v * 16);
      float dot = 0.0f;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float4 a = xv[q];
        dot = fmaf(wv[4 * q + 0], a.x, dot);
        dot = fmaf(wv[4 * q + 1], a.y, dot);
        dot = fmaf(wv[4 * q + 2], a.z, dot);
        dot = fmaf(wv[4 * q + 3], a.w, dot);
      }
      acc[t] = fmaf(dot, s, acc[t]);
    }
  }
#pragma unroll
  for (int t = 0; t < kTokens; ++t) {
    float v = acc[t];
#pragma unroll
    for (int mask = 32; mask >= 1; mask >>= 1) v += ShflXor(v, mask);
    if (lane == 0) y[static_cast<int64_t>(t) * n + row] = v;
  }
}

// ------------------------------------------------------------------ GEMM


constexpr int kTileM = 256;             // activation rows a workgroup
constexpr int kStepK = 128;             // codes a K step
constexpr int kRingB = 3;               // stages of weight tiles in LDS (of activation tiles: two or three, GemmLds)
constexpr int kTileABytes = kTileM * kStepK;  // 32 KB
constexpr int kScaleStageBytes = 1024;  // two atoms a stage, either operand

struct GemmArgs {
  const uint8_t* a;         // activations, m rows of k codes
  const uint8_t* a_scales;  // atoms
  const uint8_t* b;         // weights, n rows of k codes
  const uint8_t* b_scales;  // atoms
  void* d;
  int m, n, k;  // k: bytes of a row of either operand (the codes of a step are 128 of them)
  int bf16;     // D's elements: 0 F32, 1 BF16, 2 F16
  int tiles_m, tiles_n;
  int64_t ldd;  // elements between D's rows
};

// LDS of GemmKernel<WN>: activation tiles, weight tiles, activation scales, weight scales.
template <int WN, int RA>
struct GemmLds {
  static constexpr int kRingA = RA;
  static constexpr int kTileN = 32 * WN;
  static constexpr int kTileBBytes = kTileN * kStepK;
  static constexpr int kA = 0;
  static constexpr int kB = kA + kRingA * kTileABytes;
  static constexpr int kAScales = kB + kRingB * kTileBBytes;
  static constexpr int kBScales = kAScales + kRingA * kScaleStageBytes;
  static constexpr int kBytes = kBScales + kRingB * kScaleStageBytes;
};

// Position p of a ROWS x 128-byte tile in LDS holds row p / 8's 16-byte chunk
// (p % 8) ^ ((row / 2) % 8). Rows past the operand's end repeat the last (their results are
// never stored).

// Waits until at most `left` of this wave's vector-memory operations are outstanding.
template <int LEFT>
__device__ __forceinline__ void AwaitLoads() {
  __builtin_amdgcn_s_waitcnt(0x0F70 | (LEFT & 15) | ((LEFT >> 4) << 14));
}

// D tile of 256 activation rows by 32 WN weight rows, K step 128, by WM x 2 waves: wave (wm, wn) owns 256 / WM
// activation rows by 16 WN weight rows, the weights as the first operand of v_mfma_scale_f32_16x16x128_f8f6f4.
//
// A workgroup a compute unit goes through its tiles one after the other (two each at M 2048, N 12288). Tiles come
// by global_load_lds into rings in LDS, activations 2 stages and weights 3 (every weight byte is a compulsory HBM
// miss for the first workgroup that asks, activations mostly hit L2). In iteration s, after its barrier: activations
// s + 2 are asked for (into the stage step s used: every wave read its fragments of it during iteration s - 1), then
// weights s + 3, a load after every third product (a CU's path to LDS takes 64 bytes a cycle; its four waves' loads
// after every product would ask for 128); the fragments of step s + 1 are read while step s is multiplied, one read
// after a product (GemmRegs); and at the end all loads but the weights just asked for have landed, so that after the
// next barrier step s + 2 is whole in LDS. One barrier a step; no wave waits for another inside a step. A tile's
// first products start its sums (no clearing), and the next tile's first stages are asked for ahead of this tile's
// stores, which take about 4 us to be accepted (every CU stores its 98 KB at once; stores marked nontemporal made a
// launch 107 us instead of 91).
//
// What bounds a step (M 2048, N 12288, K 4096; measured with a probe of the matrix pipe and with parts of the loop left out): one wave a SIMD issues a
// product every 32 cycles, and a vector move, a read of LDS or (every third product) a load to LDS between two
// products costs 0.3 to 1.2 cycles: they are issued while the product runs. But the clock does not hold: 2.4 GHz on
// zeros, 1.97 GHz with random codes in every CU's products, and 1.35-1.4 GHz when the operands also stream from L2
// at this kernel's rate (64 KB a workgroup a step): 2.7-2.8 PFLOP/s is what the device's power allows with operands
// arriving. The loop here runs at 1.04-1.12 us a step, 2.9-3.1 PFLOP/s while it multiplies, at 1.85-1.9 GHz with its
// pipes 0.75 busy: cycles taken out of it (loads 140 a step, reads of LDS 95, barrier and waits 110 of 2070) come back
// as a lower clock. Two waves a SIMD (eight waves a tile) read 216 KB of LDS a step where four read 168, and LDS's
// 128 bytes a cycle then bound the step; four waves are the default.
//
// Reads of LDS are written as instructions (the compiler would make each wait for every load into LDS in flight): a
// wave waits for them itself at the end of an iteration.

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a constant expression
// (a register number or an instruction's offset field).
template <class F, int... I>
__device__ __forceinline__ void StaticForEach(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void StaticFor(F&& f) {
  StaticForEach(f, std::make_integer_sequence<int, N>{});
}

// The loop's registers are named, not allocated: left to itself the compiler copies an accumulator before every
// product whose neighbours are loads (its D and C end up in different registers) and builds each 32-byte operand
// out of two 16-byte reads with eight moves, all of them on the one pipe that also issues the products.
// With four waves a workgroup (WM = 2, WN = 6):
//   a[4 t .. 4 t + 3], t = 8 i + j        product (i, j)'s sums (192 of the upper registers)
//   v[64 + 8 b ..], b < 9                 activation fragment j < 7 in b = j: the lane's chunks g and 4 + g of row
//                                         16 j + r; fragment 7 in b = 7 on even steps and b = 8 on odd ones
//   v[136 + 48 p + 8 i ..], i < 6         weight fragment i of a step of parity p
//   v[232 + b], v[241 + 6 p + i]          their scales, a byte each
// The second set lets the next step's weight fragments and last activation fragment be read at any time in a step,
// so a step's 42 reads of LDS go one after a product, none in a burst at the step's end. With eight waves (WM = 4)
// there is one set: a fragment's registers are refilled when its last product has been issued.
// The compiler keeps to v0 .. v63 (amdgpu_num_vgpr) and is told once that the kernel uses the rest; what it may
// not see is listed with each helper.
constexpr int GemmCompilerVgprs(int) { return 64; }

// WM waves share the tile's 256 activation rows (2 waves of weights each): 2, a wave a SIMD with 448 registers, or 4, two
// waves a SIMD with 256 each; each of the eight then reads 20 KB of fragments a step where each of four reads 28 KB.
template <int WM, int WN>
struct GemmRegs {
  static constexpr int kXFrags = 16 / WM;                    // 16-row activation fragments a wave
  static constexpr bool kTwice = WM == 2;                    // two sets of weight fragments, two places for the last activation fragment
  static constexpr int kXBuffers = kXFrags + (kTwice ? 1 : 0);
  static constexpr int kWSets = kTwice ? 2 : 1;
  static constexpr int kCompilerVgprs = GemmCompilerVgprs(WM);  // v0 .. for the compiler
  static constexpr int kX = kCompilerVgprs;
  static constexpr int kW = kX + 8 * kXBuffers;
  static constexpr int kXScale = kW + 8 * WN * kWSets;
  static constexpr int kWScale = kXScale + kXBuffers;
  static constexpr int kTop = kWScale + WN * kWSets;
  static constexpr int kSums = 4 * kXFrags * WN;
  static_assert(WM == 2 ? (kTop <= 254 && kSums <= 192) : (kTop <= 160 && kSums <= 96), "the register file");
  static_assert(!kTwice || WN >= 4, "a row of products has a slot for each of four reads");
  // Where fragment j (i) of a step of parity p lies, and its scale.
  static constexpr int XBuffer(int j, int p) { return kTwice && j == kXFrags - 1 ? j + p : j; }
  static constexpr int X(int j, int p) { return kX + 8 * XBuffer(j, p); }
  static constexpr int XScale(int j, int p) { return kXScale + XBuffer(j, p); }
  static constexpr int W(int i, int p) { return kW + 8 * (i + (kTwice ? p * WN : 0)); }
  static constexpr int WScale(int i, int p) { return kWScale + i + (kTwice ? p * WN : 0); }
};

// Fragment registers REG .. REG + 3 from LDS. In flight until the wave's next s_waitcnt lgkmcnt(0).
template <int REG, int OFFSET>
__device__ __forceinline__ void LdsToRegs16(uint32_t at) {
  asm volatile("ds_read_b128 v[%1:%1+3], %0 offset:%2" ::"v"(at), "n"(REG), "n"(OFFSET));
}
template <int REG, int OFFSET>
__device__ __forceinline__ void LdsToReg1(uint32_t at) {
  asm volatile("ds_read_u8 v[%1], %0 offset:%2" ::"v"(at), "n"(REG), "n"(OFFSET));
}
// 16 bytes a lane from `base` + `offset` (a lane's own) to LDS at `to` + 16 lane, without a register between.
__device__ __forceinline__ void GlobalToLds16(const uint8_t* base, uint32_t offset, uint32_t to) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(to), "v"(offset), "s"(base));
}

// sums(T) += weights(I) x activations(J) of a step of parity P, both scaled; FIRST: sums(T) = that product.
template <class R, int T, int I, int J, int P = 0, bool FIRST = false>
__device__ __forceinline__ void ScaledProduct() {
  if constexpr (FIRST) {
    asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 a[%0:%0+3], v[%1:%1+7], v[%2:%2+7], 0, v[%3], v[%4] op_sel_hi:[0,0,0]" ::"n"(T * 4),
                 "n"(R::W(I, P)), "n"(R::X(J, P)), "n"(R::WScale(I, P)), "n"(R::XScale(J, P)));
  } else {
    asm volatile(
        "v_mfma_scale_f32_16x16x128_f8f6f4 a[%0:%0+3], v[%1:%1+7], v[%2:%2+7], a[%0:%0+3], v[%3], v[%4] op_sel_hi:[0,0,0]" ::"n"(
            T * 4),
        "n"(R::W(I, P)), "n"(R::X(J, P)), "n"(R::WScale(I, P)), "n"(R::XScale(J, P)));
  }
}
// The same for F16 operands (a step's 128 bytes a row are 64 values: the fragment's lower chunk is one product's K,
// its upper chunk the next one's): two v_mfma_f32_16x16x32_f16 into the same sums, no scales.
template <class R, int T, int I, int J, int P = 0, bool FIRST = false>
__device__ __forceinline__ void HalfProduct() {
  if constexpr (FIRST) {
    asm volatile("v_mfma_f32_16x16x32_f16 a[%0:%0+3], v[%1:%1+3], v[%2:%2+3], 0\n\t"
                 "v_mfma_f32_16x16x32_f16 a[%0:%0+3], v[%1+4:%1+7], v[%2+4:%2+7], a[%0:%0+3]" ::"n"(T * 4),
                 "n"(R::W(I, P)), "n"(R::X(J, P)));
  } else {
    asm volatile("v_mfma_f32_16x16x32_f16 a[%0:%0+3], v[%1:%1+3], v[%2:%2+3], a[%0:%0+3]\n\t"
                 "v_mfma_f32_16x16x32_f16 a[%0:%0+3], v[%1+4:%1+7], v[%2+4:%2+7], a[%0:%0+3]" ::"n"(T * 4),
                 "n"(R::W(I, P)), "n"(R::X(J, P)));
  }
}
template <int REG>
__device__ __forceinline__ void ClearSum() {
  asm volatile("v_accvgpr_write_b32 a[%0], 0" ::"n"(REG));
}
template <int REG>
__device__ __forceinline__ float ReadSum() {
  float v;
  asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(v) : "n"(REG));
  return v;
}

// Two floats to BF16 (nearest, ties to even; a NaN stays a quiet NaN) in one dword, `lo` in the low half: one
// instruction where the shifts and adds take six a value, 192 values a lane a tile.
__device__ __forceinline__ uint32_t PackBf16(float lo, float hi) {
  uint32_t packed;
  asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(packed) : "v"(lo), "v"(hi));
  return packed;
}

// kHalf: the operands are rows of F16 values and there are no scales (the reconstruction paths' product).
template <int WM, int WN, int RA, bool kHalf = false>
__device__ __forceinline__ void GemmTiles(const GemmArgs& a) {
  using L = GemmLds<WN, RA>;
  using R = GemmRegs<WM, WN>;
  constexpr int kTileN = L::kTileN;
  constexpr int kThreads = WM * 128;
  constexpr int kXFrags = R::kXFrags;
  constexpr int kLoadsA = kTileABytes / 16 / kThreads;     // 8 or 4 a thread a stage
  constexpr int kLoadsB = L::kTileBBytes / 16 / kThreads;  // WN or half of it
  // A load after every kLoadEvery-th product: a CU's path to LDS takes 64 bytes a cycle, its four waves' loads after
  // every product would ask for 128 (1 KB a wave every 32 cycles) and hold the next products back.
  constexpr int kLoadEveryMost = kXFrags * WN / (kLoadsA + 1 + kLoadsB);
  constexpr int kLoadEvery = kLoadEveryMost;
  static_assert(L::kTileBBytes % (16 * kThreads) == 0 && (kLoadsA + 1 + kLoadsB) * kLoadEvery <= kXFrags * WN, "load slots");
  // The kernel's register counts cover the named ones.
  if constexpr (WM == 2) {
    asm volatile("" ::: "v253", "a191");
  } else {
    asm volatile("" ::: "v159", "a95");
  }
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % WM, wn = wave / WM;  // (the two waves of a SIMD, w and w + 4, differ in both)
  const int r = lane & 15, g = lane >> 4;

  // This workgroup's tiles: positions blockIdx.x, + gridDim.x, ... of the launch's order (an XCD a run of tiles, m
  // fastest), one after the other: `mine` of them.
  const int tiles = a.tiles_m * a.tiles_n;
  const int steps = a.k / kStepK;
  const int blocks = a.k / 32;
  const int mine = (tiles - static_cast<int>(blockIdx.x) + static_cast<int>(gridDim.x) - 1) / static_cast<int>(gridDim.x);
  auto origin = [&](int ord, int& m0, int& n0) {
    int tile = static_cast<int>(blockIdx.x) + ord * static_cast<int>(gridDim.x);
    if (tiles % 8 == 0) tile = (tile % 8) * (tiles / 8) + tile / 8;
    m0 = tile % a.tiles_m * kTileM;
    n0 = tile / a.tiles_m * kTileN;
  };
  const int atoms_a = (a.m + 127) / 128, atoms_b = (a.n + 127) / 128;

  // What this thread brings of a stage: position T i + tid of either tile (T threads) is row T / 8 i + tid / 8, and the chunk
  // there is the same for every i. Where its chunks come from, the step's 128 bytes aside (they go into the scalar
  // base), is kept for the whole tile: a vector instruction in the loop takes a matrix instruction's place.
  // The scales: wave 0 the activations', wave 1 the weights', two atoms a stage, 16 bytes a lane.
  const uint32_t chunk_from = static_cast<uint32_t>(((tid & 7) ^ ((tid >> 4) & 7)) * 16);
  const uint8_t* const scales_of = wave == 0 ? a.a_scales : a.b_scales;
  // Load i's rows lie 32 k bytes (T / 8 rows) after load i - 1's, but never past the operand's last row: one
  // register for the first load's place and one for the last row's, an add and a minimum a load (vector instructions
  // that are issued while a product runs), not a register a load.
  uint32_t a_from = 0, b_from = 0, scale_from = 0;
  const uint32_t a_last = static_cast<uint32_t>(a.m - 1) * static_cast<uint32_t>(a.k) + chunk_from;
  const uint32_t b_last = static_cast<uint32_t>(a.n - 1) * static_cast<uint32_t>(a.k) + chunk_from;
  const uint32_t load_stride = static_cast<uint32_t>(kThreads / 8) * static_cast<uint32_t>(a.k);
  auto aim_loads = [&](int ord) {
    int m0, n0;
    origin(ord, m0, n0);
    a_from = static_cast<uint32_t>(min(m0 + (tid >> 3), a.m - 1)) * static_cast<uint32_t>(a.k) + chunk_from;
    b_from = static_cast<uint32_t>(min(n0 + (tid >> 3), a.n - 1)) * static_cast<uint32_t>(a.k) + chunk_from;
    const int atom_mine = wave == 0 ? min(m0 / 128 + (lane >> 5), atoms_a - 1) : min(n0 / 128 + (lane >> 5), atoms_b - 1);
    scale_from = static_cast<uint32_t>(atom_mine) * static_cast<uint32_t>(blocks / 4) * 512u + (lane & 31) * 16;
  };
  const uint32_t lds_at = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds));
  const uint32_t to_mine = lds_at + static_cast<uint32_t>(wave * 64 * 16);
  auto load_a = [&](int i, int step, int stage) {
    GlobalToLds16(a.a + step * kStepK, min(a_from + static_cast<uint32_t>(i) * load_stride, a_last),
                  to_mine + static_cast<uint32_t>(L::kA + stage * kTileABytes + i * kThreads * 16));
  };
  auto load_b = [&](int i, int step, int stage) {
    GlobalToLds16(a.b + step * kStepK, min(b_from + static_cast<uint32_t>(i) * load_stride, b_last),
                  to_mine + static_cast<uint32_t>(L::kB + stage * L::kTileBBytes + i * kThreads * 16));
  };
  // The same in the loop, where a load whose place is computed just before it would wait for that result with the
  // next product behind it: each load leaves the next one's place in `load_from`.
  uint32_t load_from = 0;
  auto load_a_ahead = [&](int i, int step, int stage) {
    GlobalToLds16(a.a + step * kStepK, i == 0 ? a_from : load_from,
                  to_mine + static_cast<uint32_t>(L::kA + stage * kTileABytes + i * kThreads * 16));
    if (i + 1 < kLoadsA) load_from = min(a_from + static_cast<uint32_t>(i + 1) * load_stride, a_last);
  };
  auto load_b_ahead = [&](int i, int step, int stage) {
    GlobalToLds16(a.b + step * kStepK, i == 0 ? b_from : load_from,
                  to_mine + static_cast<uint32_t>(L::kB + stage * L::kTileBBytes + i * kThreads * 16));
    if (i + 1 < kLoadsB) load_from = min(b_from + static_cast<uint32_t>(i + 1) * load_stride, b_last);
  };
  // A stage's scales: wave 0 the activations' into stage_a, wave 1 the weights' into stage_b. (A wave-uniform branch
  // around one load each: the waits below count a wave's loads, and these waves have one more.)
  auto load_scales = [&](int step_a, int stage_a, int step_b, int stage_b) {
    if constexpr (kHalf) return;
    if (wave == 0) {
      GlobalToLds16(scales_of + step_a * 512, scale_from, lds_at + static_cast<uint32_t>(L::kAScales + stage_a * kScaleStageBytes));
    } else if (wave == 1) {
      GlobalToLds16(scales_of + step_b * 512, scale_from, lds_at + static_cast<uint32_t>(L::kBScales + stage_b * kScaleStageBytes));
    }
  };

  auto scale_at = [](int q, int atom0) { return (q / 8 - atom0) * 512 + (q % 2) * 256 + (q % 8) / 2 * 4; };
  const int scale_lane = r * 16 + g;
  // Lane (r, g) wants its row's chunks g and 4 + g; a fragment's rows are 16 f + r, whose swizzle key is r's.
  const uint32_t chunk_lo = static_cast<uint32_t>((r * 8 + (g ^ ((r >> 1) & 7))) * 16);
  const uint32_t chunk_hi = static_cast<uint32_t>((r * 8 + ((4 + g) ^ ((r >> 1) & 7))) * 16);
  const uint32_t frag_a = lds_at + L::kA + static_cast<uint32_t>(wm * kXFrags * 2048);
  const uint32_t frag_b = lds_at + L::kB + static_cast<uint32_t>(wn * WN * 2048);
  // A lane's scale bytes: the activations' at a fixed place a fragment from the wave's base, the weights' at
  // places that depend on the tile (the same for every lane: kept in scalar registers).
  const uint32_t scale_a_base = lds_at + L::kAScales + static_cast<uint32_t>(scale_at(wm * kXFrags, 0) + scale_lane);
  const uint32_t scale_b_base = lds_at + L::kBScales + static_cast<uint32_t>(scale_lane);
  int scale_b_off[WN];
  auto aim_weight_scales = [&](int ord) {
    int m0, n0;
    origin(ord, m0, n0);
#pragma unroll
    for (int i = 0; i < WN; ++i) scale_b_off[i] = __builtin_amdgcn_readfirstlane(scale_at(n0 / 16 + wn * WN + i, n0 / 128));
  };

  // The fragments' registers are refilled in place: an activation fragment's when its row of products has been
  // issued, a weight fragment's when its last product (in the last row) has.
  // (The stage's part of an address is added once an iteration, a fragment's is the instruction's offset.)
  uint32_t a_lo = 0, a_hi = 0, a_scale = 0, b_lo = 0, b_hi = 0, b_scale = 0;
  auto aim_reads = [&](int stage_a, int stage_b) {
    a_lo = frag_a + chunk_lo + static_cast<uint32_t>(stage_a * kTileABytes);
    a_hi = frag_a + chunk_hi + static_cast<uint32_t>(stage_a * kTileABytes);
    a_scale = scale_a_base + static_cast<uint32_t>(stage_a * kScaleStageBytes);
    b_lo = frag_b + chunk_lo + static_cast<uint32_t>(stage_b * L::kTileBBytes);
    b_hi = frag_b + chunk_hi + static_cast<uint32_t>(stage_b * L::kTileBBytes);
    b_scale = scale_b_base + static_cast<uint32_t>(stage_b * kScaleStageBytes);
  };
  // Fragment j (i) of the step the reads are aimed at, into the registers of parity p: its lower chunk, its upper
  // chunk and scale byte, or both.
  auto read_a_lo = [&](auto jc, auto pc) {
    constexpr int j = decltype(jc)::value, p = decltype(pc)::value;
    LdsToRegs16<R::X(j, p), j * 2048>(a_lo);
  };
  auto read_a_hi = [&](auto jc, auto pc) {
    constexpr int j = decltype(jc)::value, p = decltype(pc)::value;
    LdsToRegs16<R::X(j, p) + 4, j * 2048>(a_hi);
    if constexpr (!kHalf) LdsToReg1<R::XScale(j, p), (j % 2) * 256 + (j / 2) * 4>(a_scale);
  };
  auto read_b_lo = [&](auto ic, auto pc) {
    constexpr int i = decltype(ic)::value, p = decltype(pc)::value;
    LdsToRegs16<R::W(i, p), i * 2048>(b_lo);
  };
  auto read_b_hi = [&](auto ic, auto pc) {
    constexpr int i = decltype(ic)::value, p = decltype(pc)::value;
    LdsToRegs16<R::W(i, p) + 4, i * 2048>(b_hi);
    if constexpr (!kHalf) LdsToReg1<R::WScale(i, p), 0>(b_scale + static_cast<uint32_t>(scale_b_off[i]));
  };
  auto read_a = [&](auto jc, auto pc) {
    read_a_lo(jc, pc);
    read_a_hi(jc, pc);
  };
  auto read_b = [&](auto ic, auto pc) {
    read_b_lo(ic, pc);
    read_b_hi(ic, pc);
  };
  auto read_done = [&]() { asm volatile("s_waitcnt lgkmcnt(0)"); };
  auto barrier = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };

  // A tile's first stages: activations 0 .. RA - 1, weights 0, 1 and 2, each with its scales.
  auto first_loads = [&]() {
    StaticFor<(RA > kRingB ? RA : kRingB)>([&](auto sc) {
      constexpr int stage = decltype(sc)::value;
      const int step = min(stage, steps - 1);
      if constexpr (stage < RA) {
#pragma unroll
        for (int i = 0; i < kLoadsA; ++i) load_a(i, step, stage);
      }
      if constexpr (stage < kRingB) {
#pragma unroll
        for (int i = 0; i < kLoadsB; ++i) load_b(i, step, stage);
      }
      if constexpr (!kHalf) {
        if (wave == 0) {
          if constexpr (stage < RA) load_scales(step, stage, step, stage);
        } else if (wave == 1) {
          if constexpr (stage < kRingB) load_scales(step, stage, step, stage);
        }
      }
    });
  };
  using Even = std::integral_constant<int, 0>;
  using Odd = std::integral_constant<int, 1>;

  int stage_a = 0;  // step s's activation stage, s % RA
  int stage_b = 0;  // step s's weight stage, s % 3
  // One step, its fragments in the registers of parity P, the next step's read into those of the other parity.
  int ord = 0;  // the tile that is multiplied
  auto multiply = [&](auto pc, auto firstc, int step) {
    constexpr int P = decltype(pc)::value;
    constexpr bool kFirst = decltype(firstc)::value;  // the tile's first step starts its sums, the others add to them
    using Next = std::integral_constant<int, R::kTwice ? 1 - P : 0>;
    barrier();
    // Every wave holds step `step`'s fragments; steps up to `step` + RA - 1 (weights: + 2) are whole in LDS or on
    // their way, step + 1 whole.
    const int next_a = stage_a + 1 == RA ? 0 : stage_a + 1;      // step + 1's activations
    const int next_b = stage_b + 1 == kRingB ? 0 : stage_b + 1;  // step + 1's weights
    const int bring_a = min(step + RA, steps - 1), bring_b = min(step + 3, steps - 1);
    // After a product at most one load (activations, their scales, weights) and one read of the next step's
    // fragments. With two sets of registers: in row j the activation fragment row j - 1 was multiplied from (in row
    // 0 the last fragment, into its other place), and in the first WN rows a weight fragment each, into the other set.
    // With one: a fragment's registers are refilled when its row (the weights: the last row) has been issued.
    aim_reads(next_a, next_b);
    __builtin_amdgcn_sched_barrier(0);
    StaticFor<kXFrags>([&](auto jc) {
      constexpr int j = decltype(jc)::value;
      StaticFor<WN>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if constexpr (kHalf) {
          HalfProduct<R, kXFrags * i + j, i, j, P, kFirst>();
        } else {
          ScaledProduct<R, kXFrags * i + j, i, j, P, kFirst>();
        }
        constexpr int t = j * WN + i;
        constexpr int q = t % kLoadEvery == 0 ? t / kLoadEvery : kLoadsA + 1 + kLoadsB;  // the load after product t
        if constexpr (q < kLoadsA) {
          load_a_ahead(q, bring_a, stage_a);
        } else if constexpr (q == kLoadsA) {
          load_scales(bring_a, stage_a, bring_b, stage_b);
        } else if constexpr (q - kLoadsA - 1 < kLoadsB) {
          load_b_ahead(q - kLoadsA - 1, bring_b, stage_b);
        }
        if constexpr (R::kTwice) {
          using Before = std::integral_constant<int, j == 0 ? kXFrags - 1 : j - 1>;
          if constexpr (i == 0) read_a_lo(Before{}, Next{});
          if constexpr (i == 1) read_a_hi(Before{}, Next{});
          if constexpr (i == 2 && j < WN) read_b_lo(jc, Next{});
          if constexpr (i == 3 && j < WN) read_b_hi(jc, Next{});
        } else if constexpr (j == kXFrags - 1) {
          read_b(ic, Next{});
        }
        __builtin_amdgcn_sched_barrier(0);
      });
      if constexpr (!R::kTwice) read_a(jc, Next{});
      __builtin_amdgcn_sched_barrier(0);
    });
    read_done();
    // Step + 2 has landed: with two activation stages all but the weights just asked for (and their scales, wave 1),
    // with three everything asked for before this iteration (loads complete in the order they were asked for).
    constexpr int kLeft = RA == 2 ? kLoadsB : kLoadsA + kLoadsB;
    if (!kHalf && (wave == 1 || (RA > 2 && wave == 0))) {
      AwaitLoads<kLeft + 1>();
    } else {
      AwaitLoads<kLeft>();
    }
    stage_a = next_a;
    stage_b = next_b;
  };
  // A finished tile's sums to D: sums(8 i + j)[q] = D[m0 + wm 128 + 16 j + r][n0 + wn 16 WN + 16 i + 4 g + q]. A tile
  // inside the matrix (the common one) stores without a test an element. The sums stay as they are: the next tile's
  // first products do not add to them.
  auto store_tile = [&](int of) {
    int m0, n0;
    origin(of, m0, n0);
    const int m_first = m0 + wm * 16 * kXFrags + r, n_first = n0 + wn * 16 * WN + 4 * g;  // n is a multiple of 4 (checked on the host)
    const int64_t first = static_cast<int64_t>(m_first) * a.ldd + n_first;
    const int64_t row_step = a.ldd * 16;
    auto store = [&](auto kind, auto whole) {
      StaticFor<kXFrags>([&](auto jc) {
        constexpr int j = decltype(jc)::value;
        StaticFor<WN>([&](auto ic) {
          constexpr int i = decltype(ic)::value;
          constexpr int reg = (kXFrags * i + j) * 4;
          const float v0 = ReadSum<reg>(), v1 = ReadSum<reg + 1>(), v2 = ReadSum<reg + 2>(), v3 = ReadSum<reg + 3>();
          if (!decltype(whole)::value && (m_first + 16 * j >= a.m || n_first + 16 * i >= a.n)) return;
          const int64_t at = first + j * row_step + i * 16;
          if constexpr (decltype(kind)::value == 1) {
            uint2 packed;
            packed.x = PackBf16(v0, v1);
            packed.y = PackBf16(v2, v3);
            *reinterpret_cast<uint2*>(static_cast<uint16_t*>(a.d) + at) = packed;
          } else if constexpr (decltype(kind)::value == 2) {
            uint2 packed;
            packed.x = FloatToHalfBits(v0) | (FloatToHalfBits(v1) << 16);
            packed.y = FloatToHalfBits(v2) | (FloatToHalfBits(v3) << 16);
            *reinterpret_cast<uint2*>(static_cast<uint16_t*>(a.d) + at) = packed;
          } else {
            *reinterpret_cast<float4*>(static_cast<float*>(a.d) + at) = make_float4(v0, v1, v2, v3);
          }
        });
      });
    };
    const bool whole = m0 + kTileM <= a.m && n0 + kTileN <= a.n;
    using F32Out = std::integral_constant<int, 0>;
    using Bf16Out = std::integral_constant<int, 1>;
    using F16Out = std::integral_constant<int, 2>;
    if constexpr (kHalf) {  // F16 or F32
      if (a.bf16 == 2) {
        if (whole) {
          store(F16Out{}, std::true_type{});
        } else {
          store(F16Out{}, std::false_type{});
        }
      } else {
        if (whole) {
          store(F32Out{}, std::true_type{});
        } else {
          store(F32Out{}, std::false_type{});
        }
      }
    } else if (a.bf16) {
      if (whole) {
        store(Bf16Out{}, std::true_type{});
      } else {
        store(Bf16Out{}, std::false_type{});
      }
    } else {
      if (whole) {
        store(F32Out{}, std::true_type{});
      } else {
        store(F32Out{}, std::false_type{});
      }
    }
  };

  aim_loads(0);
  first_loads();
  for (; ord < mine; ++ord) {
    if constexpr (!kHalf) aim_weight_scales(ord);
    // The tile's first stages have landed (they were asked for ahead of the tile before's stores, which this wait
    // counts as well), for every wave. The launch's first tile has no stores behind it and starts like a step: its
    // third stage of weights, asked for last, may still be on its way (the first step's own wait takes it in).
    if (ord == 0 && RA == 2) {
      if (!kHalf && wave == 1) {
        AwaitLoads<kLoadsB + 1>();
      } else {
        AwaitLoads<kLoadsB>();
      }
    } else {
      AwaitLoads<0>();
    }
    barrier();
    aim_reads(0, 0);
    StaticFor<kXFrags>([&](auto j) { read_a(j, Even{}); });
    StaticFor<WN>([&](auto i) { read_b(i, Even{}); });
    read_done();
    stage_a = 0;
    stage_b = 0;
    multiply(Even{}, std::true_type{}, 0);
    int step = 1;
    for (; step + 1 < steps; step += 2) {
      multiply(Odd{}, std::false_type{}, step);
      multiply(Even{}, std::false_type{}, step + 1);
    }
    if (step < steps) multiply(Odd{}, std::false_type{}, step);
    // The next tile's first stages are asked for ahead of this tile's stores: they land while the stores are taken.
    // (This wave's loads still on their way, the last step asked for again, go to places of its own and land first.)
    if (ord + 1 < mine) {
      aim_loads(ord + 1);
      first_loads();
    }
    // The last products' sums are written passes after their issue: no read of them before.
    asm volatile("s_nop 15\n\ts_nop 15");
    store_tile(ord);
  }
  AwaitLoads<0>();  // nothing may land in LDS after the workgroup has gone
}

// The two tile shapes, four waves each, one a SIMD. (Eight waves of 64 x 64 on the 256 x 128 tile with three
// activation stages, two waves a SIMD issuing into each other's products, take 1.10 us a step against this form's
// 1.03: eight waves read 176 KB of LDS a step.) A kernel's register attribute cannot depend on a template's argument:
// one kernel a shape.
__global__ __launch_bounds__(256, 1) __attribute__((amdgpu_num_vgpr(GemmCompilerVgprs(2)))) void GemmKernel192(const GemmArgs a) {
  GemmTiles<2, 6, 2>(a);
}
__global__ __launch_bounds__(256, 1) __attribute__((amdgpu_num_vgpr(GemmCompilerVgprs(2)))) void GemmKernel128(const GemmArgs a) {
  GemmTiles<2, 4, 2>(a);
}
constexpr int kWavesM128 = 2, kRingA128 = 2;
// The same two shapes over F16 operands.
__global__ __launch_bounds__(256, 1) __attribute__((amdgpu_num_vgpr(GemmCompilerVgprs(2)))) void GemmKernelHalf192(const GemmArgs a) {
  GemmTiles<2, 6, 2, true>(a);
}
__global__ __launch_bounds__(256, 1) __attribute__((amdgpu_num_vgpr(GemmCompilerVgprs(2)))) void GemmKernelHalf128(const GemmArgs a) {
  GemmTiles<2, 4, 2, true>(a);
}


// A workgroup a compute unit, each through its share of the tiles (fewer workgroups where there are fewer tiles).
template <int WM, int WN, int RA, bool kHalf = false>
int LaunchGemm(void (*kernel)(const GemmArgs), GemmArgs a, int compute_units, hipStream_t stream) {
  using L = GemmLds<WN, RA>;
  static_assert(L::kBytes <= 160 * 1024, "the stages do not fit a CU's LDS");
  a.tiles_n = (a.n + L::kTileN - 1) / L::kTileN;
  static bool sized = false;  // (one a kernel: the template's arguments name it)
  if (!AllowLds(reinterpret_cast<const void*>(kernel), L::kBytes, &sized)) return LaunchStatus("mxfp8.gemm");
  const int tiles = a.tiles_m * a.tiles_n;
  hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(tiles < compute_units ? tiles : compute_units)), dim3(WM * 128), L::kBytes, stream, a);
  return LaunchStatus("mxfp8.gemm");
}

}  // namespace

// D[m][n] (rows ldd elements apart; F16 if f16_out, else F32) = A[m][k] B[n][k]^T over F16 operands whose rows follow
// each other, F32 sums: the MXFP8 product's loop with two F16 products where it has a scaled one. k a multiple of 64,
// n of 4, operands and D at 16-byte boundaries (the caller's checks). Queues one launch.
int LaunchHalfGemm(const void* a_rows, const void* b_rows, void* d, int m, int n, int k, int64_t ldd, bool f16_out,
                   int compute_units, hipStream_t stream) {
  GemmArgs a;
  a.a = static_cast<const uint8_t*>(a_rows);
  a.a_scales = nullptr;
  a.b = static_cast<const uint8_t*>(b_rows);
  a.b_scales = nullptr;
  a.d = d;
  a.m = m;
  a.n = n;
  a.k = 2 * k;
  a.bf16 = f16_out ? 2 : 0;
  a.ldd = ldd;
  a.tiles_m = (m + kTileM - 1) / kTileM;
  a.tiles_n = 0;
  const int cus = compute_units > 0 ? compute_units : 256;
  int best = 0;
  int64_t best_cost = 0;
  for (const int tile_n : {192, 128}) {
    const int64_t tiles = static_cast<int64_t>(a.tiles_m) * ((n + tile_n - 1) / tile_n);
    const int64_t cost = (tiles + cus - 1) / cus * tile_n;
    if (best == 0 || cost < best_cost) best = tile_n, best_cost = cost;
  }
  return best == 192 ? LaunchGemm<2, 6, 2, true>(GemmKernelHalf192, a, cus, stream)
                     : LaunchGemm<kWavesM128, 4, kRingA128, true>(GemmKernelHalf128, a, cus, stream);
}

}  // namespace llmp_hip

using namespace llmp_hip;

extern "C" int llmp_hip_mxfp8_quantize(const void* x, int x_type, int64_t x_stride, int64_t k, int64_t rows, void* codes,
                                       void* scales, void* stream) {
  BeginLaunches();
  if (x == nullptr || codes == nullptr || scales == nullptr) return Refuse(1, "mxfp8.quantize: null operand");
  if (k <= 0 || k % 128 != 0) return Refuse(1, "mxfp8.quantize: k %lld is not whole 128-value scale groups", (long long)k);
  if (rows <= 0 || rows > (1 << 24)) return Refuse(1, "mxfp8.quantize: 1 to 2^24 rows");
  if (x_type != LLMP_X_F32 && x_type != LLMP_X_BF16) return Refuse(1, "mxfp8.quantize: F32 or BF16 rows");
  if (reinterpret_cast<uintptr_t>(codes) % 16 != 0) return Refuse(1, "mxfp8.quantize: codes not 16-byte aligned");
  const int64_t padded = (rows + 127) / 128 * 128;
  const int64_t items = padded * (k / 32);
  const dim3 grid(static_cast<unsigned>((items + 255) / 256));
  const auto s = static_cast<hipStream_t>(stream);
  // Rows that start on 16-byte boundaries (and scales on 4-byte ones): eight values a lane.
  const int64_t element = x_type == LLMP_X_F32 ? 4 : 2;
  if (reinterpret_cast<uintptr_t>(x) % 16 == 0 && (x_stride * element) % 16 == 0 && reinterpret_cast<uintptr_t>(scales) % 4 == 0 &&
      reinterpret_cast<uintptr_t>(codes) % 8 == 0) {
    const int64_t wide_items = padded * (k / 8);
    const dim3 wide_grid(static_cast<unsigned>((wide_items + 255) / 256));
    if (x_type == LLMP_X_F32) {
      hipLaunchKernelGGL(QuantizeWideKernel<float>, wide_grid, dim3(256), 0, s, static_cast<const float*>(x), x_stride,
                         static_cast<uint8_t*>(codes), static_cast<uint8_t*>(scales), static_cast<int>(k),
                         static_cast<int>(rows), wide_items);
    } else {
      hipLaunchKernelGGL(QuantizeWideKernel<uint16_t>, wide_grid, dim3(256), 0, s, static_cast<const uint16_t*>(x), x_stride,
                         static_cast<uint8_t*>(codes), static_cast<uint8_t*>(scales), static_cast<int>(k),
                         static_cast<int>(rows), wide_items);
    }
    return LaunchStatus("mxfp8.quantize");
  }
  if (x_type == LLMP_X_F32) {
    hipLaunchKernelGGL(QuantizeKernel<float>, grid, dim3(256), 0, s, static_cast<const float*>(x), x_stride,
                       static_cast<uint8_t*>(codes), static_cast<uint8_t*>(scales), static_cast<int>(k),
                       static_cast<int>(rows), items);
  } else {
    hipLaunchKernelGGL(QuantizeKernel<uint16_t>, grid, dim3(256), 0, s, static_cast<const uint16_t*>(x), x_stride,
                       static_cast<uint8_t*>(codes), static_cast<uint8_t*>(scales), static_cast<int>(k),
                       static_cast<int>(rows), items);
  }
  return LaunchStatus("mxfp8.quantize");
}

extern "C" int llmp_hip_mxfp8_swizzle(const void* scales, int64_t n, int64_t k, void* out, void* stream) {
  BeginLaunches();
  if (scales == nullptr || out == nullptr) return Refuse(1, "mxfp8.swizzle: null operand");
  if (n <= 0 || k <= 0 || k % 128 != 0) return Refuse(1, "mxfp8.swizzle: k is not whole 128-value scale groups");
  const int64_t padded = (n + 127) / 128 * 128;
  const int64_t items = padded * (k / 32);
  hipLaunchKernelGGL(SwizzleKernel, dim3(static_cast<unsigned>((items + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint8_t*>(scales), static_cast<uint8_t*>(out),
                     static_cast<int>(n), static_cast<int>(k / 32), items);
  return LaunchStatus("mxfp8.swizzle");
}

extern "C" int llmp_hip_mxfp8_gemv(const void* codes, const void* scales, int64_t n, int64_t k, const float* x,
                                   int tokens, float* y, void* stream) {
  BeginLaunches();
  if (codes == nullptr || scales == nullptr || x == nullptr || y == nullptr) return Refuse(1, "mxfp8.mul_mat_vec: null operand");
  if (k <= 0 || k % 32 != 0 || n <= 0) return Refuse(1, "mxfp8.mul_mat_vec: k is not whole 32-value blocks");
  if (tokens < 1 || tokens > 16) return Refuse(1, "mxfp8.mul_mat_vec: 1 to 16 tokens, not %d", tokens);
  if ((reinterpret_cast<uintptr_t>(codes) | reinterpret_cast<uintptr_t>(x)) % 16 != 0)
    return Refuse(1, "mxfp8.mul_mat_vec: operands not 16-byte aligned");
  const dim3 grid(static_cast<unsigned>((n + 3) / 4));
  const auto s = static_cast<hipStream_t>(stream);
  const auto* c = static_cast<const uint8_t*>(codes);
  const auto* sc = static_cast<const uint8_t*>(scales);
#define LLMP_GEMV(T) \
  case T:            \
    hipLaunchKernelGGL(GemvKernel<T>, grid, dim3(256), 0, s, c, sc, x, y, static_cast<int>(n), static_cast<int>(k)); \
    break;
  switch (tokens) {
    LLMP_GEMV(1) LLMP_GEMV(2) LLMP_GEMV(3) LLMP_GEMV(4) LLMP_GEMV(5) LLMP_GEMV(6) LLMP_GEMV(7) LLMP_GEMV(8)
    LLMP_GEMV(9) LLMP_GEMV(10) LLMP_GEMV(11) LLMP_GEMV(12) LLMP_GEMV(13) LLMP_GEMV(14) LLMP_GEMV(15) LLMP_GEMV(16)
  }
#undef LLMP_GEMV
  return LaunchStatus("mxfp8.mul_mat_vec");
}

extern "C" int llmp_hip_mxfp8_gemm_available(void) { return 1; }

extern "C" size_t llmp_hip_mxfp8_gemm_scratch(const llmp_mxfp8_gemm* gemm, int compute_units) {
  (void)gemm;
  (void)compute_units;
  return 0;  // the product needs no workspace
}

extern "C" int llmp_hip_mxfp8_gemm_run(const llmp_mxfp8_gemm* gemm, int compute_units, void* stream) {
  BeginLaunches();
  if (gemm == nullptr) return Refuse(1, "mxfp8.gemm: null descriptor");
  if (gemm->a == nullptr || gemm->a_scales == nullptr || gemm->b == nullptr || gemm->b_scales == nullptr ||
      gemm->d == nullptr)
    return Refuse(1, "mxfp8.gemm: null operand");
  if (gemm->m <= 0 || gemm->n <= 0 || gemm->k <= 0) return Refuse(1, "mxfp8.gemm: empty product");
  if (gemm->k % 128 != 0) return Refuse(1, "mxfp8.gemm: k %d is not whole 128-value scale groups", gemm->k);
  if (gemm->n % 4 != 0) return Refuse(1, "mxfp8.gemm: n %d is not a multiple of 4", gemm->n);
  const uintptr_t align = reinterpret_cast<uintptr_t>(gemm->a) | reinterpret_cast<uintptr_t>(gemm->b) |
                          reinterpret_cast<uintptr_t>(gemm->d);
  if (align % 16 != 0) return Refuse(1, "mxfp8.gemm: codes or output not 16-byte aligned");
  if (static_cast<int64_t>(gemm->m) * gemm->k >= (int64_t{1} << 32) || static_cast<int64_t>(gemm->n) * gemm->k >= (int64_t{1} << 32))
    return Refuse(1, "mxfp8.gemm: an operand of 4 GiB or more");
  if ((reinterpret_cast<uintptr_t>(gemm->a_scales) | reinterpret_cast<uintptr_t>(gemm->b_scales)) % 4 != 0)
    return Refuse(1, "mxfp8.gemm: scales not 4-byte aligned");
  GemmArgs a;
  a.a = static_cast<const uint8_t*>(gemm->a);
  a.a_scales = static_cast<const uint8_t*>(gemm->a_scales);
  a.b = static_cast<const uint8_t*>(gemm->b);
  a.b_scales = static_cast<const uint8_t*>(gemm->b_scales);
  a.d = gemm->d;
  a.m = gemm->m;
  a.n = gemm->n;
  a.k = gemm->k;
  a.bf16 = gemm->bf16 != 0 ? 1 : 0;
  a.ldd = gemm->n;
  a.tiles_m = (gemm->m + kTileM - 1) / kTileM;
  a.tiles_n = 0;
  // The weight rows a workgroup takes (192 or 128): whichever leaves the fewest idle
  // compute units in the last round of workgroups, the larger on a tie.
  const int cus = compute_units > 0 ? compute_units : 256;
  int best = 0;
  int64_t best_cost = 0;
  for (const int tile_n : {192, 128}) {
    const int64_t tiles = static_cast<int64_t>(a.tiles_m) * ((gemm->n + tile_n - 1) / tile_n);
    if (tiles > (1 << 30)) return Refuse(1, "mxfp8.gemm: too many tiles");
    const int64_t cost = (tiles + cus - 1) / cus * tile_n;
    if (best == 0 || cost < best_cost) best = tile_n, best_cost = cost;
  }
  const hipStream_t on = static_cast<hipStream_t>(stream);
  const int status = best == 192 ? LaunchGemm<2, 6, 2>(GemmKernel192, a, cus, on) : LaunchGemm<kWavesM128, 4, kRingA128>(GemmKernel128, a, cus, on);
  return status;  // negative: the launch failed after the checks (the caller's fault path)
}

