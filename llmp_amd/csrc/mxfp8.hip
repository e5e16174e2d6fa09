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

typedef int V8i __attribute__((ext_vector_type(8)));
typedef float V4f __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* LdsPointer;
typedef const __attribute__((address_space(1))) void* GlobalPointer;

constexpr int kTileM = 256;             // activation rows a workgroup
constexpr int kStepK = 128;             // codes a K step
constexpr int kGemmThreads = 512;       // 8 waves: 4 along m, 2 along n
constexpr int kGroupThreads = 256;      // a group: the four waves with the same position along n
constexpr int kRingA = 2;               // stages of activation tiles in LDS
constexpr int kRingB = 3;               // stages of weight tiles
constexpr int kTileABytes = kTileM * kStepK;  // 32 KB
constexpr int kLoadsA = kTileABytes / 16 / kGroupThreads;  // 8 a thread of group 1 a stage
constexpr int kScaleStageBytes = 1024;  // two atoms a stage, either operand

struct GemmArgs {
  const uint8_t* a;         // activations, m rows of k codes
  const uint8_t* a_scales;  // atoms
  const uint8_t* b;         // weights, n rows of k codes
  const uint8_t* b_scales;  // atoms
  void* d;
  int m, n, k;
  int bf16;
  int tiles_m, tiles_n;
};

// Timeline instrumentation for tuning, compiled only with -DLLMP_GEMM_TRACE (never into the library): lane 0 of
// every wave stores the 100 MHz clock at up to eight points of its tile, eight 64-bit words a wave.
#ifdef LLMP_GEMM_TRACE
__device__ unsigned long long* g_gemm_trace = nullptr;
#define GEMM_TRACE(slot)                                                                                          \
  do {                                                                                                            \
    if (g_gemm_trace != nullptr && (threadIdx.x & 63) == 0)                                                       \
      g_gemm_trace[(static_cast<size_t>(blockIdx.x) * (blockDim.x / 64) + threadIdx.x / 64) * 8 + (slot)] = wall_clock64(); \
  } while (0)
// ... or the shader clock's counter (slots 1 and 6: the kernel's cycles between them give its clock).
#define GEMM_TRACE_CYCLES(slot)                                                                                   \
  do {                                                                                                            \
    if (g_gemm_trace != nullptr && (threadIdx.x & 63) == 0)                                                       \
      g_gemm_trace[(static_cast<size_t>(blockIdx.x) * (blockDim.x / 64) + threadIdx.x / 64) * 8 + (slot)] = __builtin_readcyclecounter(); \
  } while (0)
#else
#define GEMM_TRACE(slot) \
  do {                   \
  } while (0)
#define GEMM_TRACE_CYCLES(slot) \
  do {                          \
  } while (0)
#endif

// LDS of GemmKernel<WN>: activation tiles, weight tiles, activation scales, weight scales.
template <int WN>
struct GemmLds {
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

// A 16-row fragment: the lane's two 16-byte chunks, at lo and hi bytes into it.
__device__ __forceinline__ V8i ReadFragment(const uint8_t* fragment, int lo_at, int hi_at) {
  const U32x4 lo = *reinterpret_cast<const U32x4*>(fragment + lo_at);
  const U32x4 hi = *reinterpret_cast<const U32x4*>(fragment + hi_at);
  V8i v;
  v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w;
  v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
  return v;
}

// Waits until at most `left` of this wave's vector-memory operations are outstanding.
template <int LEFT>
__device__ __forceinline__ void AwaitLoads() {
  __builtin_amdgcn_s_waitcnt(0x0F70 | (LEFT & 15) | ((LEFT >> 4) << 14));
}

// D tile of 256 activation rows by 32 WN weight rows, K step 128. Wave (wm, wn) of 4 x 2 owns
// 64 x 16 WN of it: WN x 4 MFMA tiles, the weights as the first operand.
//
// The two waves of a SIMD (wn 0 and 1: the hardware places waves 0-3 and 4-7 of a workgroup
// one on each SIMD) work half a step apart. A step of a wave is a read phase (its 4 + WN
// fragments and their scales from LDS into registers) and a multiply phase (4 WN MFMAs);
// every phase ends at a workgroup barrier, and group 1 sits the first phase out, so that
// while one wave of a SIMD multiplies the other reads: the matrix pipe and LDS both stay
// busy. Phases, counted from 0: group 0 reads step s in phase 2 s and multiplies in 2 s + 1,
// group 1 reads in 2 s + 1 and multiplies in 2 s + 2.
//
// Tiles come by global_load_lds, issued between the MFMAs of the multiply phases (the only
// time a wave has issue slots to spare): group 1 brings activations s + 2 while it
// multiplies step s, into the stage step s used (ring of 2; free since the barrier that ended
// phase 2 s + 1), and waits for them at the end of its next read phase, before the barrier
// that opens phase 2 s + 4. Group 0 brings weights s + 2 while it multiplies step s, into the
// stage step s - 1 used (ring of 3: every weight byte is a compulsory HBM miss for the first
// workgroup that asks, activations mostly hit L2), and waits for weights s + 1, leaving s + 2
// in flight, before the barrier that ends its multiply phase.
template <int WN>
__global__ __launch_bounds__(kGemmThreads, 1) void GemmKernel(const GemmArgs a) {
  using L = GemmLds<WN>;
  constexpr int kTileN = L::kTileN;
  constexpr int kLoadsB = L::kTileBBytes / 16 / kGroupThreads;  // WN a thread of group 0 a stage
  constexpr int kLoadEvery = WN / 2;  // MFMAs between two loads: 8 loads fit 4 WN MFMAs
  static_assert(kLoadsB <= kLoadsA && kLoadsA * kLoadEvery <= 4 * WN, "the loads do not fit a multiply phase");
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  GEMM_TRACE(0);  // the wave's start
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 3, wn = wave >> 2;
  const int group = wn;
  const int r = lane & 15, g = lane >> 4;

  // Workgroups go round-robin to the eight XCDs, each with its own L2: give every XCD a
  // contiguous run of tiles, walking m fastest, so the workgroups resident on an XCD share
  // weight tiles (all m of a few n) and every activation tile.
  int tile = blockIdx.x;
  const int tiles = a.tiles_m * a.tiles_n;
  if (tiles % 8 == 0) tile = (tile % 8) * (tiles / 8) + tile / 8;
  const int tm = tile % a.tiles_m, tn = tile / a.tiles_m;
  const int m0 = tm * kTileM, n0 = tn * kTileN;
  const int steps = a.k / kStepK;
  const int blocks = a.k / 32;

  // What this thread brings: group 1 the activation tile, group 0 the weight tile; the
  // group's first wave also the operand's scales, two atoms (128 rows by the step's four
  // blocks each) a stage. An atom past the operand's padded rows repeats the last.
  const int loads = group == 1 ? kLoadsA : kLoadsB;
  const uint8_t* const matrix = group == 1 ? a.a : a.b;
  // Its position p = 256 i + t of a tile is row 32 i + t / 8, and the chunk there is the same
  // for every i (the swizzle key of 32 i + t / 8 is that of t / 8).
  const int thread = tid & (kGroupThreads - 1);
  const int row_first = (group == 1 ? m0 : n0) + (thread >> 3);
  const int row_last = (group == 1 ? a.m : a.n) - 1;
  const uint32_t chunk_from = static_cast<uint32_t>(((thread & 7) ^ ((thread >> 4) & 7)) * 16);
  const int atom_b0 = n0 / 128;
  const int atoms = ((group == 1 ? a.m : a.n) + 127) / 128;
  const int atom_mine = min((group == 1 ? m0 / 128 : atom_b0) + (lane >> 5), atoms - 1);
  const uint8_t* const from_scale = (group == 1 ? a.a_scales : a.b_scales) +
                                    static_cast<int64_t>(atom_mine) * (blocks / 4) * 512 + (lane & 31) * 16;
  const int tile_base = group == 1 ? L::kA : L::kB;
  const int tile_bytes = group == 1 ? kTileABytes : L::kTileBBytes;
  const int scale_base = group == 1 ? L::kAScales : L::kBScales;
  // Load i of this wave of its operand's tile of K step `step` into ring stage `stage`.
  auto load = [&](int i, int step, int stage) {
    uint8_t* to = lds + tile_base + stage * tile_bytes + (i * kGroupThreads + wm * 64) * 16;
    // Recomputed at every use: eight 64-bit addresses kept across the steps would not fit the
    // register file beside the accumulators and fragments.
    int row = row_first;
    asm volatile("" : "+v"(row));
    const uint32_t from = static_cast<uint32_t>(min(row + 32 * i, row_last)) * static_cast<uint32_t>(a.k) + chunk_from;
    __builtin_amdgcn_global_load_lds((GlobalPointer)(matrix + step * kStepK + from), (LdsPointer)to, 16, 0, 0);
  };
  auto load_scales = [&](int step, int stage) {
    if (wm == 0) {
      __builtin_amdgcn_global_load_lds((GlobalPointer)(from_scale + step * 512),
                                       (LdsPointer)(lds + scale_base + stage * kScaleStageBytes), 16, 0, 0);
    }
  };

  // Where a lane's scale bytes sit in a scale stage. Row 16 q + r of an operand has its four
  // scales at atom q / 8, byte (q % 2) 256 + r 16 + (q % 8) / 2 * 4: a part per 16 rows that
  // is the same for every lane, plus 16 r + g.
  auto scale_at = [](int q, int atom0) { return (q / 8 - atom0) * 512 + (q % 2) * 256 + (q % 8) / 2 * 4; };
  const int scale_lane = r * 16 + g;
  int scale_x[4], scale_w[WN];
#pragma unroll
  for (int j = 0; j < 4; ++j) scale_x[j] = scale_at(wm * 4 + j, 0);
#pragma unroll
  for (int i = 0; i < WN; ++i) scale_w[i] = scale_at(n0 / 16 + wn * WN + i, atom_b0);

  // Lane (r, g) wants its row's chunks g and 4 + g; a fragment's rows are 16 f + r, whose
  // swizzle key is r's.
  const int chunk_lo = (r * 8 + (g ^ ((r >> 1) & 7))) * 16;
  const int chunk_hi = (r * 8 + ((4 + g) ^ ((r >> 1) & 7))) * 16;

  V4f acc[WN][4];
#pragma unroll
  for (int i = 0; i < WN; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = V4f{0.0f, 0.0f, 0.0f, 0.0f};
  V8i xf[4], wf[WN];
  int xscale[4], wscale[WN];

  // Step s's fragments and scales into registers. Fragment f of a tile is 2 KB further on for
  // every lane; a lane's scale is one byte.
  auto read = [&](int stage_a, int stage_b) {
    const uint8_t* tile_a = lds + L::kA + stage_a * kTileABytes + wm * 4 * 2048;
    const uint8_t* tile_b = lds + L::kB + stage_b * L::kTileBBytes + wn * WN * 2048;
    const uint8_t* scales_a = lds + L::kAScales + stage_a * kScaleStageBytes + scale_lane;
    const uint8_t* scales_b = lds + L::kBScales + stage_b * kScaleStageBytes + scale_lane;
#pragma unroll
    for (int j = 0; j < 4; ++j) xscale[j] = scales_a[scale_x[j]];
#pragma unroll
    for (int i = 0; i < WN; ++i) wscale[i] = scales_b[scale_w[i]];
#pragma unroll
    for (int j = 0; j < 4; ++j) xf[j] = ReadFragment(tile_a + j * 2048, chunk_lo, chunk_hi);
#pragma unroll
    for (int i = 0; i < WN; ++i) wf[i] = ReadFragment(tile_b + i * 2048, chunk_lo, chunk_hi);
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): in registers before the barrier that lets the stage go
    __builtin_amdgcn_sched_barrier(0);
  };
  // The 4 WN MFMAs of a step, with this wave's loads of K step `step` into ring stage `stage`
  // between them. Past the last step the last is asked for again, into a stage nobody reads
  // any more: no branch on it, and the loads a wave has in flight stay the same number.
  auto multiply = [&](int step, int stage) {
    const int bring = min(step, steps - 1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < WN; ++i) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[i], xf[j], acc[i][j], 0, 0, 0, wscale[i], 0, xscale[j]);
        // Pins the MFMA here in program order (the compiler would otherwise sink all of them
        // below the loads, which have side effects and so keep their place).
        asm volatile("" : "+v"(acc[i][j]));
        const int t = i * 4 + j;
        if (t % kLoadEvery == kLoadEvery - 1 && t / kLoadEvery < kLoadsA) {
          if (t / kLoadEvery < loads) load(t / kLoadEvery, bring, stage);
        }
      }
    }
    load_scales(bring, stage);
    __builtin_amdgcn_sched_barrier(0);
  };
  auto barrier = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };

  // Before the first phase: activations 0 and 1, weights 0 and 1.
#pragma unroll
  for (int i = 0; i < kLoadsA; ++i)
    if (i < loads) load(i, 0, 0);
  load_scales(0, 0);
  if (steps > 1) {
#pragma unroll
    for (int i = 0; i < kLoadsA; ++i)
      if (i < loads) load(i, 1, 1);
    load_scales(1, 1);
  }
  GEMM_TRACE_CYCLES(1);  // the first two stages asked for
  AwaitLoads<0>();
  barrier();
  GEMM_TRACE(2);  // ... and landed, for every wave
  if (group == 1) barrier();
  int stage_b = 0;  // step s's weight stage, s % 3
  for (int step = 0; step < steps; ++step) {
    if (step == 1) GEMM_TRACE(3);
    if (step == steps / 2) GEMM_TRACE(4);
    read(step & 1, stage_b);
    // Group 1: activations step + 1, asked for while multiplying step - 1, have landed.
    if (group == 1) AwaitLoads<0>();
    barrier();
    int to = stage_b + 2;  // (step + 2) % 3
    if (to >= kRingB) to -= kRingB;
    multiply(step + 2, group == 1 ? (step & 1) : to);
    // Group 0: weights step + 1 have landed; step + 2, just asked for, may stay in flight.
    if (group == 0) {
      if (wm == 0) {
        AwaitLoads<kLoadsB + 1>();
      } else {
        AwaitLoads<kLoadsB>();
      }
    }
    barrier();
    if (++stage_b == kRingB) stage_b = 0;
  }
  GEMM_TRACE(5);  // the last step multiplied
  if (group == 0) barrier();
  AwaitLoads<0>();  // nothing may land in LDS after the workgroup has gone
  GEMM_TRACE_CYCLES(6);

  // acc[i][j][q] = D[m0 + wm 64 + 16 j + r][n0 + wn 16 WN + 16 i + 4 g + q]
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int m = m0 + wm * 64 + j * 16 + r;
    if (m >= a.m) continue;
#pragma unroll
    for (int i = 0; i < WN; ++i) {
      const int n = n0 + wn * 16 * WN + i * 16 + 4 * g;
      if (n >= a.n) continue;  // n is a multiple of 4 (checked on the host)
      const V4f v = acc[i][j];
      if (a.bf16) {
        uint2 packed;
        packed.x = FloatToBf16Bits(v[0]) | (FloatToBf16Bits(v[1]) << 16);
        packed.y = FloatToBf16Bits(v[2]) | (FloatToBf16Bits(v[3]) << 16);
        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(a.d) + static_cast<int64_t>(m) * a.n + n) = packed;
      } else {
        *reinterpret_cast<float4*>(static_cast<float*>(a.d) + static_cast<int64_t>(m) * a.n + n) =
            make_float4(v[0], v[1], v[2], v[3]);
      }
    }
  }
  GEMM_TRACE(7);  // the tile's stores queued
}

template <int WN>
int LaunchGemm(GemmArgs a, hipStream_t stream) {
  using L = GemmLds<WN>;
  static_assert(L::kBytes <= 160 * 1024, "the stages do not fit a CU's LDS");
  a.tiles_n = (a.n + L::kTileN - 1) / L::kTileN;
  static bool sized = false;
  if (!AllowLds(reinterpret_cast<const void*>(&GemmKernel<WN>), L::kBytes, &sized)) return LaunchStatus("mxfp8.gemm");
  hipLaunchKernelGGL((GemmKernel<WN>), dim3(static_cast<unsigned>(a.tiles_m * a.tiles_n)), dim3(kGemmThreads), L::kBytes,
                     stream, a);
  return LaunchStatus("mxfp8.gemm");
}

}  // namespace
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
  const int status = best == 192 ? LaunchGemm<6>(a, on) : LaunchGemm<4>(a, on);
  return status;  // negative: the launch failed after the checks (the caller's fault path)
}

#ifdef LLMP_GEMM_TRACE
// The tuning build's switch: where the GEMM's waves put their timestamps (device memory), or null.
extern "C" int llmp_hip_gemm_trace_set(unsigned long long* buffer) {
  return static_cast<int>(hipMemcpyToSymbol(HIP_SYMBOL(llmp_hip::g_gemm_trace), &buffer, sizeof(buffer)));
}
#endif
