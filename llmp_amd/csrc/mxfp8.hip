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

constexpr int kTile = 128;              // rows of either operand a workgroup
constexpr int kStepK = 128;             // codes a K step
constexpr int kOperandBytes = kTile * kStepK;  // 16 KB
constexpr int kStageBytes = 2 * kOperandBytes;
constexpr int kGemmThreads = 256;

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

// Queues one operand's 128 x 128-byte tile of K step `step` into LDS at `to`: position
// P = 256 i + thread holds row P / 8's chunk (P % 8) ^ ((row / 2) % 8).
__device__ __forceinline__ void FetchOperand(const uint8_t* matrix, int row0, int rows, int k, int step, uint8_t* to,
                                             int tid, int wave) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int p = i * kGemmThreads + tid;
    const int row = p >> 3;
    const int chunk = (p & 7) ^ ((row >> 1) & 7);
    const int source = min(row0 + row, rows - 1);  // rows past the end repeat the last (never stored)
    const uint8_t* from = matrix + static_cast<int64_t>(source) * k + step * kStepK + chunk * 16;
    __builtin_amdgcn_global_load_lds((GlobalPointer)from, (LdsPointer)(to + (i * kGemmThreads + wave * 64) * 16), 16, 0,
                                     0);
  }
}

// Fragment f (16 rows) of an operand tile: lane (r, g) gets its row's chunks g and 4 + g.
__device__ __forceinline__ V8i ReadFragment(const uint8_t* tile, int f, int r, int g) {
  const int row = f * 16 + r;
  const int key = (row >> 1) & 7;
  const U32x4 lo = *reinterpret_cast<const U32x4*>(tile + (row * 8 + (g ^ key)) * 16);
  const U32x4 hi = *reinterpret_cast<const U32x4*>(tile + (row * 8 + ((4 + g) ^ key)) * 16);
  V8i v;
  v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w;
  v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
  return v;
}

__global__ __launch_bounds__(kGemmThreads, 2) void GemmKernel(const GemmArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 1, wn = wave >> 1;
  const int r = lane & 15, g = lane >> 4;

  // Workgroups go round-robin to the eight XCDs, each with its own L2: give every XCD a
  // contiguous run of tiles (walking M fastest, so a run shares weight tiles).
  int tile = blockIdx.x;
  const int tiles = a.tiles_m * a.tiles_n;
  if (tiles % 8 == 0) tile = (tile % 8) * (tiles / 8) + tile / 8;
  const int tm = tile % a.tiles_m, tn = tile / a.tiles_m;
  const int m0 = tm * kTile, n0 = tn * kTile;
  const int steps = a.k / kStepK;
  const int blocks = a.k / 32;

  V4f acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = V4f{0.0f, 0.0f, 0.0f, 0.0f};

  // A row's four scales of a K step are one dword of the atoms; the lane wants byte g.
  const int64_t scale_step = 512;  // bytes between a tile's atoms of consecutive K steps
  const uint8_t* ws[4];
  const uint8_t* xs[4];
#pragma unroll
  for (int f = 0; f < 4; ++f) {
    ws[f] = a.b_scales + AtomOffset(n0 + wn * 64 + f * 16 + r, 0, blocks);
    xs[f] = a.a_scales + AtomOffset(m0 + wm * 64 + f * 16 + r, 0, blocks);
  }

  FetchOperand(a.b, n0, a.n, a.k, 0, lds, tid, wave);
  FetchOperand(a.a, m0, a.m, a.k, 0, lds + kOperandBytes, tid, wave);
  for (int step = 0; step < steps; ++step) {
    uint8_t* now = lds + (step & 1) * kStageBytes;
    uint8_t* next = lds + ((step + 1) & 1) * kStageBytes;
    uint32_t wscale[4], xscale[4];
#pragma unroll
    for (int f = 0; f < 4; ++f) {
      wscale[f] = *reinterpret_cast<const uint32_t*>(ws[f] + step * scale_step) >> (8 * g);
      xscale[f] = *reinterpret_cast<const uint32_t*>(xs[f] + step * scale_step) >> (8 * g);
    }
    if (step + 1 < steps) {
      FetchOperand(a.b, n0, a.n, a.k, step + 1, next, tid, wave);
      FetchOperand(a.a, m0, a.m, a.k, step + 1, next + kOperandBytes, tid, wave);
      __builtin_amdgcn_s_waitcnt(0x0F70 | 8);  // vmcnt(8): all but the next step's loads
    } else {
      __builtin_amdgcn_s_waitcnt(0x0F70);
    }
    __syncthreads();  // every wave's part of this step has landed
    V8i wf[4];
#pragma unroll
    for (int f = 0; f < 4; ++f) wf[f] = ReadFragment(now, wn * 4 + f, r, g);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const V8i xf = ReadFragment(now + kOperandBytes, wm * 4 + j, r, g);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[i], xf, acc[i][j], 0, 0, 0,
                                                                      static_cast<int>(wscale[i]), 0,
                                                                      static_cast<int>(xscale[j]));
      }
    }
    __syncthreads();  // this step's buffer may be refilled
  }

  // acc[i][j][q] = D[m0 + wm 64 + 16 j + r][n0 + wn 64 + 16 i + 4 g + q]
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int m = m0 + wm * 64 + j * 16 + r;
    if (m >= a.m) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = n0 + wn * 64 + i * 16 + 4 * g;
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
}

}  // namespace
}  // namespace llmp_hip

using namespace llmp_hip;

extern "C" int llmp_hip_mxfp8_quantize(const void* x, int x_type, int64_t x_stride, int64_t k, int64_t rows, void* codes,
                                       void* scales, void* stream) {
  if (x == nullptr || codes == nullptr || scales == nullptr) return Refuse(1, "mxfp8.quantize: null operand");
  if (k <= 0 || k % 128 != 0) return Refuse(1, "mxfp8.quantize: k %lld is not whole 128-value scale groups", (long long)k);
  if (rows <= 0 || rows > (1 << 24)) return Refuse(1, "mxfp8.quantize: 1 to 2^24 rows");
  if (x_type != LLMP_X_F32 && x_type != LLMP_X_BF16) return Refuse(1, "mxfp8.quantize: F32 or BF16 rows");
  if (reinterpret_cast<uintptr_t>(codes) % 16 != 0) return Refuse(1, "mxfp8.quantize: codes not 16-byte aligned");
  const int64_t padded = (rows + 127) / 128 * 128;
  const int64_t items = padded * (k / 32);
  const dim3 grid(static_cast<unsigned>((items + 255) / 256));
  const auto s = static_cast<hipStream_t>(stream);
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
  (void)compute_units;
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
  a.bf16 = gemm->bf16;
  a.tiles_m = (gemm->m + kTile - 1) / kTile;
  a.tiles_n = (gemm->n + kTile - 1) / kTile;
  const int64_t tiles = static_cast<int64_t>(a.tiles_m) * a.tiles_n;
  if (tiles > (1 << 30)) return Refuse(1, "mxfp8.gemm: too many tiles");
  static bool sized = false;
  if (!sized) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&GemmKernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                              2 * kStageBytes);
    sized = true;
  }
  hipLaunchKernelGGL(GemmKernel, dim3(static_cast<unsigned>(tiles)), dim3(kGemmThreads), 2 * kStageBytes,
                     static_cast<hipStream_t>(stream), a);
  const int status = LaunchStatus("mxfp8.gemm");
  return status;  // negative: the launch failed after the checks (the caller's fault path)
}
