// llmp.moe.gemm's product: the block-scaled NVFP4 grouped GEMM over routed rows sorted by expert, behind the
// reference's three calls (src/kernels/ggml/moe_cutlass.h:48-76: GroupedGemmAvailable, GroupedGemmScratch,
// RunGroupedGemm over a GroupedGemm of device addresses).
//
// One group an expert e: D_e[M_e, n] = A_e[M_e, k] B_e[n, k]^T with M_e = offsets[e + 1] - offsets[e]. Both
// operands are E2M1 codes (k / 2 bytes a row, element 2i in the low nibble) with one UE4M3 scale per 16 elements
// in 128-row by 4-scale atoms (SfOffset): A's scales for expert e in a block of rows starting at sf_rows[e], B_e's
// at weights + e * expert_stride + scales_offset over n rows. D is BF16, accumulated in F32.
//
// gfx950's scaled matrix instructions take one E8M0 scale per 32 values, which is not this format's UE4M3 per 16,
// so the operands are decoded instead: an E2M1 value (two significant bits) times a UE4M3 scale (four) is exact in
// BF16, and the product runs on v_mfma_f32_16x16x32_bf16 over exactly the values the format defines. The group
// sizes are known only on the device: a fixed grid of workgroups walks the list of 64 x 64 output tiles that the
// offsets imply (no host synchronization, no arguments built on the device, no scratch), which also makes the
// launch replay-invariant for a captured graph. A tile's K is walked 64 values at a time: 256 threads decode the
// two 64 x 64 pieces into LDS (a thread sixteen values: eight bytes of codes and one scale), then each of four
// waves multiplies its sixteen rows by the tile's 64 columns.

#include <hip/hip_runtime.h>

#include "common.h"
#include "llmp_hip.h"

namespace llmp_hip {
namespace {

typedef float Float2 __attribute__((ext_vector_type(2)));
typedef float Float4 __attribute__((ext_vector_type(4)));
typedef __bf16 Bf8 __attribute__((ext_vector_type(8)));

constexpr int kTile = 64;            // rows and columns of an output tile, and the K values of a step
constexpr int kRowBytes = 144;       // an LDS row of 64 BF16 values, padded: sixteen lanes' 16-byte reads miss each other
constexpr int kThreads = 256;

// moe_cutlass.h:42-46.
__host__ __device__ __forceinline__ uint64_t SfOffset(uint64_t row, uint64_t block, uint64_t blocks) {
  return (((row / 128) * (blocks / 4)) + (block / 4)) * 512 + ((row % 32) * 16) + (((row % 128) / 32) * 4) + (block % 4);
}

// src/kernels/reference/decode.cc:407-411: E4M3's value up to 0x7E, NaN from 0x7F.
__device__ __forceinline__ float Ue4m3(uint32_t bits) {
  const float value = __builtin_amdgcn_cvt_pk_f32_fp8(bits, false)[0];
  return bits < 0x7Fu ? value : __builtin_nanf("");
}

// Sixteen values (eight bytes of codes, element 2i in byte i's low nibble) times their scale, as BF16 (exact).
__device__ __forceinline__ void DecodeSixteen(uint2 codes, float scale, uint32_t (&out)[8]) {
  const uint32_t words[2] = {codes.x, codes.y};
#pragma unroll
  for (int w = 0; w < 2; ++w) {
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      Float2 pair;
      switch (b) {
        case 0: pair = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(words[w], 1.0f, 0); break;
        case 1: pair = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(words[w], 1.0f, 1); break;
        case 2: pair = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(words[w], 1.0f, 2); break;
        default: pair = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(words[w], 1.0f, 3); break;
      }
      out[4 * w + b] = FloatToBf16Bits(pair[0] * scale) | (FloatToBf16Bits(pair[1] * scale) << 16);
    }
  }
}

struct GroupedArgs {
  llmp_grouped_gemm g;
};

__global__ __launch_bounds__(kThreads) void GroupedNvfp4Kernel(const GroupedArgs args) {
  const llmp_grouped_gemm& g = args.g;
  __shared__ __attribute__((aligned(16))) uint8_t a_tile[kTile * kRowBytes];
  __shared__ __attribute__((aligned(16))) uint8_t b_tile[kTile * kRowBytes];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int n16 = lane & 15, q = lane >> 4;
  const int tiles_n = (g.n + kTile - 1) / kTile;
  const uint64_t row_bytes = static_cast<uint64_t>(g.k) / 2;
  const uint64_t blocks = static_cast<uint64_t>(g.k) / 16;
  const int piece_row = tid >> 2, piece_seg = tid & 3;  // the thread's sixteen values of each 64 x 64 piece

  int base = 0;  // tiles of the groups before this one
  for (int e = 0; e < g.groups; ++e) {
    const int first = g.offsets[e];
    const int rows = g.offsets[e + 1] - first;
    if (rows <= 0) continue;
    const int tiles = ((rows + kTile - 1) / kTile) * tiles_n;
    const uint8_t* weights = static_cast<const uint8_t*>(g.weights) + static_cast<uint64_t>(e) * g.expert_stride;
    const uint8_t* b_codes = weights + g.codes_offset;
    const uint8_t* b_scales = weights + g.scales_offset;
    const uint64_t scale_row0 = static_cast<uint64_t>(g.sf_rows[e]);
    // This workgroup's tiles of the group: every gridDim.x-th of the whole list.
    int t = (static_cast<int>(blockIdx.x) - base % static_cast<int>(gridDim.x) + static_cast<int>(gridDim.x)) % static_cast<int>(gridDim.x);
    for (; t < tiles; t += gridDim.x) {
      const int row0 = (t / tiles_n) * kTile, col0 = (t % tiles_n) * kTile;
      Float4 acc[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[c] = Float4{0.0f, 0.0f, 0.0f, 0.0f};
      const bool a_live = row0 + piece_row < rows;
      const bool b_live = col0 + piece_row < g.n;
      const uint8_t* a_from = static_cast<const uint8_t*>(g.a) + static_cast<uint64_t>(first + row0 + piece_row) * row_bytes + piece_seg * 8;
      const uint8_t* b_from = b_codes + static_cast<uint64_t>(col0 + piece_row) * row_bytes + piece_seg * 8;
      const uint8_t* a_scale = static_cast<const uint8_t*>(g.a_scales);
      for (int k0 = 0; k0 < g.k; k0 += kTile) {
        uint32_t a16[8] = {0, 0, 0, 0, 0, 0, 0, 0}, b16[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        const uint64_t block = static_cast<uint64_t>(k0 / 16 + piece_seg);
        if (a_live) {
          const uint2 codes = *reinterpret_cast<const uint2*>(a_from + k0 / 2);
          DecodeSixteen(codes, Ue4m3(a_scale[SfOffset(scale_row0 + row0 + piece_row, block, blocks)]), a16);
        }
        if (b_live) {
          const uint2 codes = *reinterpret_cast<const uint2*>(b_from + k0 / 2);
          DecodeSixteen(codes, Ue4m3(b_scales[SfOffset(col0 + piece_row, block, blocks)]), b16);
        }
        __syncthreads();  // the last step's readers
        U32x4* a_to = reinterpret_cast<U32x4*>(a_tile + piece_row * kRowBytes + piece_seg * 32);
        U32x4* b_to = reinterpret_cast<U32x4*>(b_tile + piece_row * kRowBytes + piece_seg * 32);
        a_to[0] = U32x4{a16[0], a16[1], a16[2], a16[3]}, a_to[1] = U32x4{a16[4], a16[5], a16[6], a16[7]};
        b_to[0] = U32x4{b16[0], b16[1], b16[2], b16[3]}, b_to[1] = U32x4{b16[4], b16[5], b16[6], b16[7]};
        __syncthreads();
        // Lane (n16, q) holds k = 16 q + [0, 8) and 16 q + [8, 16) of its row on both sides: the same labels, so
        // the instruction's sum over its 32 slots is the step's sum over those 32 values, twice for all 64.
        const U32x4* mine = reinterpret_cast<const U32x4*>(a_tile + (16 * wave + n16) * kRowBytes + q * 32);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const U32x4 x8 = mine[j];
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const U32x4 w8 = reinterpret_cast<const U32x4*>(b_tile + (16 * c + n16) * kRowBytes + q * 32)[j];
            acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(Bf8, x8), __builtin_bit_cast(Bf8, w8), acc[c], 0, 0, 0);
          }
        }
      }
      // acc[c][i] = D[row 16 wave + 4 q + i][column 16 c + n16], rounded to BF16 once.
      uint16_t* d = static_cast<uint16_t*>(g.d);
#pragma unroll
      for (int c = 0; c < 4; ++c) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int row = row0 + 16 * wave + 4 * q + i, col = col0 + 16 * c + n16;
          if (row < rows && col < g.n) d[static_cast<uint64_t>(first + row) * g.n + col] = static_cast<uint16_t>(FloatToBf16Bits(acc[c][i]));
        }
      }
    }
    base += tiles;
  }
}

}  // namespace
}  // namespace llmp_hip

using namespace llmp_hip;

extern "C" int llmp_hip_grouped_gemm_available(void) { return 1; }

extern "C" size_t llmp_hip_grouped_gemm_scratch(int groups, int compute_units) {
  (void)groups, (void)compute_units;
  return 0;  // the workgroups read the offsets themselves: no arguments are built on the device
}

extern "C" int llmp_hip_grouped_gemm_run(const llmp_grouped_gemm* gemm, int compute_units, void* stream) {
  BeginLaunches();
  if (gemm == nullptr) return Refuse(1, "moe.gemm: null descriptor");
  if (gemm->groups < 1 || gemm->groups > 65536) return Refuse(1, "moe.gemm: 1 to 65536 groups, not %d", gemm->groups);
  if (gemm->n < 1 || gemm->k < 64 || gemm->k % 64 != 0)
    return Refuse(1, "moe.gemm: n %d, k %d: k in whole 64-value scale atoms (four scales of sixteen)", gemm->n, gemm->k);
  if (gemm->offsets == nullptr || gemm->sf_rows == nullptr || gemm->a == nullptr || gemm->a_scales == nullptr ||
      gemm->weights == nullptr || gemm->d == nullptr)
    return Refuse(1, "moe.gemm: null operand");
  if ((reinterpret_cast<uintptr_t>(gemm->a) | reinterpret_cast<uintptr_t>(gemm->weights) | gemm->expert_stride | gemm->codes_offset) % 8 != 0)
    return Refuse(1, "moe.gemm: codes not 8-byte aligned");
  if (reinterpret_cast<uintptr_t>(gemm->d) % 2 != 0 || (reinterpret_cast<uintptr_t>(gemm->offsets) | reinterpret_cast<uintptr_t>(gemm->sf_rows)) % 4 != 0)
    return Refuse(1, "moe.gemm: output or offsets misaligned");
  const uint64_t codes_bytes = static_cast<uint64_t>(gemm->n) * (gemm->k / 2);
  const uint64_t scales_bytes = (static_cast<uint64_t>(gemm->n) + 127) / 128 * 128 * (gemm->k / 16);
  const bool apart = gemm->codes_offset + codes_bytes <= gemm->scales_offset || gemm->scales_offset + scales_bytes <= gemm->codes_offset;
  if (!apart) return Refuse(1, "moe.gemm: an expert's codes and scales overlap");
  if (gemm->groups > 1 && gemm->expert_stride < (gemm->codes_offset > gemm->scales_offset ? gemm->codes_offset + codes_bytes
                                                                                          : gemm->scales_offset + scales_bytes))
    return Refuse(1, "moe.gemm: experts overlap");
  const int cus = compute_units > 0 ? compute_units : 256;
  GroupedArgs args{*gemm};
  hipLaunchKernelGGL(GroupedNvfp4Kernel, dim3(static_cast<unsigned>(4 * cus)), dim3(kThreads), 0, static_cast<hipStream_t>(stream), args);
  const int status = LaunchStatus("moe.gemm");
  return status;
}
