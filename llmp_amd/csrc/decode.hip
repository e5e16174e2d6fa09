// llmp.decode.vector and llmp.decode.vector_glu for gfx950: products over weights in their stored
// encodings, a block decoder per encoding and layout under one kernel template
// (src/kernels/decode/products.h:96-139, decoders.cuh, templates.cuh and operand.h of the reference). y[t][j] = tensor_scale(first + j) * sum_k
// W[first + j][k] x[t][k] for 1 to 16 F32 input rows; every decoder decodes a value as the
// reference's CPU decoder does (src/kernels/reference/decode.cc), the products are F32.
//
// A wave takes two output rows at a time, its lanes the rows' 16-value segments; the pass's
// input rows are staged in LDS once a workgroup (a segment's 64 bytes every 80, so that the
// lanes' 16-byte reads fall in different banks) and each staged segment multiplies both rows.
// E2M1 codes are converted by v_cvt_scalef32_pk_f32_fp4 (two values an instruction), E4M3
// codes by v_cvt_pk_f32_fp8; a segment's block scale multiplies its sum once. An input row's
// outputs do not depend on the rows beside it: each row's sums are formed alone, in one order.

#include <hip/hip_runtime.h>

#include "common.h"
#include "llmp_hip.h"

namespace llmp_hip {
namespace {

typedef float Float2 __attribute__((ext_vector_type(2)));
typedef uint32_t U32x2 __attribute__((ext_vector_type(2)));

constexpr int kDecodeWaves = 16;  // a workgroup's waves with several input rows staged; four with one
constexpr int kGroupedWaves = 8;  // of the expert worklist's kernel
constexpr int kRowsAWave = 2;
constexpr int kSegmentStride = 80;           // bytes from a staged segment to the next
constexpr size_t kDecodeLdsLimit = 80 * 1024;  // two workgroups a CU

struct DecodeArgs {
  llmp_decode_operand w;
  llmp_decode_operand up;  // the GLU form's second weight (w is its gate)
  uint32_t up_first;
  int glu;                 // ir::GluKind
  float limit;
  uint32_t first;
  uint32_t outputs;
  uint32_t token0;  // the pass's first input row
  const float* x;
  uint64_t x_stride;
  float* y;
  uint64_t y_stride;
};

// operand.h:62-67: row `row`'s scale of block `block` in CUTLASS's scale atoms.
__device__ __forceinline__ uint64_t AtomAt(uint64_t row, uint64_t block, uint64_t blocks) {
  return (((row / 128) * (blocks / 4)) + (block / 4)) * 512 + ((row % 32) * 16) + (((row % 128) / 32) * 4) + (block % 4);
}

// decode.cc:407-411: E4M3's value up to 0x7E, NaN from 0x7F.
__device__ __forceinline__ float Ue4m3ToFloat(uint32_t bits) {
  const float value = __builtin_amdgcn_cvt_pk_f32_fp8(bits, false)[0];  // OCP E4M3 on this device; no branches
  return bits < 0x7Fu ? value : __builtin_nanf("");
}

// Eight E2M1 codes, value 2 i in byte i's low nibble (decoders.cuh:57-72), into v[0..7].
__device__ __forceinline__ void Fp4Adjacent(uint32_t word, float* v) {
  const Float2 a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 0);
  const Float2 b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 1);
  const Float2 c = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 2);
  const Float2 d = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 3);
  v[0] = a[0], v[1] = a[1], v[2] = b[0], v[3] = b[1], v[4] = c[0], v[5] = c[1], v[6] = d[0], v[7] = d[1];
}
// Four bytes of GGML's block_nvfp4: byte j holds values j (low nibble) and j + 8.
__device__ __forceinline__ void Fp4Halves(uint32_t word, float* low, float* high) {
  const Float2 a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 0);
  const Float2 b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 1);
  const Float2 c = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 2);
  const Float2 d = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(word, 1.0f, 3);
  low[0] = a[0], low[1] = b[0], low[2] = c[0], low[3] = d[0];
  high[0] = a[1], high[1] = b[1], high[2] = c[1], high[3] = d[1];
}
__device__ __forceinline__ void Fp8Four(uint32_t word, float* v) {
  const Float2 a = __builtin_amdgcn_cvt_pk_f32_fp8(word, false);
  const Float2 b = __builtin_amdgcn_cvt_pk_f32_fp8(word, true);
  v[0] = a[0], v[1] = a[1], v[2] = b[0], v[3] = b[1];
}

// src/kernels/decode/templates.cuh:73-90 of the reference; ir::GluKind: SwiGLU 0, GeGLU (erf) 1, GeGLU (tanh) 2,
// SwiGLU with a clamp 3.
__device__ __forceinline__ float DecodeGlu(int kind, float g, float u, float limit) {
#pragma clang fp contract(off)
  switch (kind) {
    case 1:
      return 0.5f * g * (1.0f + erff(g * 0.70710678118654752f)) * u;
    case 2:
      return 0.5f * g * (1.0f + tanhf(0.79788456080286536f * (g + (0.044715f * g * g * g)))) * u;
    case 3: {
      const float gc = fminf(g, limit);
      const float uc = fminf(fmaxf(u, -limit), limit);
      return gc / (1.0f + expf(-gc)) * uc;
    }
    default:
      return g / (1.0f + expf(-g)) * u;
  }
}

// A segment as loaded, before any arithmetic: its codes (up to 32 bytes; the row-interleaved
// layout's eight single bytes), its scale's bits and, for the affine encoding, its bias's or zero
// point's. Loading and decoding are apart so that a kernel can queue several segments' loads,
// and other work, before it waits for the first.
struct RawSegment {
  U32x4 a, b;
  uint32_t scale, extra;
};

template <int D>
__device__ __forceinline__ RawSegment FetchSegment(const llmp_decode_operand& w, uint32_t row, uint32_t seg) {
  RawSegment r;
  r.a = U32x4{0, 0, 0, 0}, r.b = U32x4{0, 0, 0, 0}, r.scale = 0, r.extra = 0;
  const uint8_t* data = w.data + static_cast<uint64_t>(row) * w.row_bytes;
  if constexpr (D == LLMP_DECODER_BF16_DENSE || D == LLMP_DECODER_F16_DENSE) {
    const U32x4* src = reinterpret_cast<const U32x4*>(data + seg * 32u);
    r.a = __builtin_nontemporal_load(src), r.b = __builtin_nontemporal_load(src + 1);
  } else if constexpr (D == LLMP_DECODER_Q8_0_BLOCKS) {
    // block_q8_0 is 34 bytes: only two-byte loads are aligned. A segment is half a block.
    const uint8_t* block = data + static_cast<uint64_t>(seg / 2u) * 34u;
    const uint16_t* q = reinterpret_cast<const uint16_t*>(block + 2 + (seg & 1u) * 16u);
    r.scale = *reinterpret_cast<const uint16_t*>(block);
    r.a = U32x4{q[0], q[1], q[2], q[3]}, r.b = U32x4{q[4], q[5], q[6], q[7]};
  } else if constexpr (D == LLMP_DECODER_NVFP4_INTERLEAVED) {
    // A row is its K / 2 code bytes, then its K / 16 scales: no alignment beyond a byte.
    const uint8_t* c = data + seg * 8u;
    r.a = U32x4{c[0], c[1], c[2], c[3]}, r.b = U32x4{c[4], c[5], c[6], c[7]};
    r.scale = data[w.k / 2u + seg];
  } else if constexpr (D == LLMP_DECODER_NVFP4_GGML_BLOCKS) {
    // block_nvfp4: four UE4M3 scales, then 32 bytes; a segment is a 16-value sub-block.
    const uint8_t* block = data + static_cast<uint64_t>(seg / 4u) * 36u;
    const uint32_t* c = reinterpret_cast<const uint32_t*>(block + 4 + (seg & 3u) * 8u);
    r.a.x = c[0], r.a.y = c[1];
    r.scale = *reinterpret_cast<const uint32_t*>(block);
  } else if constexpr (D == LLMP_DECODER_MXFP8_SPLIT || D == LLMP_DECODER_MXFP8_ATOMS) {
    r.a = __builtin_nontemporal_load(reinterpret_cast<const U32x4*>(data + seg * 16u));
    const uint64_t at = D == LLMP_DECODER_MXFP8_SPLIT ? static_cast<uint64_t>(row) * (w.k / 32u) + seg / 2u
                                                      : AtomAt(row, seg / 2u, w.k / 32u);
    r.scale = w.scales[at];
  } else if constexpr (D == LLMP_DECODER_AFFINE_SPLIT) {
    const uint32_t g = seg * 16u / w.group;
    const uint64_t scale_row = static_cast<uint64_t>(row) * w.scale_row_bytes;
    const bool wide = (w.scale_type & 0x7Fu) == 3u;
    auto element = [&](const uint8_t* base) -> uint32_t {
      return wide ? *reinterpret_cast<const uint32_t*>(base + scale_row + g * 4u)
                  : *reinterpret_cast<const uint16_t*>(base + scale_row + g * 2u);
    };
    r.scale = element(w.scales);
    if ((w.scale_type & 0x80u) != 0) {
      const uint64_t zero_row = (static_cast<uint64_t>(w.k / w.group) * w.bits + 7) / 8;
      r.extra = w.biases[row * zero_row + (w.bits == 4 ? g / 2u : g)];
    } else if (w.biases != nullptr) {
      r.extra = element(w.biases);
    }
    if (w.bits == 4) {
      const U32x2 c = __builtin_nontemporal_load(reinterpret_cast<const U32x2*>(data + seg * 8u));
      r.a.x = c.x, r.a.y = c.y;
    } else {
      r.a = __builtin_nontemporal_load(reinterpret_cast<const U32x4*>(data + seg * 16u));
    }
  } else {
    // NVFP4 and MXFP4 codes as rows of K / 2 bytes: a segment is eight bytes.
    const U32x2 c = __builtin_nontemporal_load(reinterpret_cast<const U32x2*>(data + seg * 8u));
    r.a.x = c.x, r.a.y = c.y;
    if constexpr (D == LLMP_DECODER_NVFP4_SPLIT) {
      r.scale = w.scales[static_cast<uint64_t>(row) * (w.k / 16u) + seg];
    } else if constexpr (D == LLMP_DECODER_NVFP4_ATOMS) {
      r.scale = w.scales[AtomAt(row, seg, w.k / 16u)];
    } else if constexpr (D == LLMP_DECODER_MXFP4_SPLIT) {
      r.scale = w.scales[static_cast<uint64_t>(row) * (w.k / 32u) + seg / 2u];
    } else {
      r.scale = w.scales[AtomAt(row, seg / 2u, w.k / 32u)];
    }
  }
  return r;
}

// The segment's sixteen values before the block scale, and that scale.
template <int D>
__device__ __forceinline__ void DecodeSegment(const llmp_decode_operand& w, uint32_t seg, const RawSegment& r,
                                              float (&v)[16], float& s) {
  if constexpr (D == LLMP_DECODER_BF16_DENSE || D == LLMP_DECODER_F16_DENSE) {
    const uint32_t word[8] = {r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if constexpr (D == LLMP_DECODER_BF16_DENSE) {
        v[2 * i] = __builtin_bit_cast(float, word[i] << 16);
        v[2 * i + 1] = __builtin_bit_cast(float, word[i] & 0xFFFF0000u);
      } else {
        v[2 * i] = HalfBitsToFloat(word[i] & 0xFFFFu);
        v[2 * i + 1] = HalfBitsToFloat(word[i] >> 16);
      }
    }
    s = 1.0f;
  } else if constexpr (D == LLMP_DECODER_Q8_0_BLOCKS) {
    const uint32_t pair[8] = {r.a.x, r.a.y, r.a.z, r.a.w, r.b.x, r.b.y, r.b.z, r.b.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      v[2 * i] = static_cast<float>(static_cast<int8_t>(pair[i] & 0xFFu));
      v[2 * i + 1] = static_cast<float>(static_cast<int8_t>(pair[i] >> 8));
    }
    s = HalfBitsToFloat(r.scale);
  } else if constexpr (D == LLMP_DECODER_NVFP4_INTERLEAVED) {
    Fp4Adjacent(r.a.x | (r.a.y << 8) | (r.a.z << 16) | (r.a.w << 24), v);
    Fp4Adjacent(r.b.x | (r.b.y << 8) | (r.b.z << 16) | (r.b.w << 24), v + 8);
    s = Ue4m3ToFloat(r.scale);
  } else if constexpr (D == LLMP_DECODER_NVFP4_GGML_BLOCKS) {
    Fp4Halves(r.a.x, v, v + 8);
    Fp4Halves(r.a.y, v + 4, v + 12);
    s = Ue4m3ToFloat((r.scale >> (8u * (seg & 3u))) & 0xFFu);
  } else if constexpr (D == LLMP_DECODER_MXFP8_SPLIT || D == LLMP_DECODER_MXFP8_ATOMS) {
    Fp8Four(r.a.x, v), Fp8Four(r.a.y, v + 4), Fp8Four(r.a.z, v + 8), Fp8Four(r.a.w, v + 12);
    s = E8m0ToFloat(r.scale);
  } else if constexpr (D == LLMP_DECODER_AFFINE_SPLIT) {
    // Unsigned codes of 4 or 8 bits, a scale and a bias (or a zero point) a group of values along the
    // row; a segment lies within one group. s * q + b rounded once, or s * (q - z)
    // (src/kernels/reference/decode.cc:197-220).
#pragma clang fp contract(off)
    const uint32_t scale_type = w.scale_type & 0x7Fu;
    auto element = [&](uint32_t bits) {
      return scale_type == 3u ? __builtin_bit_cast(float, bits)
                              : scale_type == 2u ? __builtin_bit_cast(float, bits << 16) : HalfBitsToFloat(bits);
    };
    const float scale = element(r.scale);
    const bool zero_point = (w.scale_type & 0x80u) != 0;
    const uint32_t g = seg * 16u / w.group;
    const int32_t z = zero_point ? (w.bits == 4 ? (r.extra >> (4u * (g & 1u))) & 15u : r.extra) : 0;
    const float b = !zero_point && w.biases != nullptr ? element(r.extra) : 0.0f;
    uint32_t code[16];
    if (w.bits == 4) {
#pragma unroll
      for (int i = 0; i < 16; ++i) code[i] = ((i < 8 ? r.a.x : r.a.y) >> (4 * (i % 8))) & 15u;
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) code[i] = (r.a[i / 4] >> (8 * (i % 4))) & 0xFFu;
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      v[i] = zero_point ? scale * static_cast<float>(static_cast<int32_t>(code[i]) - z)
                        : fmaf(scale, static_cast<float>(code[i]), b);
    }
    s = 1.0f;
  } else {
    Fp4Adjacent(r.a.x, v);
    Fp4Adjacent(r.a.y, v + 8);
    if constexpr (D == LLMP_DECODER_NVFP4_SPLIT || D == LLMP_DECODER_NVFP4_ATOMS) {
      s = Ue4m3ToFloat(r.scale);
    } else {
      s = E8m0ToFloat(r.scale);
    }
  }
}

// Segment `seg` (16 values) of row `row`: the values before the block scale, and that scale.
template <int D>
__device__ __forceinline__ void LoadSegment(const llmp_decode_operand& w, uint32_t row, uint32_t seg, float (&v)[16],
                                            float& s) {
  DecodeSegment<D>(w, seg, FetchSegment<D>(w, row, seg), v, s);
}

// grid: workgroups of four waves (one input row) or sixteen, persistent over pairs of output rows; LDS: T input rows.
// kGlu: a wave's two rows are gate row first + j and up row up_first + j of output j; the up weight's decoder DU may
// differ from the gate's D (the pairs src/kernels/decode/implementations.cc:73-81 of the reference lists).
template <int D, int T, bool kGlu, int DU = D>
__global__ __launch_bounds__(kDecodeWaves * 64) void DecodeVectorKernel(const DecodeArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t segs = a.w.k / 16u;
  const uint32_t quarters = a.w.k / 4u;  // 16-byte pieces of an input row

  const uint32_t waves = blockDim.x / 64;
  for (uint32_t c = tid; c < T * quarters; c += blockDim.x) {
    const uint32_t t = c / quarters, q = c - t * quarters;
    const float4 piece = *reinterpret_cast<const float4*>(a.x + (a.token0 + t) * a.x_stride + q * 4u);
    *reinterpret_cast<float4*>(lds + static_cast<size_t>(t * segs + q / 4u) * kSegmentStride + (q & 3u) * 16u) = piece;
  }
  __syncthreads();  // the only one: from here the waves run alone

  if constexpr (T <= 3) {
    // One to three input rows: four or eight waves a workgroup and two or more workgroups a CU; their number hides the
    // loads (at three rows 22 us for MXFP8 4096 x 14336 against 24 with the loads ahead).
    const uint32_t pairs = kGlu ? a.outputs : (a.outputs + kRowsAWave - 1) / kRowsAWave;
    for (uint32_t pair = blockIdx.x * waves + wave; pair < pairs; pair += gridDim.x * waves) {
      const uint32_t out0 = kGlu ? pair : pair * kRowsAWave;
      float acc[kRowsAWave][T];
  #pragma unroll
      for (int r = 0; r < kRowsAWave; ++r) {
  #pragma unroll
        for (int t = 0; t < T; ++t) acc[r][t] = 0.0f;
      }
      for (uint32_t seg = lane; seg < segs; seg += 64) {
        float v[kRowsAWave][16], s[kRowsAWave];
  #pragma unroll
        for (int r = 0; r < kRowsAWave; ++r) {
          if constexpr (kGlu) {
            if (r == 0) {
              LoadSegment<D>(a.w, a.first + out0, seg, v[r], s[r]);
            } else {
              LoadSegment<DU>(a.up, a.up_first + out0, seg, v[r], s[r]);
            }
          } else {
            // A lone last row is decoded twice: its second copy's sums are not stored.
            const uint32_t out = min(out0 + r, a.outputs - 1);
            LoadSegment<D>(a.w, a.first + out, seg, v[r], s[r]);
          }
        }
  #pragma unroll
        for (int t = 0; t < T; ++t) {
          const float4* xs = reinterpret_cast<const float4*>(lds + static_cast<size_t>(t * segs + seg) * kSegmentStride);
          const float4 x0 = xs[0], x1 = xs[1], x2 = xs[2], x3 = xs[3];
          const float x[16] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w, x2.x, x2.y, x2.z, x2.w, x3.x, x3.y, x3.z, x3.w};
  #pragma unroll
          for (int r = 0; r < kRowsAWave; ++r) {
            float dot = 0.0f;
  #pragma unroll
            for (int i = 0; i < 16; ++i) dot = fmaf(v[r][i], x[i], dot);
            acc[r][t] = fmaf(dot, s[r], acc[r][t]);
          }
        }
      }
      if constexpr (kGlu) {
        const float gate_scale = a.w.tensor_scale != nullptr ? a.w.tensor_scale[(a.first + out0) / a.w.rows_per_scale] : 1.0f;
        const float up_scale = a.up.tensor_scale != nullptr ? a.up.tensor_scale[(a.up_first + out0) / a.up.rows_per_scale] : 1.0f;
  #pragma unroll
        for (int t = 0; t < T; ++t) {
          float gate = acc[0][t], up = acc[1][t];
  #pragma unroll
          for (int mask = 32; mask >= 1; mask >>= 1) {
            gate += ShflXor(gate, mask);
            up += ShflXor(up, mask);
          }
          if (lane == 0) a.y[(a.token0 + t) * a.y_stride + out0] = DecodeGlu(a.glu, gate * gate_scale, up * up_scale, a.limit);
        }
        continue;
      }
  #pragma unroll
      for (int r = 0; r < kRowsAWave; ++r) {
        const uint32_t out = out0 + r;
        float scale = 1.0f;
        if (a.w.tensor_scale != nullptr && out < a.outputs) scale = a.w.tensor_scale[(a.first + out) / a.w.rows_per_scale];
  #pragma unroll
        for (int t = 0; t < T; ++t) {
          float total = acc[r][t];
  #pragma unroll
          for (int mask = 32; mask >= 1; mask >>= 1) total += ShflXor(total, mask);
          if (lane == 0 && out < a.outputs) a.y[(a.token0 + t) * a.y_stride + out] = total * scale;
        }
      }
    }
    return;
  }
  // The wave's work as one run of steps, (pair of rows, 64 segments) each: a step's two segments are asked for two
  // steps before they are multiplied (several input rows: the staged rows fill LDS and a CU holds one workgroup),
  // past the last step the last again, so that no load sits under a branch (three steps ahead measured the same).
  // What a lane adds, and in which order, is what the plain loop over its pairs and segments adds.
  const uint32_t pairs = kGlu ? a.outputs : (a.outputs + kRowsAWave - 1) / kRowsAWave;
  const uint32_t first_pair = blockIdx.x * waves + wave, pair_step = gridDim.x * waves;
  if (first_pair >= pairs) return;
  const uint32_t seg_steps = (segs + 63u) / 64u;
  const uint32_t total = ((pairs - first_pair + pair_step - 1) / pair_step) * seg_steps;
  struct Step {
    RawSegment raw[kRowsAWave];
  };
  auto fetch = [&](uint32_t it) {
    it = min(it, total - 1);
    const uint32_t p = it / seg_steps;
    const uint32_t out0 = kGlu ? first_pair + p * pair_step : (first_pair + p * pair_step) * kRowsAWave;
    const uint32_t seg = min((it - p * seg_steps) * 64u + lane, segs - 1);
    Step step;
#pragma unroll
    for (int r = 0; r < kRowsAWave; ++r) {
      if constexpr (kGlu) {
        if (r == 0) {
          step.raw[r] = FetchSegment<D>(a.w, a.first + out0, seg);
        } else {
          step.raw[r] = FetchSegment<DU>(a.up, a.up_first + out0, seg);
        }
      } else {
        // A lone last row is decoded twice: its second copy's sums are not stored.
        step.raw[r] = FetchSegment<D>(a.w, a.first + min(out0 + r, a.outputs - 1), seg);
      }
    }
    return step;
  };
  float acc[kRowsAWave][T];
#pragma unroll
  for (int r = 0; r < kRowsAWave; ++r) {
#pragma unroll
    for (int t = 0; t < T; ++t) acc[r][t] = 0.0f;
  }
  auto multiply = [&](uint32_t it, const Step& step) {
    const uint32_t p = it / seg_steps, part = it - p * seg_steps;
    const uint32_t out0 = kGlu ? first_pair + p * pair_step : (first_pair + p * pair_step) * kRowsAWave;
    const uint32_t seg = part * 64u + lane;
    if (seg < segs) {
      float v[kRowsAWave][16], s[kRowsAWave];
#pragma unroll
      for (int r = 0; r < kRowsAWave; ++r) {
        if constexpr (kGlu) {
          if (r == 0) {
            DecodeSegment<D>(a.w, seg, step.raw[r], v[r], s[r]);
          } else {
            DecodeSegment<DU>(a.up, seg, step.raw[r], v[r], s[r]);
          }
        } else {
          DecodeSegment<D>(a.w, seg, step.raw[r], v[r], s[r]);
        }
      }
#pragma unroll
      for (int t = 0; t < T; ++t) {
        const float4* xs = reinterpret_cast<const float4*>(lds + static_cast<size_t>(t * segs + seg) * kSegmentStride);
        const float4 x0 = xs[0], x1 = xs[1], x2 = xs[2], x3 = xs[3];
        const float x[16] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w, x2.x, x2.y, x2.z, x2.w, x3.x, x3.y, x3.z, x3.w};
#pragma unroll
        for (int r = 0; r < kRowsAWave; ++r) {
          float dot = 0.0f;
#pragma unroll
          for (int i = 0; i < 16; ++i) dot = fmaf(v[r][i], x[i], dot);
          acc[r][t] = fmaf(dot, s[r], acc[r][t]);
        }
      }
    }
    if (part + 1 < seg_steps) return;
    // The pair's last step: the lanes' sums meet and the outputs are stored.
    if constexpr (kGlu) {
      const float gate_scale = a.w.tensor_scale != nullptr ? a.w.tensor_scale[(a.first + out0) / a.w.rows_per_scale] : 1.0f;
      const float up_scale = a.up.tensor_scale != nullptr ? a.up.tensor_scale[(a.up_first + out0) / a.up.rows_per_scale] : 1.0f;
#pragma unroll
      for (int t = 0; t < T; ++t) {
        float gate = acc[0][t], up = acc[1][t];
#pragma unroll
        for (int mask = 32; mask >= 1; mask >>= 1) {
          gate += ShflXor(gate, mask);
          up += ShflXor(up, mask);
        }
        if (lane == 0) a.y[(a.token0 + t) * a.y_stride + out0] = DecodeGlu(a.glu, gate * gate_scale, up * up_scale, a.limit);
        acc[0][t] = 0.0f, acc[1][t] = 0.0f;
      }
    } else {
#pragma unroll
      for (int r = 0; r < kRowsAWave; ++r) {
        const uint32_t out = out0 + r;
        float scale = 1.0f;
        if (a.w.tensor_scale != nullptr && out < a.outputs) scale = a.w.tensor_scale[(a.first + out) / a.w.rows_per_scale];
#pragma unroll
        for (int t = 0; t < T; ++t) {
          float total_sum = acc[r][t];
#pragma unroll
          for (int mask = 32; mask >= 1; mask >>= 1) total_sum += ShflXor(total_sum, mask);
          if (lane == 0 && out < a.outputs) a.y[(a.token0 + t) * a.y_stride + out] = total_sum * scale;
          acc[r][t] = 0.0f;
        }
      }
    }
  };
  Step even = fetch(0), odd = fetch(1);
  for (uint32_t it = 0; it < total; it += 2) {
    const Step now = even;
    even = fetch(it + 2);
    multiply(it, now);
    if (it + 1 < total) {
      const Step then = odd;
      odd = fetch(it + 3);
      multiply(it + 1, then);
    }
  }
}

// out[i][:] = W[ids[i]][:] as F32, times the row's tensor scale; an id outside the matrix writes
// zeros and sets *bad (products.h:172-183). A wave a gathered row, its lanes the segments.
template <int D>
__global__ __launch_bounds__(256) void DecodeRowsKernel(const llmp_decode_operand w, const int32_t* __restrict__ ids,
                                                      uint32_t count, float* __restrict__ out, uint64_t out_stride,
                                                      int32_t* __restrict__ bad) {
#pragma clang fp contract(off)
  const int lane = threadIdx.x & 63;
  const uint32_t i = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (i >= count) return;  // whole waves
  const int32_t id = ids[i];
  const bool known = id >= 0 && static_cast<uint32_t>(id) < w.rows;
  float4* row = reinterpret_cast<float4*>(out + i * out_stride);
  if (!known && bad != nullptr && lane == 0) *bad = 1;
  const float scale = known && w.tensor_scale != nullptr ? w.tensor_scale[static_cast<uint32_t>(id) / w.rows_per_scale] : 1.0f;
  for (uint32_t seg = lane; seg < w.k / 16u; seg += 64) {
    float v[16] = {};
    if (known) {
      float s;
      LoadSegment<D>(w, static_cast<uint32_t>(id), seg, v, s);
#pragma unroll
      for (int j = 0; j < 16; ++j) v[j] = (v[j] * s) * scale;
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) row[seg * 4u + q] = make_float4(v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]);
  }
}

// An expert worklist's products (products.h:141-170): expert e = blockIdx.y takes its pairs
// offsets[e] .. offsets[e + 1], T at a time: their input rows staged, then every wave its output
// row pairs. An expert whose operand's K or N is not the format's is skipped, as are pairs past
// `pairs` and pairs naming a row past x_rows or y_rows.
struct GroupedArgs {
  const llmp_decode_operand* experts;
  uint32_t k, n, first, outputs;
  const int32_t* offsets;
  const int32_t* pair_rows;
  const int32_t* pair_out;  // or null: pair p writes row p
  uint32_t pairs, x_rows, y_rows;
  const float* x;
  uint64_t x_stride;
  float* y;
  uint64_t y_stride;
};

template <int D, int T>
__global__ __launch_bounds__(kGroupedWaves * 64) void DecodeGroupedKernel(const GroupedArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  __shared__ int32_t out_row[T];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t waves = blockDim.x / 64;
  const llmp_decode_operand w = a.experts[blockIdx.y];
  if (w.k != a.k || w.rows != a.n) return;  // uniform over the workgroup
  const uint32_t segs = a.k / 16u, quarters = a.k / 4u;
  int64_t begin = a.offsets[blockIdx.y], end = a.offsets[blockIdx.y + 1];
  if (begin < 0) begin = 0;
  if (end > static_cast<int64_t>(a.pairs)) end = a.pairs;
  const uint32_t row_pairs = (a.outputs + kRowsAWave - 1) / kRowsAWave;
  for (int64_t p0 = begin; p0 < end; p0 += T) {
    const int m = static_cast<int>(end - p0 < T ? end - p0 : T);
    if (p0 > begin) __syncthreads();  // the last pass's readers of the staged rows
    // Where each pair's sums go (-1: nowhere), and its input row (zeros for a pair that is skipped).
    if (tid < m) {
      const int64_t p = p0 + tid;
      const int64_t from = a.pair_rows[p];
      const int64_t to = a.pair_out != nullptr ? a.pair_out[p] : p;
      out_row[tid] = from >= 0 && from < a.x_rows && to >= 0 && to < a.y_rows ? static_cast<int32_t>(to) : -1;
    }
    for (uint32_t c = tid; c < m * quarters; c += blockDim.x) {
      const uint32_t t = c / quarters, q = c - t * quarters;
      const int64_t from = a.pair_rows[p0 + t];
      float4 piece = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      if (from >= 0 && from < a.x_rows) piece = *reinterpret_cast<const float4*>(a.x + from * a.x_stride + q * 4u);
      *reinterpret_cast<float4*>(lds + static_cast<size_t>(t * segs + q / 4u) * kSegmentStride + (q & 3u) * 16u) = piece;
    }
    __syncthreads();
    for (uint32_t pair = blockIdx.x * waves + wave; pair < row_pairs; pair += gridDim.x * waves) {
      const uint32_t out0 = pair * kRowsAWave;
      float acc[kRowsAWave][T];
#pragma unroll
      for (int r = 0; r < kRowsAWave; ++r) {
#pragma unroll
        for (int t = 0; t < T; ++t) acc[r][t] = 0.0f;
      }
      for (uint32_t seg = lane; seg < segs; seg += 64) {
        float v[kRowsAWave][16], s[kRowsAWave];
#pragma unroll
        for (int r = 0; r < kRowsAWave; ++r) LoadSegment<D>(w, a.first + min(out0 + r, a.outputs - 1), seg, v[r], s[r]);
#pragma unroll
        for (int t = 0; t < T; ++t) {
          if (t < m) {
            const float4* xs = reinterpret_cast<const float4*>(lds + static_cast<size_t>(t * segs + seg) * kSegmentStride);
            const float4 x0 = xs[0], x1 = xs[1], x2 = xs[2], x3 = xs[3];
            const float x[16] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w, x2.x, x2.y, x2.z, x2.w, x3.x, x3.y, x3.z, x3.w};
#pragma unroll
            for (int r = 0; r < kRowsAWave; ++r) {
              float dot = 0.0f;
#pragma unroll
              for (int i = 0; i < 16; ++i) dot = fmaf(v[r][i], x[i], dot);
              acc[r][t] = fmaf(dot, s[r], acc[r][t]);
            }
          }
        }
      }
#pragma unroll
      for (int r = 0; r < kRowsAWave; ++r) {
        const uint32_t out = out0 + r;
        float scale = 1.0f;
        if (w.tensor_scale != nullptr && out < a.outputs) scale = w.tensor_scale[(a.first + out) / w.rows_per_scale];
#pragma unroll
        for (int t = 0; t < T; ++t) {
          if (t < m) {
            float total = acc[r][t];
#pragma unroll
            for (int mask = 32; mask >= 1; mask >>= 1) total += ShflXor(total, mask);
            const int32_t to = out_row[t];
            if (lane == 0 && out < a.outputs && to >= 0) a.y[static_cast<int64_t>(to) * a.y_stride + out] = total * scale;
          }
        }
      }
    }
  }
}

// ------------------------------------------------------------------ matrix
// RunMatrix's tensor-core path (products.h:111-118, templates.cuh's Matrix): tiles of 64 outputs by 64
// input rows, the weights decoded and, like the inputs, rounded to the decoder's matrix element
// (F16 for F16 and Q8_0 weights, BF16 otherwise), F32 sums on the matrix cores
// (v_mfma_f32_16x16x32: D[input row][output] += x[input row][k] W[output][k]).
// A workgroup takes 256 outputs by 64 input rows, a wave 64 of the outputs in four groups of 16; a lane (n = lane % 16, q = lane / 16) decodes segment
// 4 c + q of output n of each group for chunk c of 64 values of K: its sixteen values are the second operands of
// two instructions whose k labels run over the four lanes' segments, and the inputs' first
// operands follow the same labels, so no lane exchange is needed. The inputs' chunk is staged in
// LDS in the matrix element, rows 144 bytes apart (conflict-free 16-byte reads), in two buffers: the
// next chunk's inputs and weights are loaded while this one multiplies, one barrier a chunk.
typedef short Short8 __attribute__((ext_vector_type(8)));
typedef float Float4 __attribute__((ext_vector_type(4)));
constexpr int kMatrixRowBytes = 144;   // 64 two-byte elements and 16 bytes

// Nearest even, by the hardware's conversions (v_cvt_f16_f32, v_cvt_pk_bf16_f32).
template <bool kHalf>
__device__ __forceinline__ uint32_t ToElement(float v) {
  if constexpr (kHalf) {
    return FloatToHalfBits(v);
  } else {
    return __builtin_bit_cast(uint16_t, static_cast<__bf16>(v));
  }
}

// G: groups of 16 outputs a wave; M: groups of 16 input rows (a workgroup takes 64 G outputs by 16 M input rows).
// Decoding a segment costs some sixty vector instructions whatever M is, so the large tile is what
// lets the matrix cores, not the decoding, set the pace; the small one is for products with few tiles, where
// each wave waits on memory instead: it loads two chunks ahead, the large one (short of registers) one.
template <int D, int G, int M>
__global__ __launch_bounds__(256) void DecodeMatrixKernel(const DecodeArgs a, const uint32_t rows) {
  constexpr bool kHalf = D == LLMP_DECODER_F16_DENSE || D == LLMP_DECODER_Q8_0_BLOCKS;
  constexpr int kAhead = G == 1 ? 2 : 1;
  constexpr int kTileBytes = 16 * M * kMatrixRowBytes;
  __shared__ __attribute__((aligned(16))) uint8_t tiles[2 * kTileBytes];  // this chunk's inputs and the next's
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, q = lane >> 4;
  const uint32_t out0 = (blockIdx.x * 4 + wave) * (16 * G), t0 = blockIdx.y * (16 * M);
  const uint32_t segs = a.w.k / 16u, chunks = (segs + 3u) / 4u;
  Float4 acc[G][M];  // [outputs' group][input rows' group]
#pragma unroll
  for (int g = 0; g < G; ++g) {
#pragma unroll
    for (int m = 0; m < M; ++m) acc[g][m] = Float4{0.0f, 0.0f, 0.0f, 0.0f};
  }
  // A chunk's share of a thread: M pieces of four input values, and the lane's segment of each of
  // its groups of outputs. Loads without branches: a row past the inputs or a column past K reads a
  // valid address nearby and is zeroed when it is used; the same for a segment past the row's last.
  auto load_inputs = [&](uint32_t chunk, float4 (&piece)[M]) {
#pragma unroll
    for (int i = 0; i < M; ++i) {
      const uint32_t c = tid + i * 256;
      const uint32_t row = min(t0 + (c >> 4), rows - 1), column = min(chunk * 64u + (c & 15u) * 4u, a.w.k - 4u);
      piece[i] = *reinterpret_cast<const float4*>(a.x + static_cast<uint64_t>(row) * a.x_stride + column);
    }
  };
  auto fetch_weights = [&](uint32_t chunk, RawSegment (&raw)[G]) {
    const uint32_t seg = min(chunk * 4u + q, segs - 1);
#pragma unroll
    for (int g = 0; g < G; ++g) raw[g] = FetchSegment<D>(a.w, a.first + min(out0 + 16 * g + n, a.outputs - 1), seg);
  };
  // Scaled and rounded to the element: two operands of eight a group.
  auto decode_weights = [&](uint32_t chunk, const RawSegment (&raw)[G], Short8 (&b)[G][2]) {
    const uint32_t seg = chunk * 4u + q;
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float v[16], s;
      DecodeSegment<D>(a.w, min(seg, segs - 1), raw[g], v, s);
#pragma unroll
      for (int j = 0; j < 2; ++j) {
#pragma unroll
        for (int i = 0; i < 8; ++i) b[g][j][i] = static_cast<short>(ToElement<kHalf>(seg < segs ? v[8 * j + i] * s : 0.0f));
      }
    }
  };

  // Loads run kAhead chunks ahead of their use, in as many sets of registers (by the chunk's parity when
  // two): a chunk's multiplies are shorter than a trip to memory. Loads past the last chunk read its
  // addresses and are dropped.
  float4 piece[kAhead][M];
  RawSegment raw[kAhead][G];
  Short8 b[G][2];
  auto step = [&](uint32_t chunk, auto slot) {
    constexpr int P = decltype(slot)::value, kNext = (P + 1) % kAhead;
    uint8_t* tile = tiles + (chunk & 1u) * kTileBytes;
#pragma unroll
    for (int i = 0; i < M; ++i) {
      const uint32_t c = tid + i * 256;
      const bool live = t0 + (c >> 4) < rows && chunk * 64u + (c & 15u) * 4u < a.w.k;
      uint2 packed;
      packed.x = live ? ToElement<kHalf>(piece[P][i].x) | (ToElement<kHalf>(piece[P][i].y) << 16) : 0u;
      packed.y = live ? ToElement<kHalf>(piece[P][i].z) | (ToElement<kHalf>(piece[P][i].w) << 16) : 0u;
      *reinterpret_cast<uint2*>(tile + (c >> 4) * kMatrixRowBytes + (c & 15u) * 8u) = packed;
    }
    // One barrier a chunk: this buffer is complete, and the other's readers (the last chunk's) are done.
    __syncthreads();
    load_inputs(chunk + kAhead, piece[P]);
    if constexpr (kAhead == 1) fetch_weights(chunk + 1, raw[0]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int m = 0; m < M; ++m) {
      const U32x4* mine = reinterpret_cast<const U32x4*>(tile + (16 * m + n) * kMatrixRowBytes + q * 32);
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const U32x4 x8 = mine[j];
#pragma unroll
        for (int g = 0; g < G; ++g) {
          if constexpr (kHalf) {
            typedef _Float16 Half8 __attribute__((ext_vector_type(8)));
            acc[g][m] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(Half8, x8),
                                                               __builtin_bit_cast(Half8, b[g][j]), acc[g][m], 0, 0, 0);
          } else {
            typedef __bf16 Bf8 __attribute__((ext_vector_type(8)));
            acc[g][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(Bf8, x8),
                                                                __builtin_bit_cast(Bf8, b[g][j]), acc[g][m], 0, 0, 0);
          }
        }
      }
    }
    __builtin_amdgcn_sched_barrier(0);  // the loads' first use stays behind the multiplies
    decode_weights(chunk + 1, raw[kNext], b);
    if constexpr (kAhead == 2) fetch_weights(chunk + 3, raw[kNext]);
    __builtin_amdgcn_sched_barrier(0);
  };
  load_inputs(0, piece[0]);
  fetch_weights(0, raw[0]);
  if constexpr (kAhead == 2) {
    load_inputs(1, piece[1]);
    fetch_weights(1, raw[1]);
  }
  decode_weights(0, raw[0], b);
  if constexpr (kAhead == 2) fetch_weights(2, raw[0]);
  for (uint32_t chunk = 0; chunk < chunks; chunk += kAhead) {  // every wave: the same count of barriers
    step(chunk, std::integral_constant<int, 0>{});
    if constexpr (kAhead == 2) {
      if (chunk + 1 < chunks) step(chunk + 1, std::integral_constant<int, 1>{});
    }
  }
  // acc[g][m][i] = D[input row 16 m + 4 q + i][output 16 g + n].
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const uint32_t out = out0 + 16 * g + n;
    if (out < a.outputs) {
      const float scale = a.w.tensor_scale != nullptr ? a.w.tensor_scale[(a.first + out) / a.w.rows_per_scale] : 1.0f;
#pragma unroll
      for (int m = 0; m < M; ++m) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t t = t0 + 16 * m + 4 * q + i;
          if (t < rows) a.y[t * a.y_stride + out] = acc[g][m][i] * scale;
        }
      }
    }
  }
}

// The large product: a workgroup of eight waves takes 256 outputs by 128 input rows. A segment of the
// weights is decoded once a workgroup, by one thread, into an LDS tile laid out like the inputs' (rows of 64
// elements, 144 bytes apart), and every wave reads its operands of both sides from LDS: a wave (rows' half
// w / 4, outputs' quarter w % 4) multiplies 64 rows by 64 outputs. Two stages of both tiles: after a chunk's one
// barrier a wave queues the loads of the chunk after the next, and decodes the next chunk (loaded a step ago)
// into the other stage among this chunk's matrix instructions.
// MR: groups of 16 input rows a wave (4: the tile is 128 input rows; 8: 256, where the inputs have that many and the
// tiles still fill the device: a decoded segment then serves twice the matrix instructions, and a wave reads 24
// operands of LDS for 64 instructions instead of 16 for 32).
constexpr int kSharedOutputs = 256;
constexpr int SharedStageBytes(int mr) { return (32 * mr + kSharedOutputs) * kMatrixRowBytes; }

template <int D, int MR>
__global__ __launch_bounds__(512) void DecodeMatrixSharedKernel(const DecodeArgs a, const uint32_t rows) {
  constexpr bool kHalf = D == LLMP_DECODER_F16_DENSE || D == LLMP_DECODER_Q8_0_BLOCKS;
  constexpr int kSharedRows = 32 * MR;
  constexpr int kSharedInputBytes = kSharedRows * kMatrixRowBytes, kSharedStageBytes = SharedStageBytes(MR);
  extern __shared__ __attribute__((aligned(16))) uint8_t stages[];  // two of inputs' tile, weights' tile
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n = lane & 15, q = lane >> 4;
  const uint32_t out0 = blockIdx.x * kSharedOutputs, t0 = blockIdx.y * kSharedRows;
  const uint32_t row_half = (wave >> 2) * (16 * MR), out_quarter = (wave & 3) * 64;
  const uint32_t segs = a.w.k / 16u, chunks = (segs + 3u) / 4u;
  Float4 acc[4][MR];  // [outputs' group][input rows' group]
#pragma unroll
  for (int g = 0; g < 4; ++g) {
#pragma unroll
    for (int m = 0; m < MR; ++m) acc[g][m] = Float4{0.0f, 0.0f, 0.0f, 0.0f};
  }
  // A thread's share of a chunk: MR pieces of four input values (row c / 16, columns 4 (c % 16) + [0, 4) for
  // c = tid + 512 i) and two segments of weights (output e / 4, segment e % 4 for e = tid + 512 u). Loads
  // without branches: past the inputs, the outputs or K they read a valid address nearby, zeroed when staged.
  struct Share {
    float4 piece[MR];
    RawSegment raw[2];
  };
  auto load_inputs = [&](uint32_t chunk, Share& share) {
    // (The tall tile of the decoders with the most state a thread works its pieces' places out again every chunk,
    // from a thread number the compiler cannot see through: kept across the loop they are sixteen registers, which
    // it spills and reloads from scratch memory among the loop's loads. BF16 at 2048 rows: 489 -> 467 us. The
    // other decoders' kernels do not spill and are faster as they are.)
    constexpr bool kAgain = MR > 4 && (D == LLMP_DECODER_BF16_DENSE || D == LLMP_DECODER_F16_DENSE ||
                                       D == LLMP_DECODER_Q8_0_BLOCKS || D == LLMP_DECODER_NVFP4_INTERLEAVED ||
                                       D == LLMP_DECODER_MXFP8_ATOMS || D == LLMP_DECODER_AFFINE_SPLIT);
    uint32_t thread = tid;
    if constexpr (kAgain) asm volatile("" : "+v"(thread));
#pragma unroll
    for (int i = 0; i < MR; ++i) {
      const uint32_t c = thread + i * 512;
      const uint32_t row = min(t0 + (c >> 4), rows - 1), column = min(chunk * 64u + (c & 15u) * 4u, a.w.k - 4u);
      share.piece[i] = *reinterpret_cast<const float4*>(a.x + static_cast<uint64_t>(row) * a.x_stride + column);
    }
  };
  auto load_weights = [&](uint32_t chunk, Share& share) {
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const uint32_t e = tid + u * 512;
      share.raw[u] = FetchSegment<D>(a.w, a.first + min(out0 + (e >> 2), a.outputs - 1), min(chunk * 4u + (e & 3u), segs - 1));
    }
  };
  auto load = [&](uint32_t chunk, Share& share) {
    load_inputs(chunk, share);
    load_weights(chunk, share);
  };
  auto stage_inputs = [&](uint32_t chunk, const Share& share) {
    uint8_t* inputs = stages + (chunk & 1u) * kSharedStageBytes;
#pragma unroll
    for (int i = 0; i < MR; ++i) {
      const uint32_t c = tid + i * 512;
      const bool live = t0 + (c >> 4) < rows && chunk * 64u + (c & 15u) * 4u < a.w.k;
      uint2 packed;
      packed.x = live ? ToElement<kHalf>(share.piece[i].x) | (ToElement<kHalf>(share.piece[i].y) << 16) : 0u;
      packed.y = live ? ToElement<kHalf>(share.piece[i].z) | (ToElement<kHalf>(share.piece[i].w) << 16) : 0u;
      *reinterpret_cast<uint2*>(inputs + (c >> 4) * kMatrixRowBytes + (c & 15u) * 8u) = packed;
    }
  };
  auto stage_weights = [&](uint32_t chunk, const Share& share) {
    uint8_t* weights = stages + (chunk & 1u) * kSharedStageBytes + kSharedInputBytes;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const uint32_t e = tid + u * 512;
      const uint32_t seg = chunk * 4u + (e & 3u);
      float v[16], s;
      DecodeSegment<D>(a.w, min(seg, segs - 1), share.raw[u], v, s);
      U32x4 half[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t two = ToElement<kHalf>(v[8 * j + 2 * i] * s) | (ToElement<kHalf>(v[8 * j + 2 * i + 1] * s) << 16);
          half[j][i] = seg < segs ? two : 0u;
        }
      }
      U32x4* to = reinterpret_cast<U32x4*>(weights + (e >> 2) * kMatrixRowBytes + (e & 3u) * 32u);
      to[0] = half[0], to[1] = half[1];
    }
  };
  auto stage = [&](uint32_t chunk, const Share& share) {
    stage_inputs(chunk, share);
    stage_weights(chunk, share);
  };
  auto multiply = [&](uint32_t chunk) {
    const uint8_t* inputs = stages + (chunk & 1u) * kSharedStageBytes;
    const uint8_t* weights = inputs + kSharedInputBytes;
    // A half of the chunk's K at a time: the outputs' four operands stay, the rows' pass by.
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      U32x4 b[4];
#pragma unroll
      for (int g = 0; g < 4; ++g)
        b[g] = reinterpret_cast<const U32x4*>(weights + (out_quarter + 16 * g + n) * kMatrixRowBytes + q * 32)[j];
      // (The rows' operands are read one group ahead of their use and no further: left to itself the compiler
      // reads all of them first and the tall tile's registers spill.)
      auto rows_operand = [&](int m) {
        return reinterpret_cast<const U32x4*>(inputs + (row_half + 16 * m + n) * kMatrixRowBytes + q * 32)[j];
      };
      U32x4 ahead = rows_operand(0);
#pragma unroll
      for (int m = 0; m < MR; ++m) {
        const U32x4 x8 = ahead;
        if (m + 1 < MR) ahead = rows_operand(m + 1);
        if constexpr (MR > 4) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          if constexpr (kHalf) {
            typedef _Float16 Half8 __attribute__((ext_vector_type(8)));
            acc[g][m] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(Half8, x8),
                                                               __builtin_bit_cast(Half8, b[g]), acc[g][m], 0, 0, 0);
          } else {
            typedef __bf16 Bf8 __attribute__((ext_vector_type(8)));
            acc[g][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(Bf8, x8),
                                                                __builtin_bit_cast(Bf8, b[g]), acc[g][m], 0, 0, 0);
          }
        }
      }
    }
  };
  Share share[2];  // by the chunk's parity
  load(0, share[0]);
  if constexpr (MR > 4) {
    load_weights(1, share[1]);
  } else {
    load(1, share[1]);
  }
  stage(0, share[0]);
  auto step = [&](uint32_t chunk, auto parity) {
    constexpr int P = decltype(parity)::value;
    // One barrier a chunk: its stage is complete, and the other stage's readers (the last chunk's) are done.
    __syncthreads();
    if constexpr (MR > 4) {
      // The tall tile's registers hold one chunk's inputs, not two: the next chunk's are asked for here, a chunk's
      // multiplies ahead of their staging, into the set the weights' loads two chunks ahead do not use.
      load_weights(chunk + 2, share[P]);
      load_inputs(chunk + 1, share[0]);
      multiply(chunk);
      stage_inputs(chunk + 1, share[0]);
      stage_weights(chunk + 1, share[1 - P]);
    } else {
      load(chunk + 2, share[P]);
      multiply(chunk);
      stage(chunk + 1, share[1 - P]);
    }
  };
  for (uint32_t chunk = 0; chunk < chunks; chunk += 2) {  // every wave: the same count of barriers
    step(chunk, std::integral_constant<int, 0>{});
    if (chunk + 1 < chunks) step(chunk + 1, std::integral_constant<int, 1>{});
  }
  // acc[g][m][i] = D[input row 16 m + 4 q + i][output 16 g + n] of the wave's 64 by 64.
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const uint32_t out = out0 + out_quarter + 16 * g + n;
    if (out < a.outputs) {
      const float scale = a.w.tensor_scale != nullptr ? a.w.tensor_scale[(a.first + out) / a.w.rows_per_scale] : 1.0f;
#pragma unroll
      for (int m = 0; m < MR; ++m) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t t = t0 + row_half + 16 * m + 4 * q + i;
          if (t < rows) a.y[t * a.y_stride + out] = acc[g][m][i] * scale;
        }
      }
    }
  }
}

template <int D, int MR>
void LaunchMatrixShared(const DecodeArgs& a, dim3 grid, uint32_t rows, hipStream_t stream) {
  static bool sized = false;  // more than 64 KB of dynamic LDS must be asked for once
  if (!AllowLds(reinterpret_cast<const void*>(&DecodeMatrixSharedKernel<D, MR>), 2 * SharedStageBytes(MR), &sized)) return;
  hipLaunchKernelGGL((DecodeMatrixSharedKernel<D, MR>), grid, dim3(512), 2 * SharedStageBytes(MR), stream, a, rows);
}

size_t DecodeLds(int tokens, uint32_t k) { return static_cast<size_t>(tokens) * (k / 16u) * kSegmentStride; }

template <int D, int T, bool kGlu, int DU = D>
void LaunchDecode(const DecodeArgs& a, int groups, int waves, hipStream_t stream) {
  static bool sized = false;  // more than 64 KB of dynamic LDS must be asked for once
  if (!AllowLds(reinterpret_cast<const void*>(&DecodeVectorKernel<D, T, kGlu, DU>), static_cast<int>(kDecodeLdsLimit), &sized)) return;
  hipLaunchKernelGGL((DecodeVectorKernel<D, T, kGlu, DU>), dim3(static_cast<unsigned>(groups)), dim3(waves * 64),
                     DecodeLds(T, a.w.k), stream, a);
}

// The GLU of two different decoders.
template <int D, int DU>
void LaunchMixedGlu(const DecodeArgs& a, int tokens, int groups, int waves, hipStream_t stream) {
  switch (tokens) {
    case 1: LaunchDecode<D, 1, true, DU>(a, groups, waves, stream); break;
    case 2: LaunchDecode<D, 2, true, DU>(a, groups, waves, stream); break;
    case 3: LaunchDecode<D, 3, true, DU>(a, groups, waves, stream); break;
    default: LaunchDecode<D, 4, true, DU>(a, groups, waves, stream); break;
  }
}
// The mixed pairs the reference instantiates (decode_mixed.cu by src/kernels/decode/implementations.cc:73-81): a
// block-scaled or affine gate with a BF16 or Q8_0 up.
constexpr int kMixedGlu[6][2] = {{LLMP_DECODER_MXFP8_SPLIT, LLMP_DECODER_BF16_DENSE},  {LLMP_DECODER_NVFP4_SPLIT, LLMP_DECODER_Q8_0_BLOCKS},
                                 {LLMP_DECODER_NVFP4_SPLIT, LLMP_DECODER_BF16_DENSE},  {LLMP_DECODER_MXFP4_SPLIT, LLMP_DECODER_BF16_DENSE},
                                 {LLMP_DECODER_MXFP4_SPLIT, LLMP_DECODER_Q8_0_BLOCKS}, {LLMP_DECODER_AFFINE_SPLIT, LLMP_DECODER_BF16_DENSE}};
bool MixedGluBuilt(int gate, int up) {
  for (const auto& pair : kMixedGlu)
    if (pair[0] == gate && pair[1] == up) return true;
  return false;
}

template <int D, bool kGlu>
void LaunchTokens(const DecodeArgs& a, int tokens, int groups, int waves, hipStream_t stream) {
  switch (tokens) {
    case 1: LaunchDecode<D, 1, kGlu>(a, groups, waves, stream); break;
    case 2: LaunchDecode<D, 2, kGlu>(a, groups, waves, stream); break;
    case 3: LaunchDecode<D, 3, kGlu>(a, groups, waves, stream); break;
    default: LaunchDecode<D, 4, kGlu>(a, groups, waves, stream); break;
  }
}

template <int D>
void LaunchDecoder(const DecodeArgs& a, bool glu, int tokens, int groups, int waves, hipStream_t stream) {
  if (glu) {
    LaunchTokens<D, true>(a, tokens, groups, waves, stream);
  } else {
    LaunchTokens<D, false>(a, tokens, groups, waves, stream);
  }
}

// The multiple of K a decoder's rows must be (DecoderKMultiple, products.h:88-90): its blocks,
// scale atoms and 16-value segments.
uint32_t KMultiple(int decoder) {
  switch (decoder) {
    case LLMP_DECODER_Q8_0_BLOCKS: case LLMP_DECODER_MXFP8_SPLIT: case LLMP_DECODER_MXFP4_SPLIT: return 32;
    case LLMP_DECODER_NVFP4_ATOMS: case LLMP_DECODER_NVFP4_GGML_BLOCKS: return 64;
    case LLMP_DECODER_MXFP8_ATOMS: case LLMP_DECODER_MXFP4_ATOMS: return 128;
    default: return 16;
  }
}
// The alignment a decoder's loads of `data` need (products.h:38-43); the affine decoder's by its
// code width (16 bytes for 8-bit codes, 8 for 4-bit).
uint32_t DataAlignment(int decoder) {
  switch (decoder) {
    case LLMP_DECODER_BF16_DENSE: case LLMP_DECODER_F16_DENSE: case LLMP_DECODER_MXFP8_SPLIT:
    case LLMP_DECODER_MXFP8_ATOMS: return 16;
    case LLMP_DECODER_NVFP4_SPLIT: case LLMP_DECODER_NVFP4_ATOMS: case LLMP_DECODER_MXFP4_SPLIT:
    case LLMP_DECODER_MXFP4_ATOMS: return 8;
    case LLMP_DECODER_NVFP4_GGML_BLOCKS: return 4;
    case LLMP_DECODER_Q8_0_BLOCKS: return 2;
    default: return 1;
  }
}
bool SplitScales(int decoder) {
  return decoder == LLMP_DECODER_NVFP4_SPLIT || decoder == LLMP_DECODER_NVFP4_ATOMS || decoder == LLMP_DECODER_MXFP8_SPLIT ||
         decoder == LLMP_DECODER_MXFP8_ATOMS || decoder == LLMP_DECODER_MXFP4_SPLIT || decoder == LLMP_DECODER_MXFP4_ATOMS;
}

int CheckOperand(const char* what, int decoder, const llmp_decode_operand* w, uint64_t first, uint64_t outputs) {
  if (w == nullptr) return Refuse(1, "%s: null operand", what);
  if (decoder < 0 || decoder > LLMP_DECODER_AFFINE_SPLIT) return Refuse(1, "%s: decoder %d has no kernel", what, decoder);
  if (w->data == nullptr) return Refuse(1, "%s: null operand", what);
  if (decoder == LLMP_DECODER_AFFINE_SPLIT) {
    const uint32_t element = w->scale_type & 0x7Fu;
    if ((w->bits != 4 && w->bits != 8) || (w->group != 32 && w->group != 64 && w->group != 128) || element < 1 || element > 3)
      return Refuse(1, "%s: affine codes of 4 or 8 bits, groups of 32, 64 or 128 values, F16, BF16 or F32 scales", what);
    if (w->scales == nullptr || ((w->scale_type & 0x80u) != 0 && w->biases == nullptr))
      return Refuse(1, "%s: the affine encoding's scales or zero points are missing", what);
    if (w->k == 0 || w->k % w->group != 0) return Refuse(1, "%s: k %u is not whole groups of %u", what, w->k, w->group);
    const uint32_t step = element == 3u ? 4u : 2u;
    if ((reinterpret_cast<uintptr_t>(w->scales) | w->scale_row_bytes) % step != 0 ||
        ((w->scale_type & 0x80u) == 0 && w->biases != nullptr && reinterpret_cast<uintptr_t>(w->biases) % step != 0))
      return Refuse(1, "%s: the affine scales are not aligned to their element", what);
  }
  if (SplitScales(decoder) && w->scales == nullptr) return Refuse(1, "%s: the layout's block scales are missing", what);
  if (w->k == 0 || w->k % KMultiple(decoder) != 0)
    return Refuse(1, "%s: k %u is not a multiple of the decoder's %u", what, w->k, KMultiple(decoder));
  if (outputs == 0 || first > w->rows || outputs > w->rows - first)
    return Refuse(1, "%s: outputs [%llu, %llu) of %u", what, static_cast<unsigned long long>(first),
                  static_cast<unsigned long long>(first + outputs), w->rows);
  if (w->tensor_scale != nullptr && w->rows_per_scale == 0) return Refuse(1, "%s: tensor scales of no rows", what);
  const uint32_t alignment = decoder == LLMP_DECODER_AFFINE_SPLIT ? (w->bits == 8 ? 16u : 8u) : DataAlignment(decoder);
  if (reinterpret_cast<uintptr_t>(w->data) % alignment != 0 || w->row_bytes % alignment != 0)
    return Refuse(1, "%s: the weight's rows are not aligned for its decoder's loads (%u bytes)", what, alignment);
  return 0;
}

// The launches of a product whose operands have been checked: four input rows a pass, or
// fewer of a long row.
int LaunchProduct(const char* what, int decoder, bool glu, DecodeArgs& a, uint64_t rows, hipStream_t s, int up_decoder = -1) {
  const uint32_t k = a.w.k;
  if (rows == 0 || rows > 16) return Refuse(1, "%s: rows %llu (1 to 16)", what, static_cast<unsigned long long>(rows));
  if (reinterpret_cast<uintptr_t>(a.x) % 16 != 0 || a.x_stride % 4 != 0 || a.x_stride < k || a.y_stride < a.outputs ||
      reinterpret_cast<uintptr_t>(a.y) % 4 != 0)
    return Refuse(1, "%s: input rows are 16-byte aligned, a multiple of 4 floats apart and at least k long", what);
  int pass = rows < 4 ? static_cast<int>(rows) : 4;
  while (pass > 1 && DecodeLds(pass, k) > kDecodeLdsLimit) --pass;
  if (DecodeLds(pass, k) > kDecodeLdsLimit)
    return Refuse(1, "%s: a row of %u values does not fit the staging area (16384 at most)", what, k);
  const int cus = llmp_hip_compute_units();
  const size_t lds = DecodeLds(pass, k);
  // One input row: four waves a workgroup and more workgroups; two or three: eight; four: sixteen waves share the
  // staged rows (which then fill LDS: one workgroup a CU, its loads two steps ahead: MXFP8 4096 x 14336 at four rows
  // 34.5 -> 22.8 us, at sixteen 135 -> 88; NVFP4 30 -> 19.6 and 117 -> 74).
  const int waves = pass == 1 ? 4 : pass < 4 ? 8 : kDecodeWaves;
  int resident = static_cast<int>(160 * 1024 / (lds + 1024));
  if (resident > 32 / waves) resident = 32 / waves;  // a CU holds 32 waves
  if (resident < 1) resident = 1;
  const uint64_t pairs = glu ? a.outputs : (a.outputs + kRowsAWave - 1) / kRowsAWave;
  uint64_t groups = (pairs + waves - 1) / waves;
  const uint64_t most = static_cast<uint64_t>(cus > 0 ? cus : 256) * resident;
  if (groups > most) groups = most;
  for (uint64_t token0 = 0; token0 < rows; token0 += pass) {
    const int tokens = static_cast<int>(rows - token0 < static_cast<uint64_t>(pass) ? rows - token0 : pass);
    a.token0 = static_cast<uint32_t>(token0);
    if (up_decoder >= 0 && up_decoder != decoder) {
#define LLMP_MIXED(G, U) \
  if (decoder == G && up_decoder == U) LaunchMixedGlu<G, U>(a, tokens, static_cast<int>(groups), waves, s);
      LLMP_MIXED(LLMP_DECODER_MXFP8_SPLIT, LLMP_DECODER_BF16_DENSE)
      LLMP_MIXED(LLMP_DECODER_NVFP4_SPLIT, LLMP_DECODER_Q8_0_BLOCKS)
      LLMP_MIXED(LLMP_DECODER_NVFP4_SPLIT, LLMP_DECODER_BF16_DENSE)
      LLMP_MIXED(LLMP_DECODER_MXFP4_SPLIT, LLMP_DECODER_BF16_DENSE)
      LLMP_MIXED(LLMP_DECODER_MXFP4_SPLIT, LLMP_DECODER_Q8_0_BLOCKS)
      LLMP_MIXED(LLMP_DECODER_AFFINE_SPLIT, LLMP_DECODER_BF16_DENSE)
#undef LLMP_MIXED
      const int status = LaunchStatus(what);
      if (status != 0) return token0 == 0 ? status : (status > 0 ? -status : status);
      continue;
    }
    switch (decoder) {
#define LLMP_DECODER(ID) \
  case ID: LaunchDecoder<ID>(a, glu, tokens, static_cast<int>(groups), waves, s); break;
      LLMP_DECODER(LLMP_DECODER_BF16_DENSE)
      LLMP_DECODER(LLMP_DECODER_F16_DENSE)
      LLMP_DECODER(LLMP_DECODER_Q8_0_BLOCKS)
      LLMP_DECODER(LLMP_DECODER_NVFP4_SPLIT)
      LLMP_DECODER(LLMP_DECODER_NVFP4_ATOMS)
      LLMP_DECODER(LLMP_DECODER_NVFP4_INTERLEAVED)
      LLMP_DECODER(LLMP_DECODER_NVFP4_GGML_BLOCKS)
      LLMP_DECODER(LLMP_DECODER_MXFP8_SPLIT)
      LLMP_DECODER(LLMP_DECODER_MXFP8_ATOMS)
      LLMP_DECODER(LLMP_DECODER_MXFP4_SPLIT)
      LLMP_DECODER(LLMP_DECODER_MXFP4_ATOMS)
      LLMP_DECODER(LLMP_DECODER_AFFINE_SPLIT)
#undef LLMP_DECODER
    }
    const int status = LaunchStatus(what);
    if (status != 0) return token0 == 0 ? status : (status > 0 ? -status : status);
  }
  return 0;
}

}  // namespace
}  // namespace llmp_hip

using namespace llmp_hip;

extern "C" int llmp_hip_decode_vector(int decoder, const llmp_decode_operand* w, uint64_t first, uint64_t outputs,
                                      const float* x, uint64_t rows, uint64_t x_stride, float* y, uint64_t y_stride,
                                      void* stream) {
  BeginLaunches();
  if (const int bad = CheckOperand("decode.vector", decoder, w, first, outputs); bad != 0) return bad;
  if (x == nullptr || y == nullptr) return Refuse(1, "decode.vector: null operand");
  DecodeArgs a{};
  a.w = *w;
  a.first = static_cast<uint32_t>(first);
  a.outputs = static_cast<uint32_t>(outputs);
  a.x = x, a.x_stride = x_stride, a.y = y, a.y_stride = y_stride;
  return LaunchProduct("decode.vector", decoder, false, a, rows, static_cast<hipStream_t>(stream));
}

extern "C" int llmp_hip_decode_vector_glu(int gate_decoder, const llmp_decode_operand* gate, uint64_t gate_first,
                                          int up_decoder, const llmp_decode_operand* up, uint64_t up_first,
                                          uint64_t outputs, int glu, float limit, const float* x, uint64_t rows,
                                          uint64_t x_stride, float* y, uint64_t y_stride, void* stream) {
  BeginLaunches();
  if (const int bad = CheckOperand("decode.vector_glu gate", gate_decoder, gate, gate_first, outputs); bad != 0) return bad;
  if (const int bad = CheckOperand("decode.vector_glu up", up_decoder, up, up_first, outputs); bad != 0) return bad;
  if (gate_decoder != up_decoder && !MixedGluBuilt(gate_decoder, up_decoder))
    return Refuse(1, "decode.vector_glu: no instantiation for gate decoder %d with up decoder %d", gate_decoder, up_decoder);
  if (gate->k != up->k) return Refuse(1, "decode.vector_glu: gate's K %u and up's %u differ", gate->k, up->k);
  if (glu < 0 || glu > 3) return Refuse(1, "decode.vector_glu: unknown GLU");
  if (x == nullptr || y == nullptr) return Refuse(1, "decode.vector_glu: null operand");
  DecodeArgs a{};
  a.w = *gate;
  a.up = *up;
  a.first = static_cast<uint32_t>(gate_first);
  a.up_first = static_cast<uint32_t>(up_first);
  a.outputs = static_cast<uint32_t>(outputs);
  a.glu = glu, a.limit = limit;
  a.x = x, a.x_stride = x_stride, a.y = y, a.y_stride = y_stride;
  return LaunchProduct("decode.vector_glu", gate_decoder, true, a, rows, static_cast<hipStream_t>(stream), up_decoder);
}

extern "C" int llmp_hip_decode_rows(int decoder, const llmp_decode_operand* w, const int32_t* ids, uint64_t count,
                                    float* out, uint64_t out_stride, int32_t* bad, void* stream) {
  BeginLaunches();
  if (const int status = CheckOperand("decode.rows", decoder, w, 0, 1); status != 0) return status;
  if (ids == nullptr || out == nullptr) return Refuse(1, "decode.rows: null operand");
  if (count == 0 || count > (uint64_t{1} << 31)) return Refuse(1, "decode.rows: 1 to 2^31 rows");
  if (reinterpret_cast<uintptr_t>(out) % 16 != 0 || out_stride % 4 != 0 || out_stride < w->k ||
      reinterpret_cast<uintptr_t>(ids) % 4 != 0 || reinterpret_cast<uintptr_t>(bad) % 4 != 0)
    return Refuse(1, "decode.rows: output rows are 16-byte aligned, a multiple of 4 floats apart and at least k long");
  const dim3 grid(static_cast<unsigned>((count + 3) / 4));
  const auto s = static_cast<hipStream_t>(stream);
  switch (decoder) {
#define LLMP_DECODER(ID)                                                                                          \
  case ID:                                                                                                        \
    hipLaunchKernelGGL((DecodeRowsKernel<ID>), grid, dim3(256), 0, s, *w, ids, static_cast<uint32_t>(count), out, \
                       out_stride, bad);                                                                          \
    break;
    LLMP_DECODER(LLMP_DECODER_BF16_DENSE)
    LLMP_DECODER(LLMP_DECODER_F16_DENSE)
    LLMP_DECODER(LLMP_DECODER_Q8_0_BLOCKS)
    LLMP_DECODER(LLMP_DECODER_NVFP4_SPLIT)
    LLMP_DECODER(LLMP_DECODER_NVFP4_ATOMS)
    LLMP_DECODER(LLMP_DECODER_NVFP4_INTERLEAVED)
    LLMP_DECODER(LLMP_DECODER_NVFP4_GGML_BLOCKS)
    LLMP_DECODER(LLMP_DECODER_MXFP8_SPLIT)
    LLMP_DECODER(LLMP_DECODER_MXFP8_ATOMS)
    LLMP_DECODER(LLMP_DECODER_MXFP4_SPLIT)
    LLMP_DECODER(LLMP_DECODER_MXFP4_ATOMS)
    LLMP_DECODER(LLMP_DECODER_AFFINE_SPLIT)
#undef LLMP_DECODER
  }
  return LaunchStatus("decode.rows");
}

namespace llmp_hip {
namespace {

template <int D, int T>
void LaunchGrouped(const GroupedArgs& a, dim3 grid, hipStream_t stream) {
  static bool sized = false;  // more than 64 KB of dynamic LDS must be asked for once
  if (!AllowLds(reinterpret_cast<const void*>(&DecodeGroupedKernel<D, T>), static_cast<int>(kDecodeLdsLimit), &sized)) return;
  hipLaunchKernelGGL((DecodeGroupedKernel<D, T>), grid, dim3(kGroupedWaves * 64), DecodeLds(T, a.k), stream, a);
}

template <int D>
void LaunchGroupedDecoder(const GroupedArgs& a, int pass, dim3 grid, hipStream_t stream) {
  switch (pass) {
    case 1: LaunchGrouped<D, 1>(a, grid, stream); break;
    case 2: LaunchGrouped<D, 2>(a, grid, stream); break;
    default: LaunchGrouped<D, 4>(a, grid, stream); break;
  }
}

}  // namespace
}  // namespace llmp_hip

extern "C" int llmp_hip_decode_grouped(int decoder, const llmp_decode_operand* experts, uint64_t experts_count, uint32_t k,
                                       uint32_t n, uint64_t first, uint64_t outputs, const int32_t* offsets,
                                       const int32_t* pair_rows, const int32_t* pair_out, uint64_t pairs, const float* x,
                                       uint64_t x_rows, uint64_t x_stride, float* y, uint64_t y_rows, uint64_t y_stride,
                                       uint64_t rows_hint, void* stream) {
  BeginLaunches();
  (void)rows_hint;  // picks the reference's tile; the passes here are of up to four pairs whatever it is
  if (decoder < 0 || decoder > LLMP_DECODER_AFFINE_SPLIT) return Refuse(1, "decode.grouped: decoder %d has no kernel", decoder);
  if (experts == nullptr || offsets == nullptr || pair_rows == nullptr || x == nullptr || y == nullptr)
    return Refuse(1, "decode.grouped: null operand");
  if (experts_count == 0 || experts_count > 65535) return Refuse(1, "decode.grouped: 1 to 65535 experts");
  if (k == 0 || k % KMultiple(decoder) != 0)
    return Refuse(1, "decode.grouped: k %u is not a multiple of the decoder's %u", k, KMultiple(decoder));
  if (outputs == 0 || first > n || outputs > n - first)
    return Refuse(1, "decode.grouped: outputs [%llu, %llu) of %u", static_cast<unsigned long long>(first),
                  static_cast<unsigned long long>(first + outputs), n);
  if (pairs == 0 || pairs >= (uint64_t{1} << 31) || x_rows >= (uint64_t{1} << 31) || y_rows >= (uint64_t{1} << 31))
    return Refuse(1, "decode.grouped: 1 to 2^31 pairs and rows");
  if (reinterpret_cast<uintptr_t>(x) % 16 != 0 || x_stride % 4 != 0 || x_stride < k || y_stride < outputs ||
      reinterpret_cast<uintptr_t>(y) % 4 != 0 || reinterpret_cast<uintptr_t>(experts) % 8 != 0)
    return Refuse(1, "decode.grouped: input rows are 16-byte aligned, a multiple of 4 floats apart and at least k long");
  int pass = 4;
  while (pass > 1 && DecodeLds(pass, k) > kDecodeLdsLimit) pass /= 2;
  if (DecodeLds(pass, k) > kDecodeLdsLimit)
    return Refuse(1, "decode.grouped: a row of %u values does not fit the staging area (16384 at most)", k);
  GroupedArgs a;
  a.experts = experts;
  a.k = k, a.n = n, a.first = static_cast<uint32_t>(first), a.outputs = static_cast<uint32_t>(outputs);
  a.offsets = offsets, a.pair_rows = pair_rows, a.pair_out = pair_out;
  a.pairs = static_cast<uint32_t>(pairs), a.x_rows = static_cast<uint32_t>(x_rows), a.y_rows = static_cast<uint32_t>(y_rows);
  a.x = x, a.x_stride = x_stride, a.y = y, a.y_stride = y_stride;
  const int cus = llmp_hip_compute_units();
  uint64_t groups = 2 * static_cast<uint64_t>(cus > 0 ? cus : 256) / experts_count;
  const uint64_t most = ((outputs + kRowsAWave - 1) / kRowsAWave + kGroupedWaves - 1) / kGroupedWaves;
  if (groups > most) groups = most;
  if (groups < 1) groups = 1;
  const dim3 grid(static_cast<unsigned>(groups), static_cast<unsigned>(experts_count));
  const auto s = static_cast<hipStream_t>(stream);
  switch (decoder) {
#define LLMP_DECODER(ID) \
  case ID: LaunchGroupedDecoder<ID>(a, pass, grid, s); break;
    LLMP_DECODER(LLMP_DECODER_BF16_DENSE)
    LLMP_DECODER(LLMP_DECODER_F16_DENSE)
    LLMP_DECODER(LLMP_DECODER_Q8_0_BLOCKS)
    LLMP_DECODER(LLMP_DECODER_NVFP4_SPLIT)
    LLMP_DECODER(LLMP_DECODER_NVFP4_ATOMS)
    LLMP_DECODER(LLMP_DECODER_NVFP4_INTERLEAVED)
    LLMP_DECODER(LLMP_DECODER_NVFP4_GGML_BLOCKS)
    LLMP_DECODER(LLMP_DECODER_MXFP8_SPLIT)
    LLMP_DECODER(LLMP_DECODER_MXFP8_ATOMS)
    LLMP_DECODER(LLMP_DECODER_MXFP4_SPLIT)
    LLMP_DECODER(LLMP_DECODER_MXFP4_ATOMS)
    LLMP_DECODER(LLMP_DECODER_AFFINE_SPLIT)
#undef LLMP_DECODER
  }
  return LaunchStatus("decode.grouped");
}

extern "C" int llmp_hip_decode_matrix(int decoder, const llmp_decode_operand* w, uint64_t first, uint64_t outputs,
                                      const float* x, uint64_t rows, uint64_t x_stride, float* y, uint64_t y_stride,
                                      int path, void* stream) {
  BeginLaunches();
  if (const int bad = CheckOperand("decode.matrix", decoder, w, first, outputs); bad != 0) return bad;
  if (x == nullptr || y == nullptr) return Refuse(1, "decode.matrix: null operand");
  if (path != 0) return Refuse(1, "decode.matrix: the FMA path is for devices without matrix cores; this one has them");
  if (rows == 0 || rows > 65535ull * 64ull) return Refuse(1, "decode.matrix: rows %llu (1 to 4194240)", static_cast<unsigned long long>(rows));
  if (reinterpret_cast<uintptr_t>(x) % 16 != 0 || x_stride % 4 != 0 || x_stride < w->k || y_stride < outputs ||
      reinterpret_cast<uintptr_t>(y) % 4 != 0)
    return Refuse(1, "decode.matrix: input rows are 16-byte aligned, a multiple of 4 floats apart and at least k long");
  if (rows * x_stride >= (uint64_t{1} << 32) || rows * y_stride >= (uint64_t{1} << 32))
    return Refuse(1, "decode.matrix: inputs or outputs of 2^32 values or more");
  DecodeArgs a{};
  a.w = *w;
  a.first = static_cast<uint32_t>(first);
  a.outputs = static_cast<uint32_t>(outputs);
  a.x = x, a.x_stride = x_stride, a.y = y, a.y_stride = y_stride;
  // Tiles of 256 outputs by 128 input rows where those still give every other CU a workgroup; else 64 by 64.
  const int cus = llmp_hip_compute_units();
  const uint64_t units = static_cast<uint64_t>(cus > 0 ? cus : 256);
  const bool wide = 2 * ((outputs + 255) / 256 * ((rows + 127) / 128)) >= units;
  // Tiles of 256 input rows where the inputs have them and the tiles still give every CU one.
  const bool tall = wide && rows >= 256 && (outputs + 255) / 256 * ((rows + 255) / 256) >= units;
  const uint64_t per = wide ? 256 : 64, tile = tall ? 256 : wide ? 128 : 64;
  const dim3 grid(static_cast<unsigned>((outputs + per - 1) / per), static_cast<unsigned>((rows + tile - 1) / tile));
  const auto s = static_cast<hipStream_t>(stream);
  switch (decoder) {
#define LLMP_DECODER(ID)                                                                                          \
  case ID:                                                                                                        \
    if (tall) {                                                                                                   \
      LaunchMatrixShared<ID, 8>(a, grid, static_cast<uint32_t>(rows), s);                                        \
    } else if (wide) {                                                                                            \
      LaunchMatrixShared<ID, 4>(a, grid, static_cast<uint32_t>(rows), s);                                        \
    } else {                                                                                                      \
      hipLaunchKernelGGL((DecodeMatrixKernel<ID, 1, 4>), grid, dim3(256), 0, s, a, static_cast<uint32_t>(rows)); \
    }                                                                                                             \
    break;
    LLMP_DECODER(LLMP_DECODER_BF16_DENSE)
    LLMP_DECODER(LLMP_DECODER_F16_DENSE)
    LLMP_DECODER(LLMP_DECODER_Q8_0_BLOCKS)
    LLMP_DECODER(LLMP_DECODER_NVFP4_SPLIT)
    LLMP_DECODER(LLMP_DECODER_NVFP4_ATOMS)
    LLMP_DECODER(LLMP_DECODER_NVFP4_INTERLEAVED)
    LLMP_DECODER(LLMP_DECODER_NVFP4_GGML_BLOCKS)
    LLMP_DECODER(LLMP_DECODER_MXFP8_SPLIT)
    LLMP_DECODER(LLMP_DECODER_MXFP8_ATOMS)
    LLMP_DECODER(LLMP_DECODER_MXFP4_SPLIT)
    LLMP_DECODER(LLMP_DECODER_MXFP4_ATOMS)
    LLMP_DECODER(LLMP_DECODER_AFFINE_SPLIT)
#undef LLMP_DECODER
  }
  return LaunchStatus("decode.matrix");
}
