// llmp.set_rows.quant for gfx950: F32 rows stored into a Q8_0 or Q4_0 cache at given row
// indices (src/kernels/ggml/kv_quant.h:28-60 of the reference). Each block of 32 values is
// quantized by one thread with the arithmetic of src/kernels/ggml/kv_quant.cuh:27-69, GGML's
// reference quantizers step by step: every operation an IEEE one rounded to nearest, none
// contracted (this unit builds without fast math).

#include <hip/hip_runtime.h>

#include "common.h"
#include "llmp_hip.h"

namespace llmp_hip {
namespace {

constexpr int kStoreThreads = 256;  // kQuantStoreThreads, kv_quant.h:78

// kv_quant.cuh:27-43: d = amax / 127, codes round-half-away(x * (1 / d)).
__device__ __forceinline__ void StoreQ8_0(const float (&x)[32], uint8_t* to) {
#pragma clang fp contract(off)
  float amax = 0.0f;
#pragma unroll
  for (int j = 0; j < 32; ++j) {
    const float v = fabsf(x[j]);
    amax = amax > v ? amax : v;
  }
  const float d = amax / 127.0f;
  const float id = d != 0.0f ? 1.0f / d : 0.0f;
  uint16_t* out = reinterpret_cast<uint16_t*>(to);
  out[0] = static_cast<uint16_t>(FloatToHalfBits(d));
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const int q0 = static_cast<int8_t>(roundf(x[2 * j] * id));
    const int q1 = static_cast<int8_t>(roundf(x[2 * j + 1] * id));
    out[1 + j] = static_cast<uint16_t>((q0 & 0xFF) | ((q1 & 0xFF) << 8));
  }
}

// kv_quant.cuh:45-69: the value of largest magnitude (the first among equals) over -8 as the
// scale, codes min(15, trunc(x * (1 / d) + 8.5)), value j in byte j's low nibble and value
// j + 16 in its high one.
__device__ __forceinline__ void StoreQ4_0(const float (&x)[32], uint8_t* to) {
#pragma clang fp contract(off)
  float amax = 0.0f, vmax = 0.0f;
#pragma unroll
  for (int j = 0; j < 32; ++j) {
    const float v = x[j];
    if (amax < fabsf(v)) {
      amax = fabsf(v);
      vmax = v;
    }
  }
  float d = vmax / -8.0f;
  // The quotient as a value of its own before it is rounded to F16: folded into one fused
  // conversion (vmax * -0.125 + 0) a zero block's scale would come out +0 where 0 / -8 is -0.
  asm volatile("" : "+v"(d));
  const float id = d != 0.0f ? 1.0f / d : 0.0f;
  uint16_t* out = reinterpret_cast<uint16_t*>(to);
  out[0] = static_cast<uint16_t>(FloatToHalfBits(d));
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    uint32_t pair = 0;
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const float x0 = x[2 * j + b] * id;
      const float x1 = x[16 + 2 * j + b] * id;
      const int xi0 = min(15, static_cast<int>(static_cast<int8_t>(x0 + 8.5f)));
      const int xi1 = min(15, static_cast<int>(static_cast<int8_t>(x1 + 8.5f)));
      pair |= static_cast<uint32_t>((xi0 | (xi1 << 4)) & 0xFF) << (8 * b);
    }
    out[1 + j] = static_cast<uint16_t>(pair);
  }
}

// A thread a block of 32 values; grid covers rows x blocks.
template <typename Index>
__global__ __launch_bounds__(kStoreThreads) void SetRowsQuantKernel(const float* __restrict__ x, int64_t x_stride,
                                                                   const Index* __restrict__ ids,
                                                                   uint8_t* __restrict__ destination, int64_t row_bytes,
                                                                   int blocks, int64_t total, int type) {
  const int64_t at = static_cast<int64_t>(blockIdx.x) * kStoreThreads + threadIdx.x;
  if (at >= total) return;
  const int64_t row = at / blocks;
  const int block = static_cast<int>(at - row * blocks);
  const float4* from = reinterpret_cast<const float4*>(x + row * x_stride + block * 32);
  float v[32];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float4 f = from[i];
    v[4 * i] = f.x, v[4 * i + 1] = f.y, v[4 * i + 2] = f.z, v[4 * i + 3] = f.w;
  }
  uint8_t* to = destination + static_cast<int64_t>(ids[row]) * row_bytes;
  if (type == LLMP_TYPE_Q8_0) {
    StoreQ8_0(v, to + block * 34);
  } else {
    StoreQ4_0(v, to + block * 18);
  }
}

// Two to sixteen stores in one launch: grid row m is store m, its descriptor in the kernel's arguments
// (src/kernels/ggml/kv_quant.h:82-84, 172-178 of the reference).
struct StoreMember {
  const float* x;
  const void* ids;
  uint8_t* destination;
  int64_t x_stride, row_bytes, total;
  int blocks, type, index_bytes;
};
struct StoreGroup {
  StoreMember member[16];
};

__global__ __launch_bounds__(kStoreThreads) void SetRowsQuantGroupKernel(const StoreGroup group) {
  const StoreMember& s = group.member[blockIdx.y];
  const int64_t at = static_cast<int64_t>(blockIdx.x) * kStoreThreads + threadIdx.x;
  if (at >= s.total) return;
  const int64_t row = at / s.blocks;
  const int block = static_cast<int>(at - row * s.blocks);
  const float4* from = reinterpret_cast<const float4*>(s.x + row * s.x_stride + block * 32);
  float v[32];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float4 f = from[i];
    v[4 * i] = f.x, v[4 * i + 1] = f.y, v[4 * i + 2] = f.z, v[4 * i + 3] = f.w;
  }
  const int64_t id = s.index_bytes == 4 ? static_cast<const int32_t*>(s.ids)[row] : static_cast<const int64_t*>(s.ids)[row];
  uint8_t* to = s.destination + id * s.row_bytes;
  if (s.type == LLMP_TYPE_Q8_0) {
    StoreQ8_0(v, to + block * 34);
  } else {
    StoreQ4_0(v, to + block * 18);
  }
}

// llmp.rope.set_rows_quant: a forward NEOX RoPE of a token's heads, then the store
// (src/kernels/ggml/kv_quant_rope.cu:29-120 of the reference): a workgroup a token, a thread a block of 32 values of its row. A
// channel below n_dims is one of the pair (c, c + n_dims / 2); the pair's angle is pos * theta_scale^pair over
// the frequency factor, YaRN's ramp mixes the interpolated (freq_scale) and the extrapolated angle between the
// correction dims and raises the magnitude; channels from n_dims on pass through.
// A workgroup a token: the token's n_dims / 2 cosines and sines once, in LDS, for every head's blocks.
__global__ __launch_bounds__(kStoreThreads) void RopeSetRowsQuantKernel(const llmp_rope_store s) {
  extern __shared__ float2 rotation[];  // of pair p: magnitude * (cos, sin)
  const int64_t token = blockIdx.x;
  const int half = s.n_dims / 2;
  const float position = static_cast<float>(s.pos[token]);
  float magnitude = s.attn_factor;
  if (s.ext_factor != 0.0f) magnitude *= 1.0f + 0.1f * logf(1.0f / s.freq_scale);
  for (int pair = threadIdx.x; pair < half; pair += kStoreThreads) {
    const float factor = s.freq_factors != nullptr ? s.freq_factors[pair] : 1.0f;
    const float extrapolated = position * powf(s.theta_scale, static_cast<float>(pair)) / factor;
    const float interpolated = s.freq_scale * extrapolated;
    float theta = interpolated;
    if (s.ext_factor != 0.0f) {
      const float y = (static_cast<float>(pair) - s.corr_dims[0]) / fmaxf(0.001f, s.corr_dims[1] - s.corr_dims[0]);
      const float ramp = (1.0f - fminf(1.0f, fmaxf(0.0f, y))) * s.ext_factor;
      theta = interpolated * (1.0f - ramp) + extrapolated * ramp;
    }
    rotation[pair] = make_float2(cosf(theta) * magnitude, sinf(theta) * magnitude);
  }
  __syncthreads();  // every thread: the loop below has no barrier
  const int blocks_head = s.head_dim / 32, blocks_row = s.heads * blocks_head;
  const bool wide = half % 32 == 0 && s.x_head_stride % 4 == 0 && s.x_token_stride % 4 == 0 &&
                    reinterpret_cast<uintptr_t>(s.x) % 16 == 0;
  uint8_t* to = static_cast<uint8_t*>(s.destination) + s.ids[token] * s.row_bytes;
  for (int block = threadIdx.x; block < blocks_row; block += kStoreThreads) {
    const int head = block / blocks_head;
    const int first = (block - head * blocks_head) * 32;  // channel within the head
    const float* x = s.x + head * s.x_head_stride + token * s.x_token_stride;
    float v[32];
    if (wide) {
      // The block lies within one half of the rotated channels (or past them): its 32 values and their partners'
      // as 16-byte loads.
      const float4* own = reinterpret_cast<const float4*>(x + first);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float4 f = own[i];
        v[4 * i] = f.x, v[4 * i + 1] = f.y, v[4 * i + 2] = f.z, v[4 * i + 3] = f.w;
      }
      if (first < s.n_dims) {
        const bool lower = first < half;
        const int pair0 = lower ? first : first - half;
        const float4* other = reinterpret_cast<const float4*>(x + (lower ? first + half : pair0));
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float4 f = other[i];
          const float partner[4] = {f.x, f.y, f.z, f.w};
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const float2 r = rotation[pair0 + 4 * i + c];
            const float mine = v[4 * i + c];
            v[4 * i + c] = lower ? mine * r.x - partner[c] * r.y : partner[c] * r.y + mine * r.x;
          }
        }
      }
    } else {
#pragma unroll 8
      for (int j = 0; j < 32; ++j) {
        const int channel = first + j;
        if (channel >= s.n_dims) {
          v[j] = x[channel];
          continue;
        }
        const int pair = channel < half ? channel : channel - half;
        const float2 r = rotation[pair];
        const float x0 = x[pair], x1 = x[pair + half];
        v[j] = channel < half ? x0 * r.x - x1 * r.y : x0 * r.y + x1 * r.x;
      }
    }
    if (s.type == LLMP_TYPE_Q8_0) {
      StoreQ8_0(v, to + block * 34);
    } else {
      StoreQ4_0(v, to + block * 18);
    }
  }
}

// What one store must satisfy; its count of blocks in *total.
int CheckStore(const char* op, int type, const float* x, int64_t x_stride, const void* ids, int index_bytes,
               const void* destination, int64_t row_bytes, int64_t k, int64_t rows, int64_t* total) {
  if (x == nullptr || ids == nullptr || destination == nullptr) return Refuse(1, "%s: null operand", op);
  if (type != LLMP_TYPE_Q8_0 && type != LLMP_TYPE_Q4_0) return Refuse(1, "%s: a Q8_0 or Q4_0 destination", op);
  if (index_bytes != 4 && index_bytes != 8) return Refuse(1, "%s: I32 or I64 indices", op);
  if (k <= 0 || k % 32 != 0 || rows <= 0) return Refuse(1, "%s: rows of whole 32-value blocks", op);
  const int64_t block_bytes = type == LLMP_TYPE_Q8_0 ? 34 : 18;
  if (x_stride < k || x_stride % 4 != 0 || reinterpret_cast<uintptr_t>(x) % 16 != 0)
    return Refuse(1, "%s: source rows overlap or are not 16-byte aligned", op);
  if (row_bytes < k / 32 * block_bytes || row_bytes % 2 != 0 || reinterpret_cast<uintptr_t>(destination) % 2 != 0)
    return Refuse(1, "%s: destination rows overlap or are not 2-byte aligned", op);
  *total = rows * (k / 32);
  if (*total > 0xFFFFFFFFll / 32) return Refuse(1, "%s: more than 2^32 - 1 values", op);  // kv_quant.h:150-156
  return 0;
}

bool Meet(const void* a, int64_t a_bytes, const void* b, int64_t b_bytes) {
  const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
  return a0 < b0 + static_cast<uintptr_t>(b_bytes) && b0 < a0 + static_cast<uintptr_t>(a_bytes);
}

}  // namespace
}  // namespace llmp_hip

using namespace llmp_hip;

extern "C" int llmp_hip_set_rows_quant_group(int count, const llmp_set_rows_store* stores, void* stream) {
  BeginLaunches();
  const char* op = "set_rows.grouped_quant";
  if (stores == nullptr) return Refuse(1, "%s: null stores", op);
  if (count < 2 || count > 16) return Refuse(1, "%s: two through sixteen stores, not %d", op, count);  // kv_quant.cc:216
  StoreGroup group{};
  int64_t most = 0;
  for (int i = 0; i < count; ++i) {
    const llmp_set_rows_store& s = stores[i];
    int64_t total = 0;
    if (const int bad = CheckStore(op, s.type, s.x, s.x_stride, s.ids, s.index_bytes, s.destination, s.row_bytes, s.k,
                                   s.rows, &total);
        bad != 0)
      return bad;
    if (s.cells <= 0) return Refuse(1, "%s: a destination of no cells", op);
    group.member[i] = StoreMember{s.x, s.ids, static_cast<uint8_t*>(s.destination), s.x_stride, s.row_bytes, total,
                                  static_cast<int>(s.k / 32), s.type, s.index_bytes};
    most = total > most ? total : most;
  }
  // No destination meets another store's destination or operands (kv_quant.cc:224-233).
  for (int i = 0; i < count; ++i) {
    const llmp_set_rows_store& a = stores[i];
    const int64_t a_bytes = a.cells * a.row_bytes;
    for (int j = 0; j < count; ++j) {
      if (i == j) continue;
      const llmp_set_rows_store& b = stores[j];
      const bool meets = (j > i && Meet(a.destination, a_bytes, b.destination, b.cells * b.row_bytes)) ||
                         Meet(a.destination, a_bytes, b.x, ((b.rows - 1) * b.x_stride + b.k) * 4) ||
                         Meet(a.destination, a_bytes, b.ids, b.rows * b.index_bytes);
      if (meets) return Refuse(1, "%s: the destination of store %d overlaps store %d's destination or operands", op, i, j);
    }
  }
  const dim3 grid(static_cast<unsigned>((most + kStoreThreads - 1) / kStoreThreads), static_cast<unsigned>(count));
  hipLaunchKernelGGL(SetRowsQuantGroupKernel, grid, dim3(kStoreThreads), 0, static_cast<hipStream_t>(stream), group);
  return LaunchStatus(op);
}

extern "C" int llmp_hip_set_rows_quant(int type, const float* x, int64_t x_stride, const void* ids, int index_bytes,
                                       void* destination, int64_t row_bytes, int64_t k, int64_t rows, int64_t cells,
                                       void* stream) {
  BeginLaunches();
  const char* op = "set_rows.quant";
  int64_t total = 0;
  if (const int bad = CheckStore(op, type, x, x_stride, ids, index_bytes, destination, row_bytes, k, rows, &total); bad != 0)
    return bad;
  if (cells <= 0) return Refuse(1, "%s: a destination of no cells", op);
  // The destination's cells meet neither the values nor the indices the launch reads.
  if (Meet(destination, cells * row_bytes, x, ((rows - 1) * x_stride + k) * 4) ||
      Meet(destination, cells * row_bytes, ids, rows * index_bytes))
    return Refuse(1, "%s: the destination overlaps the values or the indices", op);
  const dim3 grid(static_cast<unsigned>((total + kStoreThreads - 1) / kStoreThreads));
  const auto s = static_cast<hipStream_t>(stream);
  auto* out = static_cast<uint8_t*>(destination);
  if (index_bytes == 4) {
    hipLaunchKernelGGL(SetRowsQuantKernel<int32_t>, grid, dim3(kStoreThreads), 0, s, x, x_stride,
                       static_cast<const int32_t*>(ids), out, row_bytes, static_cast<int>(k / 32), total, type);
  } else {
    hipLaunchKernelGGL(SetRowsQuantKernel<int64_t>, grid, dim3(kStoreThreads), 0, s, x, x_stride,
                       static_cast<const int64_t*>(ids), out, row_bytes, static_cast<int>(k / 32), total, type);
  }
  return LaunchStatus("set_rows.quant");
}

extern "C" int llmp_hip_rope_set_rows_quant(const llmp_rope_store* store, void* stream) {
  BeginLaunches();
  const char* op = "rope.set_rows_quant";
  if (store == nullptr) return Refuse(1, "%s: null store", op);
  const llmp_rope_store& s = *store;
  if (s.x == nullptr || s.pos == nullptr || s.ids == nullptr || s.destination == nullptr)
    return Refuse(1, "%s: null operand", op);
  if (s.type != LLMP_TYPE_Q8_0 && s.type != LLMP_TYPE_Q4_0) return Refuse(1, "%s: a Q8_0 or Q4_0 destination", op);
  if (s.heads <= 0 || s.head_dim <= 0 || s.head_dim % 32 != 0 || s.tokens <= 0)
    return Refuse(1, "%s: heads of whole 32-value blocks", op);  // kv_quant.h:180-185
  if (s.n_dims <= 0 || s.n_dims % 2 != 0 || s.n_dims > s.head_dim)
    return Refuse(1, "%s: an even number of rotated dims, at most the head's %d", op, s.head_dim);
  const int64_t block_bytes = s.type == LLMP_TYPE_Q8_0 ? 34 : 18;
  const int64_t blocks_row = static_cast<int64_t>(s.heads) * (s.head_dim / 32);
  if (s.row_bytes < blocks_row * block_bytes || s.row_bytes % 2 != 0 || reinterpret_cast<uintptr_t>(s.destination) % 2 != 0)
    return Refuse(1, "%s: destination rows overlap or are not 2-byte aligned", op);
  if (s.x_head_stride < s.head_dim || s.x_token_stride < s.head_dim || reinterpret_cast<uintptr_t>(s.x) % 4 != 0)
    return Refuse(1, "%s: heads or tokens overlap", op);
  if (!(s.freq_scale > 0.0f) || !(s.theta_scale > 0.0f)) return Refuse(1, "%s: a positive frequency and angle scale", op);
  const int64_t total = s.tokens * blocks_row;
  if (total > 0xFFFFFFFFll / 32) return Refuse(1, "%s: more than 2^32 - 1 values", op);
  if (s.tokens > 0x7FFFFFFFll || s.n_dims > 8192) return Refuse(1, "%s: more than 2^31 - 1 tokens or 8192 rotated dims", op);
  hipLaunchKernelGGL(RopeSetRowsQuantKernel, dim3(static_cast<unsigned>(s.tokens)), dim3(kStoreThreads),
                     static_cast<size_t>(s.n_dims / 2) * sizeof(float2), static_cast<hipStream_t>(stream), s);
  return LaunchStatus(op);
}
