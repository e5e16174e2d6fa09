// The routed-expert operations around llmp.vecq for gfx950: the router (softmax, top-k,
// renormalized weights), the expert grouping of (token, slot) pairs, the gathering Q8_1
// quantizer of the sorted rows, and the ordered weighted combine. All deterministic: fixed
// summation orders, no atomics on results.
//
// Reference behaviour restated here: src/kernels/reference/exec.cc:279-315,1728-1856
// (route and reduce definitions), src/kernels/ggml/llmp_fused.cu:1307-1407 (router kernel),
// :200-240 (combine), src/kernels/ggml/llmp_moe.cu:81-163 (grouping), :390-427 (sorted
// combine), src/kernels/ggml/moe_layout.h:46-70 (the route buffer).

#include <hip/hip_runtime.h>

#include "common.h"
#include "llmp_hip.h"
#include "moe_router.h"
#include "vecq_common.h"

namespace llmp_hip {
namespace {

constexpr int kRouterWaves = 4;
constexpr int kRouterSlots = 16;  // experts / 64 at most: up to 1024 experts
constexpr int kRouteChunk = 64;   // tokens a counting workgroup (moe_layout.h kRouteChunk)
constexpr int kScaleRows = 128;   // moe_layout.h kScaleRows

// A token a wave (moe_router.h).
template <int SLOTS>
__global__ __launch_bounds__(kRouterWaves* kWave) void RouterKernel(const float* __restrict__ logits,
                                                                   int32_t* __restrict__ ids,
                                                                   float* __restrict__ weights, int tokens, int experts,
                                                                   int used, int normalize, float scale) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t t = static_cast<int64_t>(blockIdx.x) * kRouterWaves + threadIdx.x / kWave;
  if (t >= tokens) return;  // whole waves
  int my_index = 0;
  float my_weight = 0.0f;
  RouteToken<SLOTS>(logits + t * experts, experts, used, normalize, scale, lane, &my_index, &my_weight);
  if (lane < used) {
    ids[t * used + lane] = my_index;
    weights[t * used + lane] = my_weight;
  }
}

// ---------------------------------------------------------------- grouping

struct Route {
  int32_t* offsets;
  int32_t* scale_rows;
  int32_t* position;
  int32_t* token;
  int32_t* expert;
  int32_t* counts;
  int experts, used, tokens, chunks;
};

// Each workgroup counts its chunk's ids per expert: one thread an expert, the chunk's slots
// in order (no atomics: a thread owns its counter).
// The chunk's ids into LDS (chunk tokens x used ints): every thread then walks all of them.
__device__ __forceinline__ int StageChunkIds(const int32_t* __restrict__ ids, int ids_stride, const Route& r, int t0,
                                             int t1, int32_t* staged) {
  const int n = (t1 - t0) * r.used;
  for (int i = threadIdx.x; i < n; i += blockDim.x)
    staged[i] = ids[static_cast<int64_t>(t0 + i / r.used) * ids_stride + i % r.used];
  // Padded to whole groups of four with an id nothing equals: the walks read four at a time.
  if (threadIdx.x < 4 && n + threadIdx.x < ((n + 3) & ~3)) staged[n + threadIdx.x] = INT32_MIN;
  __syncthreads();
  return n;
}

// How many of staged[0 .. end) equal e, four ids a read (end a multiple of four, or the padded
// count).
__device__ __forceinline__ int CountEqual(const int32_t* staged, int end, int e) {
  const int4* four = reinterpret_cast<const int4*>(staged);
  int n = 0;
#pragma unroll 4
  for (int i = 0; i < end / 4; ++i) {
    const int4 v = four[i];
    n += (v.x == e) + (v.y == e) + (v.z == e) + (v.w == e);
  }
  return n;
}

__global__ void RouteCount(const int32_t* __restrict__ ids, int ids_stride, Route r) {
  extern __shared__ __attribute__((aligned(16))) int32_t staged[];
  const int c = blockIdx.x;
  const int t0 = c * kRouteChunk;
  const int t1 = min(t0 + kRouteChunk, r.tokens);
  const int slots = StageChunkIds(ids, ids_stride, r, t0, t1, staged);
  for (int e = threadIdx.x; e < r.experts; e += blockDim.x)
    r.counts[static_cast<int64_t>(c) * r.experts + e] = CountEqual(staged, (slots + 3) & ~3, e);
}

// One workgroup: each expert's chunk counts become the chunks' bases, then the experts'
// offsets and scale rows.
__global__ void RouteScan(Route r) {
  extern __shared__ int total[];
  for (int e = threadIdx.x; e < r.experts; e += blockDim.x) {
    int running = 0;
    // Eight chunks' counts in flight at a time (a load after a store to the same array would
    // otherwise wait for it).
    for (int c0 = 0; c0 < r.chunks; c0 += 8) {
      int v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        v[u] = r.counts[static_cast<int64_t>(min(c0 + u, r.chunks - 1)) * r.experts + e];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (c0 + u < r.chunks) {
          r.counts[static_cast<int64_t>(c0 + u) * r.experts + e] = running;
          running += v[u];
        }
      }
    }
    total[e] = running;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int offset = 0, scale_row = 0;
    r.offsets[0] = 0;
    r.scale_rows[0] = 0;
    for (int e = 0; e < r.experts; ++e) {
      offset += total[e];
      scale_row += (total[e] + kScaleRows - 1) / kScaleRows * kScaleRows;
      r.offsets[e + 1] = offset;
      r.scale_rows[e + 1] = scale_row;
    }
  }
}

// Each workgroup places its chunk's slots, one thread a slot: the slot's row is its expert's
// first row, plus the expert's slots in earlier chunks, plus those before it in this chunk
// (token order, then slot order: every thread walks the staged ids before its own).
__global__ void RouteAssign(const int32_t* __restrict__ ids, int ids_stride, Route r) {
  extern __shared__ __attribute__((aligned(16))) int32_t staged[];
  const int c = blockIdx.x;
  const int t0 = c * kRouteChunk;
  const int t1 = min(t0 + kRouteChunk, r.tokens);
  const int slots = StageChunkIds(ids, ids_stride, r, t0, t1, staged);
  for (int i = threadIdx.x; i < slots; i += blockDim.x) {
    const int e = staged[i];
    if (e < 0 || e >= r.experts) {  // ids outside the experts have no row
      r.position[t0 * r.used + i] = -1;
      continue;
    }
    int before = CountEqual(staged, i & ~3, e);
    for (int j = i & ~3; j < i; ++j) before += staged[j] == e;
    const int row = r.offsets[e] + r.counts[static_cast<int64_t>(c) * r.experts + e] + before;
    r.position[t0 * r.used + i] = row;
    r.token[row] = t0 + i / r.used;
    r.expert[row] = e;
  }
}

// The whole grouping by one workgroup, for problems whose ids and per-run counters fit LDS
// (up to 8192 slots and runs x experts up to 8192): the slots are cut into runs of 64 in slot
// order; a run's ids are counted per expert with LDS integer atomics (a count does not depend
// on their order), a thread an expert turns the runs' counts into bases, one thread the
// experts' totals into offsets, and a thread a slot then takes its expert's first row, plus
// its run's base, plus the equal ids before it in its run (at most 63 compares).
// LDS: the ids, padded to fours; runs x experts counters; experts + 1 offsets.
constexpr int kRouteOneSlots = 8192;
constexpr int kRouteOneCounters = 8192;
constexpr int kRouteOneThreads = 1024;

__global__ __launch_bounds__(kRouteOneThreads) void RouteOne(const int32_t* __restrict__ ids, int ids_stride, Route r) {
  extern __shared__ __attribute__((aligned(16))) int32_t staged[];
  const int slots = r.tokens * r.used;
  const int runs = (slots + 63) / 64;
  int32_t* counters = staged + ((slots + 3) & ~3);  // [run][expert]
  int32_t* offsets = counters + runs * r.experts;    // [expert + 1]
  const int tid = threadIdx.x;
  for (int i = tid; i < slots; i += kRouteOneThreads) staged[i] = ids[static_cast<int64_t>(i / r.used) * ids_stride + i % r.used];
  if (tid < 4 && slots + tid < ((slots + 3) & ~3)) staged[slots + tid] = INT32_MIN;
  for (int i = tid; i < runs * r.experts; i += kRouteOneThreads) counters[i] = 0;
  __syncthreads();
  for (int i = tid; i < slots; i += kRouteOneThreads) {
    const int e = staged[i];
    if (e >= 0 && e < r.experts) atomicAdd(&counters[(i / 64) * r.experts + e], 1);
  }
  __syncthreads();
  for (int e = tid; e < r.experts; e += kRouteOneThreads) {
    int running = 0;
    // Sixteen runs' counts read together (a read after a write to the same array would
    // otherwise wait for it), then their bases written.
    for (int run0 = 0; run0 < runs; run0 += 16) {
      int v[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) v[u] = counters[min(run0 + u, runs - 1) * r.experts + e];
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        if (run0 + u < runs) {
          counters[(run0 + u) * r.experts + e] = running;
          running += v[u];
        }
      }
    }
    offsets[e + 1] = running;  // the expert's total, for now
  }
  __syncthreads();
  // The experts' totals into offsets: each lane of the first wave a block of consecutive
  // experts, the blocks' sums scanned across the wave.
  if (tid < kWave) {
    const int per = (r.experts + kWave - 1) / kWave;
    const int e0 = min(tid * per, r.experts), e1 = min(e0 + per, r.experts);
    int rows = 0, scale_rows = 0;
    for (int e = e0; e < e1; ++e) {
      const int total = offsets[e + 1];
      rows += total;
      scale_rows += (total + kScaleRows - 1) / kScaleRows * kScaleRows;
    }
    int rows_before = rows, scale_before = scale_rows;  // inclusive scans
#pragma unroll
    for (int step = 1; step < kWave; step <<= 1) {
      const int a = __shfl_up(rows_before, step, kWave);
      const int b = __shfl_up(scale_before, step, kWave);
      if (tid >= step) rows_before += a, scale_before += b;
    }
    int offset = rows_before - rows, scale_row = scale_before - scale_rows;
    if (tid == 0) {
      offsets[0] = 0;
      r.offsets[0] = 0;
      r.scale_rows[0] = 0;
    }
    for (int e = e0; e < e1; ++e) {
      const int total = offsets[e + 1];
      offset += total;
      scale_row += (total + kScaleRows - 1) / kScaleRows * kScaleRows;
      offsets[e + 1] = offset;
      r.offsets[e + 1] = offset;
      r.scale_rows[e + 1] = scale_row;
    }
  }
  __syncthreads();
  for (int i = tid; i < slots; i += kRouteOneThreads) {
    const int e = staged[i];
    if (e < 0 || e >= r.experts) {  // ids outside the experts have no row
      r.position[i] = -1;
      continue;
    }
    const int run0 = i & ~63;
    int before = CountEqual(staged + run0, (i - run0) & ~3, e);
    for (int j = i & ~3; j < i; ++j) before += staged[j] == e;
    const int row = offsets[e] + counters[(i / 64) * r.experts + e] + before;
    r.position[i] = row;
    r.token[row] = i / r.used;
    r.expert[row] = e;
  }
}

// ------------------------------------------------------- gathering quantizer

// Output row r is the Q8_1 of input row rows[r] (or r): eight lanes a block.
__global__ __launch_bounds__(kThreads) void QuantizeGatherKernel(const float* __restrict__ x,
                                                                const int32_t* __restrict__ rows,
                                                                uint8_t* __restrict__ out, int64_t k, int64_t padded_k,
                                                                int64_t row_stride) {
  const int lane8 = threadIdx.x & 7;
  const int64_t block = static_cast<int64_t>(blockIdx.x) * 32 + (threadIdx.x >> 3);
  const int64_t blocks = padded_k / 32;
  if (block >= blocks) return;  // whole 8-lane groups
  const int64_t r = blockIdx.y;
  const int64_t source = rows != nullptr ? rows[r] : r;
  float v[4];
  Load4<LLMP_X_F32>(x + source * row_stride, block * 32 + lane8 * 4, k, v);
  const Q8Block q = QuantizeQ8Block(v[0], v[1], v[2], v[3]);
  uint8_t* dst = out + (r * blocks + block) * kQ8Block;
  *reinterpret_cast<uint32_t*>(dst + 4 + lane8 * 4) = q.codes;
  if (lane8 == 0) *reinterpret_cast<uint32_t*>(dst) = FloatToHalfBits(q.d) | (FloatToHalfBits(q.sum) << 16);
}

// ------------------------------------------------------------------ combine

// out[t] = sum_j x[row(t, j)] * w[t, j] in slot order, the first term assigned: four columns
// a thread. row(t, j) is t * used + j, or position[t * used + j] for sorted rows (a negative
// position contributes nothing).
__global__ void CombineKernel(const float4* __restrict__ x, const float* __restrict__ weights,
                              const int32_t* __restrict__ position, float4* __restrict__ out, int width4, int used,
                              int64_t total4) {
#pragma clang fp contract(off)
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total4) return;
  const int64_t t = i / width4;
  const int64_t c4 = i % width4;
  float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  bool first = true;
  // Eight slots' loads in flight at a time; the terms are still added in slot order.
  for (int j0 = 0; j0 < used; j0 += 8) {
    int64_t row[8];
    float w[8];
    float4 d[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int j = min(j0 + u, used - 1);
      row[u] = t * used + j;
      w[u] = weights[row[u]];
      if (position != nullptr) row[u] = position[row[u]];
      if (j0 + u >= used) row[u] = -1;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) d[u] = x[max(row[u], int64_t{0}) * width4 + c4];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (row[u] < 0) continue;
      const float4 e = make_float4(d[u].x * w[u], d[u].y * w[u], d[u].z * w[u], d[u].w * w[u]);
      acc = first ? e : make_float4(acc.x + e.x, acc.y + e.y, acc.z + e.z, acc.w + e.w);
      first = false;
    }
  }
  out[i] = acc;
}

Route RouteOf(int32_t* base, int experts, int used, int tokens) {
  const int64_t slots = static_cast<int64_t>(used) * tokens;
  const int chunks = (tokens + kRouteChunk - 1) / kRouteChunk;
  Route r;
  r.offsets = base;
  r.scale_rows = base + experts + 1;
  r.position = base + 2 * (experts + 1);
  r.token = r.position + slots;
  r.expert = r.token + slots;
  r.counts = r.expert + slots;
  r.experts = experts;
  r.used = used;
  r.tokens = tokens;
  r.chunks = chunks;
  return r;
}

}  // namespace
}  // namespace llmp_hip

using namespace llmp_hip;

extern "C" int llmp_hip_moe_router(const float* logits, int experts, int used, int tokens, int normalize, float scale,
                                   int32_t* ids, float* weights, void* stream) {
  BeginLaunches();
  if (logits == nullptr || ids == nullptr || weights == nullptr) return Refuse(1, "moe.router: null operand");
  if (experts < 1 || experts > kRouterSlots * kWave) return Refuse(1, "moe.router: 1 to %d experts", kRouterSlots * kWave);
  if (used < 1 || used > experts || used > kWave) return Refuse(1, "moe.router: 1 to min(experts, 64) picks, not %d", used);
  if (tokens < 1) return Refuse(1, "moe.router: no tokens");
  const dim3 grid(static_cast<unsigned>((tokens + kRouterWaves - 1) / kRouterWaves));
  const auto s = static_cast<hipStream_t>(stream);
  const dim3 block(kRouterWaves * kWave);
  if (experts <= 2 * kWave) {
    hipLaunchKernelGGL(RouterKernel<2>, grid, block, 0, s, logits, ids, weights, tokens, experts, used, normalize, scale);
  } else if (experts <= 4 * kWave) {
    hipLaunchKernelGGL(RouterKernel<4>, grid, block, 0, s, logits, ids, weights, tokens, experts, used, normalize, scale);
  } else if (experts <= 8 * kWave) {
    hipLaunchKernelGGL(RouterKernel<8>, grid, block, 0, s, logits, ids, weights, tokens, experts, used, normalize, scale);
  } else {
    hipLaunchKernelGGL(RouterKernel<kRouterSlots>, grid, block, 0, s, logits, ids, weights, tokens, experts, used,
                       normalize, scale);
  }
  return LaunchStatus("moe.router");
}

extern "C" int64_t llmp_hip_moe_route_ints(int experts, int used, int tokens) {
  const int64_t slots = static_cast<int64_t>(used) * tokens;
  const int64_t chunks = (tokens + kRouteChunk - 1) / kRouteChunk;
  return 2 * (static_cast<int64_t>(experts) + 1) + 3 * slots + chunks * experts;
}

extern "C" int llmp_hip_moe_route(const int32_t* ids, int ids_stride, int experts, int used, int tokens,
                                  int32_t* route, void* stream) {
  BeginLaunches();
  if (ids == nullptr || route == nullptr) return Refuse(1, "moe.route: null operand");
  if (experts < 1 || used < 1 || tokens < 1 || ids_stride < used) return Refuse(1, "moe.route: empty or overlapping ids");
  if (used > 128) return Refuse(1, "moe.route: more than 128 slots a token");  // a chunk's ids are staged in LDS
  if (static_cast<int64_t>(used) * tokens > (1 << 24)) return Refuse(1, "moe.route: more than 2^24 slots");
  const Route r = RouteOf(route, experts, used, tokens);
  const auto s = static_cast<hipStream_t>(stream);
  const int64_t slots = static_cast<int64_t>(used) * tokens;
  const int64_t runs = (slots + 63) / 64;
  if (slots <= kRouteOneSlots && runs * experts <= kRouteOneCounters) {
    const size_t bytes = static_cast<size_t>(((slots + 3) & ~int64_t{3}) + runs * experts + experts + 1) * sizeof(int32_t);
    static bool sized = false;  // more than 64 KB of dynamic LDS must be asked for once
    if (!AllowLds(reinterpret_cast<const void*>(&RouteOne), (kRouteOneSlots + kRouteOneCounters + kRouteOneCounters + 4) * 4, &sized))
      return LaunchStatus("moe.route");
    hipLaunchKernelGGL(RouteOne, dim3(1), dim3(kRouteOneThreads), bytes, s, ids, ids_stride, r);
    return LaunchStatus("moe.route");
  }
  const int threads = experts < 256 ? (experts + 63) / 64 * 64 : 256;
  const size_t chunk_bytes = (static_cast<size_t>(kRouteChunk) * used + 4) * sizeof(int32_t);  // padded to fours
  hipLaunchKernelGGL(RouteCount, dim3(r.chunks), dim3(threads), chunk_bytes, s, ids, ids_stride, r);
  if (const int bad = LaunchStatus("moe.route count"); bad != 0) return bad;
  hipLaunchKernelGGL(RouteScan, dim3(1), dim3(threads), static_cast<size_t>(experts) * sizeof(int), s, r);
  hipLaunchKernelGGL(RouteAssign, dim3(r.chunks), dim3(256), chunk_bytes, s, ids, ids_stride, r);
  return LaunchStatus("moe.route");
}

extern "C" int llmp_hip_q8_1_quantize_rows(const float* x, const int32_t* rows, void* out, int64_t k, int64_t padded_k,
                                           int64_t row_stride, int64_t count, void* stream) {
  BeginLaunches();
  if (x == nullptr || out == nullptr) return Refuse(1, "q8_1: null operand");
  if (k <= 0 || count <= 0 || count > 65535) return Refuse(1, "q8_1: 1 to 65535 rows");
  if (padded_k < k || padded_k % 32 != 0) return Refuse(1, "q8_1: padded k below k or not whole blocks");
  const dim3 grid(static_cast<unsigned>((padded_k / 32 + 31) / 32), static_cast<unsigned>(count));
  hipLaunchKernelGGL(QuantizeGatherKernel, grid, dim3(kThreads), 0, static_cast<hipStream_t>(stream), x, rows,
                     static_cast<uint8_t*>(out), k, padded_k, row_stride);
  return LaunchStatus("q8_1 rows");
}

extern "C" int llmp_hip_moe_combine(const float* x, const float* weights, const int32_t* position, int width, int used,
                                    int tokens, float* out, void* stream) {
  BeginLaunches();
  if (x == nullptr || weights == nullptr || out == nullptr) return Refuse(1, "moe.combine: null operand");
  if (width < 4 || width % 4 != 0 || used < 1 || tokens < 1) return Refuse(1, "moe.combine: width a multiple of 4");
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) % 16 != 0)
    return Refuse(1, "moe.combine: operands not 16-byte aligned");
  const int64_t total4 = static_cast<int64_t>(tokens) * (width / 4);
  hipLaunchKernelGGL(CombineKernel, dim3(static_cast<unsigned>((total4 + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), reinterpret_cast<const float4*>(x), weights, position,
                     reinterpret_cast<float4*>(out), width / 4, used, total4);
  return LaunchStatus("moe.combine");
}
