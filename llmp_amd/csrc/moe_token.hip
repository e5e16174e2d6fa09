// One token through a routed-expert FFN layer in one launch (Q4_K experts): the router, the picked experts' gate/up
// products with their GLU, the down products and the ordered weighted sum, which the reference runs as separate
// operations (src/ir/decompose.cc:1080-1109: kRoute, kMatMulId, kGlu, kMatMulId, kExpertReduce) and this library's
// llmp_hip_moe_router / llmp_hip_vecq_fused (twice) / llmp_hip_moe_combine run as four launches. At one token the layer
// streams 21 MB and every launch is a latency chain of 4 to 8 us; here the chain is paid once.
//
// A workgroup a compute unit, eight waves. Every workgroup routes the token itself (its first wave, the router's own
// arithmetic: moe_router.h) and stages the token's Q8_1 records, so nothing waits for another workgroup before the
// first weights are asked for. First phase: a wave a tile of four rows of an expert's gate and up matrices, llmp.vecq's
// flat form (vecq_flat.h: the same tile, products, row sums and GLU, so the same bits), its h values to device memory.
// Between the phases the grid meets at words in device memory; a wave's tile of the down matrix is asked for
// before it waits there (it needs the expert, not h). Second phase: a workgroup's waves are the token's slots, each
// with its expert's rows of the down matrix for the same outputs and its own slot's h quantized into its own records;
// their sums meet in LDS and one thread an output adds them in slot order, the first term assigned, as
// llmp_hip_moe_combine does.
//
// The meeting. h and the meeting's words are written and read with agent-scope relaxed atomic operations, which reach memory
// past the XCDs' L2s; a wave waits for its h stores to be acknowledged before its workgroup counts itself in; nothing
// is fenced (a fence at agent scope writes back or empties an XCD's L2: hundreds of them cost more than the launches
// saved). Every workgroup keeps a word of its own with the number of meetings it has come to, adds one when it
// arrives, and its first wave reads all the words until they agree: launches and graph replays follow each other
// without a reset by the host, as long as they use the same grid. Every workgroup of the grid must be resident at
// once (one a compute unit: the grid is never larger); the poll is bounded, and a workgroup that gives up sets an error word and goes on (wrong results, no hang).
// `phase` 1 and 2 run the two halves as two launches with the launch boundary in place of the meeting: on an MI355X
// that is the faster form (16.7 us against 19.3; a store and a load at agent scope each take a microsecond or two to
// cross the device, a launch boundary about 2.5 us in all), so it is what callers get by default.
#include "moe_router.h"
#include "vecq_flat.h"

namespace llmp_hip {
namespace {

constexpr int kTokenWaves = 8;
constexpr int kTokenThreads = kTokenWaves * kWave;
constexpr int kPollLimit = 1 << 16;

struct MoeTokenArgs {
  llmp_moe_token d;
  int phase;  // 0: both phases, meeting in between; 1, 2: one of them
  int rows_a, rows_b, tiles_a, tiles_b;
};

__device__ __forceinline__ void StoreShared(float* at, float v) {
  __hip_atomic_store(reinterpret_cast<uint32_t*>(at), __builtin_bit_cast(uint32_t, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float LoadShared(const float* at) {
  return __builtin_bit_cast(float, __hip_atomic_load(reinterpret_cast<const uint32_t*>(at), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}

template <int SLOTS, int XT>
__global__ __launch_bounds__(kTokenThreads, 1) void MoeTokenKernel(const MoeTokenArgs a) {
  using F = FormatQ4K;
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  __shared__ int picked[kWave];
  __shared__ float picked_weight[kWave];
  __shared__ uint32_t generation;
  const llmp_moe_token& d = a.d;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int nsb_a = d.hidden / 256, nsb_b = d.ffn / 256;
  uint32_t* const words = static_cast<uint32_t*>(d.sync);  // word 2: a workgroup gave up; from word 4: a word a workgroup

  // LDS: the token's records (first phase), or a record area a wave (second phase); then a tile buffer a wave; then
  // the slots' sums of a tile of outputs.
  const int records_a = nsb_a * F::kRecord, records_b = kTokenWaves * nsb_b * F::kRecord;
  const int records = ((records_a > records_b ? records_a : records_b) + 15) & ~15;
  uint8_t* const ring = lds + records + wave * (kWave * F::kUnitBytes);
  float* const meet = reinterpret_cast<float*>(lds + records + kTokenWaves * (kWave * F::kUnitBytes));  // [slot][row of the tile]

  constexpr int kHeldSweeps = 4;
  FrontWords held[kHeldSweeps];
  const bool h_ahead = a.phase == 2 && d.ffn / 32 <= kHeldSweeps * (kWave >> 3);
  // ---- the token's experts: routed here, or (second launch of two) read back.
  if (a.phase != 2) {
    if (tid == 0) generation = __hip_atomic_load(words + 4 + blockIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (wave == 0) {
      int index = 0;
      float weight = 0.0f;
      RouteToken<SLOTS>(d.logits, d.experts, d.used, d.normalize, d.route_scale, lane, &index, &weight);
      if (lane < d.used) {
        picked[lane] = index;
        picked_weight[lane] = weight;
        if (blockIdx.x == 0) {
          d.ids[lane] = index;
          d.weights[lane] = weight;
        }
      }
    }
  } else {
    // The second launch of two: a wave's slot's h (the launch before wrote it) is asked for here, ahead of the
    // picks' loads (one trip to memory for both) and of the tile's, by instructions; quantized after the tile's
    // loads are queued, with its records written by instructions, it no longer waits for the tile to land and
    // then for a trip to memory a sweep (the compiler holds a write to LDS back while a load into LDS is in flight,
    // so every sweep's loads waited for the one before). Rows of up to kHeldSweeps x 8 blocks.
    // (One straight run of instructions from the loads to their wait, every lane taking part with its index held
    // within bounds: a branch between them gave the compiler a place to copy the registers before the data was
    // there, which the build's check of the assembly refuses.)
    const int slot = min(wave, d.used - 1);
#pragma unroll
    for (int i = 0; i < kHeldSweeps; ++i) {
      const int b = min((lane >> 3) + i * (kWave >> 3), d.ffn / 32 - 1);
      const float* from = d.h + slot * d.ffn + b * 32 + (lane & 7) * 4;
      asm volatile("global_load_dwordx4 %0, %1, off" : "=&v"(held[i]) : "v"(from) : "memory");
    }
    uint32_t pick, pick_weight;
    {
      const int32_t* from_ids = d.ids + min(tid, d.used - 1);
      const float* from_weights = d.weights + min(tid, d.used - 1);
      asm volatile("global_load_dword %0, %1, off" : "=&v"(pick) : "v"(from_ids) : "memory");
      asm volatile("global_load_dword %0, %1, off" : "=&v"(pick_weight) : "v"(from_weights) : "memory");
    }
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+v"(held[0]), "+v"(held[1]), "+v"(held[2]), "+v"(held[3]), "+v"(pick), "+v"(pick_weight)
                 :
                 : "memory");
    if (tid < d.used) {
      picked[tid] = static_cast<int>(pick);
      picked_weight[tid] = __builtin_bit_cast(float, pick_weight);
    }
  }
  if (a.phase != 2) {
    // ---- first phase: the token's records, then h = GLU(gate x, up x) of every slot.
    const FrontX front = LoadFrontX<XT>(d.x, d.hidden);
    __syncthreads();  // the picks are known
    const int waves_all = gridDim.x * kTokenWaves;
    const int first_tile = blockIdx.x * kTokenWaves + wave;
    const int tiles_a_expert = (d.ffn + a.rows_a - 1) / a.rows_a;
    const int half = a.rows_a * nsb_a;
    const bool gate_lane = lane >= half;
    const int f = gate_lane ? lane - half : lane;
    const int row = f / nsb_a, sb = f - row * nsb_a;
    const bool placed = lane < 2 * half;
    const int gate_at = half * F::kUnitBytes;
    const uint8_t* my_block = ring + (gate_lane ? gate_at + f * F::kUnitBytes : lane * F::kUnitBytes);
    llmp_vecq_desc tile_of;  // what FetchTile reads: the two matrices and their rows' pitch
    tile_of.g = d.gate_up;
    tile_of.w = static_cast<const uint8_t*>(d.gate_up) + static_cast<int64_t>(d.ffn) * nsb_a * F::kBlockBytes;
    tile_of.stride_row = nsb_a;
    auto fetch_a = [&](int tile) {
      const int slot = tile / tiles_a_expert, row0 = (tile - slot * tiles_a_expert) * a.rows_a;
      FetchTile<F, true, true>(tile_of, static_cast<int64_t>(picked[slot]) * d.gate_up_stride, row0, min(a.rows_a, d.ffn - row0), nsb_a, gate_at,
                               ring, lane);
    };
    if (first_tile < a.tiles_a) fetch_a(first_tile);
    StageRecordsX<F, XT>(d.x, d.hidden, front, lds);
    __syncthreads();  // the records are staged
    for (int tile = first_tile; tile < a.tiles_a; tile += waves_all) {
      const int slot = tile / tiles_a_expert, row0 = (tile - slot * tiles_a_expert) * a.rows_a;
      const bool live = placed && row0 + row < d.ffn;
      AwaitTile();
      float out[1];
      if (live) F::template DotAt<1, false>(my_block, lds + sb * F::kRecord, records_a, 1, out, nullptr);
      float v = live ? out[0] : 0.0f;
      for (int off = 1; off < nsb_a; off <<= 1) {
        const float other = __shfl_down(v, off, kWave);
        if (sb + off < nsb_a) v += other;
      }
      const float gate = __shfl_down(v, half, kWave);
      if (live && !gate_lane && sb == 0) StoreShared(d.h + slot * d.ffn + row0 + row, Glu(d.glu, gate, v, d.limit));
      __builtin_amdgcn_wave_barrier();
      if (tile + waves_all < a.tiles_a) fetch_a(tile + waves_all);
    }
    if (a.phase == 1) return;
    // The wave's h values have reached memory before its workgroup is counted in.
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
  } else {
    __syncthreads();  // the picks are read
  }

  // ---- second phase: out = sum over the slots of (down h) * weight, in slot order.
  const int row_b = lane / nsb_b, sb_b = lane - row_b * nsb_b;
  const bool placed_b = lane < a.rows_b * nsb_b && wave < d.used;
  llmp_vecq_desc down_of;
  down_of.w = d.down;
  down_of.g = nullptr;
  down_of.stride_row = nsb_b;
  auto fetch_b = [&](int tile) {
    const int row0 = tile * a.rows_b;
    if (wave < d.used)
      FetchTile<F, false, true>(down_of, static_cast<int64_t>(picked[wave]) * d.down_stride, row0, min(a.rows_b, d.hidden - row0), nsb_b, 0, ring, lane);
  };
  if (static_cast<int>(blockIdx.x) < a.tiles_b) fetch_b(blockIdx.x);  // on its way while the grid meets
  if (a.phase == 0) {
    __syncthreads();  // every wave's h is in memory
    // The meeting: a word a workgroup that holds the number of meetings it has come to. A workgroup adds one to its
    // own (a store: nothing is read, modified and written at one address by 256 workgroups in turn, which alone took
    // 5 us) and its first wave reads all the words until every one holds that number.
    const uint32_t mine = generation + 1;
    if (tid == 0) __hip_atomic_store(words + 4 + blockIdx.x, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (wave == 0) {
      int polls = 0;
      for (;;) {
        bool all = true;
        for (int j = lane; j < static_cast<int>(gridDim.x); j += kWave)
          all = all && __hip_atomic_load(words + 4 + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == mine;
        if (__all(all)) break;
        if (++polls > kPollLimit) {
          if (lane == 0) __hip_atomic_store(words + 2, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          break;
        }
        __builtin_amdgcn_s_sleep(4);
      }
    }
    __syncthreads();
  }
  // This wave's slot's h into its own records: eight lanes a block, the quantizer of llmp.q8_1.
  uint8_t* const my_records = lds + wave * (nsb_b * F::kRecord);
  if (h_ahead && wave < d.used) {
#pragma unroll
    for (int i = 0; i < kHeldSweeps; ++i) {
      const int b = (lane >> 3) + i * (kWave >> 3);
      if (b < d.ffn / 32) {  // whole 8-lane groups together
        const uint32_t x0 = held[i].x, x1 = held[i].y, x2 = held[i].z, x3 = held[i].w;
        const float v[4] = {__builtin_bit_cast(float, x0), __builtin_bit_cast(float, x1), __builtin_bit_cast(float, x2),
                            __builtin_bit_cast(float, x3)};
        F::StageXAsm(v, b, my_records);
      }
    }
  } else if (wave < d.used) {
    const float* from = d.h + wave * d.ffn;
    for (int b = lane >> 3; b < d.ffn / 32; b += kWave >> 3) {
      float v[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) v[c] = LoadShared(from + b * 32 + (lane & 7) * 4 + c);
      F::StageX(v, b, my_records);
    }
  }
  __builtin_amdgcn_wave_barrier();
  for (int tile = blockIdx.x; tile < a.tiles_b; tile += gridDim.x) {
    const int row0 = tile * a.rows_b;
    const int rows = min(a.rows_b, d.hidden - row0);
    const bool live = placed_b && row_b < rows;
    AwaitTile();
    float out[1];
    if (live) F::template DotAt<1, false>(ring + lane * F::kUnitBytes, my_records + sb_b * F::kRecord, 0, 1, out, nullptr);
    float v = live ? out[0] : 0.0f;
    for (int off = 1; off < nsb_b; off <<= 1) {
      const float other = __shfl_down(v, off, kWave);
      if (sb_b + off < nsb_b) v += other;
    }
    if (live && sb_b == 0) meet[wave * a.rows_b + row_b] = v;
    __syncthreads();
    if (tid < rows) {
#pragma clang fp contract(off)
      float acc = meet[tid] * picked_weight[0];
      for (int u = 1; u < d.used; ++u) acc = acc + meet[u * a.rows_b + tid] * picked_weight[u];
      d.out[row0 + tid] = acc;
    }
    __syncthreads();  // the sums are read before the next tile's are written
    if (tile + static_cast<int>(gridDim.x) < a.tiles_b) fetch_b(tile + gridDim.x);
  }
}

template <int XT>
void LaunchToken(const MoeTokenArgs& a, int groups, size_t lds, hipStream_t stream) {
  const dim3 grid(static_cast<unsigned>(groups)), block(kTokenThreads);
  static bool sized[3] = {false, false, false};
  const int experts = a.d.experts;
  if (experts <= 2 * kWave) {
    if (!AllowLds(reinterpret_cast<const void*>(&MoeTokenKernel<2, XT>), static_cast<int>(kDeepLdsLimit), &sized[0])) return;
    hipLaunchKernelGGL((MoeTokenKernel<2, XT>), grid, block, lds, stream, a);
  } else if (experts <= 4 * kWave) {
    if (!AllowLds(reinterpret_cast<const void*>(&MoeTokenKernel<4, XT>), static_cast<int>(kDeepLdsLimit), &sized[1])) return;
    hipLaunchKernelGGL((MoeTokenKernel<4, XT>), grid, block, lds, stream, a);
  } else {
    if (!AllowLds(reinterpret_cast<const void*>(&MoeTokenKernel<16, XT>), static_cast<int>(kDeepLdsLimit), &sized[2])) return;
    hipLaunchKernelGGL((MoeTokenKernel<16, XT>), grid, block, lds, stream, a);
  }
}

}  // namespace
}  // namespace llmp_hip

using namespace llmp_hip;

extern "C" size_t llmp_hip_moe_token_scratch(const llmp_moe_token* op) {
  if (op == nullptr || op->used < 1 || op->ffn < 1) return 0;
  return static_cast<size_t>(op->used) * op->ffn * sizeof(float);
}

extern "C" int llmp_hip_moe_token(const llmp_moe_token* op, int launches, int cus, void* stream) {
  BeginLaunches();
  if (op == nullptr) return Refuse(1, "moe.token: null operands");
  if (op->type != LLMP_TYPE_Q4_K) return Refuse(1, "moe.token: Q4_K experts, not type %d", op->type);
  if (op->logits == nullptr || op->x == nullptr || op->gate_up == nullptr || op->down == nullptr || op->out == nullptr ||
      op->ids == nullptr || op->weights == nullptr || op->h == nullptr || op->sync == nullptr)
    return Refuse(1, "moe.token: null operand");
  if (op->x_type != LLMP_X_F32 && op->x_type != LLMP_X_BF16) return Refuse(1, "moe.token: F32 or BF16 activations");
  if (op->experts < 1 || op->experts > 1024 || op->used < 1 || op->used > kTokenWaves || op->used > op->experts)
    return Refuse(1, "moe.token: up to 1024 experts and %d picks (a pick a wave), not %d and %d", kTokenWaves, op->experts, op->used);
  if (op->hidden < 256 || op->hidden % 256 != 0 || op->hidden > 8192 || op->ffn < 256 || op->ffn % 256 != 0 || op->ffn > 16384)
    return Refuse(1, "moe.token: hidden in whole super-blocks up to 8192 and ffn up to 16384, not %d and %d", op->hidden, op->ffn);
  if (op->glu != LLMP_GLU_SWIGLU && op->glu != LLMP_GLU_SWIGLU_CLAMP && op->glu != LLMP_GLU_GEGLU) return Refuse(1, "moe.token: a GLU");
  if (launches != 1 && launches != 2) return Refuse(1, "moe.token: one launch or two, not %d", launches);
  if ((reinterpret_cast<uintptr_t>(op->gate_up) | reinterpret_cast<uintptr_t>(op->down) | reinterpret_cast<uintptr_t>(op->x)) % 16 != 0 ||
      (reinterpret_cast<uintptr_t>(op->h) | reinterpret_cast<uintptr_t>(op->out) | reinterpret_cast<uintptr_t>(op->sync)) % 16 != 0)
    return Refuse(1, "moe.token: operands at 16-byte boundaries");
  if (op->gate_up_stride < static_cast<int64_t>(2) * op->ffn * (op->hidden / 256) || op->down_stride < static_cast<int64_t>(op->hidden) * (op->ffn / 256))
    return Refuse(1, "moe.token: an expert's stride holds its matrices");
  MoeTokenArgs a;
  a.d = *op;
  const int nsb_a = op->hidden / 256, nsb_b = op->ffn / 256;
  const int groups = cus > 0 ? cus : 256;
  a.rows_a = kWave / 2 / nsb_a;  // rows of each matrix a tile: 32 lanes a matrix
  a.tiles_a = op->used * ((op->ffn + a.rows_a - 1) / a.rows_a);
  // Outputs a tile of the second phase: a tile a workgroup where the lanes allow.
  const int most = kWave / nsb_b;
  if (most < 1) return Refuse(1, "moe.token: ffn beyond a wave's 64 super-blocks");
  a.rows_b = (op->hidden + groups - 1) / groups;
  if (a.rows_b > most) a.rows_b = most;
  a.tiles_b = (op->hidden + a.rows_b - 1) / a.rows_b;
  const size_t records_a = static_cast<size_t>(nsb_a) * FormatQ4K::kRecord, records_b = static_cast<size_t>(kTokenWaves) * nsb_b * FormatQ4K::kRecord;
  const size_t lds = (((records_a > records_b ? records_a : records_b) + 15) & ~static_cast<size_t>(15)) +
                     static_cast<size_t>(kTokenWaves) * kWave * FormatQ4K::kUnitBytes + static_cast<size_t>(kTokenWaves) * a.rows_b * sizeof(float);
  if (lds > kDeepLdsLimit) return Refuse(1, "moe.token: %zu bytes of LDS", lds);
  const hipStream_t on = static_cast<hipStream_t>(stream);
  for (int phase = launches == 1 ? 0 : 1; phase <= (launches == 1 ? 0 : 2); ++phase) {
    a.phase = phase;
    op->x_type == LLMP_X_F32 ? LaunchToken<LLMP_X_F32>(a, groups, lds, on) : LaunchToken<LLMP_X_BF16>(a, groups, lds, on);
  }
  return LaunchStatus("moe.token");
}
