// ggml.flash_attn_ext.vec_q8_0 / vec_q4_0 (FlashAttnVecQuant, src/kernels/ggml/kv_quant.h:9-26, 146-160 of the
// reference): attention whose K and V are read as the Q8_0 or Q4_0 blocks the cache stores of kv_quant.hip wrote,
// nothing expanded into device memory. The reference launches GGML's vector kernel; this is a gfx950 kernel with the
// same operands and the same outline (Q quantized to Q8_1 in LDS for the K product; an online softmax; F32 output).
//
// A workgroup of four waves (eight at D 256) takes one KV head, a run of cells (a split) and up to eight queries that
// share that KV head (the head's group of query heads times a few rows), so K and V are read once for all of them. A
// wave takes tiles of 64 cells (32 at D 256 and 512): its K and V rows come by global_load_lds as 16-byte (4-byte at
// D 64) pieces, packed rows in LDS, every cache line asked for once. K product: a lane a cell (two lanes a cell, half
// a row each, in tiles of 32); the row's dwords multiply, as they
// lie, with an image of the quantized query that holds its codes where the row holds codes and zeros where it holds
// the blocks' scales (Q4_0: one image for the low nibbles, one for the high), v_dot4_i32_i8 by v_dot4_i32_i8; every
// dword holds codes of one block only, so a block's integer sum is complete at a known dword and is scaled there. V
// product: a lane D / 64 consecutive values of every row, the tile's probabilities broadcast from LDS. The waves'
// (max, sum, values) meet in LDS, a split's go to scratch, and a second launch combines the splits (and the sinks).
// The loads into LDS are written as instructions and waited for by count: the compiler would make every LDS read
// wait for all of them.
#include <hip/hip_runtime.h>

#include <cmath>
#include <type_traits>
#include <utility>

#include "common.h"
#include "llmp_hip.h"
#include "vecq_common.h"

namespace llmp_hip {
namespace {

// Waves a workgroup and cells a tile by head size: 4 waves of 64 cells at D 64, 8 of 32 at D 256 (two waves a SIMD:
// the tile's vector work of one wave runs under the other's waits), 4 of 32 at D 512.
constexpr int AttnWavesOf(int head_dim) { return head_dim == 256 ? 8 : 4; }
constexpr int AttnTileOf(int head_dim) { return head_dim >= 256 ? 32 : 64; }
constexpr int kMostQueries = 8;  // queries of a workgroup: a KV head's query heads times rows

template <int TYPE, int D>
struct AttnGeo {
  static constexpr bool kQ8 = TYPE == LLMP_TYPE_Q8_0;
  static constexpr int kBlock = kQ8 ? 34 : 18;        // bytes of a block of 32 values
  static constexpr int kBlocks = D / 32;
  static constexpr int kRow = kBlocks * kBlock;       // bytes of a (cell, head) row
  static constexpr int kDwords = kRow / 4;
  static constexpr bool kWide = kRow % 16 == 0;       // rows of whole 16-byte pieces (D 256, 512)
  static constexpr int kPiece = kWide ? 16 : 4;       // bytes a lane brings a load
  static constexpr int kRead = kWide ? 4 : 1;         // dwords a read of LDS
  static constexpr int kWaves = AttnWavesOf(D);
  static constexpr int kThreads = kWaves * kWave;
  static constexpr int kTile = AttnTileOf(D);         // cells a tile
  static constexpr int kTileBytes = kTile * kRow;
  static constexpr int kLoads = (kTileBytes + kWave * kPiece - 1) / (kWave * kPiece);  // loads a tile of K or of V
  static constexpr int kLastLanes = (kTileBytes - (kLoads - 1) * kWave * kPiece) / kPiece;  // lanes of the last one
  // A tile of 32 cells leaves half the wave without a cell: the K product then splits a row between two lanes (whole
  // blocks each). (The V product keeps a lane at D / 64 values of every cell: twice the values of half the cells has
  // two rows' reads of LDS in the same banks, and took longer.)
  static constexpr int kHalves = kWave / kTile;       // lanes a cell in the K product
  static constexpr int kHalfRow = kRow / kHalves, kHalfDwords = kDwords / kHalves, kHalfBlocks = kBlocks / kHalves;
  static constexpr int kPer = D / kWave;              // values of a V row a lane
  static constexpr int kImage = (kQ8 ? 1 : 2) * kRow; // bytes of a query's image(s)
  static constexpr int kQuery = kImage + kBlocks * 8; // ... and its blocks' scales and code sums
  static constexpr int kQueries = (kMostQueries * kQuery + 15) & ~15;
  static constexpr int kMaskBytes = kMostQueries * kTile * 2;                   // a tile's mask values, a row a query row
  static constexpr int kWaveBytes = 2 * kTileBytes + kMostQueries * kTile * 4 + kMaskBytes;  // K, V, probabilities, mask
  static constexpr int kLoadsWithMask = kLoads + kMostQueries;  // a tile of K and its mask rows
  static constexpr int kLds = kQueries + kWaves * kWaveBytes;
  static_assert(kTileBytes % kPiece == 0 && kRow % 4 == 0 && kPer >= 1 && 32 % kPer == 0 && kHalfRow % kBlock == 0 && (kHalves == 1 || kHalfRow % 8 == 0), "geometry");
  // The block whose codes dword w holds: its last byte's, unless that byte is a scale's.
  static constexpr int BlockOf(int w) { return (4 * w + 3) % kBlock >= 2 ? (4 * w + 3) / kBlock : (4 * w) / kBlock; }
  static constexpr bool LastOf(int w) { return w + 1 == kHalfDwords || BlockOf(w + 1) != BlockOf(w); }
  // Whether dword w holds a block's scale, and in which half.
  static constexpr bool HasScale(int w) { return (4 * w) % kBlock == 0 || (4 * w + 2) % kBlock == 0; }
  static constexpr int ScaleShift(int w) { return (4 * w) % kBlock == 0 ? 0 : 16; }
  static constexpr int ScaleBlock(int w) { return (4 * w) % kBlock == 0 ? 4 * w / kBlock : (4 * w + 2) / kBlock; }
};

template <class F, int... I>
__device__ __forceinline__ void AttnForEach(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void AttnFor(F&& f) {
  AttnForEach(f, std::make_integer_sequence<int, N>{});
}

// `bytes` a lane from `from` (a lane's own address) to LDS at `to` + bytes * lane, no register between. In flight
// until the wave's vmcnt says otherwise.
// `base` the same in every lane (scalar registers), `offset` a lane's own.
template <int BYTES, int OFFSET>
__device__ __forceinline__ void ToLds(const uint8_t* base, uint32_t offset, uint32_t to) {
  if constexpr (BYTES == 16) {
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(to), "v"(offset), "s"(base), "n"(OFFSET) : "memory", "scc");
  } else {
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(to), "v"(offset), "s"(base), "n"(OFFSET) : "memory", "scc");
  }
}
// The same pointer known to the compiler as the same in every lane.
__device__ __forceinline__ const uint8_t* UniformPointer(const uint8_t* p) {
  const uint64_t bits = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bits));
  const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(bits >> 32));
  return reinterpret_cast<const uint8_t*>((static_cast<uint64_t>(hi) << 32) | lo);
}

template <int LEFT>
__device__ __forceinline__ void AwaitAllBut() {
  __builtin_amdgcn_s_waitcnt(0x0F70 | (LEFT & 15) | ((LEFT >> 4) << 14));
  asm volatile("" ::: "memory");
}

struct AttnArgs {
  llmp_attn_vec_quant d;
  float* partial;  // [rows][heads][splits][D + 2]: max, sum, values
  int splits, split_cells, group, rows_a_pass;
};

// Over a wave's 64 lanes, the same in every lane: within a row of 16 lanes by data-parallel moves (lane ^ 1, lane ^ 2,
// the mirrored half row, the mirrored row), across the four rows by lane reads; no permute through LDS.
template <int CONTROL>
__device__ __forceinline__ float Dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), CONTROL, 0xF, 0xF, true));
}
__device__ __forceinline__ float LaneValue(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
__device__ __forceinline__ float WaveMax(float v) {
  v = fmaxf(v, Dpp<0xB1>(v));
  v = fmaxf(v, Dpp<0x4E>(v));
  v = fmaxf(v, Dpp<0x141>(v));
  v = fmaxf(v, Dpp<0x140>(v));
  return fmaxf(fmaxf(LaneValue(v, 0), LaneValue(v, 16)), fmaxf(LaneValue(v, 32), LaneValue(v, 48)));
}
__device__ __forceinline__ float WaveSum(float v) {
  v += Dpp<0xB1>(v);
  v += Dpp<0x4E>(v);
  v += Dpp<0x141>(v);
  v += Dpp<0x140>(v);
  return (LaneValue(v, 0) + LaneValue(v, 16)) + (LaneValue(v, 32) + LaneValue(v, 48));
}

// grid (splits, KV heads, passes of rows); 256 threads.
// NQ: the queries the loops are unrolled for, at least the pass's; those beyond it multiply images of zeros and are
// never written out.
template <int TYPE, int D, int NQ>
__global__ __launch_bounds__(AttnWavesOf(D) * kWave, 1) void AttnVecQuantKernel(const AttnArgs a) {
  using G = AttnGeo<TYPE, D>;
  constexpr int kAttnWaves = G::kWaves, kAttnThreads = G::kThreads;
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const llmp_attn_vec_quant& d = a.d;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int split = blockIdx.x, kv_head = blockIdx.y;
  const int row0 = blockIdx.z * a.rows_a_pass;
  const int rows_here = min(a.rows_a_pass, d.rows - row0);
  const int nq = a.group * rows_here;  // query q: head kv_head * group + q / rows_here, row row0 + q % rows_here

  // ---- this wave's tiles of the split.
  const uint32_t lds_at = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(lds)));
  uint8_t* const mine = lds + G::kQueries + wave * G::kWaveBytes;
  const uint32_t mine_at = lds_at + G::kQueries + wave * G::kWaveBytes;
  uint8_t* const k_tile = mine;
  uint8_t* const v_tile = mine + G::kTileBytes;
  float* const probs = reinterpret_cast<float*>(mine + 2 * G::kTileBytes);  // [query][cell of the tile]
  const int cell_first = split * a.split_cells;
  const int tiles = min(a.split_cells, d.cells - cell_first) / G::kTile;
  // A lane's piece of every load: piece p = 64 i + lane of a tile is row p / (pieces a row), piece p % (...): where
  // it lies from the tile's first row is the same for every tile (a register a load; the tile's place is scalar).
  constexpr int kPieces = G::kRow / G::kPiece;
  uint32_t k_from[G::kLoads], v_from[G::kLoads];
#pragma unroll
  for (int i = 0; i < G::kLoads; ++i) {
    const int p = i * kWave + lane;
    const int r = p / kPieces, c = p - r * kPieces;
    k_from[i] = static_cast<uint32_t>(r * d.k_cell_stride + c * G::kPiece);
    v_from[i] = static_cast<uint32_t>(r * d.v_cell_stride + c * G::kPiece);
  }
  auto fetch = [&](const void* base, int64_t cell_stride, int64_t head_stride, const uint32_t (&from)[G::kLoads], int tile, uint32_t to) {
    const int cell0 = cell_first + tile * G::kTile;
    const uint8_t* first = UniformPointer(static_cast<const uint8_t*>(base) + kv_head * head_stride + cell0 * cell_stride);
    AttnFor<G::kLoads>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      // (The last load of a tile that is no whole number of loads is the lower lanes' alone: an instruction all the
      // same, counted by the waits like the others.)
      if (i + 1 < G::kLoads || G::kLastLanes == kWave || lane < G::kLastLanes) ToLds<G::kPiece, i * kWave * G::kPiece>(first, from[i], to);
    });
  };

  // A tile's mask values: query row r's 64 halves by lanes 0 to 31, always kMostQueries loads (rows past the pass's
  // repeat its last) so that the waits count the same loads whatever the pass holds.
  const uint32_t mask_at = mine_at + 2 * G::kTileBytes + kMostQueries * G::kTile * 4;
  const uint16_t* const mask_tile = reinterpret_cast<const uint16_t*>(mine + 2 * G::kTileBytes + kMostQueries * G::kTile * 4);
  auto fetch_keys = [&](int tile) {
    fetch(d.k, d.k_cell_stride, d.k_head_stride, k_from, tile, mine_at);
    const int cell0 = cell_first + tile * G::kTile;
    AttnFor<kMostQueries>([&](auto rc) {
      constexpr int r = decltype(rc)::value;
      const int row = row0 + min(r, rows_here - 1);
      const uint8_t* first = UniformPointer(reinterpret_cast<const uint8_t*>(static_cast<const uint16_t*>(d.mask) + row * d.mask_row_stride + cell0));
      if (lane < G::kTile / 2) ToLds<4, r * G::kTile * 2>(first, static_cast<uint32_t>(4 * lane), mask_at);
    });
  };

  // The queries' loads first, then the wave's first tiles, then the staging: the loads are written as instructions
  // and waited for by count (they are older than the tiles' loads), so that the tiles are on their way while the
  // queries are quantized.
  typedef float F4 __attribute__((ext_vector_type(4)));
  constexpr int kGroups = kAttnThreads >> 3;                                         // 8-lane groups, a block each a sweep
  constexpr int kSweeps = (kMostQueries * G::kBlocks + kGroups - 1) / kGroups;
  F4 held[kSweeps];
#pragma unroll
  for (int i = 0; i < kSweeps; ++i) {
    const int b = (tid >> 3) + i * kGroups;
    held[i] = F4{0.0f, 0.0f, 0.0f, 0.0f};
    if (b < nq * G::kBlocks) {
      const int q = b / G::kBlocks, blk = b - q * G::kBlocks;
      const int head = kv_head * a.group + q / rows_here, row = row0 + q % rows_here;
      const float* src = static_cast<const float*>(d.q) + head * d.q_head_stride + row * d.q_row_stride + blk * 32 + (tid & 7) * 4;
      asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(held[i]) : "v"(src) : "memory");
    }
  }
  for (int i = tid; i < G::kQueries / 4; i += kAttnThreads) reinterpret_cast<uint32_t*>(lds)[i] = 0;
  if (wave < tiles) {
    fetch_keys(wave);
    fetch(d.v, d.v_cell_stride, d.v_head_stride, v_from, wave, mine_at + G::kTileBytes);
  }
  // The queries have landed once no more than the tiles' loads are outstanding (the registers are tied to the wait).
  if (wave < tiles) {
    if constexpr (kSweeps == 1) asm volatile("s_waitcnt vmcnt(%1)" : "+v"(held[0]) : "n"(G::kLoadsWithMask + G::kLoads));
    if constexpr (kSweeps == 2) asm volatile("s_waitcnt vmcnt(%2)" : "+v"(held[0]), "+v"(held[1]) : "n"(G::kLoadsWithMask + G::kLoads));
    if constexpr (kSweeps == 4)
      asm volatile("s_waitcnt vmcnt(%4)" : "+v"(held[0]), "+v"(held[1]), "+v"(held[2]), "+v"(held[3]) : "n"(G::kLoadsWithMask + G::kLoads));
  } else {
    if constexpr (kSweeps == 1) asm volatile("s_waitcnt vmcnt(0)" : "+v"(held[0]));
    if constexpr (kSweeps == 2) asm volatile("s_waitcnt vmcnt(0)" : "+v"(held[0]), "+v"(held[1]));
    if constexpr (kSweeps == 4) asm volatile("s_waitcnt vmcnt(0)" : "+v"(held[0]), "+v"(held[1]), "+v"(held[2]), "+v"(held[3]));
  }
  static_assert(kSweeps == 1 || kSweeps == 2 || kSweeps == 4, "the sweeps the waits are written for");
  __syncthreads();  // the images are zero

  // ---- the queries: Q8_1 blocks (eight lanes a block), laid out as images of a K row.
#pragma unroll
  for (int i = 0; i < kSweeps; ++i) {
    const int b = (tid >> 3) + i * kGroups;
    if (b < nq * G::kBlocks) {  // whole 8-lane groups together
      const int q = b / G::kBlocks, blk = b - q * G::kBlocks;
      const Q8Block packed = QuantizeQ8Block(held[i].x, held[i].y, held[i].z, held[i].w);
      uint8_t* image = lds + q * G::kQuery;
      const int lane8 = tid & 7;
      // Values 4 lane8 .. + 3 of the block: against the row's codes (Q4_0: the low nibbles hold values 0 to 15, the
      // high ones 16 to 31 of the same bytes).
      const int at = G::kQ8 ? blk * G::kBlock + 2 + 4 * lane8 : (lane8 >> 2) * G::kRow + blk * G::kBlock + 2 + 4 * (lane8 & 3);
      *reinterpret_cast<uint16_t*>(image + at) = static_cast<uint16_t>(packed.codes);
      *reinterpret_cast<uint16_t*>(image + at + 2) = static_cast<uint16_t>(packed.codes >> 16);
      int total = Dot4(0x01010101, static_cast<int>(packed.codes), 0);
      total += ShflXor(total, 1);
      total += ShflXor(total, 2);
      total += ShflXor(total, 4);
      if (lane8 == 0) {
        float* scales = reinterpret_cast<float*>(image + G::kImage);
        scales[blk] = HalfBitsToFloat(FloatToHalfBits(packed.d));  // the scale as a Q8_1 block stores it
        scales[G::kBlocks + blk] = static_cast<float>(total);
      }
    }
  }
  __syncthreads();

  float top[NQ], sum[NQ], corr[NQ], acc[NQ][G::kPer];
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    top[q] = -INFINITY;
    sum[q] = 0.0f;
    corr[q] = 0.0f;
#pragma unroll
    for (int j = 0; j < G::kPer; ++j) acc[q][j] = 0.0f;
  }
  const bool capped = d.softcap > 0.0f;
  const float cap_inverse = capped ? 1.0f / d.softcap : 0.0f;
  // Where a lane's values of a V row lie: block, first byte and, for Q4_0, the nibble.
  const int v_block = lane * G::kPer / 32, v_in = lane * G::kPer % 32;
  const int v_scale_at = v_block * G::kBlock;
  const int v_codes_at = v_scale_at + 2 + (G::kQ8 ? v_in : v_in % 16);
  const int v_shift = G::kQ8 ? 0 : (v_in / 16) * 4;

  for (int tile = wave; tile < tiles; tile += kAttnWaves) {
    AwaitAllBut<G::kLoads>();  // K and the mask have landed, V may be on its way
    __builtin_amdgcn_wave_barrier();
    // The mask's values into registers: their place is refilled before they are used.
    float bias[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      bias[q] = 0.0f;
      if (lane < G::kTile) bias[q] = HalfBitsToFloat(mask_tile[(q % rows_here) * G::kTile + lane]);
    }
    // ---- scores: a lane a cell.
    float score[NQ];
    int part[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) score[q] = 0.0f, part[q] = 0;
    {
      // (A tile of 32 cells: lanes 32 to 63 take the rows' upper halves, whole blocks like the lower ones.)
      const int k_half = lane / G::kTile;
      const uint8_t* row = k_tile + (lane & (G::kTile - 1)) * G::kRow + k_half * G::kHalfRow;
      // One or two queries' images stay in registers from tile to tile (the compiler finds their reads the same in
      // every iteration); more do not fit, so their place is hidden from it here and they are read again a tile.
      uint32_t images_at = 0;
      if constexpr (NQ > 2) asm volatile("" : "+v"(images_at));
      const uint8_t* images = lds + images_at + k_half * G::kHalfRow;
      const int scales_from = k_half * G::kHalfBlocks;
      uint32_t kd[G::kRead];
      uint32_t low[NQ][G::kRead], high[G::kQ8 ? 1 : NQ][G::kRead];  // the images' dwords beside the row's
      float dk = 0.0f;
      AttnFor<G::kHalfDwords>([&](auto wc) {
        constexpr int w = decltype(wc)::value;
        // (The reads of LDS stay with their group of dwords: hoisted to the front of the unrolled row they take
        // more registers than there are.)
        if constexpr (w % (2 * G::kRead) == 0 && w > 0) __builtin_amdgcn_sched_barrier(0);
        if constexpr (w % G::kRead == 0) {
          if constexpr (G::kWide) {
            // (Half rows begin at 8-byte boundaries: two 8-byte reads each. A row's last read may run past its half.)
            auto four = [](const uint8_t* at, uint32_t (&into)[G::kRead]) {
              if constexpr (G::kHalfRow % 16 == 0) {
                const uint4 x = *reinterpret_cast<const uint4*>(at);
                into[0] = x.x, into[1] = x.y, into[2] = x.z, into[3] = x.w;
              } else {
                const uint2 x = *reinterpret_cast<const uint2*>(at), y = *reinterpret_cast<const uint2*>(at + 8);
                into[0] = x.x, into[1] = x.y, into[2] = y.x, into[3] = y.y;
              }
            };
            four(row + 4 * w, kd);
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
              four(images + q * G::kQuery + 4 * w, low[q]);
              if constexpr (!G::kQ8) four(images + q * G::kQuery + G::kRow + 4 * w, high[q]);
            }
          } else {
            kd[0] = *reinterpret_cast<const uint32_t*>(row + 4 * w);
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
              low[q][0] = *reinterpret_cast<const uint32_t*>(images + q * G::kQuery + 4 * w);
              if constexpr (!G::kQ8) high[q][0] = *reinterpret_cast<const uint32_t*>(images + q * G::kQuery + G::kRow + 4 * w);
            }
          }
        }
        const uint32_t x = kd[w % G::kRead];
        constexpr int blk = G::BlockOf(w);
        // A scale in the dword's upper half is the next block's: it takes effect once this block's sum is scaled.
        if constexpr (G::HasScale(w) && G::ScaleBlock(w) == blk) dk = HalfBitsToFloat((x >> G::ScaleShift(w)) & 0xFFFFu);
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
          if constexpr (G::kQ8) {
            part[q] = Dot4(static_cast<int>(x), static_cast<int>(low[q][w % G::kRead]), part[q]);
          } else {
            part[q] = Dot4(static_cast<int>(x & 0x0F0F0F0Fu), static_cast<int>(low[q][w % G::kRead]), part[q]);
            part[q] = Dot4(static_cast<int>((x >> 4) & 0x0F0F0F0Fu), static_cast<int>(high[q][w % G::kRead]), part[q]);
          }
          if constexpr (G::LastOf(w)) {
            const float* scales = reinterpret_cast<const float*>(lds + images_at + q * G::kQuery + G::kImage) + scales_from;
            // Q4_0: values are codes minus 8, so eight times the query's code sum comes off.
            const float whole = G::kQ8 ? static_cast<float>(part[q]) : static_cast<float>(part[q]) - 8.0f * scales[G::kBlocks + blk];
            score[q] += (dk * scales[blk]) * whole;
            part[q] = 0;
          }
        }
        if constexpr (G::HasScale(w) && G::ScaleBlock(w) != blk) dk = HalfBitsToFloat((x >> G::ScaleShift(w)) & 0xFFFFu);
        // The sums are taken where they are computed: pure as they are, the compiler otherwise moves every product
        // to the row's end and keeps all the row's and images' dwords until then.
        if constexpr ((w + 1) % G::kRead == 0 || w + 1 == G::kHalfDwords) {
#pragma unroll
          for (int q = 0; q < NQ; ++q) asm volatile("" : "+v"(part[q]), "+v"(score[q]));
        }
      });
    }
    if constexpr (G::kHalves == 2) {
#pragma unroll
      for (int q = 0; q < NQ; ++q) score[q] += __shfl_xor(score[q], 32);  // a cell's two half rows
    }
    // K's buffer is free: the wave's next tile of K on its way.
    const int next = tile + kAttnWaves;
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    if (next < tiles) fetch_keys(next);
    // ---- online softmax over the tile.
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      float s = score[q] * d.scale;
      if (capped) s = d.softcap * tanhf(s * cap_inverse);
      s = lane < G::kTile ? s + bias[q] : -INFINITY;
      const float peak = fmaxf(top[q], WaveMax(s));
      const float p = peak == -INFINITY ? 0.0f : __expf(s - peak);
      const float keep = peak == -INFINITY ? 1.0f : __expf(top[q] - peak);  // exp(-inf) is 0: a first tile keeps nothing
      sum[q] = sum[q] * keep + WaveSum(p);
      corr[q] *= keep;
#pragma unroll
      for (int j = 0; j < G::kPer; ++j) acc[q][j] *= keep;
      top[q] = peak;
      if (lane < G::kTile) probs[q * G::kTile + lane] = p;
    }
    if (next < tiles) {
      AwaitAllBut<G::kLoadsWithMask>();  // V has landed (the next K and mask may be on their way)
    } else {
      AwaitAllBut<0>();
    }
    __builtin_amdgcn_wave_barrier();
    // ---- values: a lane kPer consecutive values of every row of the tile.
#pragma unroll 1
    for (int c4 = 0; c4 < G::kTile; c4 += 4) {
      float4 four_probs[NQ];  // the probabilities of four cells, broadcast
#pragma unroll
      for (int q = 0; q < NQ; ++q) four_probs[q] = *reinterpret_cast<const float4*>(probs + q * G::kTile + c4);
#pragma unroll
      for (int cc = 0; cc < 4; ++cc) {
        const uint8_t* row = v_tile + (c4 + cc) * G::kRow;
        const float dv = HalfBitsToFloat(*reinterpret_cast<const uint16_t*>(row + v_scale_at));
        float value[G::kPer];
        if constexpr (G::kPer == 1) {
          const uint32_t byte = row[v_codes_at];
          value[0] = G::kQ8 ? static_cast<float>(byte ^ 0x80u) : static_cast<float>((byte >> v_shift) & 0xFu);
        } else {
#pragma unroll
          for (int j = 0; j < G::kPer; j += 4) {
            uint32_t four = *reinterpret_cast<const uint16_t*>(row + v_codes_at + j) |
                            (static_cast<uint32_t>(*reinterpret_cast<const uint16_t*>(row + v_codes_at + j + 2)) << 16);
            four = G::kQ8 ? four ^ 0x80808080u : (four >> v_shift) & 0x0F0F0F0Fu;
            value[j] = static_cast<float>(four & 0xFFu);
            value[j + 1] = static_cast<float>((four >> 8) & 0xFFu);
            value[j + 2] = static_cast<float>((four >> 16) & 0xFFu);
            value[j + 3] = static_cast<float>(four >> 24);
          }
        }
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
          const float p = cc == 0 ? four_probs[q].x : cc == 1 ? four_probs[q].y : cc == 2 ? four_probs[q].z : four_probs[q].w;
          const float weight = p * dv;
          corr[q] += weight;
#pragma unroll
          for (int j = 0; j < G::kPer; ++j) acc[q][j] = fmaf(weight, value[j], acc[q][j]);
        }
      }
    }
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    if (next < tiles) fetch(d.v, d.v_cell_stride, d.v_head_stride, v_from, next, mine_at + G::kTileBytes);
  }
  AwaitAllBut<0>();
  __syncthreads();

  // ---- the waves' results meet in LDS (the tile buffers are free): values minus the offset the codes carried.
  constexpr float kOffset = G::kQ8 ? 128.0f : 8.0f;
  float* const meet = reinterpret_cast<float*>(lds + G::kQueries);  // [wave][query][D + 2]
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    if (q < nq) {
      float* out = meet + (wave * kMostQueries + q) * (D + 2);
      if (lane == 0) out[0] = top[q], out[1] = sum[q];
#pragma unroll
      for (int j = 0; j < G::kPer; ++j) out[2 + lane * G::kPer + j] = acc[q][j] - kOffset * corr[q];
    }
  }
  __syncthreads();
  for (int i = tid; i < nq * D; i += kAttnThreads) {
    const int q = i / D, j = i - q * D;
    float peak = -INFINITY;
#pragma unroll
    for (int w = 0; w < kAttnWaves; ++w) peak = fmaxf(peak, meet[(w * kMostQueries + q) * (D + 2)]);
    float total = 0.0f, value = 0.0f;
#pragma unroll
    for (int w = 0; w < kAttnWaves; ++w) {
      const float* from = meet + (w * kMostQueries + q) * (D + 2);
      const float keep = from[0] == -INFINITY ? 0.0f : __expf(from[0] - peak);
      total += from[1] * keep;
      value += from[2 + j] * keep;
    }
    const int head = kv_head * a.group + q / rows_here, row = row0 + q % rows_here;
    float* out = a.partial + ((static_cast<int64_t>(row) * d.heads + head) * a.splits + split) * (D + 2);
    if (j == 0) out[0] = peak, out[1] = total;
    out[2 + j] = value;
  }
}

// grid (heads, rows); D threads: the splits' partial results into one row of the output. The splits' maxima and sums
// through LDS (a thread a split), then every thread its value over the splits, in split order.
constexpr int kMostSplits = 512;
template <int D>
__global__ __launch_bounds__(D) void AttnCombineKernel(const AttnArgs a) {
  __shared__ float peaks[kMostSplits], totals[kMostSplits];
  const llmp_attn_vec_quant& d = a.d;
  const int head = blockIdx.x, row = blockIdx.y, j = threadIdx.x;
  const float* from = a.partial + (static_cast<int64_t>(row) * d.heads + head) * a.splits * (D + 2);
  for (int s = j; s < a.splits; s += D) peaks[s] = from[s * (D + 2)], totals[s] = from[s * (D + 2) + 1];
  __syncthreads();
  const bool sunk = d.sinks != nullptr;
  float peak = sunk ? static_cast<const float*>(d.sinks)[head] : -INFINITY;
  for (int s = 0; s < a.splits; ++s) peak = fmaxf(peak, peaks[s]);
  float total = sunk ? __expf(static_cast<const float*>(d.sinks)[head] - peak) : 0.0f, value = 0.0f;
  // (Thirty-two loads in flight: a launch of sixteen workgroups is a chain of round trips, and eight at a time made
  // four of them at 32 splits. Asking for them ahead of the maxima's trip through LDS measured slower.)
#pragma unroll 32
  for (int s = 0; s < a.splits; ++s) {
    const float keep = peaks[s] == -INFINITY ? 0.0f : __expf(peaks[s] - peak);
    total += totals[s] * keep;
    value += from[s * (D + 2) + 2 + j] * keep;
  }
  // A row that sees nothing (and has no sink) is zero, as the reference's SoftmaxRow has it.
  static_cast<float*>(d.out)[(static_cast<int64_t>(row) * d.heads + head) * D + j] =
      peak == -INFINITY || !(total > 0.0f) ? 0.0f : value / total;
}

struct AttnPlan {
  int group, rows_a_pass, passes, splits, split_cells;
};

template <int TYPE, int D, int NQ>
void LaunchAttnFor(const AttnArgs& args, const AttnPlan& plan, hipStream_t stream) {
  using G = AttnGeo<TYPE, D>;
  static bool sized = false;
  if (!AllowLds(reinterpret_cast<const void*>(&AttnVecQuantKernel<TYPE, D, NQ>), G::kLds, &sized)) return;
  const dim3 grid(static_cast<unsigned>(plan.splits), static_cast<unsigned>(args.d.kv_heads), static_cast<unsigned>(plan.passes));
  hipLaunchKernelGGL((AttnVecQuantKernel<TYPE, D, NQ>), grid, dim3(G::kThreads), G::kLds, stream, args);
}

template <int TYPE, int D>
void LaunchAttn(const AttnArgs& args, const AttnPlan& plan, hipStream_t stream) {
  const int queries = plan.group * plan.rows_a_pass;  // of a full pass
  if (queries <= 1) {
    LaunchAttnFor<TYPE, D, 1>(args, plan, stream);
  } else if (queries <= 2) {
    LaunchAttnFor<TYPE, D, 2>(args, plan, stream);
  } else if (queries <= 4) {
    LaunchAttnFor<TYPE, D, 4>(args, plan, stream);
  } else {
    LaunchAttnFor<TYPE, D, 8>(args, plan, stream);
  }
  hipLaunchKernelGGL((AttnCombineKernel<D>), dim3(static_cast<unsigned>(args.d.heads), static_cast<unsigned>(args.d.rows)), dim3(D), 0,
                     stream, args);
}

// 0 and the plan, or a refusal: every check of the reference's CheckFlashAttnVecQuant (src/kernels/ggml/kv_quant.cc:81-170)
// that applies to these operands, and this kernel's own.
int PlanAttn(const llmp_attn_vec_quant* op, int cus, AttnPlan* plan) {
  if (op == nullptr) return Refuse(1, "attn_vec_quant: null operands");
  if (op->type != LLMP_TYPE_Q8_0 && op->type != LLMP_TYPE_Q4_0)
    return Refuse(1, "attn_vec_quant: K and V are both Q8_0 or both Q4_0, not type %d", op->type);
  if (op->head_dim != 64 && op->head_dim != 256 && (op->head_dim != 512 || op->type != LLMP_TYPE_Q8_0))
    return Refuse(1, "attn_vec_quant: head sizes 64 and 256 (and 512 for Q8_0), not %d", op->head_dim);
  if (op->heads < 1 || op->kv_heads < 1 || op->rows < 1 || op->cells < 1 || op->heads % op->kv_heads != 0)
    return Refuse(1, "attn_vec_quant: a whole number of query heads a KV head (%d, %d), rows %d, cells %d", op->heads, op->kv_heads, op->rows, op->cells);
  if (op->heads / op->kv_heads > kMostQueries)
    return Refuse(1, "attn_vec_quant: at most %d query heads a KV head, not %d", kMostQueries, op->heads / op->kv_heads);
  if (op->cells % 256 != 0) return Refuse(1, "attn_vec_quant: the attended cells are padded to 256, not %d", op->cells);
  if (op->q == nullptr || op->k == nullptr || op->v == nullptr || op->mask == nullptr || op->out == nullptr)
    return Refuse(1, "attn_vec_quant: null operand (Q, K, V, the mask and the output are all required)");
  if (!(op->scale > 0.0f) || !std::isfinite(op->scale)) return Refuse(1, "attn_vec_quant: a positive finite scale");
  if (op->softcap != 0.0f && !(op->head_dim == 256 && op->softcap > 0.0f && std::isfinite(op->softcap) && std::isfinite(op->scale / op->softcap)))
    return Refuse(1, "attn_vec_quant: a finite positive softcap, at head size 256 only");
  const int block = op->type == LLMP_TYPE_Q8_0 ? 34 : 18;
  const int64_t row_bytes = static_cast<int64_t>(op->head_dim / 32) * block;
  for (const int64_t stride : {op->k_cell_stride, op->k_head_stride, op->v_cell_stride, op->v_head_stride}) {
    if (stride < row_bytes || stride % block != 0 || stride % 4 != 0)
      return Refuse(1, "attn_vec_quant: K's and V's strides are whole blocks at 4-byte boundaries holding a row, not %lld bytes", (long long)stride);
  }
  if ((reinterpret_cast<uintptr_t>(op->k) | reinterpret_cast<uintptr_t>(op->v)) % 4 != 0 ||
      (row_bytes % 16 == 0 && ((reinterpret_cast<uintptr_t>(op->k) | reinterpret_cast<uintptr_t>(op->v) | op->k_cell_stride | op->k_head_stride |
                                 op->v_cell_stride | op->v_head_stride) % 16 != 0)))
    return Refuse(1, "attn_vec_quant: K and V at 4-byte boundaries, rows of whole 16-byte pieces at 16-byte boundaries");
  if (reinterpret_cast<uintptr_t>(op->q) % 16 != 0 || op->q_row_stride % 4 != 0 || op->q_head_stride % 4 != 0 ||
      reinterpret_cast<uintptr_t>(op->out) % 16 != 0)
    return Refuse(1, "attn_vec_quant: Q and the output at 16-byte boundaries");
  if (op->mask_row_stride < op->cells || op->mask_row_stride % 2 != 0 || reinterpret_cast<uintptr_t>(op->mask) % 16 != 0)
    return Refuse(1, "attn_vec_quant: one F16 mask row of at least %d cells a query row, at 16-byte boundaries", op->cells);
  if (static_cast<int64_t>(op->cells) * op->k_cell_stride > INT32_MAX || static_cast<int64_t>(op->cells) * op->v_cell_stride > INT32_MAX)
    return Refuse(1, "attn_vec_quant: K and V within 2 GiB");
  const int group = op->heads / op->kv_heads;
  plan->group = group;
  plan->rows_a_pass = op->rows < kMostQueries / group ? op->rows : (kMostQueries / group < 1 ? 1 : kMostQueries / group);
  plan->passes = (op->rows + plan->rows_a_pass - 1) / plan->rows_a_pass;
  // Splits: about two workgroups a compute unit over the launch, each at least a tile a wave where the cells allow.
  const int tile = AttnTileOf(op->head_dim), waves = AttnWavesOf(op->head_dim);
  const int tiles = op->cells / tile;
  const int others = op->kv_heads * plan->passes;
  int splits = (2 * (cus > 0 ? cus : 256) + others - 1) / others;
  const int most = (tiles + waves - 1) / waves;
  if (splits > most) splits = most;
  if (splits > kMostSplits) splits = kMostSplits;
  if (splits < 1) splits = 1;
  const int tiles_a_split = (tiles + splits - 1) / splits;
  plan->split_cells = tiles_a_split * tile;
  plan->splits = (tiles + tiles_a_split - 1) / tiles_a_split;
  return 0;
}

}  // namespace
}  // namespace llmp_hip

using namespace llmp_hip;

extern "C" size_t llmp_hip_attn_vec_quant_scratch(const llmp_attn_vec_quant* op, int cus) {
  AttnPlan plan;
  if (PlanAttn(op, cus, &plan) != 0) return 0;
  return static_cast<size_t>(op->rows) * op->heads * plan.splits * (op->head_dim + 2) * sizeof(float);
}

extern "C" int llmp_hip_attn_vec_quant(const llmp_attn_vec_quant* op, void* scratch, size_t scratch_bytes, int cus, void* stream) {
  BeginLaunches();
  AttnPlan plan;
  if (const int bad = PlanAttn(op, cus, &plan); bad != 0) return bad;
  const size_t needs = static_cast<size_t>(op->rows) * op->heads * plan.splits * (op->head_dim + 2) * sizeof(float);
  if (scratch == nullptr || scratch_bytes < needs || reinterpret_cast<uintptr_t>(scratch) % 16 != 0)
    return Refuse(1, "attn_vec_quant: %zu bytes of scratch at a 16-byte boundary, %zu given", needs, scratch_bytes);
  AttnArgs args;
  args.d = *op;
  args.partial = static_cast<float*>(scratch);
  args.splits = plan.splits;
  args.split_cells = plan.split_cells;
  args.group = plan.group;
  args.rows_a_pass = plan.rows_a_pass;
  const hipStream_t on = static_cast<hipStream_t>(stream);
  if (op->type == LLMP_TYPE_Q8_0) {
    if (op->head_dim == 64) LaunchAttn<LLMP_TYPE_Q8_0, 64>(args, plan, on);
    if (op->head_dim == 256) LaunchAttn<LLMP_TYPE_Q8_0, 256>(args, plan, on);
    if (op->head_dim == 512) LaunchAttn<LLMP_TYPE_Q8_0, 512>(args, plan, on);
  } else {
    if (op->head_dim == 64) LaunchAttn<LLMP_TYPE_Q4_0, 64>(args, plan, on);
    if (op->head_dim == 256) LaunchAttn<LLMP_TYPE_Q4_0, 256>(args, plan, on);
  }
  return LaunchStatus("attn_vec_quant");
}
