// llmp.vecq over Q4_K weights, the form the default launches take: one lane owns
// one whole 144-byte super-block; every wave streams its own tiles through LDS
// with global-to-LDS loads and never waits for another wave.
//
// A tile is R consecutive rows of the weights (of both matrices with a GLU), at
// most 64 super-blocks: lane t of a wave owns super-block t of the tile's flat
// list (the up rows' super-blocks, then the gate rows'). With packed rows a
// matrix's part of the list is one contiguous byte range; the wave fetches the
// list as 16-byte chunks with global_load_lds_dwordx4, chunk 64 j + lane by its
// j-th load, which lands at 16 * (64 j + lane) of the wave's LDS buffer: every
// cache line is requested once, by neighbouring lanes, and no register holds
// weights in flight. After s_waitcnt vmcnt(0) each lane reads its own
// super-block, nine 16-byte reads 144 bytes apart (36 dwords: sixteen lanes'
// reads fall in distinct banks). A workgroup (8 wave64s) stages its tokens'
// activations once (quantizing them to Q8_1 itself in the fused form) while the
// waves' first tiles are in flight; after that one barrier its waves are
// independent: wave w of the grid takes tiles w, w + waves, .... Sixteen waves a
// CU alternate between waiting for a tile and computing one, so a CU always has
// tiles in flight.
//
// Staged activations, per token and super-block, a record of 336 bytes (84
// dwords, so that consecutive super-blocks start 20 banks apart and sixteen
// lanes' 16-byte reads of the same field never share a bank):
//   [0, 256)    the 256 int8 codes;
//   [256, 288)  the eight sub-blocks' scales d8 as floats;
//   [288, 320)  d8 * sum(codes) of each sub-block as floats (the minimum term);
//   [320, 336)  sum(codes) of each sub-block as int16 (read by the test dump).
// A lane's super-block sum is d * sum_g sc_g * d8_g * prod_g - dmin * sum_g m_g *
// d8_g * sum_g (tests/unit/dsv4_fast_test.cc:179-193), prod_g eight v_dot4_i32_i8.
// Row sums: the lanes' partials go to the wave's LDS buffer and one lane a row
// adds them in super-block order, so a (token, row) value never depends on its
// neighbours or on which wave computed it.

#include <hip/hip_runtime.h>

#include "common.h"
#include "llmp_hip.h"
#include "vecq_common.h"

namespace llmp_hip {
namespace {

constexpr int kRecord = 336;     // bytes a staged super-block
constexpr int kGroup = 512;      // threads a workgroup
constexpr int kWaves = kGroup / kWave;
constexpr int kRing = kWave * 9 * 16;  // bytes of a wave's tile buffer
constexpr int kChunks = 9;       // 16-byte chunks a super-block

struct SuperBlock {
  U32x4 header;  // d, dmin, scales[12]
  U32x4 codes[8];
};

// ---- staging into records

template <int XT>
__device__ __forceinline__ void StageRecordsX(const void* __restrict__ x, int k, uint8_t* token) {
  constexpr int kStep = kGroup / 8;
  constexpr int kAhead = 4;
  const int lane8 = threadIdx.x & 7;
  const int blocks = k / 32;
  const bool wide = reinterpret_cast<uintptr_t>(x) % (XT == LLMP_X_F32 ? 16 : 8) == 0;
  for (int b0 = threadIdx.x >> 3; b0 < blocks; b0 += kStep * kAhead) {
    float v[kAhead][4];
#pragma unroll
    for (int i = 0; i < kAhead; ++i) {
      const int b = b0 + i * kStep;
      if (b < blocks) Load4Wide<XT>(x, static_cast<int64_t>(b) * 32 + lane8 * 4, k, wide, v[i]);
    }
#pragma unroll
    for (int i = 0; i < kAhead; ++i) {
      const int b = b0 + i * kStep;
      if (b >= blocks) break;  // whole 8-lane groups leave together
      const Q8Block q = QuantizeQ8Block(v[i][0], v[i][1], v[i][2], v[i][3]);
      uint8_t* record = token + (b >> 3) * kRecord;
      const int g = b & 7;
      *reinterpret_cast<uint32_t*>(record + g * 32 + lane8 * 4) = q.codes;
      int s = Dot4(0x01010101, static_cast<int>(q.codes), 0);
      s += ShflXor(s, 1);
      s += ShflXor(s, 2);
      s += ShflXor(s, 4);
      if (lane8 == 0) {
        // The products read the scale as a Q8_1 block stores it: rounded to F16.
        const float d8 = HalfBitsToFloat(FloatToHalfBits(q.d));
        reinterpret_cast<float*>(record + 256)[g] = d8;
        reinterpret_cast<float*>(record + 288)[g] = d8 * static_cast<float>(s);
        reinterpret_cast<int16_t*>(record + 320)[g] = static_cast<int16_t>(s);
      }
    }
  }
}

__device__ __forceinline__ void StageRecordsQ8(const uint8_t* __restrict__ y, int blocks, uint8_t* token) {
  for (int b = threadIdx.x; b < blocks; b += kGroup) {
    const uint32_t* src = reinterpret_cast<const uint32_t*>(y + static_cast<int64_t>(b) * kQ8Block);
    uint32_t w[9];
#pragma unroll
    for (int i = 0; i < 9; ++i) w[i] = src[i];
    uint8_t* record = token + (b >> 3) * kRecord;
    const int g = b & 7;
    uint4* dst = reinterpret_cast<uint4*>(record + g * 32);
    dst[0] = make_uint4(w[1], w[2], w[3], w[4]);
    dst[1] = make_uint4(w[5], w[6], w[7], w[8]);
    int s = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) s = Dot4(0x01010101, static_cast<int>(w[1 + i]), s);
    const float d8 = HalfBitsToFloat(w[0] & 0xFFFFu);
    reinterpret_cast<float*>(record + 256)[g] = d8;
    reinterpret_cast<float*>(record + 288)[g] = d8 * static_cast<float>(s);
    reinterpret_cast<int16_t*>(record + 320)[g] = static_cast<int16_t>(s);
  }
}

// ---- one super-block times the staged tokens

__device__ __forceinline__ float ByteToFloat(uint32_t word, int byte) {
  return static_cast<float>((word >> (8 * byte)) & 0xFFu);  // v_cvt_f32_ubyteN
}

template <int P, bool kDump>
__device__ __forceinline__ void DotSuperBlock(const SuperBlock& b, const uint8_t* records, int token_stride, int m,
                                              float (&out)[P], int32_t* dump) {
#pragma clang fp contract(off)
  const uint32_t s0 = b.header.y, s1 = b.header.z, s2 = b.header.w;
  // Bytes g of sc[0], sc[1]: the scales of sub-blocks g and 4 + g; mn likewise.
  const uint32_t sc[2] = {s0 & 0x3F3F3F3Fu, (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u)};
  const uint32_t mn[2] = {s1 & 0x3F3F3F3Fu, ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u)};
  const float d = HalfBitsToFloat(b.header.x & 0xFFFFu);
  const float dmin = HalfBitsToFloat(b.header.x >> 16);
  float main[P];
#pragma unroll
  for (int t = 0; t < P; ++t) main[t] = 0.0f;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    // Pair p: 32 bytes, the low nibbles sub-block 2p, the high ones 2p + 1.
    int lo[8], hi[8];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const U32x4 raw = b.codes[2 * p + i];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        lo[4 * i + c] = static_cast<int>(raw[c] & 0x0F0F0F0Fu);
        hi[4 * i + c] = static_cast<int>((raw[c] >> 4) & 0x0F0F0F0Fu);
      }
    }
    const float sc0 = ByteToFloat(sc[(2 * p) >> 2], (2 * p) & 3);
    const float sc1 = ByteToFloat(sc[(2 * p + 1) >> 2], (2 * p + 1) & 3);
#pragma unroll
    for (int t = 0; t < P; ++t) {
      if (t < m) {
        const uint8_t* record = records + t * token_stride;
        const uint4* a = reinterpret_cast<const uint4*>(record + p * 64);
        const uint4 a0 = a[0], a1 = a[1], a2 = a[2], a3 = a[3];
        const float2 d8 = *reinterpret_cast<const float2*>(record + 256 + p * 8);
        int prod0 = Dot4(lo[0], static_cast<int>(a0.x), 0);
        prod0 = Dot4(lo[1], static_cast<int>(a0.y), prod0);
        prod0 = Dot4(lo[2], static_cast<int>(a0.z), prod0);
        prod0 = Dot4(lo[3], static_cast<int>(a0.w), prod0);
        prod0 = Dot4(lo[4], static_cast<int>(a1.x), prod0);
        prod0 = Dot4(lo[5], static_cast<int>(a1.y), prod0);
        prod0 = Dot4(lo[6], static_cast<int>(a1.z), prod0);
        prod0 = Dot4(lo[7], static_cast<int>(a1.w), prod0);
        int prod1 = Dot4(hi[0], static_cast<int>(a2.x), 0);
        prod1 = Dot4(hi[1], static_cast<int>(a2.y), prod1);
        prod1 = Dot4(hi[2], static_cast<int>(a2.z), prod1);
        prod1 = Dot4(hi[3], static_cast<int>(a2.w), prod1);
        prod1 = Dot4(hi[4], static_cast<int>(a3.x), prod1);
        prod1 = Dot4(hi[5], static_cast<int>(a3.y), prod1);
        prod1 = Dot4(hi[6], static_cast<int>(a3.z), prod1);
        prod1 = Dot4(hi[7], static_cast<int>(a3.w), prod1);
        if (kDump && dump != nullptr) {
          dump[2 * p] = prod0;
          dump[2 * p + 1] = prod1;
          const int16_t* sums = reinterpret_cast<const int16_t*>(record + 320);
          dump[8 + 2 * p] = sums[2 * p];
          dump[8 + 2 * p + 1] = sums[2 * p + 1];
        }
        main[t] = fmaf(static_cast<float>(prod0), sc0 * d8.x, main[t]);
        main[t] = fmaf(static_cast<float>(prod1), sc1 * d8.y, main[t]);
      }
    }
  }
#pragma unroll
  for (int t = 0; t < P; ++t) {
    if (t < m) {
      const float4* ds = reinterpret_cast<const float4*>(records + t * token_stride + 288);
      const float4 lo4 = ds[0], hi4 = ds[1];
      float mins = ByteToFloat(mn[0], 0) * lo4.x;
      mins = fmaf(ByteToFloat(mn[0], 1), lo4.y, mins);
      mins = fmaf(ByteToFloat(mn[0], 2), lo4.z, mins);
      mins = fmaf(ByteToFloat(mn[0], 3), lo4.w, mins);
      mins = fmaf(ByteToFloat(mn[1], 0), hi4.x, mins);
      mins = fmaf(ByteToFloat(mn[1], 1), hi4.y, mins);
      mins = fmaf(ByteToFloat(mn[1], 2), hi4.z, mins);
      mins = fmaf(ByteToFloat(mn[1], 3), hi4.w, mins);
      out[t] = fmaf(d, main[t], -(dmin * mins));
    }
  }
}

struct Tile {
  int row0;
  int half;   // super-blocks of one matrix: rows * nsb
  int total;  // of both
};

template <bool kGlu>
__device__ __forceinline__ Tile TileOf(int index, int rows_per_tile, int nrows, int nsb) {
  Tile t;
  t.row0 = index * rows_per_tile;
  t.half = min(rows_per_tile, nrows - t.row0) * nsb;
  t.total = kGlu ? 2 * t.half : t.half;
  return t;
}

typedef __attribute__((address_space(3))) void* LdsPointer;
typedef const __attribute__((address_space(1))) void* GlobalPointer;

// Queues the tile's chunks into the wave's buffer: chunk 64 j + lane at byte 16 (64 j + lane).
// kPacked: rows follow each other without a gap, so a matrix's part of the tile is one range.
template <bool kGlu, bool kPacked>
__device__ __forceinline__ void FetchTile(const llmp_vecq_desc& d, int64_t expert_block, const Tile& tile, int nsb,
                                          uint8_t* ring, int lane) {
  const int64_t first = expert_block + static_cast<int64_t>(tile.row0) * d.stride_row;
  const uint8_t* up = static_cast<const uint8_t*>(d.w) + first * 144;
  const uint8_t* gate = kGlu ? static_cast<const uint8_t*>(d.g) + first * 144 : nullptr;
  const int half = tile.half * kChunks;
  const int total = tile.total * kChunks;
#pragma unroll
  for (int j = 0; j < kChunks; ++j) {
    int c = j * kWave + lane;
    if (c < total) {
      const uint8_t* matrix = up;
      if (kGlu && c >= half) {
        matrix = gate;
        c -= half;
      }
      int64_t at;
      if constexpr (kPacked) {
        at = static_cast<int64_t>(c) * 16;
      } else {
        const int f = c / kChunks;
        const int row = f / nsb;
        at = (static_cast<int64_t>(row) * d.stride_row + (f - row * nsb)) * 144 + (c - f * kChunks) * 16;
      }
      __builtin_amdgcn_global_load_lds((GlobalPointer)(matrix + at), (LdsPointer)(ring + j * kWave * 16), 16, 0, 0);
    }
  }
}

// The tile has landed: all of this wave's memory operations are complete.
__device__ __forceinline__ void AwaitTile() {
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
  __builtin_amdgcn_wave_barrier();
  asm volatile("" ::: "memory");
}

__device__ __forceinline__ SuperBlock ReadSuperBlock(const uint8_t* ring, int lane) {
  SuperBlock b;
  const U32x4* mine = reinterpret_cast<const U32x4*>(ring + lane * 144);
  b.header = mine[0];
#pragma unroll
  for (int i = 0; i < 8; ++i) b.codes[i] = mine[1 + i];
  return b;
}

// grid (workgroups, slots); LDS: P tokens' records, then a tile buffer a wave.
template <int P, bool kGlu, int XT, bool kDump, bool kPacked>
__global__ __launch_bounds__(kGroup, 4) void VecQFlatQ4K(const VecQArgs a, const int rows_per_tile) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  __shared__ int pairs[kMaxPairs];
  __shared__ int count;

  const llmp_vecq_desc& d = a.d;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int nsb = d.ncols_x / 256;
  const int token_stride = nsb * kRecord;
  const int tiles = (d.nrows + rows_per_tile - 1) / rows_per_tile;
  uint8_t* ring = lds + P * token_stride + wave * kRing;
  float* partial = reinterpret_cast<float*>(ring);  // [P][64], once the super-blocks are read

  // A routed product's workgroup first learns whether it owns its expert.
  int expert = blockIdx.y;
  if (d.ids != nullptr) {
    expert = ResolvePairs(d, blockIdx.y, pairs, &count);
    if (count == 0) return;  // uniform over the workgroup
  }
  const int64_t expert_block = static_cast<int64_t>(expert) * d.stride_expert;
  const int first_tile = blockIdx.x * kWaves + wave;
  const int tile_step = gridDim.x * kWaves;
  if (d.ids == nullptr) ResolvePairs(d, blockIdx.y, pairs, &count);
  const int n = count;

  for (int p0 = 0; p0 < n; p0 += P) {
    const int m = min(P, n - p0);
    if (p0 > 0) __syncthreads();  // the last pass's readers of the records
    // The wave's first tile leaves before the activations are staged.
    int index = first_tile;
    Tile tile{};
    if (index < tiles) {
      tile = TileOf<kGlu>(index, rows_per_tile, d.nrows, nsb);
      FetchTile<kGlu, kPacked>(d, expert_block, tile, nsb, ring, lane);
    }
    for (int j = 0; j < m; ++j) {
      const int pr = pairs[p0 + j];
      const int token = pr >> 8;
      const int slot = pr & 0xFF;
      uint8_t* records = lds + j * token_stride;
      if constexpr (XT < 0) {
        const uint8_t* y = static_cast<const uint8_t*>(d.y) +
                           (static_cast<int64_t>(token) * d.y_token + static_cast<int64_t>(slot) * d.y_slot) * kQ8Block;
        StageRecordsQ8(y, d.ncols_x / 32, records);
      } else {
        const int64_t at = token * a.x_token + slot * a.x_slot;
        const void* x = XT == LLMP_X_F32 ? static_cast<const void*>(static_cast<const float*>(a.x) + at)
                                         : static_cast<const void*>(static_cast<const uint16_t*>(a.x) + at);
        StageRecordsX<XT>(x, d.ncols_x, records);
      }
    }
    __syncthreads();  // the records are staged; from here the waves run alone

    while (index < tiles) {
      AwaitTile();
      float out[P];
      if (lane < tile.total) {
        const int f = (kGlu && lane >= tile.half) ? lane - tile.half : lane;
        const int row = f / nsb;
        const int sb = f - row * nsb;
        const SuperBlock block = ReadSuperBlock(ring, lane);
        int32_t* dump = kDump ? a.dump + (static_cast<int64_t>(tile.row0 + row) * nsb + sb) * 16 : nullptr;
        DotSuperBlock<P, kDump>(block, lds + sb * kRecord, token_stride, m, out, dump);
      }
      // Every lane's reads of the buffer precede these writes in the wave's LDS order.
      if (lane < tile.total) {
#pragma unroll
        for (int t = 0; t < P; ++t) {
          if (t < m) partial[t * kWave + lane] = out[t];
        }
      }
      __builtin_amdgcn_wave_barrier();
      asm volatile("" ::: "memory");
      // One lane a (token, row): the row's super-block sums added in order.
      const int rows = tile.half / nsb;
      for (int item = lane; item < m * rows; item += kWave) {
        const int t = item / rows;
        const int r = item - t * rows;
        const float* pu = partial + t * kWave + r * nsb;
        float su = 0.0f, sg = 0.0f;
        for (int s = 0; s < nsb; ++s) {
          su += pu[s];
          if constexpr (kGlu) sg += pu[tile.half + s];
        }
        const int pr = pairs[p0 + t];
        float* dst =
            d.dst + static_cast<int64_t>(pr >> 8) * d.dst_token + static_cast<int64_t>(pr & 0xFF) * d.dst_slot;
        dst[tile.row0 + r] = kGlu ? Glu(d.glu, sg, su, d.limit) : su;
      }
      __builtin_amdgcn_wave_barrier();
      asm volatile("" ::: "memory");
      index += tile_step;
      if (index < tiles) {
        tile = TileOf<kGlu>(index, rows_per_tile, d.nrows, nsb);
        FetchTile<kGlu, kPacked>(d, expert_block, tile, nsb, ring, lane);
      }
    }
  }
}

// The rows of a tile: as many as a wave's 64 lanes hold (half of them a matrix with a GLU).
struct FlatPlan {
  int rows;
  size_t lds;
};

FlatPlan PlanFlat(int pass, int nsb, bool glu) {
  FlatPlan p;
  p.rows = (glu ? kWave / 2 : kWave) / nsb;
  p.lds = static_cast<size_t>(pass) * nsb * kRecord + static_cast<size_t>(kWaves) * kRing;
  return p;
}

constexpr size_t kFlatLdsLimit = 80 * 1024;  // two workgroups share a CU's 160 KB
int g_compute_units = 0;

template <int P, bool kGlu, int XT, bool kDump, bool kPacked>
void LaunchK(const VecQArgs& a, dim3 grid, const FlatPlan& plan, hipStream_t stream) {
  static bool sized = false;  // more than 64 KB of dynamic LDS must be asked for once
  if (!sized) {
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&VecQFlatQ4K<P, kGlu, XT, kDump, kPacked>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kFlatLdsLimit));
    sized = true;
  }
  hipLaunchKernelGGL((VecQFlatQ4K<P, kGlu, XT, kDump, kPacked>), grid, dim3(kGroup), plan.lds, stream, a, plan.rows);
}

template <int P, bool kGlu, int XT>
void LaunchT(const VecQArgs& a, dim3 grid, const FlatPlan& plan, hipStream_t stream) {
  const bool packed = a.d.stride_row == a.d.ncols_x / 256;
  if (a.dump != nullptr) {
    if constexpr (P == 1 && !kGlu && XT < 0) LaunchK<P, kGlu, XT, true, false>(a, grid, plan, stream);
    return;
  }
  if (packed) {
    LaunchK<P, kGlu, XT, false, true>(a, grid, plan, stream);
  } else {
    LaunchK<P, kGlu, XT, false, false>(a, grid, plan, stream);
  }
}

template <int P>
void LaunchP(const VecQArgs& a, int x_type, dim3 grid, const FlatPlan& plan, hipStream_t stream) {
  const bool glu = a.d.g != nullptr;
  switch (x_type) {
    case -1:
      glu ? LaunchT<P, true, -1>(a, grid, plan, stream) : LaunchT<P, false, -1>(a, grid, plan, stream);
      break;
    case LLMP_X_F32:
      glu ? LaunchT<P, true, LLMP_X_F32>(a, grid, plan, stream) : LaunchT<P, false, LLMP_X_F32>(a, grid, plan, stream);
      break;
    default:
      glu ? LaunchT<P, true, LLMP_X_BF16>(a, grid, plan, stream)
          : LaunchT<P, false, LLMP_X_BF16>(a, grid, plan, stream);
      break;
  }
}

}  // namespace

bool FlatQ4KTakes(const llmp_vecq_desc& d) {
  const int nsb = d.ncols_x / 256;
  const bool glu = d.g != nullptr;
  return nsb >= 1 && nsb <= (glu ? kWave / 2 : kWave) && PlanFlat(1, nsb, glu).lds <= kFlatLdsLimit;
}

void LaunchFlatQ4K(const VecQArgs& a, int x_type, int pass, hipStream_t stream) {
  const llmp_vecq_desc& d = a.d;
  const int nsb = d.ncols_x / 256;
  const bool glu = d.g != nullptr;
  if (pass > 1 && PlanFlat(4, nsb, glu).lds > kFlatLdsLimit) pass = 1;
  const FlatPlan plan = PlanFlat(pass > 1 ? 4 : 1, nsb, glu);
  if (g_compute_units == 0) {
    const int units = llmp_hip_compute_units();
    g_compute_units = units > 0 ? units : 256;
  }
  const int slots = d.ids != nullptr ? d.used * d.tokens : d.used;
  const int tiles = (d.nrows + plan.rows - 1) / plan.rows;
  // What is resident at once: two workgroups a CU, shared by the slots that have work.
  const int live_slots = d.ids != nullptr ? (d.used < slots ? d.used : slots) : slots;
  int groups = 2 * g_compute_units / (live_slots > 0 ? live_slots : 1);
  if (groups < 1) groups = 1;
  if (groups > (tiles + kWaves - 1) / kWaves) groups = (tiles + kWaves - 1) / kWaves;
  const dim3 grid(static_cast<unsigned>(groups), static_cast<unsigned>(slots));
  if (pass > 1) {
    LaunchP<4>(a, x_type, grid, plan, stream);
  } else {
    LaunchP<1>(a, x_type, grid, plan, stream);
  }
}

}  // namespace llmp_hip
