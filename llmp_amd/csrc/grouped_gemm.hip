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
// so the operands are decoded instead: an E2M1 value (two significant bits, 0.5 to 6) times a UE4M3 scale (four
// significant bits, 2^-9 to 448) has six significant bits between 2^-10 and 2688, exact in F16, and the product runs
// on v_mfma_f32_16x16x32_f16 over exactly the values the format defines (v_cvt_scalef32_pk_f16_fp4 makes two halves
// of a byte of codes, one packed multiply applies the scale: an operation a value). The group sizes are known only on
// the device: a fixed grid of workgroups walks the list of 64 x 64 output tiles that the offsets imply (no host
// synchronization, no arguments built on the device, no scratch), which also makes the launch replay-invariant for a
// captured graph. A tile's K is walked 128 values at a time. A's 64 x 128 piece is decoded into LDS by the 256
// threads (32 values each: sixteen bytes of codes and two scales; only the sixteens of rows that hold a row of the
// group), two buffers, one barrier a step. Wave w multiplies the tile's columns 16 w + [0, 16) by those rows, and B's
// values for it are decoded by the lanes that multiply them, straight into the instruction's operand: no other wave
// wants them, so they do not pass through LDS. Codes and scales are asked for three steps ahead, held in registers,
// every load made whatever the tile's edges (from a place inside the operand, its values then given the scale zero):
// a load under a branch makes every later wait a wait for all loads. The groups' offsets are read into LDS a chunk
// at a time and a tile's group found by a search there: at the routed layers' sizes (128 groups of some 32 rows) a
// walk over the offsets in device memory, a round trip a group for every workgroup, took longer than the products.

#include <hip/hip_runtime.h>

#include <type_traits>

#include "common.h"
#include "llmp_hip.h"

namespace llmp_hip {
namespace {

typedef float Float4 __attribute__((ext_vector_type(4)));
typedef _Float16 Half2 __attribute__((ext_vector_type(2)));
typedef _Float16 Half8 __attribute__((ext_vector_type(8)));

constexpr int kTile = 64;            // rows and columns of an output tile
constexpr int kStepK = 128;          // K values of a step
// An LDS row of 128 F16 values: chunk j (32 values, 64 bytes) at 64 j + 32 (j / 2), rows 304 bytes (76 dwords) apart.
// Eight lanes' 16-byte accesses then cover all 32 banks once, both for the readers (eight rows, one chunk: 12 i mod 32
// are the eight multiples of four) and for the writers (two rows' four chunks: 0, 16, 8, 24 and the same plus 12).
constexpr int kRowBytes = 304;
__host__ __device__ constexpr int ChunkAt(int j) { return 64 * j + 32 * (j >> 1); }
constexpr int kPieceBytes = kTile * kRowBytes;
constexpr int kGroupedLds = 2 * kPieceBytes;  // A's piece, two buffers
constexpr int kAhead = 3;            // steps whose codes and scales are on their way
constexpr int kThreads = 256;
constexpr int kChunk = 128;          // groups whose offsets are in LDS at a time

// moe_cutlass.h:42-46.
__host__ __device__ __forceinline__ uint64_t SfOffset(uint64_t row, uint64_t block, uint64_t blocks) {
  return (((row / 128) * (blocks / 4)) + (block / 4)) * 512 + ((row % 32) * 16) + (((row % 128) / 32) * 4) + (block % 4);
}

// src/kernels/reference/decode.cc:407-411: E4M3's value up to 0x7E, NaN from 0x7F on. Exact in F16. Two scales (the
// low two bytes of `bits`) at once: the hardware's E4M3 has its NaN at 0x7F and negative values from 0x80, which are
// made NaN here.
__device__ __forceinline__ Half2 Ue4m3Pair(uint32_t bits) {
  const Half2 value = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(bits, 1.0f, false);
  const uint32_t nan = 0x7E007E00u;
  const uint32_t signs = bits & 0x8080u;  // bit 7 of byte 0 and bit 15 of byte 1
  uint32_t out = __builtin_bit_cast(uint32_t, value);
  if (signs & 0x80u) out = (out & 0xFFFF0000u) | (nan & 0xFFFFu);
  if (signs & 0x8000u) out = (out & 0xFFFFu) | (nan & 0xFFFF0000u);
  return __builtin_bit_cast(Half2, out);
}
__device__ __forceinline__ Half2 BothLow(Half2 v) { return Half2{v[0], v[0]}; }
__device__ __forceinline__ Half2 BothHigh(Half2 v) { return Half2{v[1], v[1]}; }

// What a thread brings of one step for one operand: 32 values of a row, and the dword of four scales that holds
// their two.
struct Brought {
  U32x4 codes;
  uint32_t scales;
};

// Sixteen values (two dwords of codes, element 2i in byte i's low nibble) times their scale, as F16 (exact).
__device__ __forceinline__ void DecodeSixteen(uint32_t w0, uint32_t w1, Half2 scale, U32x4& lo, U32x4& hi) {
  Half2 v[8];
  v[0] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w0, 1.0f, 0) * scale;
  v[1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w0, 1.0f, 1) * scale;
  v[2] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w0, 1.0f, 2) * scale;
  v[3] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w0, 1.0f, 3) * scale;
  v[4] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w1, 1.0f, 0) * scale;
  v[5] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w1, 1.0f, 1) * scale;
  v[6] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w1, 1.0f, 2) * scale;
  v[7] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w1, 1.0f, 3) * scale;
  lo = U32x4{__builtin_bit_cast(uint32_t, v[0]), __builtin_bit_cast(uint32_t, v[1]), __builtin_bit_cast(uint32_t, v[2]),
             __builtin_bit_cast(uint32_t, v[3])};
  hi = U32x4{__builtin_bit_cast(uint32_t, v[4]), __builtin_bit_cast(uint32_t, v[5]), __builtin_bit_cast(uint32_t, v[6]),
             __builtin_bit_cast(uint32_t, v[7])};
}

// A thread's 32 values of one operand into its place of a piece (`to`: its row's chunk `seg`).
__device__ __forceinline__ void DecodeInto(uint8_t* to_bytes, const U32x4& codes, uint32_t scales) {
  U32x4* to = reinterpret_cast<U32x4*>(to_bytes);
  const Half2 pair = Ue4m3Pair(scales);
  U32x4 lo, hi;
  DecodeSixteen(codes.x, codes.y, BothLow(pair), lo, hi);
  to[0] = lo, to[1] = hi;
  DecodeSixteen(codes.z, codes.w, BothHigh(pair), lo, hi);
  to[2] = lo, to[3] = hi;
}

struct GroupedArgs {
  llmp_grouped_gemm g;
};

__global__ __launch_bounds__(kThreads, 3) void GroupedNvfp4Kernel(const GroupedArgs args) {
  const llmp_grouped_gemm& g = args.g;
  extern __shared__ __attribute__((aligned(16))) uint8_t pieces[];  // [buffer][64 rows] of A
  __shared__ int s_first[kChunk + 1];    // the chunk's groups' first rows (and the last's end)
  __shared__ int s_scale_rows[kChunk];   // their first rows among the activations' scales
  __shared__ int s_before[kChunk + 1];   // the tiles of the chunk's groups before each (and of all)
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int n16 = lane & 15, q = lane >> 4;
  const int tiles_n = (g.n + kTile - 1) / kTile;
  const uint64_t row_bytes = static_cast<uint64_t>(g.k) / 2;
  const uint64_t blocks = static_cast<uint64_t>(g.k) / 16;
  const int steps = (g.k + kStepK - 1) / kStepK;       // k is a multiple of 64: the last step may be half
  const int piece_row = tid >> 2, piece_seg = tid & 3;  // the thread's 32 values of each 64 x 128 piece
  const int scales_shift = (piece_seg & 1) * 16;        // its two scales in the dword of four

  // The groups' offsets are read a chunk at a time into LDS, where their tile counts are summed: a workgroup then
  // finds the group of each of its tiles by a search there. (Read one after the other from device memory, every
  // group's offsets cost every workgroup a round trip: 128 groups took longer than the products.)
  int base = 0;  // tiles of the chunks before this one
  for (int chunk0 = 0; chunk0 < g.groups; chunk0 += kChunk) {
    const int count = min(kChunk, g.groups - chunk0);
    __syncthreads();  // the last chunk's readers
    for (int i = tid; i <= count; i += kThreads) s_first[i] = g.offsets[chunk0 + i];
    for (int i = tid; i < count; i += kThreads) s_scale_rows[i] = g.sf_rows[chunk0 + i];
    __syncthreads();
    if (wave == 0) {
      // Lane l sums groups 2 l and 2 l + 1 of the chunk; the lanes' totals are scanned across the wave.
      static_assert(kChunk == 128, "two groups a lane");
      int mine[2];
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int i = 2 * lane + j;
        const int rows = i < count ? s_first[i + 1] - s_first[i] : 0;
        mine[j] = rows > 0 ? ((rows + kTile - 1) / kTile) * tiles_n : 0;
      }
      int before = mine[0] + mine[1];  // becomes the tiles of the lanes before this one
      const int own = before;
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const int other = __shfl_up(before, off, 64);
        if (lane >= off) before += other;
      }
      before -= own;
      s_before[2 * lane] = before;
      s_before[2 * lane + 1] = before + mine[0];
      if (lane == 63) s_before[kChunk] = before + own;
    }
    __syncthreads();
    const int total = s_before[kChunk];
    // This workgroup's tiles of the chunk: every gridDim.x-th place of the whole list, a place p holding tile
    // (p % 8) * ceil(total / 8) + p / 8. Workgroups go to the device's eight dies in turn, so with a grid that is a multiple of
    // eight (the usual compute-unit counts) a die takes a run of consecutive tiles: a group's tiles, which read the same rows of A, share that
    // die's L2 (spread over the dies, every die fetched A for itself: 1.4 times the bytes).
    const int run = (total + 7) / 8;
    int place = (static_cast<int>(blockIdx.x) - base % static_cast<int>(gridDim.x) + static_cast<int>(gridDim.x)) % static_cast<int>(gridDim.x);
    for (; place < 8 * run; place += gridDim.x) {
      const int t = (place & 7) * run + (place >> 3);
      if (t >= total) continue;
      // The last group whose tiles start at or before t (groups without tiles share their start with the next).
      int lo = 0, hi = count - 1;
      while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (s_before[mid] <= t) lo = mid; else hi = mid - 1;
      }
      const int e_in = __builtin_amdgcn_readfirstlane(lo);
      const int e = chunk0 + e_in;
      const int first = __builtin_amdgcn_readfirstlane(s_first[e_in]);
      const int rows = __builtin_amdgcn_readfirstlane(s_first[e_in + 1]) - first;
      const int tile = t - __builtin_amdgcn_readfirstlane(s_before[e_in]);
      const uint8_t* weights = static_cast<const uint8_t*>(g.weights) + static_cast<uint64_t>(e) * g.expert_stride;
      const uint8_t* b_codes = weights + g.codes_offset;
      const uint8_t* b_scales = weights + g.scales_offset;
      const uint64_t scale_row0 = static_cast<uint64_t>(__builtin_amdgcn_readfirstlane(s_scale_rows[e_in]));
      const int row0 = (tile / tiles_n) * kTile, col0 = (tile % tiles_n) * kTile;
      // Wave w multiplies the tile's columns 16 w + [0, 16) by every sixteen rows that hold a row of the group (one to
      // four; the routed layers' groups have some 32 rows): it reads its quarter of B and the live part of A.
      const int live = min(4, (rows - row0 + 15) / 16);
      Float4 acc[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[r] = Float4{0.0f, 0.0f, 0.0f, 0.0f};
      const bool a_wanted = piece_row < 16 * live;  // the same for a wave's threads: they share sixteen rows
      // Every load is made, from a place inside the operand (a row past the tile's last is the last row, a half
      // step's missing half its first), and what must be zero gets the scale zero at its decoding: a load under a
      // branch would make every later wait a wait for all loads, and the steps ahead would not be ahead.
      // B: lane (n16, q) of wave w brings and decodes what it multiplies itself, column 16 w + n16's values 32 q + [0, 32)
      // of a step, straight into the instruction's operand: no other wave wants them, so they do not pass through LDS.
      const bool a_live = row0 + piece_row < rows;
      const bool b_live = col0 + 16 * wave + n16 < g.n;
      const int a_row = min(row0 + piece_row, rows - 1), b_row = min(col0 + 16 * wave + n16, g.n - 1);
      const uint8_t* a_from = static_cast<const uint8_t*>(g.a) + static_cast<uint64_t>(first + a_row) * row_bytes;
      const uint8_t* b_from = b_codes + static_cast<uint64_t>(b_row) * row_bytes;
      // The thread's two scales of a step are blocks 8 step + 2 seg and the next: neighbours in an atom's row.
      const uint8_t* a_scale_from = static_cast<const uint8_t*>(g.a_scales) + SfOffset(scale_row0 + a_row, 0, blocks);
      const uint8_t* b_scale_from = b_scales + SfOffset(b_row, 0, blocks);
      auto in_k = [&](int step, int seg) { return step * kStepK + seg * 32 < g.k; };
      // Blocks 8 step + 2 seg, + 1: atom step * 2 + seg / 2 of the row's (512 bytes an atom), places 2 (seg % 2), + 1:
      // the dword of the four is loaded (a narrower load's widening would be placed at the load, and wait there).
      auto bring = [&](const uint8_t* codes, const uint8_t* scales, int step, int seg) {
        const bool whole = in_k(step, seg);
        Brought x;
        x.codes = *reinterpret_cast<const U32x4*>(codes + (whole ? static_cast<uint32_t>(step * (kStepK / 2) + seg * 16) : 0u));
        x.scales = *reinterpret_cast<const uint32_t*>(scales + (whole ? static_cast<uint32_t>((step * 2 + (seg >> 1)) * 512) : 0u));
        return x;
      };
      // Both operands' codes and scales are asked for three steps ahead. (A column's next four steps asked for
      // together, 256 consecutive bytes of its row at a time, were no faster.)
      Brought ring[kAhead + 1], b_ring[kAhead + 1];
#pragma unroll
      for (int i = 0; i < kAhead; ++i) {
        ring[i] = bring(a_from, a_scale_from, min(i, steps - 1), piece_seg);
        b_ring[i] = bring(b_from, b_scale_from, min(i, steps - 1), q);
      }
      __syncthreads();  // the last tile's readers of both buffers
      // (The count of live row groups a constant in the loop: reads under a branch each would each be waited for.)
      auto walk = [&](auto live_c) {
      constexpr int kLive = decltype(live_c)::value;
      for (int s0 = 0; s0 < steps; s0 += kAhead + 1) {
#pragma unroll
        for (int u = 0; u <= kAhead; ++u) {
          const int step = s0 + u;
          ring[(u + kAhead) % (kAhead + 1)] = bring(a_from, a_scale_from, min(step + kAhead, steps - 1), piece_seg);
          b_ring[(u + kAhead) % (kAhead + 1)] = bring(b_from, b_scale_from, min(step + kAhead, steps - 1), q);
          if (step < steps) {  // (the same for every thread; no load inside)
            uint8_t* a_piece = pieces + (u & 1) * kPieceBytes;
            if (a_wanted) {
              DecodeInto(a_piece + piece_row * kRowBytes + ChunkAt(piece_seg), ring[u].codes,
                         a_live && in_k(step, piece_seg) ? ring[u].scales >> scales_shift : 0u);
            }
            U32x4 w8[4];
            DecodeInto(reinterpret_cast<uint8_t*>(w8), b_ring[u].codes, b_live && in_k(step, q) ? b_ring[u].scales >> ((q & 1) * 16) : 0u);
            __syncthreads();  // the piece is whole; the other buffer's readers (a step ago) passed the barrier before
            // Lane (n16, q) holds k = 32 q + 8 j + [0, 8) of its row on both sides: the same labels, so the
            // instruction's sum over its 32 slots is the sum over those 32 values, and the four the step's.
            const uint8_t* x_from = a_piece + n16 * kRowBytes + ChunkAt(q);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
              for (int r = 0; r < kLive; ++r) {
                const U32x4 x8 = *reinterpret_cast<const U32x4*>(x_from + r * 16 * kRowBytes + j * 16);
                acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(Half8, x8), __builtin_bit_cast(Half8, w8[j]), acc[r], 0, 0, 0);
              }
            }
          }
        }
      }
      };
      switch (live) {
        case 1: walk(std::integral_constant<int, 1>{}); break;
        case 2: walk(std::integral_constant<int, 2>{}); break;
        case 3: walk(std::integral_constant<int, 3>{}); break;
        default: walk(std::integral_constant<int, 4>{}); break;
      }
      // acc[r][i] = D[row 16 r + 4 q + i][column 16 wave + n16], rounded to BF16 once.
      uint16_t* d = static_cast<uint16_t*>(g.d);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int row = row0 + 16 * r + 4 * q + i, col = col0 + 16 * wave + n16;
          if (row < rows && col < g.n) d[static_cast<uint64_t>(first + row) * g.n + col] = static_cast<uint16_t>(FloatToBf16Bits(acc[r][i]));
        }
      }
    }
    base += 8 * run;
  }
}

bool g_grouped_sized = false;

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
  if ((reinterpret_cast<uintptr_t>(gemm->a) | reinterpret_cast<uintptr_t>(gemm->weights) | gemm->expert_stride | gemm->codes_offset) % 16 != 0)
    return Refuse(1, "moe.gemm: codes not 16-byte aligned");
  if ((reinterpret_cast<uintptr_t>(gemm->a_scales) | gemm->scales_offset) % 4 != 0) return Refuse(1, "moe.gemm: scales not 4-byte aligned");
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
  if (!AllowLds(reinterpret_cast<const void*>(&GroupedNvfp4Kernel), kGroupedLds, &g_grouped_sized)) return LaunchStatus("moe.gemm");
  // Three workgroups a compute unit are resident (registers): that many walk the tiles.
  hipLaunchKernelGGL(GroupedNvfp4Kernel, dim3(static_cast<unsigned>(3 * cus)), dim3(kThreads), kGroupedLds, static_cast<hipStream_t>(stream), args);
  const int status = LaunchStatus("moe.gemm");
  return status;
}
