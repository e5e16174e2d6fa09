// llmp.q8_1 and llmp.vecq for gfx950: the Q8_1 activation quantizer and the
// quantized mat-vec over Q8_0 / Q4_K weights (dense rows, grouped matrices,
// routed experts; with or without a fused gate/up GLU; 1..16 tokens).
//
// Shape of the product kernel. A workgroup is 4 wave64s. The tokens of a pass
// (P of them) are staged once into LDS as split Q8_1: the codes as a byte
// stream (16-byte aligned per 32-value block), the block scales as floats and,
// for Q4_K, the code sums of each 16-value half block. They come either from
// Q8_1 blocks in memory or, in the fused form, from the unquantized rows,
// quantized in the workgroup with the quantizer kernel's arithmetic. Then every
// group of LPR lanes streams one weight row: a lane owns a fixed 16-byte slice
// of each Q4_K super-block (two half sub-blocks of nibbles) or one pair of Q8_0
// blocks (68 bytes, 4-byte aligned), loads it straight from global memory a few
// units ahead of its use, multiplies it with the staged codes by v_dot4_i32_i8
// and folds the scales in fp32. A (token, row) sum never depends on what else
// the workgroup computes: per-lane sums in unit order, then a fixed xor
// butterfly over the row's lanes. No atomics on the result path.
//
// Reference behaviour restated here: src/kernels/ggml/vecq.cu:457-665 (kernel
// forms, pair ownership for routed experts), :186-195 (GLU), :398-418 (Q8_0
// dot), tests/unit/dsv4_fast_test.cc:167-195 (Q4_K dot).

#include <hip/hip_runtime.h>

#include "common.h"
#include "llmp_hip.h"
#include "vecq_common.h"

namespace llmp_hip {
namespace {

// grid (ceil(blocks / 32), rows, planes), 256 threads: 32 blocks a workgroup.
__global__ __launch_bounds__(kThreads) void QuantizeQ8Kernel(const float* __restrict__ x, uint8_t* __restrict__ out,
                                                            int64_t k, int64_t padded_k, int64_t row_stride,
                                                            int64_t rows, int64_t plane_stride) {
  const int lane8 = threadIdx.x & 7;
  const int64_t block = static_cast<int64_t>(blockIdx.x) * 32 + (threadIdx.x >> 3);
  const int64_t blocks = padded_k / 32;
  const int64_t row = blockIdx.y;
  const int64_t plane = blockIdx.z;
  // Whole 8-lane groups leave together: the shuffles below stay within a group.
  if (block >= blocks) return;
  const float* src = x + plane * plane_stride + row * row_stride;
  float v[4];
  Load4<LLMP_X_F32>(src, block * 32 + lane8 * 4, k, v);
  const Q8Block q = QuantizeQ8Block(v[0], v[1], v[2], v[3]);
  uint8_t* dst = out + ((plane * rows + row) * blocks + block) * kQ8Block;
  *reinterpret_cast<uint32_t*>(dst + 4 + lane8 * 4) = q.codes;
  if (lane8 == 0) *reinterpret_cast<uint32_t*>(dst) = FloatToHalfBits(q.d) | (FloatToHalfBits(q.sum) << 16);
}

// The staged activations of a pass.
struct Staged {
  const uint8_t* codes;    // [P][kp]
  const float* scales;     // [P][kp / 32]
  const uint32_t* halves;  // [P][kp / 32]: Q4_K, per (super-block, lane slice) two int16 sums
};

// Stages token slot j from Q8_1 blocks in memory: a thread a block.
template <bool kQ4K>
__device__ __forceinline__ void StageQ8(const uint8_t* __restrict__ y, int blocks, int kp, int j, uint8_t* codes,
                                        float* scales, uint32_t* halves) {
  for (int b = threadIdx.x; b < blocks; b += kThreads) {
    const uint32_t* src = reinterpret_cast<const uint32_t*>(y + static_cast<int64_t>(b) * kQ8Block);
    uint32_t w[9];
#pragma unroll
    for (int i = 0; i < 9; ++i) w[i] = src[i];
    uint4* dst = reinterpret_cast<uint4*>(codes + static_cast<int64_t>(j) * kp + b * 32);
    dst[0] = make_uint4(w[1], w[2], w[3], w[4]);
    dst[1] = make_uint4(w[5], w[6], w[7], w[8]);
    scales[j * (kp / 32) + b] = HalfBitsToFloat(w[0] & 0xFFFFu);
    if constexpr (kQ4K) {
      int lo = 0, hi = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        lo = Dot4(0x01010101, static_cast<int>(w[1 + i]), lo);
        hi = Dot4(0x01010101, static_cast<int>(w[5 + i]), hi);
      }
      // Sub-block g = b % 8 of its super-block: slice 2(g / 2) + h, half g % 2.
      auto* h16 = reinterpret_cast<int16_t*>(halves + j * (kp / 32));
      const int at = ((b & ~7) + ((b & 7) >> 1) * 2) * 2 + (b & 1);
      h16[at] = static_cast<int16_t>(lo);
      h16[at + 2] = static_cast<int16_t>(hi);
    }
  }
}

// Stages token slot j from an unquantized row: eight lanes a block, the loads of four
// blocks a lane issued together (one memory round trip for rows up to 4096 values).
template <bool kQ4K, int XT>
__device__ __forceinline__ void StageX(const void* __restrict__ x, int k, int kp, int j, uint8_t* codes, float* scales,
                                       uint32_t* halves) {
  constexpr int kStep = kThreads / 8;  // blocks a sweep of the workgroup
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
      *reinterpret_cast<uint32_t*>(codes + static_cast<int64_t>(j) * kp + b * 32 + lane8 * 4) = q.codes;
      // The products read the scale as the Q8_1 block stores it: rounded to F16.
      if (lane8 == 0) scales[j * (kp / 32) + b] = HalfBitsToFloat(FloatToHalfBits(q.d));
      if constexpr (kQ4K) {
        int s = Dot4(0x01010101, static_cast<int>(q.codes), 0);
        s += ShflXor(s, 1);
        s += ShflXor(s, 2);
        if ((lane8 & 3) == 0) {
          auto* h16 = reinterpret_cast<int16_t*>(halves + j * (kp / 32));
          const int h = lane8 >> 2;
          h16[((b & ~7) + ((b & 7) >> 1) * 2 + h) * 2 + (b & 1)] = static_cast<int16_t>(s);
        }
      }
    }
  }
}

// ---- Q4_K: a lane's 16-byte slice j of a super-block holds values
// 16h .. 16h + 15 of sub-blocks 2p (low nibbles) and 2p + 1 (high), p = j / 2,
// h = j % 2.
struct Q4KUnit {
  U32x4 header;  // d, dmin, scales[12]
  U32x4 codes;
};

__device__ __forceinline__ Q4KUnit LoadQ4K(const uint8_t* row, int unit) {
  const uint8_t* block = row + static_cast<int64_t>(unit >> 3) * 144;
  Q4KUnit u;
  u.header = __builtin_nontemporal_load(reinterpret_cast<const U32x4*>(block));
  u.codes = __builtin_nontemporal_load(reinterpret_cast<const U32x4*>(block + 16 + (unit & 7) * 16));
  return u;
}

struct Q4KScales {
  float dsc0, dsc1, dm0, dm1;
};

__device__ __forceinline__ Q4KScales DecodeQ4KScales(const U32x4& header, int p) {
#pragma clang fp contract(off)
  const int shift = 16 * (p & 1);
  const uint32_t a = (header.y >> shift) & 0xFFFFu;  // scales[0..3]
  const uint32_t b = (header.z >> shift) & 0xFFFFu;  // scales[4..7]
  const uint32_t c = (header.w >> shift) & 0xFFFFu;  // scales[8..11]
  uint32_t sc, mn;
  if (p < 2) {
    sc = a & 0x3F3Fu;
    mn = b & 0x3F3Fu;
  } else {
    sc = (c & 0x0F0Fu) | ((a >> 2) & 0x3030u);
    mn = ((c >> 4) & 0x0F0Fu) | ((b >> 2) & 0x3030u);
  }
  const float d = HalfBitsToFloat(header.x & 0xFFFFu);
  const float dmin = HalfBitsToFloat(header.x >> 16);
  Q4KScales s;
  s.dsc0 = d * static_cast<float>(sc & 0xFFu);
  s.dsc1 = d * static_cast<float>(sc >> 8);
  s.dm0 = dmin * static_cast<float>(mn & 0xFFu);
  s.dm1 = dmin * static_cast<float>(mn >> 8);
  return s;
}

template <int P, bool kDump>
__device__ __forceinline__ void DotQ4K(const Q4KUnit& u, int unit, int m, const Staged& act, int kp, float (&acc)[P],
                                       int32_t* dump) {
#pragma clang fp contract(off)
  const int j = unit & 7;
  const int sb = unit >> 3;
  const int p = j >> 1;
  const int h = j & 1;
  const Q4KScales s = DecodeQ4KScales(u.header, p);
  const uint32_t raw[4] = {u.codes.x, u.codes.y, u.codes.z, u.codes.w};
  int lo[4], hi[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    lo[i] = static_cast<int>(raw[i] & 0x0F0F0F0Fu);
    hi[i] = static_cast<int>((raw[i] >> 4) & 0x0F0F0F0Fu);
  }
#pragma unroll
  for (int t = 0; t < P; ++t) {
    if (t < m) {
      const uint8_t* codes = act.codes + static_cast<int64_t>(t) * kp + sb * 256 + p * 64 + h * 16;
      const uint4 a0 = *reinterpret_cast<const uint4*>(codes);
      const uint4 a1 = *reinterpret_cast<const uint4*>(codes + 32);
      const float2 d8 = *reinterpret_cast<const float2*>(act.scales + t * (kp / 32) + sb * 8 + p * 2);
      const uint32_t sums = act.halves[t * (kp / 32) + sb * 8 + j];
      int prod0 = Dot4(lo[0], static_cast<int>(a0.x), 0);
      prod0 = Dot4(lo[1], static_cast<int>(a0.y), prod0);
      prod0 = Dot4(lo[2], static_cast<int>(a0.z), prod0);
      prod0 = Dot4(lo[3], static_cast<int>(a0.w), prod0);
      int prod1 = Dot4(hi[0], static_cast<int>(a1.x), 0);
      prod1 = Dot4(hi[1], static_cast<int>(a1.y), prod1);
      prod1 = Dot4(hi[2], static_cast<int>(a1.z), prod1);
      prod1 = Dot4(hi[3], static_cast<int>(a1.w), prod1);
      const int sum0 = static_cast<int16_t>(sums & 0xFFFFu);
      const int sum1 = static_cast<int16_t>(sums >> 16);
      if (kDump && dump != nullptr) {
        int32_t* out = dump + static_cast<int64_t>(sb) * 16;
        atomicAdd(out + 2 * p, prod0);
        atomicAdd(out + 2 * p + 1, prod1);
        atomicAdd(out + 8 + 2 * p, sum0);
        atomicAdd(out + 8 + 2 * p + 1, sum1);
      }
      // Spelled out so that every instantiation rounds at the same places.
      const float t0 = fmaf(s.dsc0, static_cast<float>(prod0), -(s.dm0 * static_cast<float>(sum0)));
      const float t1 = fmaf(s.dsc1, static_cast<float>(prod1), -(s.dm1 * static_cast<float>(sum1)));
      acc[t] = fmaf(d8.y, t1, fmaf(d8.x, t0, acc[t]));
    }
  }
}

// ---- Q8_0: a unit is a pair of blocks, 68 bytes at a 4-byte boundary:
// {d0, q0[0:2]} q0[2:30] {q0[30:32], d1} q1[0:32].
struct Q8Pair {
  uint32_t w[17];
};

__device__ __forceinline__ Q8Pair LoadQ8Pair(const uint8_t* row, int unit) {
  const uint8_t* at = row + static_cast<int64_t>(unit) * 68;
  Q8Pair u;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const U32x4 v = __builtin_nontemporal_load(reinterpret_cast<const U32x4A4*>(at) + i);
    u.w[4 * i + 0] = v.x;
    u.w[4 * i + 1] = v.y;
    u.w[4 * i + 2] = v.z;
    u.w[4 * i + 3] = v.w;
  }
  u.w[16] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(at) + 16);
  return u;
}

template <int P, bool kDump>
__device__ __forceinline__ void DotQ8Pair(const Q8Pair& u, int unit, int m, const Staged& act, int kp, float (&acc)[P],
                                          int32_t* dump) {
#pragma clang fp contract(off)
  const float d0 = HalfBitsToFloat(u.w[0] & 0xFFFFu);
  const float d1 = HalfBitsToFloat(u.w[8] >> 16);
  int q0[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) q0[i] = static_cast<int>(__builtin_amdgcn_alignbyte(u.w[i + 1], u.w[i], 2));
#pragma unroll
  for (int t = 0; t < P; ++t) {
    if (t < m) {
      const uint4* codes = reinterpret_cast<const uint4*>(act.codes + static_cast<int64_t>(t) * kp + unit * 64);
      const float2 d8 = *reinterpret_cast<const float2*>(act.scales + t * (kp / 32) + unit * 2);
      int prod0 = 0, prod1 = 0;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const uint4 a = codes[i];
        prod0 = Dot4(q0[4 * i + 0], static_cast<int>(a.x), prod0);
        prod0 = Dot4(q0[4 * i + 1], static_cast<int>(a.y), prod0);
        prod0 = Dot4(q0[4 * i + 2], static_cast<int>(a.z), prod0);
        prod0 = Dot4(q0[4 * i + 3], static_cast<int>(a.w), prod0);
        const uint4 b = codes[2 + i];
        prod1 = Dot4(static_cast<int>(u.w[9 + 4 * i + 0]), static_cast<int>(b.x), prod1);
        prod1 = Dot4(static_cast<int>(u.w[9 + 4 * i + 1]), static_cast<int>(b.y), prod1);
        prod1 = Dot4(static_cast<int>(u.w[9 + 4 * i + 2]), static_cast<int>(b.z), prod1);
        prod1 = Dot4(static_cast<int>(u.w[9 + 4 * i + 3]), static_cast<int>(b.w), prod1);
      }
      if (kDump && dump != nullptr) {
        atomicAdd(dump + 2 * unit, prod0);
        atomicAdd(dump + 2 * unit + 1, prod1);
      }
      // src/kernels/ggml/vecq.cu:416
      acc[t] = fmaf(d1 * d8.y, static_cast<float>(prod1), fmaf(d0 * d8.x, static_cast<float>(prod0), acc[t]));
    }
  }
}

// A single Q8_0 block at a 2-byte boundary (rows of an odd block count, or
// strides that break the pairs' alignment).
struct Q8Single {
  uint16_t h[17];
};

__device__ __forceinline__ Q8Single LoadQ8Single(const uint8_t* row, int unit) {
  const uint16_t* at = reinterpret_cast<const uint16_t*>(row + static_cast<int64_t>(unit) * 34);
  Q8Single u;
#pragma unroll
  for (int i = 0; i < 17; ++i) u.h[i] = at[i];
  return u;
}

template <int P, bool kDump>
__device__ __forceinline__ void DotQ8Single(const Q8Single& u, int unit, int m, const Staged& act, int kp,
                                            float (&acc)[P], int32_t* dump) {
#pragma clang fp contract(off)
  const float d0 = HalfBitsToFloat(u.h[0]);
  int q[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) q[i] = static_cast<int>(u.h[1 + 2 * i] | (static_cast<uint32_t>(u.h[2 + 2 * i]) << 16));
#pragma unroll
  for (int t = 0; t < P; ++t) {
    if (t < m) {
      const uint4* codes = reinterpret_cast<const uint4*>(act.codes + static_cast<int64_t>(t) * kp + unit * 32);
      const float d8 = act.scales[t * (kp / 32) + unit];
      const uint4 a = codes[0];
      const uint4 b = codes[1];
      int prod = Dot4(q[0], static_cast<int>(a.x), 0);
      prod = Dot4(q[1], static_cast<int>(a.y), prod);
      prod = Dot4(q[2], static_cast<int>(a.z), prod);
      prod = Dot4(q[3], static_cast<int>(a.w), prod);
      prod = Dot4(q[4], static_cast<int>(b.x), prod);
      prod = Dot4(q[5], static_cast<int>(b.y), prod);
      prod = Dot4(q[6], static_cast<int>(b.z), prod);
      prod = Dot4(q[7], static_cast<int>(b.w), prod);
      if (kDump && dump != nullptr) atomicAdd(dump + unit, prod);
      acc[t] = fmaf(d0 * d8, static_cast<float>(prod), acc[t]);
    }
  }
}

enum Form { kFormQ4K = 0, kFormQ8Pair = 1, kFormQ8Single = 2 };

template <int FORM>
struct FormTraits;
template <>
struct FormTraits<kFormQ4K> {
  using Unit = Q4KUnit;
  static constexpr int kBlockBytes = 144;
  __device__ static Unit Load(const uint8_t* row, int unit) { return LoadQ4K(row, unit); }
  template <int P, bool kDump>
  __device__ static void Dot(const Unit& u, int unit, int m, const Staged& a, int kp, float (&acc)[P], int32_t* dump) {
    DotQ4K<P, kDump>(u, unit, m, a, kp, acc, dump);
  }
  __host__ __device__ static int Units(int k) { return k / 256 * 8; }
  __host__ __device__ static int DumpInts(int k) { return k / 256 * 16; }
};
template <>
struct FormTraits<kFormQ8Pair> {
  using Unit = Q8Pair;
  static constexpr int kBlockBytes = 34;
  __device__ static Unit Load(const uint8_t* row, int unit) { return LoadQ8Pair(row, unit); }
  template <int P, bool kDump>
  __device__ static void Dot(const Unit& u, int unit, int m, const Staged& a, int kp, float (&acc)[P], int32_t* dump) {
    DotQ8Pair<P, kDump>(u, unit, m, a, kp, acc, dump);
  }
  __host__ __device__ static int Units(int k) { return k / 64; }
  __host__ __device__ static int DumpInts(int k) { return k / 32; }
};
template <>
struct FormTraits<kFormQ8Single> {
  using Unit = Q8Single;
  static constexpr int kBlockBytes = 34;
  __device__ static Unit Load(const uint8_t* row, int unit) { return LoadQ8Single(row, unit); }
  template <int P, bool kDump>
  __device__ static void Dot(const Unit& u, int unit, int m, const Staged& a, int kp, float (&acc)[P], int32_t* dump) {
    DotQ8Single<P, kDump>(u, unit, m, a, kp, acc, dump);
  }
  __host__ __device__ static int Units(int k) { return k / 32; }
  __host__ __device__ static int DumpInts(int k) { return k / 32; }
};

// LPR lanes a row, P tokens a pass, D units in flight a lane.
// XT < 0: activations are Q8_1 blocks; else the unquantized element type.
template <int FORM, int LPR, int P, int D, bool kGlu, int XT, bool kDump>
__global__ __launch_bounds__(kThreads) void VecQKernel(const VecQArgs a) {
  using T = FormTraits<FORM>;
  using Unit = typename T::Unit;
  constexpr bool kQ4K = FORM == kFormQ4K;
  constexpr int kRowsPerWave = kWave / LPR;
  constexpr int kRowsPerGroup = kRowsPerWave * (kThreads / kWave);

  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  __shared__ int pairs[kMaxPairs];  // token << 8 | slot
  __shared__ int count;

  const llmp_vecq_desc& d = a.d;
  const int kp = a.kp;
  uint8_t* codes = lds;
  float* scales = reinterpret_cast<float*>(lds + static_cast<int64_t>(P) * kp);
  uint32_t* halves = reinterpret_cast<uint32_t*>(scales + P * (kp / 32));
  const Staged act{codes, scales, halves};

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int expert = ResolvePairs(d, blockIdx.y, pairs, &count);
  const int n = count;
  if (n == 0) return;  // uniform over the workgroup

  const int row = blockIdx.x * kRowsPerGroup + wave * kRowsPerWave + lane / LPR;
  const int sub = lane % LPR;
  const bool live = row < d.nrows;
  const int64_t row_at =
      (static_cast<int64_t>(expert) * d.stride_expert + static_cast<int64_t>(live ? row : d.nrows - 1) * d.stride_row) *
      T::kBlockBytes;
  const uint8_t* wrow = static_cast<const uint8_t*>(d.w) + row_at;
  const uint8_t* grow = kGlu ? static_cast<const uint8_t*>(d.g) + row_at : nullptr;
  const int units = T::Units(d.ncols_x);
  int32_t* dump = kDump && live ? a.dump + static_cast<int64_t>(row) * T::DumpInts(d.ncols_x) : nullptr;

  for (int p0 = 0; p0 < n; p0 += P) {
    const int m = min(P, n - p0);
    // D units in flight: the loads of unit i + D are issued before unit i's arithmetic, and
    // the first D before the activations are staged (they depend on nothing staged).
    Unit wu[D];
    Unit gu[kGlu ? D : 1];
#pragma unroll
    for (int i = 0; i < D; ++i) {
      const int unit = sub + i * LPR;
      if (unit < units) {
        wu[i] = T::Load(wrow, unit);
        if constexpr (kGlu) gu[i] = T::Load(grow, unit);
      }
    }
    for (int j = 0; j < m; ++j) {
      const int pr = pairs[p0 + j];
      const int token = pr >> 8;
      const int slot = pr & 0xFF;
      if constexpr (XT < 0) {
        const uint8_t* y = static_cast<const uint8_t*>(d.y) +
                           (static_cast<int64_t>(token) * d.y_token + static_cast<int64_t>(slot) * d.y_slot) * kQ8Block;
        StageQ8<kQ4K>(y, d.ncols_x / 32, kp, j, codes, scales, halves);
      } else {
        const int64_t at = token * a.x_token + slot * a.x_slot;
        const void* x = XT == LLMP_X_F32 ? static_cast<const void*>(static_cast<const float*>(a.x) + at)
                                         : static_cast<const void*>(static_cast<const uint16_t*>(a.x) + at);
        StageX<kQ4K, XT>(x, d.ncols_x, kp, j, codes, scales, halves);
      }
    }
    __syncthreads();

    float acc[P];
    float accg[kGlu ? P : 1];
#pragma unroll
    for (int t = 0; t < P; ++t) acc[t] = 0.0f;
#pragma unroll
    for (int t = 0; t < (kGlu ? P : 1); ++t) accg[t] = 0.0f;

    for (int base = sub; base < units; base += D * LPR) {
#pragma unroll
      for (int i = 0; i < D; ++i) {
        const int unit = base + i * LPR;
        const Unit w_now = wu[i];
        Unit g_now;
        if constexpr (kGlu) g_now = gu[i];
        const int next = unit + D * LPR;
        if (next < units) {
          wu[i] = T::Load(wrow, next);
          if constexpr (kGlu) gu[i] = T::Load(grow, next);
        }
        if (unit < units) {
          T::template Dot<P, kDump>(w_now, unit, m, act, kp, acc, dump);
          if constexpr (kGlu) T::template Dot<P, false>(g_now, unit, m, act, kp, accg, nullptr);
        }
      }
    }

#pragma unroll
    for (int t = 0; t < P; ++t) {
#pragma unroll
      for (int mask = LPR / 2; mask >= 1; mask >>= 1) {
        acc[t] += ShflXor(acc[t], mask);
        if constexpr (kGlu) accg[t] += ShflXor(accg[t], mask);
      }
      if (t < m && sub == 0 && live) {
        const int pr = pairs[p0 + t];
        float* dst = d.dst + static_cast<int64_t>(pr >> 8) * d.dst_token + static_cast<int64_t>(pr & 0xFF) * d.dst_slot;
        dst[row] = kGlu ? Glu(d.glu, accg[t], acc[t], d.limit) : acc[t];
      }
    }
    __syncthreads();  // the next pass restages
  }
}

// ------------------------------------------------------------ host side

struct Variant {
  const char* name;
  int lanes;   // a row
  int pass;    // tokens a pass
  int flight;  // units a lane keeps in flight
};

constexpr Variant kVariants[] = {
    {"lanes8 pass1 flight4", 8, 1, 4},   {"lanes8 pass2 flight3", 8, 2, 3},   {"lanes8 pass4 flight2", 8, 4, 2},
    {"lanes8 pass8 flight2", 8, 8, 2},   {"lanes16 pass1 flight4", 16, 1, 4}, {"lanes64 pass1 flight2", 64, 1, 2},
    // A lane a whole unit of a row, a Q4_K super-block or four Q8_0 blocks (vecq_flat.hip);
    // `lanes` 0 marks the form.
    // `flight`: tile buffers a wave.
    {"flat pass1", 0, 1, 1},             {"flat pass4", 0, 4, 1},             {"flat pass1 two tiles", 0, 1, 2},
    // Q4_K sub-block products on the int8 matrix cores, 16 tokens a pass (vecq_mma.hip);
    // `lanes` -1 marks the form.
    {"mma pass16", -1, 16, 1},
    // Q4_K, a weight row a lane, 2 to 8 tokens of a dense or grouped product on the 4 x 4 x 4 int8 matrix
    // instruction (vecq_rows.hip); `lanes` -2 marks the form.
    // `flight`: the units of a row in a piece, 0 for the launcher's choice (see the variants that follow the next).
    {"rows pass8", -2, 8, 0},
    // The same over weights relaid out at import into 64-row tiles (llmp_hip_relayout_q4_k_tiles64); `lanes` -3.
    // Never a default: the layout is the caller's to declare.
    {"rows pass8 tiles64", -3, 8, 1},
    // The row-a-lane form over the file's layout with its tile named: 64 rows (a piece a unit of each), or 32 or 16 (a
    // piece two or four units of each row, for matrices of few rows).
    {"rows pass8 rows64", -2, 8, 1},
    {"rows pass8 rows32", -2, 8, 2},
    {"rows pass8 rows16", -2, 8, 4},
};
constexpr int kMmaVariant = 9;
constexpr int kRowsVariant = 10;
constexpr int kFlatFirst = 6;
constexpr int kVariantCount = sizeof(kVariants) / sizeof(kVariants[0]);

size_t LdsBytes(int pass, int kp) { return static_cast<size_t>(pass) * (kp + kp / 8 + kp / 8); }

int PaddedK(int k) { return (k + 511) / 512 * 512; }

template <int FORM, int LPR, int P, int D, bool kGlu, int XT>
void LaunchOne(const VecQArgs& a, dim3 grid, size_t lds, hipStream_t stream) {
  if (a.dump != nullptr) {
    if constexpr (P == 1 && !kGlu && XT < 0 && LPR == 8) {
      hipLaunchKernelGGL((VecQKernel<FORM, LPR, P, D, kGlu, XT, true>), grid, dim3(kThreads), lds, stream, a);
    }
    return;
  }
  hipLaunchKernelGGL((VecQKernel<FORM, LPR, P, D, kGlu, XT, false>), grid, dim3(kThreads), lds, stream, a);
}

template <int FORM, int LPR, int P, int D>
void LaunchSource(const VecQArgs& a, int x_type, dim3 grid, size_t lds, hipStream_t stream) {
  const bool glu = a.d.g != nullptr;
  switch (x_type) {
    case -1:
      glu ? LaunchOne<FORM, LPR, P, D, true, -1>(a, grid, lds, stream)
          : LaunchOne<FORM, LPR, P, D, false, -1>(a, grid, lds, stream);
      break;
    case LLMP_X_F32:
      glu ? LaunchOne<FORM, LPR, P, D, true, LLMP_X_F32>(a, grid, lds, stream)
          : LaunchOne<FORM, LPR, P, D, false, LLMP_X_F32>(a, grid, lds, stream);
      break;
    default:
      glu ? LaunchOne<FORM, LPR, P, D, true, LLMP_X_BF16>(a, grid, lds, stream)
          : LaunchOne<FORM, LPR, P, D, false, LLMP_X_BF16>(a, grid, lds, stream);
      break;
  }
}

template <int FORM>
void LaunchVariant(const VecQArgs& a, int x_type, int variant, dim3 grid, size_t lds, hipStream_t stream) {
  switch (variant) {
    case 0:
      LaunchSource<FORM, 8, 1, 4>(a, x_type, grid, lds, stream);
      break;
    case 1:
      LaunchSource<FORM, 8, 2, 3>(a, x_type, grid, lds, stream);
      break;
    case 2:
      LaunchSource<FORM, 8, 4, 2>(a, x_type, grid, lds, stream);
      break;
    case 3:
      LaunchSource<FORM, 8, 8, 2>(a, x_type, grid, lds, stream);
      break;
    case 4:
      LaunchSource<FORM, 16, 1, 4>(a, x_type, grid, lds, stream);
      break;
    default:
      LaunchSource<FORM, 64, 1, 2>(a, x_type, grid, lds, stream);
      break;
  }
}

// The default configuration of a shape: the tokens of a pass first (each pass
// streams the weights again), then enough lanes a row to fill the device.
int DefaultVariant(int type, const llmp_vecq_desc& d, int kp, bool fused) {
  const int tokens = d.tokens;
  // Several tokens of a dense or grouped product over Q8_1 blocks: the matrix cores. A routed product's pairs
  // mostly name different experts, one or two tokens each: the flat form.
  // Q4_K, 2 to 8 tokens: a weight row a lane on the 4 x 4 x 4 instruction (at 3840 x 2 x 15360 with a GLU 17.8 us
  // at two and at four tokens, 21.3 at eight, against the 16 x 16 form's 25 at any count and the flat form's
  // four-token passes' 18 / 25 / 43). More tokens, and rows that form does not take: the 16 x 16 form, whose time
  // hardly depends on the tokens; the flat form's four-token pass stays under it up to five tokens for Q8_0
  // (15 / 17 / 20 / 27 us against 29 at 4096 x 14336).
  // The row-a-lane form's time hardly depends on the tokens. Its tiles are 64 rows a workgroup of four waves, or 32 or
  // 16 where the matrix has too few rows to give most compute units a tile of 64 (Q4_K 15360 x 3840, 60 tiles of 64:
  // 12.8 / 12.6 / 19 us at two, four and eight tokens in tiles of 16 against 24.8 / 24.5 / 34 in tiles of 64 and the
  // flat form's four-token passes' 13.7 / 25 / 44; 4096 x 4096: 7.0 / 7.1 / 8.0 against 10.5 / 10.5 / 12.4 and
  // 7.0 / 9.0 / 14.5). At two tokens the four-token pass is as fast, here a tenth faster (5120 x 5120: 8.0 against
  // 9.2 us) and there a tenth slower; the row-a-lane form from two tokens keeps a token's bits the same at every count.
  // Q8_0: the same (4096 x 14336: 16.2-17.4 us at 2 to 8 tokens against 19 / 22 / 31 for the four-token passes and
  // the 16 x 16 form; 14336 x 4096 in tiles of 16 rows: 17 us at 2 to 4 tokens and 22 at 5 to 8 against 26 / 35 / 44
  // / 54-82).
  if (tokens > 1 && !fused && (type == LLMP_TYPE_Q4_K || type == LLMP_TYPE_Q8_0) && RowsTakes(type, d)) {
    // (More than eight tokens are launches of eight: for rows too long for the 16 x 16 form. Q4_K 15360 x 3840 at
    // sixteen tokens: 2 x 19 us against the four-token passes' 82.)
    if (tokens <= 8 || !MmaTakes(type, d)) return kRowsVariant;
  }
  // (A plain Q4_K product of few rows: the four-token pass up to four tokens, 9.0 us against the 16 x 16 form's 13.1
  // at 4096 x 4096.)
  const bool few_rows = static_cast<int64_t>((d.nrows + 63) / 64) * d.used < 128;
  const int flat_up_to = type == LLMP_TYPE_Q8_0 ? 5 : d.g != nullptr || few_rows ? 4 : 2;
  if (tokens > flat_up_to && d.ids == nullptr && !fused && MmaTakes(type, d)) return kMmaVariant;
  if (FlatTakes(type, d)) return tokens > 1 ? kFlatFirst + 1 : kFlatFirst;
  int pass = tokens >= 5 ? 8 : tokens >= 3 ? 4 : tokens >= 2 ? 2 : 1;
  while (pass > 1 && LdsBytes(pass, kp) > static_cast<size_t>(kLdsBudget)) pass /= 2;
  switch (pass) {
    case 8:
      return 3;
    case 4:
      return 2;
    case 2:
      return 1;
    default:
      return 0;
  }
}

int CheckDesc(int type, const llmp_vecq_desc* d, bool sorted = false) {
  if (d == nullptr) return Refuse(1, "vecq: null descriptor");
  const bool legacy = type == LLMP_TYPE_Q4_0 || type == LLMP_TYPE_Q4_1 || type == LLMP_TYPE_Q5_0 || type == LLMP_TYPE_Q5_1 ||
                      type == LLMP_TYPE_IQ4_NL;  // 18-byte blocks as Q4_0's
  if (type != LLMP_TYPE_Q8_0 && type != LLMP_TYPE_Q4_K && type != LLMP_TYPE_Q5_K && type != LLMP_TYPE_Q6_K && type != LLMP_TYPE_MXFP4 &&
      !legacy)
    return Refuse(1, "vecq: weight type %d has no kernel", type);
  const int qk = type == LLMP_TYPE_Q4_K || type == LLMP_TYPE_Q5_K || type == LLMP_TYPE_Q6_K ? 256 : 32;
  if (d->w == nullptr || d->dst == nullptr) return Refuse(1, "vecq: null weights or output");
  if (d->ncols_x <= 0 || d->ncols_x % qk != 0) return Refuse(1, "vecq: k %d is not whole %d-value blocks", d->ncols_x, qk);
  if (d->nrows <= 0) return Refuse(1, "vecq: no rows");
  if (d->tokens < 1 || d->tokens > 16) return Refuse(1, "vecq: 1 to 16 tokens, not %d", d->tokens);
  // A pair packs its slot in 8 bits; sorted rows have no pairs.
  if (d->used < 1 || (!sorted && d->used > 256)) return Refuse(1, "vecq: 1 to 256 slots, not %d", d->used);
  if (d->ids != nullptr && d->used * d->tokens > kMaxPairs)
    return Refuse(1, "vecq: %d routed pairs exceed %d", d->used * d->tokens, kMaxPairs);
  if ((d->glu != LLMP_GLU_NONE) != (d->g != nullptr)) return Refuse(1, "vecq: gate weights exactly with a GLU");
  if (d->glu < 0 || d->glu > LLMP_GLU_GEGLU) return Refuse(1, "vecq: unknown GLU %d", d->glu);
  if (d->glu == LLMP_GLU_GEGLU && d->limit != 0.0f) return Refuse(1, "vecq: GeGLU takes no clamp limit");
  if (d->stride_row < d->ncols_x / qk) return Refuse(1, "vecq: rows overlap");
  if (reinterpret_cast<uintptr_t>(d->dst) % 4 != 0) return Refuse(1, "vecq: output not 4-byte aligned");
  const uintptr_t wa = reinterpret_cast<uintptr_t>(d->w) | reinterpret_cast<uintptr_t>(d->g);
  if (type == LLMP_TYPE_Q4_K && wa % 16 != 0) return Refuse(1, "vecq: Q4_K weights not 16-byte aligned");
  if (type == LLMP_TYPE_Q6_K && !FlatTakes(type, *d))
    return Refuse(1, "vecq: Q6_K takes 16-byte aligned weights, rows up to 16384 values (8192 with a GLU), packed or of a multiple "
                     "of eight blocks, matrices and experts of a multiple of eight blocks");
  // Q5_K runs through the flat form alone.
  if (type == LLMP_TYPE_Q5_K && !FlatTakes(type, *d))
    return Refuse(1, "vecq: Q5_K takes 16-byte aligned weights and rows whose staged activations fit LDS (up to 8192 values "
                     "with a GLU)");
  if (type == LLMP_TYPE_Q8_0 && wa % 2 != 0) return Refuse(1, "vecq: Q8_0 weights not 2-byte aligned");
  // The legacy 4/5-bit blocks run through the flat form alone: rows of whole 256 values at 16-byte boundaries.
  if (legacy && !FlatTakes(type, *d))
    return Refuse(1, "vecq: Q4_0, Q4_1, Q5_0, Q5_1 and IQ4_NL take rows of whole 256 values (up to 8192 with a GLU) whose rows, "
                     "matrices and experts start on 16-byte boundaries");
  // MXFP4 likewise; its 136-byte units come in pairs.
  if (type == LLMP_TYPE_MXFP4 && !FlatTakes(type, *d))
    return Refuse(1, "vecq: MXFP4 takes rows of whole 512 values (up to 8192 with a GLU) whose rows, matrices and experts "
                     "start on 16-byte boundaries");
  return 0;
}

int Launch(int type, const llmp_vecq_desc* d, const llmp_vecq_source* x, int variant, int32_t* dump, void* stream,
           const int32_t* offsets = nullptr) {
  if (const int bad = CheckDesc(type, d, offsets != nullptr); bad != 0) return bad;
  int x_type = -1;
  VecQArgs a{};
  a.d = *d;
  if (x != nullptr) {
    if (x->x == nullptr || x->x_type < LLMP_X_F32 || x->x_type > LLMP_X_BF16)
      return Refuse(1, "vecq: unquantized activations of an unknown type");
    x_type = x->x_type;
    a.x = x->x;
    a.x_token = x->x_token;
    a.x_slot = x->x_slot;
  } else if (d->y == nullptr || reinterpret_cast<uintptr_t>(d->y) % 4 != 0) {
    return Refuse(1, "vecq: Q8_1 activations null or not 4-byte aligned");
  }
  a.kp = PaddedK(d->ncols_x);
  a.dump = dump;
  a.offsets = offsets;
  if (variant < 0) variant = DefaultVariant(type, *d, a.kp, x != nullptr);
  if (variant >= kVariantCount) return Refuse(1, "vecq: no variant %d", variant);
  const Variant& v = kVariants[variant];
  if (type != LLMP_TYPE_Q8_0 && type != LLMP_TYPE_Q4_K && v.lanes != 0)
    return Refuse(1, "vecq: the legacy 4/5-bit blocks, IQ4_NL, Q5_K, Q6_K and MXFP4 take the flat variants");
  if (offsets != nullptr && v.lanes > 0) return Refuse(1, "vecq: sorted rows take the flat or the matrix-core form");
  if (v.lanes == -3) {
    if (offsets != nullptr || x != nullptr || dump != nullptr || !RowsTiledTakes(type, *d))
      return Refuse(1, "vecq: the row-a-lane form over relaid-out weights takes what the row-a-lane form takes, in whole tiles of "
                       "64 packed rows");
    a.tiled = type == LLMP_TYPE_Q8_0 ? 2 : 1;
    LaunchRows(a, static_cast<hipStream_t>(stream));
    return LaunchStatus("vecq");
  }
  if (v.lanes == -2) {
    if (offsets != nullptr || !RowsTakes(type, *d, v.flight > 0 ? v.flight : 1))
      return Refuse(1, "vecq: the row-a-lane form takes 2 to 16 tokens of a dense or grouped Q4_K product, rows of 1024 values "
                       "or more, or of a Q8_0 product, rows of whole 256 values, 512 or more, at 16-byte boundaries; tiles of 32 "
                       "or 16 rows, rows of two or four times that");
    if (x != nullptr) return Refuse(1, "vecq: the row-a-lane form takes Q8_1 activations");
    if (dump != nullptr) return Refuse(1, "vecq: block sums are of the one-token variants");
    a.tiled = type == LLMP_TYPE_Q8_0 ? 3 : 0;
    a.parts = v.flight;
    LaunchRows(a, static_cast<hipStream_t>(stream));
    return LaunchStatus("vecq");
  }
  if (v.lanes < 0) {
    if (!MmaTakes(type, *d))
      return Refuse(1, "vecq: the matrix-core form takes Q4_K rows up to 7168 values and Q8_0 rows of whole 128 values "
                       "up to 8192 at 4-byte boundaries");
    if (x != nullptr) return Refuse(1, "vecq: the matrix-core form takes Q8_1 activations");
    if (dump != nullptr) return Refuse(1, "vecq: block sums are of the one-token variants");
    LaunchMma(type, a, static_cast<hipStream_t>(stream));
    return LaunchStatus("vecq");
  }
  if (v.lanes == 0) {
    if (!FlatTakes(type, *d, dump != nullptr))
      return Refuse(1, "vecq: the flat form takes rows whose staged activations fit LDS beside three waves' tiles (Q4_K to "
                       "41216 values, Q8_0 to 46976; 8192 and 4096 with a GLU), Q8_0 and the legacy blocks in whole 256 (MXFP4 512) "
                       "values at 16-byte boundaries; block sums, rows up to 64 units");
    if (dump != nullptr && (d->ids != nullptr || d->tokens != 1 || d->used != 1 || d->g != nullptr))
      return Refuse(1, "vecq: block sums are of a dense one-token product");
    LaunchFlat(type, a, x_type, v.pass, v.flight == 2, static_cast<hipStream_t>(stream));
    return LaunchStatus("vecq");
  }
  const size_t lds = LdsBytes(v.pass, a.kp);
  if (lds > static_cast<size_t>(kLdsBudget))
    return Refuse(1, "vecq: %d tokens of k %d do not fit the staging area", v.pass, d->ncols_x);
  if (dump != nullptr && (d->ids != nullptr || d->tokens != 1 || d->used != 1 || d->g != nullptr))
    return Refuse(1, "vecq: block sums are of a dense one-token product");
  const int slots = d->ids != nullptr ? d->used * d->tokens : d->used;
  const int rows_per_group = (kWave / v.lanes) * (kThreads / kWave);
  const dim3 grid(static_cast<unsigned>((d->nrows + rows_per_group - 1) / rows_per_group),
                  static_cast<unsigned>(slots));
  const auto s = static_cast<hipStream_t>(stream);
  if (type == LLMP_TYPE_Q4_K) {
    LaunchVariant<kFormQ4K>(a, x_type, variant, grid, lds, s);
  } else {
    const bool pairs = d->ncols_x % 64 == 0 && d->stride_row % 2 == 0 && d->stride_expert % 2 == 0 &&
                       (reinterpret_cast<uintptr_t>(d->w) | reinterpret_cast<uintptr_t>(d->g)) % 4 == 0;
    if (pairs) {
      LaunchVariant<kFormQ8Pair>(a, x_type, variant, grid, lds, s);
    } else {
      LaunchVariant<kFormQ8Single>(a, x_type, variant, grid, lds, s);
    }
  }
  return LaunchStatus("vecq");
}

}  // namespace
}  // namespace llmp_hip

using namespace llmp_hip;

extern "C" int llmp_hip_q8_1_quantize(const float* x, void* out, int64_t k, int64_t padded_k, int64_t row_stride,
                                      int64_t rows, int64_t planes, int64_t plane_stride, void* stream) {
  BeginLaunches();
  if (x == nullptr || out == nullptr) return Refuse(1, "q8_1: null operand");
  if (k <= 0 || rows <= 0 || planes <= 0) return Refuse(1, "q8_1: empty input");
  if (padded_k < k || padded_k % 32 != 0) return Refuse(1, "q8_1: padded k %lld below k or not whole blocks", (long long)padded_k);
  if (rows > 65535 || planes > 65535) return Refuse(1, "q8_1: more than 65535 rows or planes");
  if (reinterpret_cast<uintptr_t>(x) % 4 != 0 || reinterpret_cast<uintptr_t>(out) % 4 != 0)
    return Refuse(1, "q8_1: operands not 4-byte aligned");
  const int64_t blocks = padded_k / 32;
  const dim3 grid(static_cast<unsigned>((blocks + 31) / 32), static_cast<unsigned>(rows), static_cast<unsigned>(planes));
  hipLaunchKernelGGL(QuantizeQ8Kernel, grid, dim3(kThreads), 0, static_cast<hipStream_t>(stream), x,
                     static_cast<uint8_t*>(out), k, padded_k, row_stride, rows, plane_stride);
  return LaunchStatus("q8_1");
}

extern "C" int llmp_hip_vecq(int type, const llmp_vecq_desc* d, int variant, void* stream) {
  BeginLaunches();
  return Launch(type, d, nullptr, variant, nullptr, stream);
}

extern "C" int llmp_hip_vecq_fused(int type, const llmp_vecq_desc* d, const llmp_vecq_source* x, int variant,
                                   void* stream) {
  BeginLaunches();
  if (x == nullptr) return Refuse(1, "vecq: null source");
  return Launch(type, d, x, variant, nullptr, stream);
}

extern "C" int llmp_hip_vecq_block_sums(int type, const llmp_vecq_desc* d, int variant, int32_t* sums, void* stream) {
  BeginLaunches();
  if (sums == nullptr) return Refuse(1, "vecq: null sums");
  if (const int bad = CheckDesc(type, d); bad != 0) return bad;  // before any plan divides by the row's units
  if (variant < 0) variant = FlatTakes(type, *d, true) ? kFlatFirst : 0;
  if (variant != 0 && variant != kFlatFirst) return Refuse(1, "vecq: block sums are of the one-token variants");
  return Launch(type, d, nullptr, variant, sums, stream);
}

extern "C" int llmp_hip_vecq_sorted(int type, const llmp_vecq_desc* d, const int32_t* offsets, int experts, int variant,
                                    void* stream) {
  BeginLaunches();
  if (offsets == nullptr || d == nullptr) return Refuse(1, "vecq: null offsets");
  if (experts < 1 || experts > 65535) return Refuse(1, "vecq: 1 to 65535 experts");
  llmp_vecq_desc sorted = *d;
  sorted.ids = nullptr;
  sorted.used = experts;  // a workgroup row an expert
  sorted.tokens = 1;      // the row counts come from the offsets
  sorted.y_slot = 0;
  sorted.dst_slot = 0;
  if (const int bad = CheckDesc(type, &sorted, true); bad != 0) return bad;  // before any plan divides by the row's units
  if (!FlatTakes(type, sorted) && !MmaTakes(type, sorted))
    return Refuse(1, "vecq: sorted rows take weights the flat or the matrix-core form takes");
  // An expert's rows are many tokens of one matrix: the matrix cores where they apply.
  if (variant < 0) variant = MmaTakes(type, *d) ? kMmaVariant : kFlatFirst + 1;
  return Launch(type, &sorted, nullptr, variant, nullptr, stream, offsets);
}

extern "C" int llmp_hip_vecq_variants(void) { return kVariantCount; }

extern "C" const char* llmp_hip_vecq_variant_name(int variant) {
  return variant >= 0 && variant < kVariantCount ? kVariants[variant].name : "default";
}
