// Device code shared by the llmp.vecq kernels: the Q8_1 block quantizer, the launch
// arguments, the GLU, and the (token, slot) pair list of a workgroup.
#ifndef LLMP_AMD_CSRC_VECQ_COMMON_H_
#define LLMP_AMD_CSRC_VECQ_COMMON_H_

#include <hip/hip_runtime.h>

#include "common.h"
#include "llmp_hip.h"

namespace llmp_hip {

constexpr int kMaxPairs = 128;  // used * tokens of a routed product
constexpr int kThreads = 256;
constexpr int kQ8Block = 36;
constexpr int kLdsBudget = 60 * 1024;

// ------------------------------------------------------------- quantizer

// Eight lanes quantize one 32-value block, four consecutive values a lane:
// amax over the block, d = amax / 127 (IEEE), q = round-half-away(x / d), 0 for
// a zero block. `sum` is the 32 values added in a 32-lane xor butterfly's order
// (offsets 16, 8, 4, 2, 1 over one value a lane), whatever the lane mapping.
struct Q8Block {
  float d;
  float sum;
  uint32_t codes;  // four int8, the first value in the low byte
};

__device__ __forceinline__ Q8Block QuantizeQ8Block(float x0, float x1, float x2, float x3) {
#pragma clang fp contract(off)
  float amax = fmaxf(fmaxf(fabsf(x0), fabsf(x1)), fmaxf(fabsf(x2), fabsf(x3)));
  amax = fmaxf(amax, ShflXor(amax, 4));
  amax = fmaxf(amax, ShflXor(amax, 2));
  amax = fmaxf(amax, ShflXor(amax, 1));
  const float d = amax / 127.0f;
  Q8Block out;
  out.d = d;
  int q0 = 0, q1 = 0, q2 = 0, q3 = 0;
  if (amax != 0.0f) {
    q0 = static_cast<int>(roundf(x0 / d));
    q1 = static_cast<int>(roundf(x1 / d));
    q2 = static_cast<int>(roundf(x2 / d));
    q3 = static_cast<int>(roundf(x3 / d));
  }
  out.codes = (q0 & 0xFF) | ((q1 & 0xFF) << 8) | ((q2 & 0xFF) << 16) | (static_cast<uint32_t>(q3 & 0xFF) << 24);
  // value 4L + c pairs with 4(L ^ 4) + c at offset 16, 4(L ^ 2) + c at 8, 4(L ^ 1) + c at 4.
  float s0 = x0, s1 = x1, s2 = x2, s3 = x3;
#pragma unroll
  for (int mask = 4; mask >= 1; mask >>= 1) {
    s0 = s0 + ShflXor(s0, mask);
    s1 = s1 + ShflXor(s1, mask);
    s2 = s2 + ShflXor(s2, mask);
    s3 = s3 + ShflXor(s3, mask);
  }
  out.sum = (s0 + s2) + (s1 + s3);
  return out;
}

template <int XT>
__device__ __forceinline__ void Load4(const void* base, int64_t at, int64_t k, float (&v)[4]) {
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int64_t i = at + c;
    float x = 0.0f;
    if (i < k) {
      if constexpr (XT == LLMP_X_F32) {
        x = static_cast<const float*>(base)[i];
      } else if constexpr (XT == LLMP_X_BF16) {
        x = Bf16BitsToFloat(static_cast<const uint16_t*>(base)[i]);
      } else {
        x = HalfBitsToFloat(static_cast<const uint16_t*>(base)[i]);
      }
    }
    v[c] = x;
  }
}

// Four consecutive elements at `at`, zero past k; one vector load when `wide` says the
// row allows it (alignment, checked once a row).
template <int XT>
__device__ __forceinline__ void Load4Wide(const void* base, int64_t at, int64_t k, bool wide, float (&v)[4]) {
  if (wide && at + 4 <= k) {
    if constexpr (XT == LLMP_X_F32) {
      const float4 f = *reinterpret_cast<const float4*>(static_cast<const float*>(base) + at);
      v[0] = f.x, v[1] = f.y, v[2] = f.z, v[3] = f.w;
    } else {
      const uint2 u = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(base) + at);
      if constexpr (XT == LLMP_X_BF16) {
        v[0] = Bf16BitsToFloat(u.x & 0xFFFFu), v[1] = Bf16BitsToFloat(u.x >> 16);
        v[2] = Bf16BitsToFloat(u.y & 0xFFFFu), v[3] = Bf16BitsToFloat(u.y >> 16);
      } else {
        v[0] = HalfBitsToFloat(u.x & 0xFFFFu), v[1] = HalfBitsToFloat(u.x >> 16);
        v[2] = HalfBitsToFloat(u.y & 0xFFFFu), v[3] = HalfBitsToFloat(u.y >> 16);
      }
    }
    return;
  }
  Load4<XT>(base, at, k, v);
}

// ------------------------------------------------------------------ vecq

struct VecQArgs {
  llmp_vecq_desc d;
  const void* x;  // fused form: unquantized rows
  int64_t x_token;
  int64_t x_slot;
  int kp;         // k rounded up to 512: the staged codes' stride
  int32_t* dump;  // block sums, or null
  // Sorted rows: expert e computes rows offsets[e] .. offsets[e + 1] of the activations into
  // the same rows of the output (d.ids unused), or null.
  const int32_t* offsets;
  // The row-a-lane form over weights the importer relaid out (llmp_hip_relayout_q4_k_tiles64): within every 64
  // rows the blocks lie super-block after super-block, a super-block's 64 rows together.
  int tiled = 0;
  // The row-a-lane form: units of each wave's quarter of a row whose tokens are staged at a time (0: the whole row's).
  int span = 0;
  // and the super-blocks of a row in a piece: 1 (tiles of 64 rows), 2 or 4 (of 32 or 16, Q4_K); 0: the launcher's choice.
  int parts = 0;
};

__device__ __forceinline__ float Silu(float x) {
#pragma clang fp contract(off)
  return x / (1.0f + expf(-x));
}
__device__ __forceinline__ float GeluTanh(float x) {
#pragma clang fp contract(off)
  return 0.5f * x * (1.0f + tanhf(0.79788456080286535588f * x * (1.0f + 0.044715f * x * x)));
}
// src/kernels/ggml/vecq.cu:186-195
__device__ __forceinline__ float Glu(int glu, float gate, float up, float limit) {
#pragma clang fp contract(off)
  if (glu == LLMP_GLU_GEGLU) return GeluTanh(gate) * up;
  if (glu == LLMP_GLU_SWIGLU_CLAMP) {
    gate = fminf(gate, limit);
    up = fmaxf(fminf(up, limit), -limit);
  }
  return Silu(gate) * up;
}


// The pairs a workgroup computes, in pair order, and its expert: a dense or grouped
// product's slot is its matrix; of a routed product's pairs, the first naming an expert
// owns it and computes every pair that names it (src/kernels/ggml/vecq.cu:504-546, with
// 64-lane ballots). Returns the expert; `count` is 0 for a workgroup that owns nothing.
// Ends with a workgroup barrier.
__device__ __forceinline__ int ResolvePairs(const llmp_vecq_desc& d, int slot_index, int* pairs, int* count) {
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  int expert;
  if (d.ids == nullptr) {
    expert = slot_index;
    if (tid < d.tokens) pairs[tid] = (tid << 8) | expert;
    if (tid == 0) *count = d.tokens;
  } else {
    const int s = slot_index;
    expert = d.ids[(s / d.used) * d.ids_stride + (s % d.used)];
    if (tid < kWave) {
      const int total = d.tokens * d.used;
      int n = 0;
      bool owner = true;
      for (int base = 0; base < total && owner; base += kWave) {
        const int s2 = base + lane;
        const int t = s2 / d.used;
        const int u = s2 % d.used;
        const bool match = s2 < total && d.ids[t * d.ids_stride + u] == expert;
        const unsigned long long ballot = __ballot(match);
        if (n == 0 && ballot != 0) owner = base + __ffsll(ballot) - 1 == s;
        if (owner && match) pairs[n + __popcll(ballot & ((1ull << lane) - 1ull))] = (t << 8) | u;
        n += __popcll(ballot);
      }
      if (lane == 0) *count = owner ? n : 0;
    }
  }
  __syncthreads();
  return expert;
}

// The same list for a routed product whose workgroups share an expert's work instead: every pair's workgroups
// get the pairs that name their pair's expert, in pair order, and `rank`, their own pair's place among them. An
// expert that n pairs name then has n pairs' workgroups, each taking a share of its rows against all n tokens: the
// weights are still read once, and the workgroups an expert gets grow with the tokens it serves. Every wave works
// the list out for itself from one round of loads (the pairs' experts, two a lane) and writes the same words to
// `pairs`, so no wave waits for another here: a wave reads back what it wrote itself.
__device__ __forceinline__ int SharePairs(const llmp_vecq_desc& d, int slot_index, int* pairs, int* count, int* rank) {
  const int lane = threadIdx.x & (kWave - 1);
  const int s = slot_index;
  const int total = d.tokens * d.used;
  const int s0 = lane, s1 = kWave + lane;
  const int t0 = s0 / d.used, u0 = s0 - t0 * d.used;
  const int t1 = s1 / d.used, u1 = s1 - t1 * d.used;
  const int id0 = s0 < total ? d.ids[t0 * d.ids_stride + u0] : 0;
  const int id1 = s1 < total ? d.ids[t1 * d.ids_stride + u1] : 0;
  const int expert = s < kWave ? __builtin_amdgcn_readlane(id0, s) : __builtin_amdgcn_readlane(id1, s - kWave);
  const bool match0 = s0 < total && id0 == expert;
  const bool match1 = s1 < total && id1 == expert;
  const unsigned long long named0 = __ballot(match0), named1 = __ballot(match1);
  const unsigned long long below = (1ull << lane) - 1ull;
  const int n0 = __popcll(named0);
  if (match0) pairs[__popcll(named0 & below)] = (t0 << 8) | u0;
  if (match1) pairs[n0 + __popcll(named1 & below)] = (t1 << 8) | u1;
  *count = n0 + __popcll(named1);
  *rank = s < kWave ? __popcll(named0 & ((1ull << s) - 1ull)) : n0 + __popcll(named1 & ((1ull << (s - kWave)) - 1ull));
  return expert;
}

// The decoded header of a super-block: 6-bit scales and minimums as bytes g of sc[g / 4],
// mn[g / 4] (the packing of tests/unit/dsv4_fast_test.cc:180-183 of the reference).
struct Q4KHeader {
  uint32_t sc[2], mn[2];
  float d, dmin;
};

__device__ __forceinline__ Q4KHeader DecodeQ4KHeader(const U32x4& h) {
  Q4KHeader out;
  const uint32_t s0 = h.y, s1 = h.z, s2 = h.w;
  out.sc[0] = s0 & 0x3F3F3F3Fu;
  out.sc[1] = (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u);
  out.mn[0] = s1 & 0x3F3F3F3Fu;
  out.mn[1] = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
  out.d = HalfBitsToFloat(h.x & 0xFFFFu);
  out.dmin = HalfBitsToFloat(h.x >> 16);
  return out;
}

// The flat kernels' launch (vecq_flat.hip): whether a product's shape and alignment fit them,
// and the launch. x_type -1: Q8_1 activations.
bool FlatTakes(int type, const llmp_vecq_desc& d, bool whole_rows = false);
// `deep`: two tile buffers a wave where the shape allows (one token a pass, packed rows).
void LaunchFlat(int type, const VecQArgs& a, int x_type, int pass, bool deep, hipStream_t stream);

// The matrix-core kernels for 2 to 16 tokens a pass over Q8_1 activations (vecq_mma.hip).
bool MmaTakes(int type, const llmp_vecq_desc& d);
void LaunchMma(int type, const VecQArgs& a, hipStream_t stream);

// The row-a-lane kernel for 2 to 8 tokens of a dense or grouped Q4_K product over Q8_1 activations (vecq_rows.hip).
constexpr int kRowsTokensMost = 16;  // of the row-a-lane form (the operation's most): eight a launch
bool RowsTakes(int type, const llmp_vecq_desc& d, int parts = 1);  // parts: the units of a row in a piece (tiles of 64 / parts rows)
bool RowsTiledTakes(int type, const llmp_vecq_desc& d);
void LaunchRows(const VecQArgs& a, hipStream_t stream);

}  // namespace llmp_hip

#endif  // LLMP_AMD_CSRC_VECQ_COMMON_H_
