// The router's arithmetic for one token a wave (llmp.moe.router, src/kernels/ggml/llmp_fused.cu:1307-1407 of the
// reference; the definition is kRoute with kSoftmaxTopK, src/kernels/reference/exec.cc:1728-1818), shared by the router
// kernel and by the one-token expert layer, which routes in its own prologue: the same bits from both.
#ifndef LLMP_AMD_CSRC_MOE_ROUTER_H_
#define LLMP_AMD_CSRC_MOE_ROUTER_H_

#include <hip/hip_runtime.h>

#include "common.h"

namespace llmp_hip {

__device__ __forceinline__ float RouterWaveSum(float v) {
#pragma unroll
  for (int mask = 32; mask >= 1; mask >>= 1) v += ShflXor(v, mask);
  return v;
}

// Lane j < used leaves with pick j: its expert in *index and its weight in *weight. `l`: the token's `experts` logits,
// expert lane + 64 i in lane `lane`'s slot i. SLOTS: slots a lane holds (128 experts do not walk the sixteen that 1024 need).
template <int SLOTS>
__device__ __forceinline__ void RouteToken(const float* __restrict__ l, int experts, int used, int normalize, float scale, int lane,
                                           int* index_out, float* weight_out) {
  constexpr int kWave = 64;
  const int slots = (experts + kWave - 1) / kWave;
  float v[SLOTS];
  float p[SLOTS];
  float most = -INFINITY;
  bool nan = false;
#pragma unroll
  for (int i = 0; i < SLOTS; ++i) {
    const int e = i * kWave + lane;
    const bool have = i < slots && e < experts;
    v[i] = have ? l[e] : -INFINITY;
    nan = nan || (have && v[i] != v[i]);
    most = fmaxf(most, v[i]);  // ignores NaN, as std::max(max, v) does
  }
  // The maximum through keys whose unsigned order is the floats' (a NaN is no maximum here).
  const auto ordered = [](float f) {
    const uint32_t bits = __builtin_bit_cast(uint32_t, f == 0.0f ? 0.0f : f);  // -0 is +0
    return (bits & 0x80000000u) != 0 ? ~bits : bits | 0x80000000u;
  };
  {
    const uint32_t top = WaveMaxU32(most != most ? 0u : ordered(most));
    const uint32_t bits = (top & 0x80000000u) != 0 ? top & 0x7FFFFFFFu : ~top;
    most = __builtin_bit_cast(float, bits);
  }
  nan = __any(nan);
  // A row with a NaN or no finite maximum has no probabilities: every expert 0, so the first
  // `used` experts with zero weights (exec.cc:279-299 and the stable order of :303-315).
  const bool degenerate = nan || !(fabsf(most) < INFINITY);
  float sum = 0.0f;
  uint32_t key[SLOTS];  // 0: not an expert, or picked already
#pragma unroll
  for (int i = 0; i < SLOTS; ++i) {
    const int e = i * kWave + lane;
    const bool have = i < slots && e < experts;
    p[i] = have && !degenerate ? expf(v[i] - most) : 0.0f;
    sum += p[i];
    key[i] = !have ? 0u : degenerate ? 1u : ordered(v[i]);
  }
  const float total = RouterWaveSum(sum);
  const float inverse = total > 0.0f ? 1.0f / total : 0.0f;
  // Top `used` by logit (the probabilities' order without their rounding), lower index first
  // among equals; a degenerate row orders by index alone. A pick: the largest key, then the
  // lowest index among the lanes that hold it.
  float mine = 0.0f;
  float picked = 0.0f;
  int my_index = 0;
  for (int j = 0; j < used; ++j) {
    uint32_t best = 0u;
    uint32_t index = 0x7FFFFFFFu;
#pragma unroll
    for (int i = 0; i < SLOTS; ++i) {
      if (key[i] > best) {  // a lane's slots in index order: the first of equals stays
        best = key[i];
        index = static_cast<uint32_t>(i * kWave + lane);
      }
    }
    const uint32_t top = WaveMaxU32(best);
    const uint32_t chosen = WaveMinU32(best == top ? index : 0x7FFFFFFFu);
    const int owner = static_cast<int>(chosen & (kWave - 1));
    const int slot = static_cast<int>(chosen / kWave);
    float held = 0.0f;
#pragma unroll
    for (int i = 0; i < SLOTS; ++i) {
      if (i == slot) {
        held = p[i];
        if (lane == owner) key[i] = 0u;
      }
    }
    const float best_p = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, held), owner));
    const float q = best_p * inverse;
    if (lane == j) {
      mine = q;
      my_index = static_cast<int>(chosen);
    }
    picked += q;  // in pick order
  }
  const float denominator = normalize ? fmaxf(picked, 6.103515625e-5f) : 1.0f;  // 2^-14
  *index_out = my_index;
  *weight_out = mine / denominator * scale;
}

}  // namespace llmp_hip

#endif  // LLMP_AMD_CSRC_MOE_ROUTER_H_
