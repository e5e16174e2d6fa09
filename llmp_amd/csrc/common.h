// Shared host and device helpers of the gfx950 kernels.
#ifndef LLMP_AMD_CSRC_COMMON_H_
#define LLMP_AMD_CSRC_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace llmp_hip {

// ---- host: status of the calling thread's last refusal or fault.
void SetError(const char* format, ...) __attribute__((format(printf, 1, 2)));
// Called by an entry point once its checks have passed, before its first launch: forgets an error that an
// earlier, unrelated HIP call left on this thread, so that LaunchStatus judges this call's launches only.
void BeginLaunches();
// Asks once for `bytes` of dynamic LDS for a kernel that needs more than 64 KB. False: the runtime refused; the
// reason is recorded, the launch must be skipped, the next LaunchStatus returns the failure and `sized` stays
// clear so that the next call asks again.
bool AllowLds(const void* kernel, int bytes, bool* sized);
// 0 if the launches since BeginLaunches were accepted, else -(hipError_t) with the error recorded.
int LaunchStatus(const char* what);
int Refuse(int code, const char* format, ...) __attribute__((format(printf, 2, 3)));

constexpr int kWave = 64;

// ---- device: element conversions (src/kernels/device/float_formats.cuh:14-49).
__device__ __forceinline__ float HalfBitsToFloat(uint32_t bits) {
  return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(bits)));
}
__device__ __forceinline__ uint32_t FloatToHalfBits(float v) {
  return __builtin_bit_cast(uint16_t, static_cast<_Float16>(v));  // nearest even
}
__device__ __forceinline__ float Bf16BitsToFloat(uint32_t bits) {
  return __builtin_bit_cast(float, bits << 16);
}
__device__ __forceinline__ uint32_t FloatToBf16Bits(float v) {
  const uint32_t x = __builtin_bit_cast(uint32_t, v);
  const uint32_t quiet = (x >> 16) | 0x40u;                          // a NaN keeps its payload's top bits
  const uint32_t nearest = (x + 0x7FFFu + ((x >> 16) & 1u)) >> 16;  // ties to even
  return __builtin_isnan(v) ? quiet : nearest;
}
// E8M0: 2^(bits - 127); 0 is 2^-127 (a float subnormal), 0xFF NaN.
__device__ __forceinline__ float E8m0ToFloat(uint32_t bits) {
  if (bits == 0xFFu) return __builtin_nanf("");
  return bits == 0 ? __builtin_bit_cast(float, 0x00400000u) : __builtin_bit_cast(float, bits << 23);
}
// OCP E4M3 (bias 7, 0x7F/0xFF NaN, subnormals m * 2^-9).
__device__ __forceinline__ float E4m3ToFloat(uint32_t bits) {
  const uint32_t magnitude = bits & 0x7Fu;
  float v;
  if (magnitude == 0x7Fu) {
    v = __builtin_nanf("");
  } else if (magnitude < 8u) {
    v = static_cast<float>(magnitude) * 0.001953125f;
  } else {
    v = __builtin_bit_cast(float, (magnitude << 20) + (120u << 23));
  }
  return (bits & 0x80u) ? -v : v;
}

__device__ __forceinline__ int Dot4(int a, int b, int c) {
  return __builtin_amdgcn_sdot4(a, b, c, false);
}
// A 16-byte and a 4-byte-aligned 16-byte global load of weights, which are
// read once: non-temporal, so that they do not displace the activations.
typedef uint32_t U32x4 __attribute__((ext_vector_type(4)));
typedef U32x4 U32x4A4 __attribute__((aligned(4)));

// The value of lane `lane ^ mask` (every lane of the 2 * mask group active). Within a row of 16
// lanes by data-parallel moves, which cost a few cycles where a permute through LDS costs its
// latency: lane ^ 1 and lane ^ 2 are quad permutes, lane ^ 8 a rotation of the row by eight,
// lane ^ 4 a shift by four either way, each on the banks of four lanes it is right for.
template <typename T>
__device__ __forceinline__ T ShflXor(T v, int mask) {
  static_assert(sizeof(T) == 4, "32-bit values");
  const int bits = __builtin_bit_cast(int, v);
  int got;
  switch (mask) {
    case 1:
      got = __builtin_amdgcn_mov_dpp(bits, 0xB1, 0xF, 0xF, true);  // quad_perm:[1,0,3,2]
      break;
    case 2:
      got = __builtin_amdgcn_mov_dpp(bits, 0x4E, 0xF, 0xF, true);  // quad_perm:[2,3,0,1]
      break;
    case 4:
      got = __builtin_amdgcn_update_dpp(bits, bits, 0x104, 0xF, 0x5, false);  // row_shl:4, banks 0 and 2
      got = __builtin_amdgcn_update_dpp(got, bits, 0x114, 0xF, 0xA, false);   // row_shr:4, banks 1 and 3
      break;
    case 8:
      got = __builtin_amdgcn_mov_dpp(bits, 0x128, 0xF, 0xF, true);  // row_ror:8
      break;
    default:
      return __shfl_xor(v, mask, kWave);
  }
  return __builtin_bit_cast(T, got);
}

// The largest / smallest value over a full wave's 64 lanes, the same in every lane (and known to
// the compiler as such). Within a row of 16 lanes by data-parallel moves: lane ^ 1, lane ^ 2,
// then the mirrored half row and the mirrored row, whose lanes already agree within quads and
// half rows; across the four rows by lane reads.
__device__ __forceinline__ uint32_t WaveMaxU32(uint32_t v) {
  v = max(v, static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(v), 0xB1, 0xF, 0xF, true)));
  v = max(v, static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(v), 0x4E, 0xF, 0xF, true)));
  v = max(v, static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(v), 0x141, 0xF, 0xF, true)));
  v = max(v, static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(v), 0x140, 0xF, 0xF, true)));
  const uint32_t a = __builtin_amdgcn_readlane(static_cast<int>(v), 0);
  const uint32_t b = __builtin_amdgcn_readlane(static_cast<int>(v), 16);
  const uint32_t c = __builtin_amdgcn_readlane(static_cast<int>(v), 32);
  const uint32_t d = __builtin_amdgcn_readlane(static_cast<int>(v), 48);
  return max(max(a, b), max(c, d));
}
__device__ __forceinline__ uint32_t WaveMinU32(uint32_t v) { return ~WaveMaxU32(~v); }

}  // namespace llmp_hip

#endif  // LLMP_AMD_CSRC_COMMON_H_
