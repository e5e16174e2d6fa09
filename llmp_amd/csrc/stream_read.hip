// What a launch that only reads takes: the yardstick the mat-vec kernels' launch times are held against beside the
// published HBM peak. Every lane keeps eight 16-byte loads in flight, consecutive lanes consecutive chunks, a
// workgroup a contiguous run of the range; what is read is folded into one word a wave so that no load can be
// dropped.
#include <hip/hip_runtime.h>

#include "common.h"
#include "llmp_hip.h"

namespace llmp_hip {
namespace {

typedef uint32_t Chunk __attribute__((ext_vector_type(4)));

constexpr int kReadThreads = 256;
constexpr int kReadFlight = 8;

__global__ __launch_bounds__(kReadThreads) void StreamReadKernel(const Chunk* __restrict__ data, uint64_t chunks, uint32_t* sink) {
  // A workgroup's run: whole rounds of (threads x flight) chunks, the workgroups side by side.
  const uint64_t round = static_cast<uint64_t>(kReadThreads) * kReadFlight;
  const uint64_t rounds = (chunks + round - 1) / round;
  const uint64_t mine = (rounds + gridDim.x - 1) / gridDim.x;
  const uint64_t first = blockIdx.x * mine, last = min(first + mine, rounds);
  uint32_t folded = 0;
  for (uint64_t r = first; r < last; ++r) {
    Chunk v[kReadFlight];
#pragma unroll
    for (int i = 0; i < kReadFlight; ++i) {
      const uint64_t at = r * round + static_cast<uint64_t>(i) * kReadThreads + threadIdx.x;
      v[i] = at < chunks ? __builtin_nontemporal_load(data + at) : Chunk{0, 0, 0, 0};
    }
#pragma unroll
    for (int i = 0; i < kReadFlight; ++i) folded ^= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
  }
  for (int off = 32; off > 0; off >>= 1) folded ^= __shfl_xor(folded, off, 64);
  if ((threadIdx.x & 63) == 0) sink[blockIdx.x * (kReadThreads / 64) + threadIdx.x / 64] = folded;
}

}  // namespace
}  // namespace llmp_hip

using namespace llmp_hip;

extern "C" size_t llmp_hip_stream_read_sink(int compute_units) {
  return static_cast<size_t>(compute_units < 1 ? 1 : compute_units) * 8 * (kReadThreads / 64) * sizeof(uint32_t);
}

extern "C" int llmp_hip_stream_read(const void* data, size_t bytes, void* sink, int compute_units, void* stream) {
  BeginLaunches();
  if (data == nullptr || sink == nullptr) return Refuse(1, "stream_read: null operand");
  if (reinterpret_cast<uintptr_t>(data) % 16 != 0 || bytes % 16 != 0 || bytes == 0) return Refuse(1, "stream_read: whole 16-byte chunks");
  if (compute_units < 1) return Refuse(1, "stream_read: %d compute units", compute_units);
  hipLaunchKernelGGL(StreamReadKernel, dim3(static_cast<unsigned>(compute_units) * 8), dim3(kReadThreads), 0, static_cast<hipStream_t>(stream),
                     static_cast<const Chunk*>(data), static_cast<uint64_t>(bytes / 16), static_cast<uint32_t*>(sink));
  return LaunchStatus("stream_read");
}
