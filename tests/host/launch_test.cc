// The HIP device-execution provider and the launch context (include/llmp_hip_launch.hpp) driven the way the
// reference drives its own (src/kernels/ggml/launch.h:135-222 over src/providers/device_execution.h:56-98): a run of
// two launchers with the pool's scratch between them, the same run captured and replayed, lanes, fences that are
// queried and released, and every refusal the interfaces promise. "host" needs no GPU (a provider for a device that
// is not there is refused, null arguments are); "device" runs on the GPU and compares a run's, a lane's and every
// replay's result with the same launchers called directly.
//
// Usage: launch_test host | device. Exit status 0 when every check holds.
#include <hip/hip_runtime_api.h>

#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "llmp_hip_launch.hpp"

namespace {

int g_failures = 0;

#define EXPECT(condition)                                                        \
  do {                                                                           \
    if (!(condition)) {                                                          \
      std::printf("%s:%d: EXPECT(%s) failed (%s)\n", __FILE__, __LINE__, #condition, llmp_hip_last_error()); \
      ++g_failures;                                                              \
    }                                                                            \
  } while (0)

using llmp_amd::Done;
using llmp_amd::ggml::CapturedGraph;
using llmp_amd::ggml::LaunchContext;
using llmp_amd::ggml::Launched;
using llmp_amd::ggml::LaunchFailure;
using llmp_amd::providers::FenceState;
using llmp_amd::providers::HipDeviceExecution;
using llmp_amd::providers::ProviderError;

struct Rng {
  std::uint64_t state;
  std::uint64_t Next() {
    std::uint64_t z = (state += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
  }
  float Unit() { return static_cast<float>(Next() >> 40) * (1.0f / 16777216.0f); }
};

void HostChecks() {
  // No device here (or none with this ordinal): nothing is made, and the reason is named.
  auto none = HipDeviceExecution::Create(1 << 20);
  EXPECT(!none && none.error() == ProviderError::kUnsupported && !none.detail().empty());
  llmp_hip_launch* context = nullptr;
  EXPECT(llmp_hip_launch_create(nullptr, 0, 1, 0, 0, &context) == 1 && context == nullptr);
  EXPECT(llmp_hip_execution_create(0, nullptr) == LLMP_PROVIDER_INVALID);
  EXPECT(llmp_hip_execution_destroy(nullptr) == 0);
  EXPECT(llmp_hip_launch_end(nullptr) == 1);
  EXPECT(llmp_hip_launch_faulted(nullptr) == 0 && llmp_hip_launch_lanes(nullptr) == 0 && llmp_hip_graph_nodes(nullptr) == 0);
  void* stream = nullptr;
  EXPECT(llmp_hip_launch_begin(nullptr, 0, &stream) == 1);
  llmp_hip_graph_destroy(nullptr);
  llmp_hip_launch_destroy(nullptr);
}

// Waits for a fence the way the completion lane does: by asking, never by blocking in the runtime.
bool AwaitFence(HipDeviceExecution& execution, std::uint64_t fence) {
  const auto give_up = std::chrono::steady_clock::now() + std::chrono::seconds(20);
  while (std::chrono::steady_clock::now() < give_up) {
    auto state = execution.Query(fence);
    if (!state) return false;
    if (*state == FenceState::kComplete) return true;
    std::this_thread::sleep_for(std::chrono::microseconds(50));
  }
  return false;
}
bool Fence(HipDeviceExecution& execution, std::uint64_t stream) {
  auto fence = execution.Record(stream);
  if (!fence) return false;
  if (!AwaitFence(execution, *fence)) return false;
  return static_cast<bool>(execution.Release(*fence));
}

template <typename T>
T* DeviceBuffer(std::size_t count) {
  T* device = nullptr;
  if (hipMalloc(reinterpret_cast<void**>(&device), count * sizeof(T)) != hipSuccess) return nullptr;
  return device;
}
template <typename T>
std::vector<T> ToHost(const T* device, std::size_t count) {
  std::vector<T> host(count);
  (void)hipMemcpy(host.data(), device, count * sizeof(T), hipMemcpyDeviceToHost);
  return host;
}

// Host-ordered: the provider's streams do not wait for the null stream.
void Fill(void* device, int value, std::size_t bytes) {
  (void)hipMemset(device, value, bytes);
  (void)hipDeviceSynchronize();
}

void DeviceChecks() {
  auto made = HipDeviceExecution::Create(0);
  EXPECT(static_cast<bool>(made));
  if (!made) return;
  HipDeviceExecution& execution = **made;
  auto stream = execution.CreateStream();
  EXPECT(static_cast<bool>(stream));
  if (!stream) return;

  // A Q8_0 mat-vec: n rows of k codes against one token, quantized to Q8_1 blocks in the run's scratch.
  constexpr int n = 96, k = 512, blocks = k / 32;
  Rng rng{42};
  std::vector<std::uint8_t> weights(static_cast<std::size_t>(n) * blocks * 34);
  for (std::size_t at = 0; at < weights.size(); at += 34) {
    for (int i = 0; i < 34; ++i) weights[at + i] = static_cast<std::uint8_t>(rng.Next());
    weights[at] = static_cast<std::uint8_t>(rng.Next());
    weights[at + 1] = 0x1F + static_cast<std::uint8_t>(rng.Next() % 4);  // half scales near 2^-8
  }
  std::vector<float> tokens[4];
  for (auto& token : tokens) {
    token.resize(k);
    for (float& v : token) v = rng.Unit() * 2.0f - 1.0f;
  }
  auto* w = DeviceBuffer<std::uint8_t>(weights.size());
  auto* x = DeviceBuffer<float>(k);          // the pinned place a graph reads its token from
  auto* staged = DeviceBuffer<float>(4 * k);  // the four tokens, copied to x on the stream
  auto* y = DeviceBuffer<float>(n);
  auto* want_q8 = DeviceBuffer<std::uint8_t>(blocks * 36 * 16);
  auto* want_y = DeviceBuffer<float>(n);
  constexpr std::uint64_t kWorkspace = 1 << 20;
  auto* workspace = DeviceBuffer<std::uint8_t>(kWorkspace);
  EXPECT(w && x && staged && y && want_q8 && want_y && workspace);
  if (!(w && x && staged && y && want_q8 && want_y && workspace)) return;
  (void)hipMemcpy(w, weights.data(), weights.size(), hipMemcpyHostToDevice);
  for (int t = 0; t < 4; ++t) (void)hipMemcpy(staged + t * k, tokens[t].data(), k * sizeof(float), hipMemcpyHostToDevice);

  const std::uint64_t q8_bytes = static_cast<std::uint64_t>(k) / 32 * 36;  // k is whole 512-value groups
  llmp_vecq_desc desc{};
  desc.w = w;
  desc.dst = y;
  desc.ncols_x = k;
  desc.nrows = n;
  desc.stride_row = blocks;
  desc.used = 1;
  desc.tokens = 1;
  // The operation: llmp.q8_1 into a pool block, then llmp.vecq over it.
  auto operation = [&](LaunchContext::RunScope& run) {
    const std::uint64_t q8 = run.Allocate(q8_bytes);
    if (q8 == 0) return;
    if (run(llmp_hip_q8_1_quantize(x, reinterpret_cast<void*>(q8), k, k, k, 1, 1, 0, run.stream())) != 0) return;
    llmp_vecq_desc d = desc;
    d.y = reinterpret_cast<const void*>(q8);
    run(llmp_hip_vecq(LLMP_TYPE_Q8_0, &d, -1, run.stream()));
  };
  // The same launchers called directly, on the null stream, for token t.
  auto direct = [&](int t) {
    (void)hipMemcpy(x, staged + t * k, k * sizeof(float), hipMemcpyDeviceToDevice);
    llmp_vecq_desc d = desc;
    d.y = want_q8;
    d.dst = want_y;
    EXPECT(llmp_hip_q8_1_quantize(x, want_q8, k, k, k, 1, 1, 0, nullptr) == 0);
    EXPECT(llmp_hip_vecq(LLMP_TYPE_Q8_0, &d, -1, nullptr) == 0);
    EXPECT(hipDeviceSynchronize() == hipSuccess);
    return ToHost(want_y, n);
  };
  const std::vector<float> want0 = direct(0);
  {
    double norm = 0;
    for (float v : want0) norm += static_cast<double>(v) * v;
    EXPECT(norm > 0);  // the product is not a vector of zeros
  }

  // ---- the provider: copies, zeroing, fences
  EXPECT(static_cast<bool>(execution.Copy(*stream, reinterpret_cast<std::uint64_t>(x), reinterpret_cast<std::uint64_t>(staged), k * sizeof(float))));
  EXPECT(static_cast<bool>(execution.Zero(*stream, reinterpret_cast<std::uint64_t>(y) + 4, n * sizeof(float) - 7)));  // ragged ends
  {
    auto refused = execution.DestroyStream(*stream);  // work not yet behind a fence
    EXPECT(!refused && refused.error() == ProviderError::kInvalid);
  }
  auto fence = execution.Record(*stream);
  EXPECT(static_cast<bool>(fence));
  if (fence) {
    auto early = execution.Release(*fence);  // not yet seen complete
    EXPECT(!early && early.error() == ProviderError::kInvalid);
    auto still = execution.DestroyStream(*stream);  // a fence of the stream is still held
    EXPECT(!still && still.error() == ProviderError::kInvalid);
    EXPECT(AwaitFence(execution, *fence));
    EXPECT(static_cast<bool>(execution.Release(*fence)));
    auto stale = execution.Query(*fence);
    EXPECT(!stale && stale.error() == ProviderError::kInvalid);
  }
  EXPECT(ToHost(x, k) == tokens[0]);
  {
    Fill(y, 0xFF, n * sizeof(float));
    EXPECT(static_cast<bool>(execution.Zero(*stream, reinterpret_cast<std::uint64_t>(y) + 4, n * sizeof(float) - 7)));
    EXPECT(Fence(execution, *stream));
    const auto bytes = ToHost(reinterpret_cast<const std::uint8_t*>(y), n * sizeof(float));
    bool right = true;
    for (std::size_t i = 0; i < bytes.size(); ++i) right = right && bytes[i] == (i >= 4 && i < 4 + n * sizeof(float) - 7 ? 0 : 0xFF);
    EXPECT(right);
  }
  {
    auto unknown = execution.Submission(*stream + 1000);
    EXPECT(!unknown && unknown.error() == ProviderError::kInvalid);
  }

  // ---- a run
  const LaunchContext::Workspace space{reinterpret_cast<std::uint64_t>(workspace), kWorkspace};
  {
    auto wrong = LaunchContext::Create(1, execution, *stream, space);  // not the provider's device
    EXPECT(!wrong && wrong.error() == LaunchFailure::kRejected);
  }
  auto created = LaunchContext::Create(0, execution, *stream, space);
  EXPECT(static_cast<bool>(created));
  if (!created) return;
  LaunchContext& context = **created;
  EXPECT(context.UsesStream(execution, *stream) && !context.UsesStream(execution, *stream + 1) && context.device() == 0);
  EXPECT(context.scratch_size(0) == kWorkspace && context.scratch_base() == space.base && context.lanes() == 0);
  {
    auto too_much = context.Run(kWorkspace + 1, operation);  // more scratch than the workspace: nothing queued
    EXPECT(!too_much && too_much.error() == LaunchFailure::kRejected && !context.faulted());
  }
  const std::uint64_t bound = q8_bytes + 256;
  auto ran = context.Run(bound, operation);
  EXPECT(static_cast<bool>(ran));
  EXPECT(Fence(execution, *stream));
  EXPECT(ToHost(y, n) == want0);
  EXPECT(context.scratch_peak() == q8_bytes);
  context.ResetScratchPeak();
  EXPECT(context.scratch_peak() == 0);
  {
    // A launcher's refusal before anything was queued is the run's refusal; the context stays usable.
    auto refused = context.Run(bound, [&](LaunchContext::RunScope& run) {
      llmp_vecq_desc d = desc;
      d.y = nullptr;
      run(llmp_hip_vecq(LLMP_TYPE_Q8_0, &d, -1, run.stream()));
    });
    EXPECT(!refused && refused.error() == LaunchFailure::kRejected && !context.faulted());
    // So is a block past the declared bound.
    auto over = context.Run(64, operation);
    EXPECT(!over && over.error() == LaunchFailure::kRejected && !context.faulted());
    EXPECT(Fence(execution, *stream));
  }

  // ---- the run captured, and replayed with a different token each time
  auto graph = context.Capture([&](LaunchContext& recording) -> Launched<Done> {
    EXPECT(recording.capturing());
    return recording.Run(bound, operation);
  });
  EXPECT(static_cast<bool>(graph));
  if (graph) {
    EXPECT(graph->nodes() >= 2 && graph->capture_seconds() > 0 && graph->instantiate_seconds() > 0);
    EXPECT(!context.capturing());
    for (int t = 1; t < 4; ++t) {
      const std::vector<float> want = direct(t);  // eager work and a synchronization between the replays
      Fill(y, 0, n * sizeof(float));
      EXPECT(static_cast<bool>(execution.Copy(*stream, reinterpret_cast<std::uint64_t>(x), reinterpret_cast<std::uint64_t>(staged + t * k), k * sizeof(float))));
      EXPECT(static_cast<bool>(context.Launch(*graph)));
      EXPECT(Fence(execution, *stream));
      EXPECT(ToHost(y, n) == want);
    }
    // Another context on the same stream may not replay it.
    auto other = LaunchContext::Create(0, execution, *stream, space);
    EXPECT(static_cast<bool>(other));
    if (other) {
      auto foreign = (*other)->Launch(*graph);
      EXPECT(!foreign && foreign.error() == LaunchFailure::kRejected && !(*other)->faulted());
    }
  }
  {
    // A capture whose recording is refused leaves the context as it was, and nothing of it ran.
    Fill(y, 0, n * sizeof(float));
    auto refused = context.Capture([&](LaunchContext& recording) -> Launched<Done> { return recording.Run(kWorkspace + 1, operation); });
    EXPECT(!refused && refused.error() == LaunchFailure::kRejected && !context.faulted() && !context.capturing());
    EXPECT(hipDeviceSynchronize() == hipSuccess);
    EXPECT(ToHost(y, n) == std::vector<float>(n, 0.0f));
    auto again = context.Run(bound, operation);
    EXPECT(static_cast<bool>(again));
    EXPECT(Fence(execution, *stream));
  }

  // ---- lanes
  constexpr std::uint64_t kLaneScratch = 64 << 10;
  {
    auto ragged = context.ConfigureLanes(2, 1000);
    EXPECT(!ragged && ragged.error() == LaunchFailure::kRejected);
    auto too_many = context.ConfigureLanes(17, kLaneScratch);  // 17 x 64 KB do not fit 1 MB
    EXPECT(!too_many && too_many.error() == LaunchFailure::kRejected && context.lanes() == 0);
  }
  EXPECT(static_cast<bool>(context.ConfigureLanes(2, kLaneScratch)));
  EXPECT(context.lanes() == 2 && context.scratch_size(0) == kWorkspace - 2 * kLaneScratch && context.scratch_size(2) == kLaneScratch);
  {
    auto twice = context.ConfigureLanes(1, kLaneScratch);
    EXPECT(!twice && twice.error() == LaunchFailure::kRejected);
  }
  {
    const std::vector<float> want = direct(2);
    Fill(y, 0, n * sizeof(float));
    EXPECT(static_cast<bool>(execution.Copy(*stream, reinterpret_cast<std::uint64_t>(x), reinterpret_cast<std::uint64_t>(staged + 2 * k), k * sizeof(float))));
    EXPECT(static_cast<bool>(context.LaneWait(2, 0)));  // the lane waits for the copy
    context.SelectLane(2);
    EXPECT(context.scratch_base() == space.base + kWorkspace - 2 * kLaneScratch);
    auto on_lane = context.Run(bound, operation);
    EXPECT(static_cast<bool>(on_lane));
    context.SelectLane(0);
    EXPECT(static_cast<bool>(context.LaneWait(0, 2)));  // the stream's fence then covers the lane's work
    EXPECT(Fence(execution, *stream));
    EXPECT(ToHost(y, n) == want);
    auto no_lane = context.LaneWait(3, 0);
    EXPECT(!no_lane && no_lane.error() == LaunchFailure::kRejected);
  }

  // ---- a refusal after an accepted launch faults the context, which then refuses everything
  {
    auto second = execution.CreateStream();
    EXPECT(static_cast<bool>(second));
    if (second) {
      auto doomed = LaunchContext::Create(0, execution, *second, space);
      EXPECT(static_cast<bool>(doomed));
      if (doomed) {
        auto broken = (*doomed)->Run(bound, [&](LaunchContext::RunScope& run) {
          const std::uint64_t q8 = run.Allocate(q8_bytes);
          run(llmp_hip_q8_1_quantize(x, reinterpret_cast<void*>(q8), k, k, k, 1, 1, 0, run.stream()));
          llmp_vecq_desc d = desc;
          d.y = nullptr;  // refused with the quantizer's work already queued
          run(llmp_hip_vecq(LLMP_TYPE_Q8_0, &d, -1, run.stream()));
        });
        EXPECT(!broken && broken.error() == LaunchFailure::kUnknown && (*doomed)->faulted());
        auto after = (*doomed)->Run(bound, operation);
        EXPECT(!after && after.error() == LaunchFailure::kRejected);
        // The stream is the owner's to quarantine: the provider will not destroy it.
        EXPECT(hipDeviceSynchronize() == hipSuccess);
        auto kept = execution.DestroyStream(*second);
        EXPECT(!kept && kept.error() == ProviderError::kInvalid);
      }
    }
  }

  created->reset();
  EXPECT(static_cast<bool>(execution.DestroyStream(*stream)));
  EXPECT(llmp_hip_execution_destroy(execution.abi()) == LLMP_PROVIDER_INVALID);  // the quarantined stream is still its own
}

}  // namespace

int main(int argc, char** argv) {
  const std::string mode = argc > 1 ? argv[1] : "host";
  if (mode == "host") {
    HostChecks();
    std::printf("host checks: %d failure(s)\n", g_failures);
  } else if (mode == "device") {
    DeviceChecks();
    std::printf("device checks: %d failure(s)\n", g_failures);
  } else {
    std::printf("usage: launch_test host | device\n");
    return 2;
  }
  return g_failures == 0 ? 0 : 1;
}
