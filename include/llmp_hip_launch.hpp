// The HIP device-execution provider and the launch context in the reference's own C++ vocabulary
// (src/providers/device_execution.h:56-98, src/kernels/ggml/launch.h:65-240 of the reference), over
// the C ABI of llmp_hip_launch.h. Header only, C++17 (the reference's std::expected becomes
// Expected below), no HIP types: a stream is the void* the reference's NativeStream carries.
#ifndef LLMP_HIP_LAUNCH_HPP_
#define LLMP_HIP_LAUNCH_HPP_

#include <cstddef>
#include <cstdint>
#include <memory>
#include <string>
#include <utility>

#include "llmp_hip.h"
#include "llmp_hip_launch.h"

namespace llmp_amd {

// The part of std::expected<T, E> the callers of these interfaces use.
template <typename T, typename E>
class Expected {
 public:
  Expected(T value) : value_(std::move(value)), ok_(true) {}
  Expected(E error, std::string detail) : error_(error), detail_(std::move(detail)), ok_(false) {}
  explicit operator bool() const { return ok_; }
  bool has_value() const { return ok_; }
  T& operator*() { return value_; }
  const T& operator*() const { return value_; }
  T* operator->() { return &value_; }
  E error() const { return error_; }
  const std::string& detail() const { return detail_; }

 private:
  T value_{};
  E error_{};
  std::string detail_;
  bool ok_;
};
struct Done {};

namespace providers {

// src/providers/device_memory.h:84-95.
enum class ProviderError : std::uint8_t { kInvalid, kOutOfMemory, kUnsupported, kFailed, kUnknown, kUndetermined };
using StreamId = std::uint64_t;  // never reused by a provider; 0 is none
using FenceId = std::uint64_t;
enum class FenceState : std::uint8_t { kPending, kComplete };
struct NativeStream {
  void* handle = nullptr;
};
template <typename T>
using Result = Expected<T, ProviderError>;

inline ProviderError FromProviderStatus(int status) {
  switch (status) {
    case LLMP_PROVIDER_INVALID: return ProviderError::kInvalid;
    case LLMP_PROVIDER_OUT_OF_MEMORY: return ProviderError::kOutOfMemory;
    case LLMP_PROVIDER_UNSUPPORTED: return ProviderError::kUnsupported;
    case LLMP_PROVIDER_UNDETERMINED: return ProviderError::kUndetermined;
    default: return status < 0 ? ProviderError::kUnknown : ProviderError::kFailed;
  }
}

// DeviceExecution for one HIP device (device_execution.h:56-98).
class HipDeviceExecution {
 public:
  static Result<std::unique_ptr<HipDeviceExecution>> Create(int device) {
    llmp_hip_execution* made = nullptr;
    if (const int status = llmp_hip_execution_create(device, &made); status != 0) return Fail<std::unique_ptr<HipDeviceExecution>>(status);
    return std::unique_ptr<HipDeviceExecution>(new HipDeviceExecution(made));
  }
  HipDeviceExecution(const HipDeviceExecution&) = delete;
  HipDeviceExecution& operator=(const HipDeviceExecution&) = delete;
  // Like the reference's, the provider outlives its streams and fences: what is still its own when it goes is leaked,
  // never destroyed under queued work.
  ~HipDeviceExecution() { (void)llmp_hip_execution_destroy(handle_); }

  Result<StreamId> CreateStream() {
    StreamId stream = 0;
    if (const int status = llmp_hip_execution_create_stream(handle_, &stream); status != 0) return Fail<StreamId>(status);
    return stream;
  }
  Result<Done> DestroyStream(StreamId stream) { return Void(llmp_hip_execution_destroy_stream(handle_, stream)); }
  Result<Done> Copy(StreamId stream, std::uint64_t destination, std::uint64_t source, std::uint64_t size) {
    return Void(llmp_hip_execution_copy(handle_, stream, destination, source, size));
  }
  Result<Done> Zero(StreamId stream, std::uint64_t destination, std::uint64_t size) {
    return Void(llmp_hip_execution_zero(handle_, stream, destination, size));
  }
  Result<NativeStream> Submission(StreamId stream) {
    NativeStream native;
    if (const int status = llmp_hip_execution_submission(handle_, stream, &native.handle); status != 0) return Fail<NativeStream>(status);
    return native;
  }
  Result<Done> Wait(StreamId stream, FenceId fence) { return Void(llmp_hip_execution_wait(handle_, stream, fence)); }
  Result<FenceId> Record(StreamId stream) {
    FenceId fence = 0;
    if (const int status = llmp_hip_execution_record(handle_, stream, &fence); status != 0) return Fail<FenceId>(status);
    return fence;
  }
  Result<FenceState> Query(FenceId fence) {
    int complete = 0;
    if (const int status = llmp_hip_execution_query(handle_, fence, &complete); status != 0) return Fail<FenceState>(status);
    return complete != 0 ? FenceState::kComplete : FenceState::kPending;
  }
  Result<Done> Release(FenceId fence) { return Void(llmp_hip_execution_release(handle_, fence)); }

  int device() const { return llmp_hip_execution_device(handle_); }
  llmp_hip_execution* abi() const { return handle_; }

 private:
  explicit HipDeviceExecution(llmp_hip_execution* handle) : handle_(handle) {}
  template <typename T>
  static Result<T> Fail(int status) {
    return Result<T>(FromProviderStatus(status), llmp_hip_last_error());
  }
  static Result<Done> Void(int status) { return status == 0 ? Result<Done>(Done{}) : Fail<Done>(status); }
  llmp_hip_execution* handle_;
};

}  // namespace providers

namespace ggml {

// src/kernels/selected_operation.h:26-35.
enum class LaunchFailure { kRejected, kUnknown };
template <typename T>
using Launched = Expected<T, LaunchFailure>;

class LaunchContext;

// An instantiated graph a context captured (launch.h:65-109). Move only.
class CapturedGraph {
 public:
  CapturedGraph() = default;
  CapturedGraph(CapturedGraph&& other) noexcept : graph_(std::exchange(other.graph_, nullptr)) {}
  CapturedGraph& operator=(CapturedGraph&& other) noexcept {
    if (this != &other) {
      llmp_hip_graph_destroy(graph_);
      graph_ = std::exchange(other.graph_, nullptr);
    }
    return *this;
  }
  CapturedGraph(const CapturedGraph&) = delete;
  CapturedGraph& operator=(const CapturedGraph&) = delete;
  ~CapturedGraph() { llmp_hip_graph_destroy(graph_); }

  std::size_t nodes() const { return llmp_hip_graph_nodes(graph_); }
  double capture_seconds() const { return llmp_hip_graph_capture_seconds(graph_); }
  double instantiate_seconds() const { return llmp_hip_graph_instantiate_seconds(graph_); }

 private:
  friend class LaunchContext;
  explicit CapturedGraph(llmp_hip_graph* graph) : graph_(graph) {}
  llmp_hip_graph* graph_ = nullptr;
};

// launch.h:135-240. What the reference's launchers get as a ggml_backend_cuda_context they get here as a Run: the
// stream to launch on and the scratch pool, as a RunScope.
class LaunchContext {
 public:
  struct Workspace {
    std::uint64_t base = 0;
    std::uint64_t size = 0;
  };
  // Inside a run: the stream, blocks of the pool, and the launchers' return values.
  class RunScope {
   public:
    void* stream() const { return stream_; }
    // A block of the run's scratch from a 256-byte boundary; 0 if the run's declared bound has no room (the run then
    // ends refused or faulted, like a launcher's refusal).
    std::uint64_t Allocate(std::uint64_t bytes) {
      std::uint64_t address = 0;
      if (const int status = llmp_hip_launch_allocate(context_, bytes, &address); status != 0) {
        llmp_hip_launch_note(context_, status);
        return 0;
      }
      return address;
    }
    // Records a launcher's return value (llmp_hip.h) and passes it on.
    int operator()(int status) {
      llmp_hip_launch_note(context_, status);
      return status;
    }

   private:
    friend class LaunchContext;
    RunScope(llmp_hip_launch* context, void* stream) : context_(context), stream_(stream) {}
    llmp_hip_launch* context_;
    void* stream_;
  };

  static Launched<std::unique_ptr<LaunchContext>> Create(int device, providers::HipDeviceExecution& execution, providers::StreamId stream,
                                                         Workspace workspace) {
    llmp_hip_launch* made = nullptr;
    if (const int status = llmp_hip_launch_create(execution.abi(), device, stream, workspace.base, workspace.size, &made); status != 0) {
      return Fail<std::unique_ptr<LaunchContext>>(status);
    }
    return std::unique_ptr<LaunchContext>(new LaunchContext(made, &execution, stream, workspace));
  }
  LaunchContext(const LaunchContext&) = delete;
  LaunchContext& operator=(const LaunchContext&) = delete;
  ~LaunchContext() { llmp_hip_launch_destroy(context_); }

  // Calls launch(run) for launchers that together draw at most `scratch` from the pool at once (launch.h:160-173).
  template <typename Launch>
  Launched<Done> Run(std::uint64_t scratch, Launch&& launch) {
    void* stream = nullptr;
    if (const int status = llmp_hip_launch_begin(context_, scratch, &stream); status != 0) return Fail<Done>(status);
    RunScope run(context_, stream);
    std::forward<Launch>(launch)(run);
    return Void(llmp_hip_launch_end(context_));
  }

  Launched<Done> ConfigureLanes(std::uint32_t count, std::uint64_t lane_scratch) {
    return Void(llmp_hip_launch_configure_lanes(context_, count, lane_scratch));
  }
  std::uint32_t lanes() const { return llmp_hip_launch_lanes(context_); }
  void SelectLane(std::uint32_t lane) { (void)llmp_hip_launch_select_lane(context_, lane); }
  Launched<Done> LaneWait(std::uint32_t waiter, std::uint32_t on) { return Void(llmp_hip_launch_lane_wait(context_, waiter, on)); }
  std::uint64_t scratch_size(std::uint32_t lane) const { return llmp_hip_launch_scratch_size(context_, lane); }
  std::uint64_t scratch_base() const { return llmp_hip_launch_scratch_base(context_); }

  // Captures what `record(*this)` queues on the context's stream; `record` returns Launched<Done> (launch.h:201-215).
  template <typename Record>
  Launched<CapturedGraph> Capture(Record&& record) {
    if (const int status = llmp_hip_launch_begin_capture(context_); status != 0) return Fail<CapturedGraph>(status);
    Launched<Done> recorded = std::forward<Record>(record)(*this);
    llmp_hip_graph* graph = nullptr;
    const int recorded_status = recorded ? 0 : recorded.error() == LaunchFailure::kRejected ? 1 : -1;
    if (const int status = llmp_hip_launch_end_capture(context_, recorded_status, &graph); status != 0) return Fail<CapturedGraph>(status);
    return CapturedGraph(graph);
  }
  Launched<Done> Launch(const CapturedGraph& graph) { return Void(llmp_hip_launch_graph(context_, graph.graph_)); }
  bool capturing() const { return llmp_hip_launch_capturing(context_) != 0; }

  std::uint64_t scratch_peak() const { return llmp_hip_launch_scratch_peak(context_); }
  void ResetScratchPeak() { llmp_hip_launch_reset_scratch_peak(context_); }
  bool faulted() const { return llmp_hip_launch_faulted(context_) != 0; }
  bool UsesStream(const providers::HipDeviceExecution& execution, providers::StreamId stream) const {
    return execution_ == &execution && stream_ == stream;
  }
  providers::NativeStream native_stream() const { return providers::NativeStream{llmp_hip_launch_native_stream(context_)}; }
  int device() const { return llmp_hip_launch_device(context_); }
  Workspace workspace() const { return workspace_; }

 private:
  LaunchContext(llmp_hip_launch* context, providers::HipDeviceExecution* execution, providers::StreamId stream, Workspace workspace)
      : context_(context), execution_(execution), stream_(stream), workspace_(workspace) {}
  template <typename T>
  static Launched<T> Fail(int status) {
    return Launched<T>(status > 0 ? LaunchFailure::kRejected : LaunchFailure::kUnknown, llmp_hip_last_error());
  }
  static Launched<Done> Void(int status) { return status == 0 ? Launched<Done>(Done{}) : Fail<Done>(status); }

  llmp_hip_launch* context_;
  providers::HipDeviceExecution* execution_;
  providers::StreamId stream_;
  Workspace workspace_;
};

}  // namespace ggml
}  // namespace llmp_amd

#endif  // LLMP_HIP_LAUNCH_HPP_
