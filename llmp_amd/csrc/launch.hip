// The HIP device-execution provider and launch context behind include/llmp_hip_launch.h: host code over the HIP
// runtime, and one small kernel (zeroing, so that a capture records a kernel node and no memset node).
#include <atomic>
#include <chrono>
#include <mutex>
#include <unordered_map>
#include <vector>

#include <string>

#include "common.h"
#include "llmp_hip.h"
#include "llmp_hip_launch.h"

namespace llmp_hip {
namespace {

// Known failures change nothing; anything else is an outcome that nobody can vouch for.
int ProviderStatus(hipError_t e, const char* what) {
  if (e == hipSuccess) return 0;
  (void)hipGetLastError();
  SetError("%s: %s", what, hipGetErrorString(e));
  switch (e) {
    case hipErrorOutOfMemory:
      return LLMP_PROVIDER_OUT_OF_MEMORY;
    case hipErrorNotSupported:
      return LLMP_PROVIDER_UNSUPPORTED;
    case hipErrorInvalidValue:
    case hipErrorInvalidDevice:
    case hipErrorInvalidHandle:
    case hipErrorInvalidDevicePointer:
    case hipErrorNoDevice:
    case hipErrorStreamCaptureUnsupported:
    case hipErrorStreamCaptureInvalidated:
    case hipErrorStreamCaptureMerge:
    case hipErrorStreamCaptureUnmatched:
    case hipErrorStreamCaptureUnjoined:
    case hipErrorStreamCaptureIsolation:
    case hipErrorStreamCaptureImplicit:
    case hipErrorStreamCaptureWrongThread:
      return LLMP_PROVIDER_FAILED;
    default:
      return -static_cast<int>(e);
  }
}

__global__ __launch_bounds__(256) void ZeroKernel(uint8_t* to, uint64_t size) {
  // Whole 16-byte words where the range allows, the ragged ends by bytes.
  const uint64_t first = (16 - (reinterpret_cast<uintptr_t>(to) & 15)) & 15;
  const uint64_t head = first < size ? first : size;
  const uint64_t words = (size - head) / 16;
  const uint64_t thread = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const uint64_t threads = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  uint4* word = reinterpret_cast<uint4*>(to + head);
  for (uint64_t i = thread; i < words; i += threads) word[i] = make_uint4(0, 0, 0, 0);
  const uint64_t tail = head + words * 16;
  if (thread < head) to[thread] = 0;
  if (thread < size - tail) to[tail + thread] = 0;
}

struct Stream {
  hipStream_t handle = nullptr;
  int fences = 0;         // recorded and not yet released
  bool unfenced = false;  // work queued since the last fence
  bool faulted = false;
};
struct Fence {
  hipEvent_t event = nullptr;
  uint64_t stream = 0;
  bool seen = false;  // a query saw it complete
  bool faulted = false;
  int queries = 0;
};

std::atomic<uint64_t> g_context_ids{1};

// The calling thread's last reason, copied: the next Refuse writes where it lies.
std::string Reason() { return llmp_hip_last_error(); }

}  // namespace
}  // namespace llmp_hip

using namespace llmp_hip;

struct llmp_hip_execution {
  int device = 0;
  std::mutex mutex;
  uint64_t next_id = 1;
  std::unordered_map<uint64_t, Stream> streams;
  std::unordered_map<uint64_t, Fence> fences;
  std::vector<hipEvent_t> spare;  // events of released fences, kept for the next

  int Current() { return ProviderStatus(hipSetDevice(device), "making the provider's device current"); }
  // The stream's handle for a call about to queue work on it.
  int Queue(uint64_t stream, hipStream_t* handle) {
    const std::scoped_lock lock(mutex);
    auto found = streams.find(stream);
    if (found == streams.end()) return Refuse(LLMP_PROVIDER_INVALID, "stale or unknown stream %llu", (unsigned long long)stream);
    if (found->second.faulted) return Refuse(LLMP_PROVIDER_UNDETERMINED, "the stream is undetermined after an unknown outcome");
    found->second.unfenced = true;
    *handle = found->second.handle;
    return 0;
  }
  void Fault(uint64_t stream) {
    const std::scoped_lock lock(mutex);
    auto found = streams.find(stream);
    if (found != streams.end()) found->second.faulted = true;
  }
};

struct llmp_hip_graph {
  uint64_t owner = 0;
  hipGraphExec_t exec = nullptr;
  size_t nodes = 0;
  double capture_seconds = 0;
  double instantiate_seconds = 0;
};

struct llmp_hip_launch {
  struct Lane {
    hipStream_t stream = nullptr;
    hipEvent_t event = nullptr;  // for llmp_hip_launch_lane_wait on this lane
  };
  uint64_t id = 0;
  int device = 0;
  llmp_hip_execution* execution = nullptr;
  uint64_t stream = 0;
  hipStream_t native = nullptr;
  hipEvent_t stream_event = nullptr;  // the stream's, made with the lanes
  uint64_t workspace_base = 0, workspace_size = 0;
  std::vector<Lane> lanes;
  uint64_t lane_scratch = 0;
  uint32_t active = 0;
  bool faulted = false;
  bool capturing = false;
  std::chrono::steady_clock::time_point capture_started;
  // The open run.
  bool running = false;
  uint64_t bound = 0;     // the run's declared scratch
  uint64_t top = 0;       // of the pool's stack
  int accepted = 0;       // launchers that queued
  int first_status = 0;   // the first launcher status that was not 0
  uint64_t peak = 0;

  hipStream_t StreamOf(uint32_t lane) const { return lane == 0 ? native : lanes[lane - 1].stream; }
  uint64_t ScratchSize(uint32_t lane) const {
    if (lane == 0) return workspace_size - lanes.size() * lane_scratch;
    return lane <= lanes.size() ? lane_scratch : 0;
  }
  uint64_t ScratchBase(uint32_t lane) const {
    return lane == 0 ? workspace_base : workspace_base + workspace_size - lane * lane_scratch;
  }
  void ReleaseLanes() {
    for (Lane& lane : lanes) {
      if (lane.event != nullptr) (void)hipEventDestroy(lane.event);
      if (lane.stream != nullptr) (void)hipStreamDestroy(lane.stream);
    }
    lanes.clear();
    if (stream_event != nullptr) (void)hipEventDestroy(stream_event);
    stream_event = nullptr;
    lane_scratch = 0;
    active = 0;
  }
};

// ------------------------------------------------------------------------------------------- the provider

extern "C" int llmp_hip_execution_create(int device, llmp_hip_execution** out) {
  if (out == nullptr) return Refuse(LLMP_PROVIDER_INVALID, "execution: null result");
  *out = nullptr;
  int devices = 0;
  if (const hipError_t e = hipGetDeviceCount(&devices); e != hipSuccess || device < 0 || device >= devices) {
    (void)hipGetLastError();
    return Refuse(LLMP_PROVIDER_UNSUPPORTED, "execution: no device %d (%d visible)", device, e == hipSuccess ? devices : 0);
  }
  auto* execution = new llmp_hip_execution;
  execution->device = device;
  if (const int status = execution->Current(); status != 0) {
    delete execution;
    return status;
  }
  *out = execution;
  return 0;
}

extern "C" int llmp_hip_execution_destroy(llmp_hip_execution* execution) {
  if (execution == nullptr) return 0;
  {
    const std::scoped_lock lock(execution->mutex);
    if (!execution->streams.empty() || !execution->fences.empty()) {
      return Refuse(LLMP_PROVIDER_INVALID, "execution: %zu stream(s) and %zu fence(s) are still the provider's",
                    execution->streams.size(), execution->fences.size());
    }
  }
  (void)hipSetDevice(execution->device);
  for (hipEvent_t event : execution->spare) (void)hipEventDestroy(event);
  delete execution;
  return 0;
}

extern "C" int llmp_hip_execution_device(const llmp_hip_execution* execution) { return execution == nullptr ? -1 : execution->device; }

extern "C" int llmp_hip_execution_create_stream(llmp_hip_execution* execution, uint64_t* stream) {
  if (execution == nullptr || stream == nullptr) return Refuse(LLMP_PROVIDER_INVALID, "create_stream: null argument");
  if (const int status = execution->Current(); status != 0) return status;
  hipStream_t handle = nullptr;
  // Default priority: streams of different priorities do not mix on these devices.
  if (const int status = ProviderStatus(hipStreamCreateWithFlags(&handle, hipStreamNonBlocking), "hipStreamCreateWithFlags"); status != 0) {
    return status;
  }
  const std::scoped_lock lock(execution->mutex);
  *stream = execution->next_id++;
  execution->streams[*stream].handle = handle;
  return 0;
}

extern "C" int llmp_hip_execution_destroy_stream(llmp_hip_execution* execution, uint64_t stream) {
  if (execution == nullptr) return Refuse(LLMP_PROVIDER_INVALID, "destroy_stream: null provider");
  hipStream_t handle = nullptr;
  {
    const std::scoped_lock lock(execution->mutex);
    auto found = execution->streams.find(stream);
    if (found == execution->streams.end()) return Refuse(LLMP_PROVIDER_INVALID, "stale or unknown stream %llu", (unsigned long long)stream);
    if (found->second.faulted) return Refuse(LLMP_PROVIDER_INVALID, "the stream is undetermined after an unknown outcome");
    if (found->second.fences > 0 || found->second.unfenced) {
      return Refuse(LLMP_PROVIDER_INVALID, "the stream has work not yet behind a completed fence");
    }
    handle = found->second.handle;
  }
  int status = execution->Current();
  if (status == 0) status = ProviderStatus(hipStreamDestroy(handle), "hipStreamDestroy");
  const std::scoped_lock lock(execution->mutex);
  if (status != 0) {
    execution->streams[stream].faulted = status < 0;  // a known failure changed nothing
    return status;
  }
  execution->streams.erase(stream);
  return 0;
}

extern "C" int llmp_hip_execution_copy(llmp_hip_execution* execution, uint64_t stream, uint64_t destination, uint64_t source,
                                       uint64_t size) {
  if (execution == nullptr) return Refuse(LLMP_PROVIDER_INVALID, "copy: null provider");
  if (size == 0) return 0;
  if (destination == 0 || source == 0) return Refuse(LLMP_PROVIDER_INVALID, "copy: null address");
  hipStream_t handle = nullptr;
  if (const int status = execution->Queue(stream, &handle); status != 0) return status;
  if (const int status = execution->Current(); status != 0) return status;
  const int status = ProviderStatus(hipMemcpyAsync(reinterpret_cast<void*>(destination), reinterpret_cast<const void*>(source), size,
                                                   hipMemcpyDeviceToDevice, handle),
                                    "hipMemcpyAsync");
  if (status < 0) execution->Fault(stream);
  return status;
}

extern "C" int llmp_hip_execution_zero(llmp_hip_execution* execution, uint64_t stream, uint64_t destination, uint64_t size) {
  if (execution == nullptr) return Refuse(LLMP_PROVIDER_INVALID, "zero: null provider");
  if (size == 0) return 0;
  if (destination == 0) return Refuse(LLMP_PROVIDER_INVALID, "zero: null address");
  hipStream_t handle = nullptr;
  if (const int status = execution->Queue(stream, &handle); status != 0) return status;
  if (const int status = execution->Current(); status != 0) return status;
  (void)hipGetLastError();
  const uint64_t blocks = (size / 16 + 255) / 256 + 1;
  hipLaunchKernelGGL(ZeroKernel, dim3(static_cast<unsigned>(blocks < 4096 ? blocks : 4096)), dim3(256), 0, handle,
                     reinterpret_cast<uint8_t*>(destination), size);
  const int status = ProviderStatus(hipGetLastError(), "zeroing kernel");
  if (status < 0) execution->Fault(stream);
  return status;
}

extern "C" int llmp_hip_execution_submission(llmp_hip_execution* execution, uint64_t stream, void** native_stream) {
  if (execution == nullptr || native_stream == nullptr) return Refuse(LLMP_PROVIDER_INVALID, "submission: null argument");
  hipStream_t handle = nullptr;
  if (const int status = execution->Queue(stream, &handle); status != 0) return status;
  if (const int status = execution->Current(); status != 0) return status;
  *native_stream = handle;
  return 0;
}

extern "C" int llmp_hip_execution_record(llmp_hip_execution* execution, uint64_t stream, uint64_t* fence) {
  if (execution == nullptr || fence == nullptr) return Refuse(LLMP_PROVIDER_INVALID, "record: null argument");
  hipStream_t handle = nullptr;
  hipEvent_t event = nullptr;
  {
    const std::scoped_lock lock(execution->mutex);
    auto found = execution->streams.find(stream);
    if (found == execution->streams.end()) return Refuse(LLMP_PROVIDER_INVALID, "stale or unknown stream %llu", (unsigned long long)stream);
    if (found->second.faulted) return Refuse(LLMP_PROVIDER_UNDETERMINED, "the stream is undetermined after an unknown outcome");
    handle = found->second.handle;
    if (!execution->spare.empty()) {
      event = execution->spare.back();
      execution->spare.pop_back();
    }
  }
  if (const int status = execution->Current(); status != 0) return status;
  if (event == nullptr) {
    if (const int status = ProviderStatus(hipEventCreateWithFlags(&event, hipEventDisableTiming), "hipEventCreateWithFlags"); status != 0) {
      return status;
    }
  }
  if (const int status = ProviderStatus(hipEventRecord(event, handle), "hipEventRecord"); status != 0) {
    (void)hipEventDestroy(event);
    return status;
  }
  const std::scoped_lock lock(execution->mutex);
  *fence = execution->next_id++;
  Fence& made = execution->fences[*fence];
  made.event = event;
  made.stream = stream;
  Stream& of = execution->streams[stream];
  ++of.fences;
  of.unfenced = false;
  return 0;
}

extern "C" int llmp_hip_execution_wait(llmp_hip_execution* execution, uint64_t stream, uint64_t fence) {
  if (execution == nullptr) return Refuse(LLMP_PROVIDER_INVALID, "wait: null provider");
  hipEvent_t event = nullptr;
  {
    const std::scoped_lock lock(execution->mutex);
    auto found = execution->fences.find(fence);
    if (found == execution->fences.end() || found->second.faulted) return Refuse(LLMP_PROVIDER_INVALID, "stale, unknown or undetermined fence");
    event = found->second.event;
  }
  hipStream_t handle = nullptr;
  if (const int status = execution->Queue(stream, &handle); status != 0) return status;
  if (const int status = execution->Current(); status != 0) return status;
  const int status = ProviderStatus(hipStreamWaitEvent(handle, event, 0), "hipStreamWaitEvent");
  if (status < 0) execution->Fault(stream);
  return status;
}

extern "C" int llmp_hip_execution_query(llmp_hip_execution* execution, uint64_t fence, int* complete) {
  if (execution == nullptr || complete == nullptr) return Refuse(LLMP_PROVIDER_INVALID, "query: null argument");
  hipEvent_t event = nullptr;
  {
    const std::scoped_lock lock(execution->mutex);
    auto found = execution->fences.find(fence);
    if (found == execution->fences.end() || found->second.faulted) return Refuse(LLMP_PROVIDER_INVALID, "stale, unknown or undetermined fence");
    event = found->second.event;
    ++found->second.queries;  // the event stays valid until this query ends
  }
  const int current = execution->Current();
  const hipError_t e = current == 0 ? hipEventQuery(event) : hipSuccess;
  const std::scoped_lock lock(execution->mutex);
  Fence& found = execution->fences[fence];
  --found.queries;
  if (current != 0) return current;
  if (e == hipErrorNotReady) {
    (void)hipGetLastError();
    *complete = 0;
    return 0;
  }
  if (e != hipSuccess) return ProviderStatus(e, "hipEventQuery");  // the event keeps its identity: the caller may ask again
  found.seen = true;
  *complete = 1;
  return 0;
}

extern "C" int llmp_hip_execution_release(llmp_hip_execution* execution, uint64_t fence) {
  if (execution == nullptr) return Refuse(LLMP_PROVIDER_INVALID, "release: null provider");
  const std::scoped_lock lock(execution->mutex);
  auto found = execution->fences.find(fence);
  if (found == execution->fences.end() || found->second.faulted) return Refuse(LLMP_PROVIDER_INVALID, "stale, unknown or undetermined fence");
  if (!found->second.seen) return Refuse(LLMP_PROVIDER_INVALID, "the fence has not been seen complete");
  if (found->second.queries > 0) return Refuse(LLMP_PROVIDER_FAILED, "the fence is being queried; release it later");
  // Seen complete, so nothing waits on the event: it serves the next fence.
  execution->spare.push_back(found->second.event);
  --execution->streams[found->second.stream].fences;
  execution->fences.erase(found);
  return 0;
}

// ------------------------------------------------------------------------------------- the launch context

namespace {
int Faulted(llmp_hip_launch* context, int status) {
  context->faulted = true;
  context->execution->Fault(context->stream);
  return status;
}
}  // namespace

extern "C" int llmp_hip_launch_create(llmp_hip_execution* execution, int device, uint64_t stream, uint64_t workspace_base,
                                      uint64_t workspace_size, llmp_hip_launch** out) {
  if (out == nullptr) return Refuse(1, "launch context: null result");
  *out = nullptr;
  if (execution == nullptr) return Refuse(1, "launch context: null provider");
  if (device != execution->device) return Refuse(1, "launch context: device %d is not the provider's (%d)", device, execution->device);
  if (workspace_size != 0 && workspace_base == 0) return Refuse(1, "launch context: a workspace of %llu bytes at address 0", (unsigned long long)workspace_size);
  if (workspace_base + workspace_size < workspace_base) return Refuse(1, "launch context: the workspace wraps the address space");
  hipStream_t native = nullptr;
  {
    const std::scoped_lock lock(execution->mutex);
    auto found = execution->streams.find(stream);
    if (found == execution->streams.end() || found->second.faulted) return Refuse(1, "launch context: stale, unknown or undetermined stream");
    native = found->second.handle;
  }
  auto* context = new llmp_hip_launch;
  context->id = g_context_ids.fetch_add(1);
  context->device = device;
  context->execution = execution;
  context->stream = stream;
  context->native = native;
  context->workspace_base = workspace_base;
  context->workspace_size = workspace_size;
  *out = context;
  return 0;
}

extern "C" void llmp_hip_launch_destroy(llmp_hip_launch* context) {
  if (context == nullptr) return;
  (void)hipSetDevice(context->device);
  context->ReleaseLanes();
  delete context;
}

extern "C" int llmp_hip_launch_begin(llmp_hip_launch* context, uint64_t scratch, void** native_stream) {
  if (context == nullptr || native_stream == nullptr) return Refuse(1, "run: null argument");
  if (context->faulted) return Refuse(1, "run: the context is faulted");
  if (context->running) return Refuse(1, "run: a run is open");
  if (scratch > context->ScratchSize(context->active)) {
    return Refuse(1, "run: %llu bytes of scratch, the selected lane's pool has %llu", (unsigned long long)scratch,
                  (unsigned long long)context->ScratchSize(context->active));
  }
  // The stream is taken again for every run: the provider counts it as queued work.
  void* taken = nullptr;
  if (const int status = llmp_hip_execution_submission(context->execution, context->stream, &taken); status != 0) {
    return status > 0 ? Refuse(1, "run: the provider refuses the stream: %s", Reason().c_str()) : Faulted(context, status);
  }
  (void)hipGetLastError();  // an error an earlier, unrelated call left on this thread is not this run's
  context->running = true;
  context->bound = scratch;
  context->top = 0;
  context->accepted = 0;
  context->first_status = 0;
  *native_stream = context->StreamOf(context->active);
  return 0;
}

extern "C" int llmp_hip_launch_allocate(llmp_hip_launch* context, uint64_t bytes, uint64_t* address) {
  if (context == nullptr || address == nullptr) return Refuse(1, "scratch block: null argument");
  if (!context->running) return Refuse(1, "scratch block: no run is open");
  const uint64_t base = context->ScratchBase(context->active);
  // From a 256-byte boundary of the address space: the rounding counts against the run's bound.
  const uint64_t at = ((base + context->top + 255) & ~uint64_t{255}) - base;
  if (at + bytes < at || at + bytes > context->bound) {
    return Refuse(1, "scratch block: %llu bytes at offset %llu pass the run's declared %llu", (unsigned long long)bytes,
                  (unsigned long long)at, (unsigned long long)context->bound);
  }
  context->top = at + bytes;
  if (context->top > context->peak) context->peak = context->top;
  *address = base + at;
  return 0;
}

extern "C" void llmp_hip_launch_note(llmp_hip_launch* context, int status) {
  if (context == nullptr || !context->running) return;
  if (status == 0) {
    ++context->accepted;
  } else if (context->first_status == 0) {
    // A refusal after an accepted launch leaves work of an unfinished operation queued: a fault.
    context->first_status = status > 0 && context->accepted > 0 ? -static_cast<int>(hipErrorUnknown) : status;
  }
}

extern "C" int llmp_hip_launch_end(llmp_hip_launch* context) {
  if (context == nullptr) return Refuse(1, "run: null context");
  if (!context->running) return Refuse(1, "run: no run is open");
  context->running = false;
  const hipError_t sticky = hipGetLastError();
  if (context->first_status > 0) return context->first_status;  // refused before anything was queued; the reason is the launcher's
  if (context->first_status < 0) return Faulted(context, context->first_status);
  if (sticky != hipSuccess) {
    SetError("run: a launcher left %s", hipGetErrorString(sticky));
    return Faulted(context, -static_cast<int>(sticky));
  }
  return 0;
}

extern "C" int llmp_hip_launch_configure_lanes(llmp_hip_launch* context, uint32_t count, uint64_t lane_scratch) {
  if (context == nullptr) return Refuse(1, "lanes: null context");
  if (context->faulted || context->capturing || context->running) return Refuse(1, "lanes: the context is faulted, capturing or inside a run");
  if (!context->lanes.empty()) return Refuse(1, "lanes: made once");
  if (count == 0) return 0;
  if (count > 64) return Refuse(1, "lanes: %u of them", count);
  if (lane_scratch % 256 != 0) return Refuse(1, "lanes: %llu bytes a lane is not whole 256-byte blocks", (unsigned long long)lane_scratch);
  if (lane_scratch != 0 && count > context->workspace_size / lane_scratch) {
    return Refuse(1, "lanes: %u x %llu bytes do not fit the workspace's %llu", count, (unsigned long long)lane_scratch,
                  (unsigned long long)context->workspace_size);
  }
  if (const int status = context->execution->Current(); status != 0) return Refuse(1, "lanes: %s", Reason().c_str());
  int status = ProviderStatus(hipEventCreateWithFlags(&context->stream_event, hipEventDisableTiming), "hipEventCreateWithFlags");
  for (uint32_t i = 0; status == 0 && i < count; ++i) {
    llmp_hip_launch::Lane lane;
    status = ProviderStatus(hipStreamCreateWithFlags(&lane.stream, hipStreamNonBlocking), "hipStreamCreateWithFlags");
    if (status == 0) status = ProviderStatus(hipEventCreateWithFlags(&lane.event, hipEventDisableTiming), "hipEventCreateWithFlags");
    context->lanes.push_back(lane);
  }
  if (status != 0) {
    context->ReleaseLanes();
    return status > 0 ? 1 : Faulted(context, status);
  }
  context->lane_scratch = lane_scratch;
  return 0;
}

extern "C" uint32_t llmp_hip_launch_lanes(const llmp_hip_launch* context) {
  return context == nullptr ? 0 : static_cast<uint32_t>(context->lanes.size());
}

extern "C" int llmp_hip_launch_select_lane(llmp_hip_launch* context, uint32_t lane) {
  if (context == nullptr) return Refuse(1, "lanes: null context");
  if (context->running) return Refuse(1, "lanes: a run is open");
  if (lane > context->lanes.size()) return Refuse(1, "lanes: lane %u of %zu", lane, context->lanes.size());
  context->active = lane;
  return 0;
}

extern "C" int llmp_hip_launch_lane_wait(llmp_hip_launch* context, uint32_t waiter, uint32_t on) {
  if (context == nullptr) return Refuse(1, "lanes: null context");
  if (context->faulted) return Refuse(1, "lanes: the context is faulted");
  if (waiter > context->lanes.size() || on > context->lanes.size() || context->lanes.empty()) {
    return Refuse(1, "lanes: lane %u waiting for lane %u of %zu", waiter, on, context->lanes.size());
  }
  if (waiter == on) return 0;
  // Either side may be the context's stream: the provider hears that it has work again.
  void* taken = nullptr;
  if (const int status = llmp_hip_execution_submission(context->execution, context->stream, &taken); status != 0) {
    return status > 0 ? 1 : Faulted(context, status);
  }
  hipEvent_t event = on == 0 ? context->stream_event : context->lanes[on - 1].event;
  int status = ProviderStatus(hipEventRecord(event, context->StreamOf(on)), "hipEventRecord");
  if (status == 0) status = ProviderStatus(hipStreamWaitEvent(context->StreamOf(waiter), event, 0), "hipStreamWaitEvent");
  if (status == 0) return 0;
  return status > 0 && !context->capturing ? 1 : Faulted(context, status > 0 ? -static_cast<int>(hipErrorUnknown) : status);
}

extern "C" uint64_t llmp_hip_launch_scratch_size(const llmp_hip_launch* context, uint32_t lane) {
  return context == nullptr ? 0 : context->ScratchSize(lane);
}
extern "C" uint64_t llmp_hip_launch_scratch_base(const llmp_hip_launch* context) {
  return context == nullptr ? 0 : context->ScratchBase(context->active);
}

extern "C" int llmp_hip_launch_begin_capture(llmp_hip_launch* context) {
  if (context == nullptr) return Refuse(1, "capture: null context");
  if (context->faulted || context->capturing || context->running) return Refuse(1, "capture: the context is faulted, capturing or inside a run");
  if (const int status = context->execution->Current(); status != 0) return Refuse(1, "capture: %s", Reason().c_str());
  hipStreamCaptureStatus state = hipStreamCaptureStatusNone;
  if (const hipError_t e = hipStreamIsCapturing(context->native, &state); e != hipSuccess) {
    const int status = ProviderStatus(e, "hipStreamIsCapturing");
    return status > 0 ? 1 : Faulted(context, status);
  }
  if (state != hipStreamCaptureStatusNone) return Refuse(1, "capture: the stream is being captured");
  context->capture_started = std::chrono::steady_clock::now();
  // Thread-local mode: a call of this thread that a capture cannot hold fails instead of running.
  if (const hipError_t e = hipStreamBeginCapture(context->native, hipStreamCaptureModeThreadLocal); e != hipSuccess) {
    const int status = ProviderStatus(e, "hipStreamBeginCapture");
    return status > 0 ? 1 : Faulted(context, status);
  }
  context->capturing = true;
  return 0;
}

extern "C" int llmp_hip_launch_end_capture(llmp_hip_launch* context, int recorded_status, llmp_hip_graph** out) {
  if (context == nullptr || out == nullptr) return Refuse(1, "capture: null argument");
  *out = nullptr;
  if (!context->capturing) return Refuse(1, "capture: the context is not capturing");
  if (context->running) return Refuse(1, "capture: a run is open");
  context->capturing = false;
  char reason[256] = "";
  if (recorded_status != 0) snprintf(reason, sizeof(reason), "%s", Reason().c_str());
  hipGraph_t graph = nullptr;
  const hipError_t ended = hipStreamEndCapture(context->native, &graph);
  const auto captured = std::chrono::steady_clock::now();
  if (ended != hipSuccess) {
    if (graph != nullptr) (void)hipGraphDestroy(graph);
    const int status = ProviderStatus(ended, "hipStreamEndCapture");
    return status > 0 ? 1 : Faulted(context, status);
  }
  if (recorded_status != 0) {
    // Nothing of it ran: the context is as it was, unless what failed was the device.
    if (graph != nullptr) (void)hipGraphDestroy(graph);
    if (recorded_status < 0) return Faulted(context, Refuse(recorded_status, "capture: recording faulted: %s", reason));
    return Refuse(1, "capture: recording was refused: %s", reason);
  }
  if (graph == nullptr) return Refuse(1, "capture: the runtime returned no graph");
  size_t nodes = 0;
  int status = ProviderStatus(hipGraphGetNodes(graph, nullptr, &nodes), "hipGraphGetNodes");
  hipGraphExec_t exec = nullptr;
  if (status == 0) status = ProviderStatus(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0), "hipGraphInstantiate");
  (void)hipGraphDestroy(graph);
  if (status != 0) return status > 0 ? 1 : Faulted(context, status);
  // The upload queues on the stream: from here an error leaves queued work behind.
  void* taken = nullptr;
  status = llmp_hip_execution_submission(context->execution, context->stream, &taken);
  if (status == 0) status = ProviderStatus(hipGraphUpload(exec, context->native), "hipGraphUpload");
  if (status != 0) {
    (void)hipGraphExecDestroy(exec);
    return Faulted(context, status > 0 ? -static_cast<int>(hipErrorUnknown) : status);
  }
  const auto done = std::chrono::steady_clock::now();
  auto* made = new llmp_hip_graph;
  made->owner = context->id;
  made->exec = exec;
  made->nodes = nodes;
  made->capture_seconds = std::chrono::duration<double>(captured - context->capture_started).count();
  made->instantiate_seconds = std::chrono::duration<double>(done - captured).count();
  *out = made;
  return 0;
}

extern "C" int llmp_hip_launch_graph(llmp_hip_launch* context, const llmp_hip_graph* graph) {
  if (context == nullptr || graph == nullptr) return Refuse(1, "replay: null argument");
  if (context->faulted || context->capturing || context->running) return Refuse(1, "replay: the context is faulted, capturing or inside a run");
  if (graph->owner != context->id) return Refuse(1, "replay: another context captured the graph");
  void* taken = nullptr;
  if (const int status = llmp_hip_execution_submission(context->execution, context->stream, &taken); status != 0) {
    return status > 0 ? Refuse(1, "replay: the provider refuses the stream: %s", Reason().c_str()) : Faulted(context, status);
  }
  if (const hipError_t e = hipGraphLaunch(graph->exec, context->native); e != hipSuccess) {
    (void)hipGetLastError();
    SetError("hipGraphLaunch: %s", hipGetErrorString(e));
    return Faulted(context, -static_cast<int>(e));
  }
  return 0;
}

extern "C" void llmp_hip_graph_destroy(llmp_hip_graph* graph) {
  if (graph == nullptr) return;
  if (graph->exec != nullptr) (void)hipGraphExecDestroy(graph->exec);
  delete graph;
}
extern "C" size_t llmp_hip_graph_nodes(const llmp_hip_graph* graph) { return graph == nullptr ? 0 : graph->nodes; }
extern "C" double llmp_hip_graph_capture_seconds(const llmp_hip_graph* graph) { return graph == nullptr ? 0 : graph->capture_seconds; }
extern "C" double llmp_hip_graph_instantiate_seconds(const llmp_hip_graph* graph) {
  return graph == nullptr ? 0 : graph->instantiate_seconds;
}

extern "C" int llmp_hip_launch_capturing(const llmp_hip_launch* context) { return context != nullptr && context->capturing; }
extern "C" uint64_t llmp_hip_launch_scratch_peak(const llmp_hip_launch* context) { return context == nullptr ? 0 : context->peak; }
extern "C" void llmp_hip_launch_reset_scratch_peak(llmp_hip_launch* context) {
  if (context != nullptr) context->peak = 0;
}
extern "C" int llmp_hip_launch_faulted(const llmp_hip_launch* context) { return context != nullptr && context->faulted; }
extern "C" void* llmp_hip_launch_native_stream(const llmp_hip_launch* context) { return context == nullptr ? nullptr : context->native; }
extern "C" int llmp_hip_launch_device(const llmp_hip_launch* context) { return context == nullptr ? -1 : context->device; }
