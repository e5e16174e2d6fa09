/*
 * C ABI of the HIP device-execution provider and launch context: the part of the reference that
 * drives the kernels of llmp_hip.h. The provider owns streams, queues copies and zeroing on them
 * and records fences that are queried without blocking (src/providers/device_execution.h:56-98,
 * as src/providers/cuda/cuda_device_execution.cc:60-330 implements it for CUDA); a launch context
 * runs launchers on one of the provider's streams with a scratch pool over workspace the caller
 * declared, captures what they queue as a graph and replays it
 * (src/kernels/ggml/launch.h:135-222). Nothing here allocates device memory: workspace, operands
 * and everything a graph names are the caller's, mapped for as long as queued work or a graph can
 * use them.
 *
 * Return values: 0 done; > 0 refused, nothing changed and nothing queued, the value one of
 * LLMP_PROVIDER_* (the reference's ProviderError, src/providers/device_memory.h:84-95) for the
 * provider and 1 (the caller's kRejected) for a launch context; < 0 the runtime reported an error
 * whose effect is unknown, -(hipError_t) (ProviderError::kUnknown, KernelFailure::kUnknown): what
 * it names stays quarantined, a launch context is faulted and refuses further runs.
 * llmp_hip_last_error() (llmp_hip.h) names the reason of the calling thread's last non-zero return.
 *
 * Threads, as in the reference (device_execution.h:17-24, launch.h:28-32): the provider's calls
 * are safe for distinct streams and fences from any threads, and llmp_hip_execution_query may run
 * beside any other call; one thread drives a stream at a time (queueing on it, recording its fences,
 * destroying it: a record that ran beside another thread's submission on the same stream could mark
 * that work as fenced); a launch context is used by one thread at a time.
 */
#ifndef LLMP_HIP_LAUNCH_H_
#define LLMP_HIP_LAUNCH_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ProviderError (src/providers/device_memory.h:84-95) as positive return values; kUnknown is the
 * negative range. */
enum {
  LLMP_PROVIDER_INVALID = 1,       /* misuse: stale identity, work not yet behind a completed fence */
  LLMP_PROVIDER_OUT_OF_MEMORY = 2,
  LLMP_PROVIDER_UNSUPPORTED = 3,
  LLMP_PROVIDER_FAILED = 4,        /* known failure, nothing changed */
  LLMP_PROVIDER_UNDETERMINED = 5   /* refused: an earlier unknown outcome left what is named undetermined */
};

typedef struct llmp_hip_execution llmp_hip_execution;
typedef struct llmp_hip_launch llmp_hip_launch;
typedef struct llmp_hip_graph llmp_hip_graph;

/* ---------------------------------------------------------------- the provider
 * DeviceExecution for one device (device_execution.h:56-98). Stream and fence identities are
 * never reused by a provider. */
int llmp_hip_execution_create(int device, llmp_hip_execution** out);
/* Refused while the provider still has a stream or a fence. */
int llmp_hip_execution_destroy(llmp_hip_execution* execution);
int llmp_hip_execution_device(const llmp_hip_execution* execution);
/* CreateStream / DestroyStream (:65-66). A stream is destroyed only when everything queued on it
 * lies behind a fence that has been seen complete and released: destroying does not wait. */
int llmp_hip_execution_create_stream(llmp_hip_execution* execution, uint64_t* stream);
int llmp_hip_execution_destroy_stream(llmp_hip_execution* execution, uint64_t stream);
/* Copy / Zero (:70-77): queued after everything queued on the stream before; device addresses.
 * Zeroing is a kernel, not a memset node, so that a launch context's capture may record it. */
int llmp_hip_execution_copy(llmp_hip_execution* execution, uint64_t stream, uint64_t destination, uint64_t source,
                            uint64_t size);
int llmp_hip_execution_zero(llmp_hip_execution* execution, uint64_t stream, uint64_t destination, uint64_t size);
/* Submission (:78-84): the stream's hipStream_t for a kernel launcher about to queue work on it;
 * notes that work is being queued (the stream then needs a fence recorded after it, seen complete
 * and released, before it can be destroyed) and makes the provider's device current on the
 * calling thread. */
int llmp_hip_execution_submission(llmp_hip_execution* execution, uint64_t stream, void** native_stream);
/* Wait (:86): the stream waits for a fence recorded on another stream. */
int llmp_hip_execution_wait(llmp_hip_execution* execution, uint64_t stream, uint64_t fence);
/* Record (:89): a fence after everything queued on the stream so far. */
int llmp_hip_execution_record(llmp_hip_execution* execution, uint64_t stream, uint64_t* fence);
/* Query (:90-95): never blocks; *complete is 0 while pending. */
int llmp_hip_execution_query(llmp_hip_execution* execution, uint64_t fence, int* complete);
/* Release (:96-97): only once a query has seen the fence complete. */
int llmp_hip_execution_release(llmp_hip_execution* execution, uint64_t fence);

/* ------------------------------------------------------------ the launch context
 * LaunchContext::Create (launch.h:143-150): launches on `stream`, a stream of `execution` on
 * `device`, with a scratch pool over [workspace_base, workspace_base + workspace_size), device
 * memory the caller mapped and keeps mapped until a fence after the last run has completed. No
 * stream, event or memory is created. The context must not outlive the provider or the stream. */
int llmp_hip_launch_create(llmp_hip_execution* execution, int device, uint64_t stream, uint64_t workspace_base,
                           uint64_t workspace_size, llmp_hip_launch** out);
/* ~LaunchContext: destroys its lanes' streams and events. Queues nothing and waits for nothing. */
void llmp_hip_launch_destroy(llmp_hip_launch* context);

/* LaunchContext::Run's two halves (launch.h:160-173): between them the caller's launchers queue
 * work on *native_stream (the selected lane's stream) and draw blocks from the pool. Begin is
 * refused, with nothing queued, if the selected lane's pool is smaller than `scratch`, the
 * provider refuses the stream, a run is open or the context is faulted. End returns what the
 * run's launchers reported (llmp_hip_launch_note) or the runtime's sticky error: a launcher's
 * refusal before anything else of the run was queued is the run's refusal (> 0, the context stays
 * usable); a refusal after an accepted launch, or any error, faults the context (< 0), as
 * src/kernels/exl3/launch.h:144-151 promotes it. */
int llmp_hip_launch_begin(llmp_hip_launch* context, uint64_t scratch, void** native_stream);
/* A block of the run's scratch: from a 256-byte boundary (launch.h:162-164), in stack order, the
 * same addresses every run (a captured graph names them). Refused past the run's declared bound. */
int llmp_hip_launch_allocate(llmp_hip_launch* context, uint64_t bytes, uint64_t* address);
/* Records the return value of a launcher of llmp_hip.h called inside the run. */
void llmp_hip_launch_note(llmp_hip_launch* context, int status);
int llmp_hip_launch_end(llmp_hip_launch* context);

/* ConfigureLanes / SelectLane / LaneWait / scratch_size / scratch_base (launch.h:175-199): `count`
 * streams of the context's own (default priority), each with `lane_scratch` bytes carved from the
 * workspace's end, which the stream's pool then no longer uses. Made once, outside any capture.
 * Lane 0 is the context's stream. llmp_hip_launch_lane_wait makes `waiter`'s stream wait for what
 * `on`'s stream has queued so far. */
int llmp_hip_launch_configure_lanes(llmp_hip_launch* context, uint32_t count, uint64_t lane_scratch);
uint32_t llmp_hip_launch_lanes(const llmp_hip_launch* context);
int llmp_hip_launch_select_lane(llmp_hip_launch* context, uint32_t lane);
int llmp_hip_launch_lane_wait(llmp_hip_launch* context, uint32_t waiter, uint32_t on);
uint64_t llmp_hip_launch_scratch_size(const llmp_hip_launch* context, uint32_t lane);
uint64_t llmp_hip_launch_scratch_base(const llmp_hip_launch* context);

/* Capture's two halves (launch.h:201-215): between them runs and the provider's copies and zeroing
 * on the context's stream are recorded, not queued (thread-local capture mode). Begin is refused,
 * with the context as it was, if it is faulted, capturing or inside a run, or the stream is being
 * captured already. End with recorded_status != 0 (the caller's record failed), or a capture the
 * runtime cannot complete, is refused (1) and leaves the context as it was; a device fault is
 * < 0 and faults the context. On success *out is the instantiated, uploaded graph. */
int llmp_hip_launch_begin_capture(llmp_hip_launch* context);
int llmp_hip_launch_end_capture(llmp_hip_launch* context, int recorded_status, llmp_hip_graph** out);
/* LaunchContext::Launch (launch.h:217-221): one replay, one operation on the stream. Refused, with
 * nothing queued, if another context captured the graph or the context is faulted or capturing. */
int llmp_hip_launch_graph(llmp_hip_launch* context, const llmp_hip_graph* graph);
/* ~CapturedGraph, nodes, capture_seconds, instantiate_seconds (launch.h:72-99). */
void llmp_hip_graph_destroy(llmp_hip_graph* graph);
size_t llmp_hip_graph_nodes(const llmp_hip_graph* graph);
double llmp_hip_graph_capture_seconds(const llmp_hip_graph* graph);
double llmp_hip_graph_instantiate_seconds(const llmp_hip_graph* graph);

/* capturing, scratch_peak, ResetScratchPeak, faulted, native_stream, device (launch.h:222-240). */
int llmp_hip_launch_capturing(const llmp_hip_launch* context);
uint64_t llmp_hip_launch_scratch_peak(const llmp_hip_launch* context);
void llmp_hip_launch_reset_scratch_peak(llmp_hip_launch* context);
int llmp_hip_launch_faulted(const llmp_hip_launch* context);
void* llmp_hip_launch_native_stream(const llmp_hip_launch* context);
int llmp_hip_launch_device(const llmp_hip_launch* context);

#ifdef __cplusplus
}
#endif

#endif /* LLMP_HIP_LAUNCH_H_ */
