// A stand-in for the part of the HIP runtime API that libtm_hip's host logic
// (tuckmill_amd/csrc/tm_hip.cpp) uses, for its CPU build: tests/host_cpu is put
// first on the include path, so `#include <hip/hip_runtime.h>` finds this file.
// "Device" memory is host memory (so that the address sanitizer sees every copy
// and every use after free), a stream is a counter of enqueued operations that
// completes only when the test advances or synchronizes it (so that leases are
// really held while work is "in flight"), nothing computes. Implemented in
// fake_runtime.cpp; the test driver reads the counters declared at the end.
#pragma once

#include <cstddef>
#include <cstdint>

typedef int hipError_t;
enum {
    hipSuccess = 0,
    hipErrorInvalidValue = 1,
    hipErrorOutOfMemory = 2,
    hipErrorInvalidDevice = 101,
    hipErrorInvalidSymbol = 13,
    hipErrorNotReady = 600,
    hipErrorStreamCaptureUnsupported = 900
};

struct fake_stream;
struct fake_event;
struct fake_graph;
struct fake_graph_exec;
typedef fake_stream *hipStream_t;
typedef fake_event *hipEvent_t;
typedef fake_graph *hipGraph_t;
typedef fake_graph_exec *hipGraphExec_t;

enum { hipStreamNonBlocking = 1 };
enum { hipEventDisableTiming = 2 };
enum hipMemcpyKind { hipMemcpyHostToDevice = 1, hipMemcpyDeviceToHost = 2, hipMemcpyDeviceToDevice = 3 };
enum hipStreamCaptureMode { hipStreamCaptureModeRelaxed = 2 };

struct hipDeviceProp_t {
    char name[256];
    char gcnArchName[256];
    int multiProcessorCount;
    size_t totalGlobalMem;
};

const char *hipGetErrorString(hipError_t e);
hipError_t hipGetLastError();
hipError_t hipGetDeviceCount(int *n);
hipError_t hipGetDeviceProperties(hipDeviceProp_t *prop, int device);
hipError_t hipSetDevice(int device);

hipError_t hipMalloc(void **ptr, size_t bytes);
hipError_t hipFree(void *ptr);
hipError_t hipMemset(void *ptr, int value, size_t bytes);
hipError_t hipMemsetAsync(void *ptr, int value, size_t bytes, hipStream_t stream);
hipError_t hipMemcpyAsync(void *dst, const void *src, size_t bytes, hipMemcpyKind kind,
                          hipStream_t stream);

hipError_t hipStreamCreateWithFlags(hipStream_t *stream, unsigned flags);
hipError_t hipStreamDestroy(hipStream_t stream);
hipError_t hipStreamSynchronize(hipStream_t stream);
hipError_t hipStreamWaitEvent(hipStream_t stream, hipEvent_t event, unsigned flags);

hipError_t hipEventCreate(hipEvent_t *event);
hipError_t hipEventCreateWithFlags(hipEvent_t *event, unsigned flags);
hipError_t hipEventDestroy(hipEvent_t event);
hipError_t hipEventRecord(hipEvent_t event, hipStream_t stream);
hipError_t hipEventQuery(hipEvent_t event);
hipError_t hipEventElapsedTime(float *ms, hipEvent_t start, hipEvent_t stop);

hipError_t hipStreamBeginCapture(hipStream_t stream, hipStreamCaptureMode mode);
hipError_t hipStreamEndCapture(hipStream_t stream, hipGraph_t *graph);
hipError_t hipGraphInstantiate(hipGraphExec_t *exec, hipGraph_t graph, void *, void *, size_t);
hipError_t hipGraphLaunch(hipGraphExec_t exec, hipStream_t stream);
hipError_t hipGraphExecDestroy(hipGraphExec_t exec);
hipError_t hipGraphDestroy(hipGraph_t graph);

// ---- what the test driver and the recording launchers use ---------------------

namespace fake {

// One operation enqueued on a stream (a kernel launch recorded by the stand-in
// launchers, a memset, a copy, an event): the stream's count of enqueued
// operations goes up, and, while the stream records, the operation goes into the
// graph instead. Returns false when the stream is null or destroyed.
bool enqueue(hipStream_t stream, const char *what);
bool capturing(hipStream_t stream);
// A launch carries `event` as its stop event: reached when the stream has
// completed everything enqueued so far.
void attach_event(hipEvent_t event, hipStream_t stream);
// Let the oldest `n` operations still in flight on every live stream complete
// (events recorded before them read as reached).
void advance_all(uint64_t n);
// true: every enqueue completes at once (the default is to complete only at a
// synchronize or advance).
void set_eager(bool eager);
// An allocation of at least `bytes` starts at `ptr` and is live: the launchers
// call it for every pointer a launch names (and touch both ends, for the
// address sanitizer).
bool device_range_live(const void *ptr, size_t bytes);
// The allocation that holds `ptr`, by its order of allocation (the first
// hipMalloc is 1), or 0: how the test driver tells the library's buffers apart.
uint64_t serial_of(const void *ptr);

struct Counters {
    uint64_t live_allocs, live_bytes, total_allocs;
    uint64_t live_streams, live_events, live_graphs, live_execs;
    uint64_t enqueued, graph_launches;
};
Counters counters();
// makes hipMalloc fail once `n` more allocations have succeeded (0: never)
void fail_malloc_after(uint64_t n);

} // namespace fake
