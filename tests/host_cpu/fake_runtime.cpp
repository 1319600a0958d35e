// Implementation of the stand-in HIP runtime declared in hip/hip_runtime.h (see there).
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <set>
#include <string>
#include <vector>

struct fake_stream {
    uint64_t issued = 0, completed = 0;
    fake_graph *recording = nullptr;
};
struct fake_event {
    fake_stream *stream = nullptr;
    uint64_t seq = 0; // reached once stream->completed >= seq; never recorded: reached
};
struct fake_graph {
    std::vector<std::string> nodes;
};
struct fake_graph_exec {
    std::vector<std::string> nodes;
};

namespace {

std::mutex mu;
std::map<const void *, size_t> allocs;
std::map<const void *, uint64_t> serials; // allocation order, from 1
std::set<fake_stream *> streams;
std::set<fake_event *> events;
std::set<fake_graph *> graphs;
std::set<fake_graph_exec *> execs;
uint64_t total_allocs = 0, enqueued = 0, graph_launches = 0, malloc_budget = 0;
bool eager = false;

} // namespace

const char *hipGetErrorString(hipError_t e) {
    switch (e) {
    case hipSuccess: return "no error";
    case hipErrorInvalidValue: return "invalid argument";
    case hipErrorOutOfMemory: return "out of memory";
    case hipErrorNotReady: return "not ready";
    default: return "error";
    }
}
hipError_t hipGetLastError() { return hipSuccess; }
hipError_t hipGetDeviceCount(int *n) {
    *n = 1;
    return hipSuccess;
}
hipError_t hipGetDeviceProperties(hipDeviceProp_t *prop, int) {
    memset(prop, 0, sizeof *prop);
    snprintf(prop->name, sizeof prop->name, "stand-in device (no GPU)");
    snprintf(prop->gcnArchName, sizeof prop->gcnArchName, "gfx950:host-stub");
    prop->multiProcessorCount = 256;
    prop->totalGlobalMem = (size_t)288 << 30;
    return hipSuccess;
}
hipError_t hipSetDevice(int device) { return device == 0 ? hipSuccess : hipErrorInvalidDevice; }

hipError_t hipMalloc(void **ptr, size_t bytes) {
    std::lock_guard<std::mutex> g(mu);
    if (malloc_budget != 0 && --malloc_budget == 0) {
        *ptr = nullptr;
        return hipErrorOutOfMemory;
    }
    // sizes of the real workloads (gigabytes of weights) are not touched by
    // anything here: a "device" allocation is at most 1 MiB of host memory
    const size_t host = bytes < (1u << 20) ? bytes : (1u << 20);
    void *p = malloc(host ? host : 1);
    if (p == nullptr) {
        return hipErrorOutOfMemory;
    }
    allocs[p] = bytes;
    serials[p] = ++total_allocs;
    *ptr = p;
    return hipSuccess;
}
hipError_t hipFree(void *ptr) {
    if (ptr == nullptr) {
        return hipSuccess;
    }
    std::lock_guard<std::mutex> g(mu);
    auto it = allocs.find(ptr);
    if (it == allocs.end()) {
        fprintf(stderr, "fake hipFree: %p is not a live allocation\n", ptr);
        abort();
    }
    allocs.erase(it);
    serials.erase(ptr);
    free(ptr);
    return hipSuccess;
}

namespace {

// the host bytes behind a device range (allocations above 1 MiB keep 1 MiB)
size_t host_bytes_of(const void *ptr, size_t bytes) {
    std::lock_guard<std::mutex> g(mu);
    auto it = allocs.upper_bound(ptr);
    if (it == allocs.begin()) {
        return 0;
    }
    --it;
    const size_t off = (size_t)((const char *)ptr - (const char *)it->first);
    if (off > it->second || bytes > it->second - off) {
        fprintf(stderr, "fake runtime: range %p+%zu leaves its allocation of %zu bytes\n", ptr, bytes,
                it->second);
        abort();
    }
    const size_t host = it->second < (1u << 20) ? it->second : (1u << 20);
    if (off >= host) {
        return 0;
    }
    return bytes < host - off ? bytes : host - off;
}

} // namespace

bool fake::device_range_live(const void *ptr, size_t bytes) {
    const size_t n = host_bytes_of(ptr, bytes ? bytes : 1);
    if (n > 0) { // touch both ends: the address sanitizer checks them
        volatile const char *p = (const char *)ptr;
        (void)p[0];
        (void)p[n - 1];
    }
    std::lock_guard<std::mutex> g(mu);
    auto it = allocs.upper_bound(ptr);
    return it != allocs.begin();
}

uint64_t fake::serial_of(const void *ptr) {
    std::lock_guard<std::mutex> g(mu);
    auto it = allocs.upper_bound(ptr);
    if (it == allocs.begin()) {
        return 0;
    }
    --it;
    const size_t off = (size_t)((const char *)ptr - (const char *)it->first);
    return off < (it->second ? it->second : 1) ? serials[it->first] : 0;
}

bool fake::enqueue(hipStream_t stream, const char *what) {
    std::lock_guard<std::mutex> g(mu);
    if (stream == nullptr || streams.count(stream) == 0) {
        return false;
    }
    if (stream->recording != nullptr) {
        stream->recording->nodes.push_back(what);
        return true;
    }
    ++enqueued;
    ++stream->issued;
    if (eager) {
        stream->completed = stream->issued;
    }
    return true;
}
bool fake::capturing(hipStream_t stream) {
    std::lock_guard<std::mutex> g(mu);
    return stream != nullptr && stream->recording != nullptr;
}
void fake::advance_all(uint64_t n) {
    std::lock_guard<std::mutex> g(mu);
    for (fake_stream *s : streams) {
        s->completed = s->completed + n < s->issued ? s->completed + n : s->issued;
    }
}
void fake::set_eager(bool e) {
    std::lock_guard<std::mutex> g(mu);
    eager = e;
}
fake::Counters fake::counters() {
    std::lock_guard<std::mutex> g(mu);
    Counters c{};
    c.live_allocs = allocs.size();
    for (auto &a : allocs) {
        c.live_bytes += a.second;
    }
    c.total_allocs = total_allocs;
    c.live_streams = streams.size();
    c.live_events = events.size();
    c.live_graphs = graphs.size();
    c.live_execs = execs.size();
    c.enqueued = enqueued;
    c.graph_launches = graph_launches;
    return c;
}
void fake::fail_malloc_after(uint64_t n) {
    std::lock_guard<std::mutex> g(mu);
    malloc_budget = n == 0 ? 0 : n + 1;
}

hipError_t hipMemset(void *ptr, int value, size_t bytes) {
    const size_t n = host_bytes_of(ptr, bytes);
    memset(ptr, value, n);
    return hipSuccess;
}
hipError_t hipMemsetAsync(void *ptr, int value, size_t bytes, hipStream_t stream) {
    if (fake::capturing(stream)) {
        fprintf(stderr, "fake runtime: memset recorded into a graph\n");
        abort(); // the library promises kernel nodes only
    }
    if (!fake::enqueue(stream, "memset")) {
        return hipErrorInvalidValue;
    }
    return hipMemset(ptr, value, bytes);
}
hipError_t hipMemcpyAsync(void *dst, const void *src, size_t bytes, hipMemcpyKind kind,
                          hipStream_t stream) {
    if (fake::capturing(stream)) {
        fprintf(stderr, "fake runtime: copy recorded into a graph\n");
        abort();
    }
    if (!fake::enqueue(stream, "memcpy")) {
        return hipErrorInvalidValue;
    }
    size_t n = bytes;
    if (kind != hipMemcpyHostToDevice) {
        n = host_bytes_of(src, bytes) < n ? host_bytes_of(src, bytes) : n;
    }
    if (kind != hipMemcpyDeviceToHost) {
        n = host_bytes_of(dst, bytes) < n ? host_bytes_of(dst, bytes) : n;
    }
    memmove(dst, src, n); // the sanitizer checks the host side's full range below
    if (kind == hipMemcpyDeviceToHost && n < bytes) {
        memset((char *)dst + n, 0, bytes - n);
    }
    if (kind == hipMemcpyHostToDevice && n < bytes) {
        volatile const char *p = (const char *)src;
        (void)p[bytes - 1];
    }
    return hipSuccess;
}

hipError_t hipStreamCreateWithFlags(hipStream_t *stream, unsigned) {
    std::lock_guard<std::mutex> g(mu);
    *stream = new fake_stream();
    streams.insert(*stream);
    return hipSuccess;
}
hipError_t hipStreamDestroy(hipStream_t stream) {
    std::lock_guard<std::mutex> g(mu);
    if (streams.erase(stream) == 0) {
        fprintf(stderr, "fake runtime: stream destroyed twice\n");
        abort();
    }
    for (fake_event *e : events) {
        if (e->stream == stream) {
            e->stream = nullptr;
        }
    }
    delete stream;
    return hipSuccess;
}
hipError_t hipStreamSynchronize(hipStream_t stream) {
    std::lock_guard<std::mutex> g(mu);
    if (stream == nullptr || streams.count(stream) == 0) {
        return hipErrorInvalidValue;
    }
    if (stream->recording != nullptr) {
        return hipErrorStreamCaptureUnsupported;
    }
    stream->completed = stream->issued;
    return hipSuccess;
}
hipError_t hipStreamWaitEvent(hipStream_t stream, hipEvent_t event, unsigned) {
    std::lock_guard<std::mutex> g(mu);
    if (streams.count(stream) == 0 || events.count(event) == 0) {
        return hipErrorInvalidValue;
    }
    // the waited-for work is complete before anything later on `stream` runs:
    // in this model, it completes now
    if (event->stream != nullptr && event->stream->completed < event->seq) {
        event->stream->completed = event->seq;
    }
    return hipSuccess;
}

hipError_t hipEventCreate(hipEvent_t *event) { return hipEventCreateWithFlags(event, 0); }
hipError_t hipEventCreateWithFlags(hipEvent_t *event, unsigned) {
    std::lock_guard<std::mutex> g(mu);
    *event = new fake_event();
    events.insert(*event);
    return hipSuccess;
}
hipError_t hipEventDestroy(hipEvent_t event) {
    std::lock_guard<std::mutex> g(mu);
    if (events.erase(event) == 0) {
        fprintf(stderr, "fake runtime: event destroyed twice (or never created)\n");
        abort();
    }
    delete event;
    return hipSuccess;
}
hipError_t hipEventRecord(hipEvent_t event, hipStream_t stream) {
    {
        std::lock_guard<std::mutex> g(mu);
        if (events.count(event) == 0 || streams.count(stream) == 0) {
            return hipErrorInvalidValue;
        }
        if (stream->recording != nullptr) {
            fprintf(stderr, "fake runtime: event recorded into a graph\n");
            abort();
        }
    }
    fake::enqueue(stream, "event");
    std::lock_guard<std::mutex> g(mu);
    event->stream = stream;
    event->seq = stream->issued;
    return hipSuccess;
}
hipError_t hipEventQuery(hipEvent_t event) {
    std::lock_guard<std::mutex> g(mu);
    if (events.count(event) == 0) {
        fprintf(stderr, "fake runtime: query of a destroyed event\n");
        abort();
    }
    if (event->stream == nullptr || event->stream->completed >= event->seq) {
        return hipSuccess;
    }
    return hipErrorNotReady;
}
hipError_t hipEventElapsedTime(float *ms, hipEvent_t start, hipEvent_t stop) {
    if (hipEventQuery(start) != hipSuccess || hipEventQuery(stop) != hipSuccess) {
        return hipErrorNotReady;
    }
    *ms = 0.001f * (float)(stop->seq >= start->seq ? stop->seq - start->seq : 0);
    return hipSuccess;
}

// (the launchers attach a commit's stop event to its last launch: the event is
// reached when the stream has completed that launch)
namespace fake {
void attach_event(hipEvent_t event, hipStream_t stream) {
    std::lock_guard<std::mutex> g(mu);
    if (events.count(event) == 0 || streams.count(stream) == 0) {
        fprintf(stderr, "fake runtime: stop event or stream of a launch is not live\n");
        abort();
    }
    event->stream = stream;
    event->seq = stream->issued;
}
} // namespace fake

hipError_t hipStreamBeginCapture(hipStream_t stream, hipStreamCaptureMode) {
    std::lock_guard<std::mutex> g(mu);
    if (streams.count(stream) == 0 || stream->recording != nullptr) {
        return hipErrorInvalidValue;
    }
    stream->recording = new fake_graph();
    graphs.insert(stream->recording);
    return hipSuccess;
}
hipError_t hipStreamEndCapture(hipStream_t stream, hipGraph_t *graph) {
    std::lock_guard<std::mutex> g(mu);
    if (streams.count(stream) == 0 || stream->recording == nullptr) {
        return hipErrorInvalidValue;
    }
    *graph = stream->recording;
    stream->recording = nullptr;
    return hipSuccess;
}
hipError_t hipGraphInstantiate(hipGraphExec_t *exec, hipGraph_t graph, void *, void *, size_t) {
    std::lock_guard<std::mutex> g(mu);
    if (graphs.count(graph) == 0) {
        return hipErrorInvalidValue;
    }
    *exec = new fake_graph_exec();
    (*exec)->nodes = graph->nodes;
    execs.insert(*exec);
    return hipSuccess;
}
hipError_t hipGraphLaunch(hipGraphExec_t exec, hipStream_t stream) {
    size_t n;
    {
        std::lock_guard<std::mutex> g(mu);
        if (execs.count(exec) == 0 || streams.count(stream) == 0) {
            return hipErrorInvalidValue;
        }
        n = exec->nodes.size();
        ++graph_launches;
    }
    for (size_t i = 0; i < n; ++i) {
        fake::enqueue(stream, "graph node");
    }
    return hipSuccess;
}
hipError_t hipGraphExecDestroy(hipGraphExec_t exec) {
    std::lock_guard<std::mutex> g(mu);
    if (exec != nullptr && execs.erase(exec) == 0) {
        fprintf(stderr, "fake runtime: graph exec destroyed twice\n");
        abort();
    }
    delete exec;
    return hipSuccess;
}
hipError_t hipGraphDestroy(hipGraph_t graph) {
    std::lock_guard<std::mutex> g(mu);
    if (graph != nullptr && graphs.erase(graph) == 0) {
        fprintf(stderr, "fake runtime: graph destroyed twice\n");
        abort();
    }
    delete graph;
    return hipSuccess;
}
