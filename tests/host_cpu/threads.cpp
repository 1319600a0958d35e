// Thread scenario for the CPU build of libtm_hip's host logic, meant for the
// thread sanitizer: what the library promises about threads is
//   - calls on one context are serialized by its owner (the typed layers hold a
//     lock around them, crates/metal/src/lib.rs:732-745), EXCEPT
//   - tm_hip_download_after and the dispatch counters, which another thread may
//     call while the owner commits (crates/metal/src/lib.rs:2618-2633 takes no
//     lock), and
//   - different contexts may be driven from different threads at once,
//     including their calls of tm_hip_q8_0_gemm_mma_noalloc, which share one
//     static workspace per GPU.
// Two owner threads each drive a context of their own through groups of
// products, calls that allocate nothing, fences and frees; a reader thread per
// context downloads results by commit number meanwhile; a clock thread lets the
// stand-in runtime's streams complete. Exit code 0 and no sanitizer report is
// the result.
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <unistd.h>
#include <vector>

#include <hip/hip_runtime.h>

#include "tm_hip.h"

namespace {

constexpr uint32_t ROWS = 1024, COLS = 1024, BATCH = 64;
std::atomic<bool> clock_stop{false};
std::atomic<int> failures{0};

void check(int rc, const char *what, const char *err) {
    if (rc != TM_HIP_OK) {
        fprintf(stderr, "%s failed (%d): %s\n", what, rc, err);
        failures.fetch_add(1);
    }
}

struct Shared {
    tm_hip_ctx *ctx = nullptr;
    tm_hip_buffer *y = nullptr;
    std::atomic<uint64_t> target{0};
    std::atomic<bool> done{false};
};

void reader(Shared *s) {
    std::vector<float> host(ROWS);
    char err[256];
    uint64_t reads = 0;
    while (!s->done.load(std::memory_order_acquire)) {
        const uint64_t t = s->target.load(std::memory_order_acquire);
        if (t == 0) {
            usleep(50);
            continue;
        }
        check(tm_hip_download_after(s->ctx, s->y, 0, host.data(), ROWS * 4u, t, err, sizeof err),
              "download_after", err);
        if (tm_hip_completed_dispatches(s->ctx) < t || tm_hip_committed_dispatches(s->ctx) < t) {
            fprintf(stderr, "download_after returned before its target completed\n");
            failures.fetch_add(1);
        }
        ++reads;
    }
    if (reads == 0) {
        fprintf(stderr, "the reader never ran\n");
        failures.fetch_add(1);
    }
}

void owner(int index, int iterations) {
    char err[512];
    Shared s;
    s.ctx = tm_hip_create(err, sizeof err);
    if (s.ctx == nullptr) {
        fprintf(stderr, "create: %s\n", err);
        failures.fetch_add(1);
        return;
    }
    const size_t wbytes = (size_t)ROWS * (COLS / 32u) * 34u;
    std::vector<uint8_t> raw(wbytes, (uint8_t)(index + 1));
    tm_hip_buffer *w = tm_hip_buffer_new(s.ctx, wbytes, 1, err, sizeof err);
    tm_hip_buffer *x = tm_hip_buffer_new(s.ctx, (size_t)BATCH * COLS * 4u, 1, err, sizeof err);
    tm_hip_buffer *g = tm_hip_buffer_new(s.ctx, COLS * 4u, 1, err, sizeof err);
    tm_hip_buffer *h = tm_hip_buffer_new(s.ctx, (size_t)BATCH * COLS * 4u, 1, err, sizeof err);
    tm_hip_buffer *big = tm_hip_buffer_new(s.ctx, (size_t)BATCH * ROWS * 4u, 1, err, sizeof err);
    s.y = tm_hip_buffer_new(s.ctx, ROWS * 4u, 1, err, sizeof err);
    if (w == nullptr || x == nullptr || g == nullptr || h == nullptr || big == nullptr || s.y == nullptr) {
        fprintf(stderr, "buffer_new: %s\n", err);
        failures.fetch_add(1);
        return;
    }
    check(tm_hip_upload(s.ctx, w, 0, raw.data(), wbytes, err, sizeof err), "upload", err);
    check(tm_hip_q8_0_pack(s.ctx, w, ROWS, COLS, err, sizeof err), "pack", err);
    std::thread rd(reader, &s);
    for (int i = 0; i < iterations; ++i) {
        check(tm_hip_begin_group(s.ctx, err, sizeof err), "begin_group", err);
        check(tm_hip_rmsnorm_f32(s.ctx, x, g, h, 1, COLS, 1e-6f, err, sizeof err), "rmsnorm", err);
        check(tm_hip_q8_0_gemv(s.ctx, w, h, s.y, ROWS, COLS, err, sizeof err), "gemv", err);
        check(tm_hip_end_group(s.ctx, err, sizeof err), "end_group", err);
        s.target.store(tm_hip_committed_dispatches(s.ctx), std::memory_order_release);
        if (i % 3 == 0) { // the static workspace, shared with the other thread's context
            check(tm_hip_q8_0_gemm_mma_noalloc(s.ctx, w, x, big, ROWS, COLS, BATCH, 0, 0, err, sizeof err),
                  "gemm_mma_noalloc", err);
        }
        if (i % 5 == 0) { // a short-lived buffer whose last use is still in flight when it is freed
            tm_hip_buffer *t = tm_hip_buffer_new(s.ctx, ROWS * 4u, 0, err, sizeof err);
            if (t == nullptr) {
                fprintf(stderr, "buffer_new: %s\n", err);
                failures.fetch_add(1);
            } else {
                check(tm_hip_q8_0_gemv(s.ctx, w, x, t, ROWS, COLS, err, sizeof err), "gemv", err);
                tm_hip_buffer_free(s.ctx, t);
            }
        }
        if (i % 16 == 15) {
            check(tm_hip_fence(s.ctx, err, sizeof err), "fence", err);
            (void)tm_hip_last_gpu_ms(s.ctx);
        }
    }
    check(tm_hip_fence(s.ctx, err, sizeof err), "fence", err);
    s.done.store(true, std::memory_order_release);
    rd.join();
    for (tm_hip_buffer *b : {w, x, g, h, big, s.y}) {
        tm_hip_buffer_free(s.ctx, b);
    }
    if (tm_hip_allocated_bytes(s.ctx) != 0 || tm_hip_in_flight_bytes(s.ctx) != 0) {
        fprintf(stderr, "context %d: bytes left allocated or in flight\n", index);
        failures.fetch_add(1);
    }
    tm_hip_destroy(s.ctx);
}

} // namespace

int main(int argc, char **argv) {
    const int iterations = argc > 1 ? atoi(argv[1]) : 200;
    fake::set_eager(false);
    std::thread clock([] {
        while (!clock_stop.load(std::memory_order_acquire)) {
            fake::advance_all(1);
            usleep(20);
        }
    });
    std::thread a(owner, 0, iterations), b(owner, 1, iterations);
    a.join();
    b.join();
    clock_stop.store(true, std::memory_order_release);
    clock.join();
    const fake::Counters c = fake::counters();
    if (c.live_allocs != 0 || c.live_streams != 0 || c.live_events > 1) {
        fprintf(stderr, "left behind: %llu allocations, %llu streams, %llu events\n",
                (unsigned long long)c.live_allocs, (unsigned long long)c.live_streams,
                (unsigned long long)c.live_events);
        failures.fetch_add(1);
    }
    printf("{\"k\":\"exit\",\"failures\":%d,\"enqueued\":%llu}\n", failures.load(),
           (unsigned long long)c.enqueued);
    return failures.load() == 0 ? 0 : 1;
}
