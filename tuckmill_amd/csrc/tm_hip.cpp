// tm_hip.cpp — host side of the C ABI declared in include/tm_hip.h.
//
// Mirrors the contract of the reference's Metal host
// (native/metal/tm_metal.m): argument validation before any device work,
// typed refusals, buffer leases held by pending commits, grouped encoding,
// completion accounting. The execution model underneath is HIP's: one
// non-blocking stream per context, one pair of HIP events per commit, and a
// group that is scheduled at end_group (independent Q8_0 products coalesce
// into one launch of the list kernel).
//
// This file holds the host logic only: validation, leases, commits, the
// dispatch planner, recorded steps. It names no kernel and includes no device
// code; what it asks of the device goes through the HIP runtime API and the
// launch interface of tm_launch.hpp. That is what lets it build with a plain
// C++ compiler against stand-ins for both, for the CPU tests that run the
// planner and the lifetime rules under sanitizers.
#include "tm_hip.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <deque>
#include <mutex>
#include <string>
#include <type_traits>
#include <unistd.h>
#include <vector>

#include "q8_plan.hpp"
#include "tm_launch.hpp"
#include "tm_plan.hpp"

using namespace tmh;

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
// Every context of a GPU shares that GPU's static workspace
// (tmdev::scratch_on_current_device), and each launches on its own
// stream. Calls of tm_hip_q8_0_gemm_mma_noalloc are ordered across contexts:
// the context whose call used the array last is remembered per device, and a
// call from another context first makes its stream wait for that one's (an
// event recorded on the last user's stream, one per device, created with the
// device's first context; nothing is allocated per call). All under
// g_scratch_mu, which a call holds from its wait to its last launch.
hipEvent_t g_scratch_event[kMaxDevices];
::tm_hip_ctx *g_scratch_last[kMaxDevices];

constexpr int kProfileSlots = 128;
constexpr int kProfileName = 48;

void alloc_release(Alloc *a) {
    if (a != nullptr && a->refs.fetch_sub(1, std::memory_order_acq_rel) == 1) {
        (void)hipFree(a->ptr);
        delete a;
    }
}

// An operation recorded into an open group holds a reference on every
// allocation it names from the moment it is recorded (the reference's group
// leases its buffers at encode time, native/metal/tm_metal.m:673, :707-739): a
// handle may be freed before end_group and the memory lives on. The references
// are dropped once the commit (or the recorded step) has taken its own, or when
// the group is aborted.
void ops_hold(const Op &op) {
    for (int i = 0; i < op.n_alloc; ++i) {
        if (op.a[i] != nullptr) {
            op.a[i]->refs.fetch_add(1, std::memory_order_relaxed);
        }
    }
}

void ops_drop(std::vector<Op> &ops) {
    for (const Op &op : ops) {
        for (int i = 0; i < op.n_alloc; ++i) {
            alloc_release(op.a[i]);
        }
    }
    ops.clear();
}

// `start` is either an event recorded just before the commit's work or, when
// the stream was still busy with the previous commit, that commit's stop
// event (the new work starts when the old one ends; one event fewer on the
// stream per commit). A lent stop event is recycled by its borrower.
struct Commit {
    uint64_t seq = 0;
    hipEvent_t start = nullptr, stop = nullptr;
    bool stop_lent = false;
    std::vector<Alloc *> keep;
    uint64_t leased = 0;
    char label[kProfileName] = {0};
};

struct ProfileSlot {
    char name[kProfileName];
    uint64_t nanos;
    uint64_t count;
};

} // namespace

struct tm_hip_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    hipStream_t copy_stream = nullptr;
    // The workspace of ordinary commits: grown on demand, never shrunk. A buffer
    // that was outgrown stays allocated until the context goes: recorded steps may
    // still point at it.
    Workspace ws;
    std::vector<void *> bx3_retired;
    // The fixed workspace inside the device's static array, and the allocations
    // that launches of tm_hip_q8_0_gemm_mma_noalloc still use: the next commit
    // adopts them (it completes after those launches), a fence releases them.
    Workspace fixed;
    std::vector<Alloc *> noalloc_keep;
    uint64_t noalloc_leased = 0;
    std::atomic<uint64_t> allocated{0};
    std::atomic<uint64_t> leased{0};
    std::atomic<uint64_t> committed{0};
    std::atomic<uint64_t> completed{0};
    std::atomic<uint64_t> last_gpu_nanos{0};
    std::atomic<uint64_t> gpu_nanos_total{0};
    std::atomic<uint64_t> launches{0};
    std::atomic<int> profiling{0};
    bool group_active = false;
    // Work put on the stream outside any commit since the last synchronize (zero
    // fills, the tail copy of a seal, launches of the allocation-free entry
    // point): a fence has to ask the runtime, the last commit's event does not
    // cover it. Under the caller's serialization.
    bool loose_work = false;
    std::vector<Op> group_ops;
    std::vector<struct tm_hip_step *> steps; // recorded steps not yet freed
    uint64_t plan_epoch = 0;
    std::mutex q_mu; // pending commits, event pool, profile table
    std::mutex copy_mu;
    std::deque<Commit> pending;
    std::deque<Commit> retired; // completed, GPU time not read yet (measure_retired)
    std::vector<hipEvent_t> event_pool;
    ProfileSlot profile[kProfileSlots];
    uint32_t profile_used = 0;
    bool commit_log_on = false;       // under q_mu
    std::deque<uint64_t> commit_log;  // GPU nanoseconds per completed commit, oldest first
};

struct tm_hip_buffer {
    tm_hip_ctx *owner;
    Alloc *alloc;
    size_t len;
    int shared;
};

// A recorded dispatch group: its planned launches as an instantiated HIP graph
// (kernel nodes only) and a reference on every allocation they touch, held
// until the step is freed.
struct tm_hip_step {
    tm_hip_ctx *owner = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    std::vector<Alloc *> keep;
    uint32_t launches = 0;
    uint32_t operators = 0;
};

namespace {

// ------------------------------------------------------------- errors ----

int fail(char *err, size_t cap, int code, const char *fmt, ...) {
    if (err != nullptr && cap > 0) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(err, cap, fmt, ap);
        va_end(ap);
    }
    return code;
}

int check_ctx(tm_hip_ctx *ctx, char *err, size_t cap, const char *what) {
    if (ctx == nullptr) {
        return fail(err, cap, TM_HIP_ERR_UNSUPPORTED, "%s: null context", what);
    }
    return TM_HIP_OK;
}

// native/metal/tm_metal.m:153-165: ownership first, then length.
int check_buffer(tm_hip_ctx *ctx, tm_hip_buffer *b, size_t need, char *err, size_t cap,
                 const char *name) {
    if (b == nullptr || b->owner != ctx) {
        return fail(err, cap, TM_HIP_ERR_UNSUPPORTED,
                    "%s: buffer does not belong to this context (different context or null)", name);
    }
    if (need == 0 || b->len < need) {
        return fail(err, cap, TM_HIP_ERR_BOUNDS, "%s: buffer holds %zu bytes but %zu are required",
                    name, b->len, need);
    }
    return TM_HIP_OK;
}

int hip_fail(char *err, size_t cap, const char *what, hipError_t e) {
    return fail(err, cap, TM_HIP_ERR_INTERNAL, "%s: %s", what, hipGetErrorString(e));
}

// ------------------------------------------------ completion accounting --

// Launches of tm_hip_q8_0_gemm_mma_noalloc hold at most this many allocations
// between two commits or fences (the list never grows: the call is refused).
constexpr size_t kNoallocKeepCap = 3u * TM_HIP_NOALLOC_MAX_PENDING;

// The stream has passed every launch of the allocation-free entry point (the
// caller has just synchronized it): give their allocations back.
void noalloc_release(tm_hip_ctx *ctx) {
    for (Alloc *a : ctx->noalloc_keep) {
        alloc_release(a);
    }
    ctx->noalloc_keep.clear();
    ctx->leased.fetch_sub(ctx->noalloc_leased, std::memory_order_relaxed);
    ctx->noalloc_leased = 0;
}

void account_profile(tm_hip_ctx *ctx, const char *label, uint64_t nanos) {
    // q_mu held by the caller
    if (label[0] == '\0') {
        return;
    }
    uint32_t slot = 0;
    while (slot < ctx->profile_used && strcmp(ctx->profile[slot].name, label) != 0) {
        slot++;
    }
    if (slot == ctx->profile_used && slot < kProfileSlots) {
        snprintf(ctx->profile[slot].name, kProfileName, "%s", label);
        ctx->profile[slot].nanos = 0;
        ctx->profile[slot].count = 0;
        ctx->profile_used++;
    }
    if (slot < kProfileSlots) {
        ctx->profile[slot].nanos += nanos;
        ctx->profile[slot].count += 1;
    }
}

// Take the GPU times of the retired commits (q_mu held by the caller): their
// events are read here, not when the commits retire, so that retiring a long
// queue at a fence costs nothing per commit beyond its leases; the measurement
// entry points ask for the times when somebody wants them.
void measure_retired(tm_hip_ctx *ctx, size_t at_most = ~(size_t)0) {
    while (!ctx->retired.empty() && at_most-- > 0) {
        Commit &c = ctx->retired.front();
        float ms = 0.0f;
        if (hipEventElapsedTime(&ms, c.start, c.stop) != hipSuccess || ms < 0.0f) {
            (void)hipGetLastError();
            ms = 0.0f;
        }
        const uint64_t nanos = (uint64_t)((double)ms * 1e6);
        ctx->last_gpu_nanos.store(nanos, std::memory_order_relaxed);
        ctx->gpu_nanos_total.fetch_add(nanos, std::memory_order_relaxed);
        account_profile(ctx, c.label, nanos);
        if (ctx->commit_log_on) {
            if (ctx->commit_log.size() >= TM_HIP_COMMIT_LOG_CAP) {
                ctx->commit_log.pop_front();
            }
            ctx->commit_log.push_back(nanos);
        }
        ctx->event_pool.push_back(c.start);
        if (!c.stop_lent) {
            ctx->event_pool.push_back(c.stop);
        }
        ctx->retired.pop_front();
    }
}

// An event for a new commit (q_mu held by the caller). Creating one costs tens of
// microseconds, more than issuing a whole decode step: when the pool is empty
// the events of commits that have retired are taken back first, their times
// read a few commits at a time (a long loop of commits that nobody measures
// used to create two events per commit until 1024 had retired: 138 us of host
// time per step of the 197-product group instead of 45).
hipEvent_t take_event(tm_hip_ctx *ctx) {
    if (ctx->event_pool.empty() && !ctx->retired.empty()) {
        measure_retired(ctx, 32);
    }
    if (!ctx->event_pool.empty()) {
        hipEvent_t e = ctx->event_pool.back();
        ctx->event_pool.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) {
        return nullptr;
    }
    return e;
}

// Retire every commit whose stop event has been reached, in order: its leases
// end and it counts as completed. `all_done`: the caller has just synchronized
// the stream, nothing needs to be asked. May be called from any thread.
constexpr size_t kMaxUnmeasured = 1024; // retired commits whose events wait to be read

void settle(tm_hip_ctx *ctx, bool all_done = false) {
    std::vector<Alloc *> release;
    {
        std::lock_guard<std::mutex> g(ctx->q_mu);
        while (!ctx->pending.empty()) {
            Commit &c = ctx->pending.front();
            if (!all_done && hipEventQuery(c.stop) != hipSuccess) {
                (void)hipGetLastError(); // "not ready" is not an error to keep
                break;
            }
            ctx->leased.fetch_sub(c.leased, std::memory_order_relaxed);
            release.insert(release.end(), c.keep.begin(), c.keep.end());
            c.keep.clear();
            ctx->retired.push_back(std::move(c));
            ctx->pending.pop_front();
            ctx->completed.fetch_add(1, std::memory_order_release);
        }
        if (ctx->retired.size() > kMaxUnmeasured) {
            measure_retired(ctx); // gives the events back to the pool
        }
    }
    for (Alloc *a : release) {
        alloc_release(a);
    }
}

// For the entry points that report GPU times.
void settle_and_measure(tm_hip_ctx *ctx) {
    settle(ctx);
    std::lock_guard<std::mutex> g(ctx->q_mu);
    measure_retired(ctx);
}

int wait_pending(tm_hip_ctx *ctx, char *err, size_t cap) {
    // A decode step lasts about 0.1 ms and its token is wanted at once: poll the
    // last commit's stop event for a while before handing the wait to the
    // runtime, whose wake-up alone costs tens of microseconds.
    hipEvent_t last = nullptr;
    {
        std::lock_guard<std::mutex> g(ctx->q_mu);
        if (!ctx->pending.empty()) {
            last = ctx->pending.back().stop;
        }
    }
    bool reached = false;
    if (last != nullptr) {
        const auto t0 = std::chrono::steady_clock::now();
        hipError_t q;
        while ((q = hipEventQuery(last)) == hipErrorNotReady &&
               std::chrono::steady_clock::now() - t0 < std::chrono::milliseconds(2)) {
        }
        (void)hipGetLastError(); // "not ready" is not an error to keep
        reached = q == hipSuccess;
    }
    // The stream runs in order: once the last commit's stop event is reached and
    // nothing was put on the stream outside a commit, everything is done, and
    // the runtime's own synchronize (which retires its record of every launch
    // since the last one, a few microseconds each) can be left for later.
    const bool proven = !ctx->loose_work && (last == nullptr || reached);
    if (!proven) {
        const hipError_t e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess) {
            return hip_fail(err, cap, "stream synchronize", e);
        }
        ctx->loose_work = false;
    }
    noalloc_release(ctx);
    settle(ctx, true);
    if (ctx->completed.load(std::memory_order_acquire) <
        ctx->committed.load(std::memory_order_relaxed)) {
        return fail(err, cap, TM_HIP_ERR_INTERNAL,
                    "fence: stream drained but completion accounting did not settle");
    }
    return TM_HIP_OK;
}

// ------------------------------------------------------------ launches ---

// Which prefill GEMMs over sealed weights run on the bf16 matrix cores: from 17
// tokens, and when the products that share the launch have enough work units
// (256 rows x 128 or 64 tokens x K chunk) between them for the kernel to pay
// (q8::bx3_launch_tile has the rule and the measurements behind it). The kernel
// is two to three times as fast as the f32 one when it fills the chip (at 512
// tokens 14336 x 4096: 204 us against 640 us, 6144 x 2048: 69 against 133; at 96
// tokens 14336 x 4096: 73 against 173) but its units are large: 1024 x 1024 at 512
// tokens takes 48 us alone against 15 us, while the seven projections of a
// Qwen3-0.6B layer together take 78 us against 144. The choice is made per launch:
// the same group gives the same bits every time, but a product's bits may depend
// on what shares its launch (the entry point is tolerance-qualified,
// native/metal/tm_metal.h:172-175; bit-identity claims belong to q8_0_gemm).
constexpr uint32_t kBx3MinBatch = 5; // (below 17 only what q8::mma_small_batch_on_tiles lets through)
constexpr uint64_t kBx3MaxPartialFloats = 1ull << 29; // 2 GiB of partial tiles per launch

bool x_aligned_of(const Op &op) {
    return ((uintptr_t)op.a[1]->ptr + (uintptr_t)op.x_off * 4u) % 16u == 0;
}

// The product could run on the bf16 matrix cores at all (its launch decides
// whether it does).
bool bx3_admissible(const Op &op) {
    return op.kind == OP_MMA && op.packed && x_aligned_of(op) && op.batch >= kBx3MinBatch &&
           (uint64_t)op.rows * op.cols < (1ull << 32) &&
           (uint64_t)op.batch * op.cols * 6u < (1ull << 32) &&
           (uint64_t)op.batch * op.cols < (1ull << 30);
}

// The most a product can need of the workspace, however its launch is cut
// (q8::bx3_plan_launch decides the chunks once the launch's list is known).
q8::Bx3Plan bx3_plan_bound(const Op &op, uint32_t tile_tokens) {
    return q8::bx3_plan_chunked(op.rows, op.cols, op.batch, tile_tokens,
                                q8::bx3_chunk_cap(op.rows, op.cols, op.batch, tile_tokens));
}

bool bx3_fits(const Op &op, uint32_t tile_tokens) {
    const q8::Bx3Plan plan = bx3_plan_bound(op, tile_tokens);
    return plan.split_tiles <= q8::BX3_MAX_SPLIT_TILES && plan.partial_floats <= kBx3MaxPartialFloats;
}

GemvKey bx3_key(uint32_t tile_tokens) {
    GemvKey k;
    k.kind = OP_MMA;
    k.variant = V_BF16X3;
    k.p0 = (uint8_t)(tile_tokens / 64u); // 2 or 1
    k.packed = true;
    k.flag = true;
    return k;
}

// The f32 matrix-core kernel's key: tile shape and the K split over a
// workgroup's waves are chosen per product. (What else shares the launch still
// shows in a product's last bits when the launch has few output tiles: each
// tile is then shared between workgroups, q8::mma_shared_parts.)
GemvKey mma_f32_key(const Op &op) {
    GemvKey k;
    k.kind = OP_MMA;
    k.packed = op.packed;
    k.flag = x_aligned_of(op);
    const q8::MmaProduct p{nullptr, nullptr, nullptr, op.rows, op.cols, op.batch};
    const q8::MmaConfig c = q8::pick_mma_config(&p, 1);
    k.variant = V_MMA;
    k.p0 = (uint8_t)c.tmw;
    k.p1 = (uint8_t)c.tnw;
    k.p2 = (uint8_t)c.s;
    return k;
}

// The key of a product that launches on its own (for OP_MMA products inside a
// group, assign_mma_keys decides per launch instead).
GemvKey gemv_key(const Op &op) {
    GemvKey k;
    k.kind = op.kind;
    k.packed = op.packed;
    if (op.kind == OP_I8) {
        k.flag = op.a[3] != nullptr;
        const bool small_regions = (uint64_t)op.rows * op.cols < (1ull << 32) &&
                                   (uint64_t)op.batch * op.cols < (1ull << 32);
        if (op.packed && op.a[3] == nullptr && op.batch >= q8::GEMM_I8_LDS_MIN_BATCH &&
            small_regions) {
            k.variant = V_I8_LDS;
            k.p0 = (uint8_t)q8::i8_lds_shape(op.batch);
            k.p1 = (uint8_t)(op.extra & 1u); // the fused tail (the other int8 kernels have none)
        } else if (op.packed && op.batch <= q8::GEMV_I8_MAX_BATCH) {
            k.variant = V_I8_STREAM;
            k.p0 = (uint8_t)q8::gemv_i8_tokens(op.batch);
        } else {
            k.variant = V_I8_TILE;
            k.p0 = (uint8_t)q8::pick_i8_config(op.batch);
        }
        return k;
    }
    if (op.kind == OP_F16_GEMM) {
        k.variant = V_F16;
        k.p0 = (uint8_t)q8::f16_tokens(op.batch);
        k.flag = (op.cols & 7u) == 0u;
        return k;
    }
    if (op.kind == OP_MMA) {
        if (bx3_admissible(op)) {
            const q8::Bx3Shape3 one{op.rows, op.cols, op.batch};
            const uint32_t tile = q8::bx3_launch_tile(&one, 1);
            if (tile != 0u && bx3_fits(op, tile)) {
                return bx3_key(tile);
            }
        }
        return mma_f32_key(op);
    }
    k.flag = x_aligned_of(op);
    if (op.batch == 1) {
        k.variant = V_DECODE;
    } else if ((op.packed || (op.cols & 63u) == 0u) && op.cols >= 1024u && op.cols < (1u << 27)) {
        // (the kernel indexes a token group's activations and a tile's quants in
        // 32 bits: rows of 2^27 columns and more take the general form)
        // waves x tokens per wave, measured on 2B-class shapes (the
        // alternatives were within 5 %)
        k.variant = V_SPLIT;
        k.p0 = op.batch <= 4 ? 1 : op.batch <= 8 ? 2 : 4;
        k.p1 = op.batch <= 2 ? 2 : op.batch <= 16 ? 4 : 8;
        k.p2 = (op.cols & 1023u) != 0u; // the instantiation that also handles a column tail
        if (k.p2 != 0 && k.p1 == 8) {
            // With a column tail the 8-tokens-per-wave form keeps 72 dwords per
            // lane in scratch: such a product goes as two groups of up to 16
            // tokens instead (split_token_groups; a token's result does not
            // depend on which tokens share its workgroup).
            k.p1 = 4;
        }
    } else {
        k.variant = V_GENERAL;
    }
    return k;
}

// Kernel launches a planned launch stands for.
uint32_t kernel_launches_of(const Launch &l) {
    if (l.single != nullptr || l.key.variant != V_BF16X3) {
        return 1u;
    }
    const uint32_t all = l.bx3_inputs >= 32 ? 0xffffffffu : (1u << l.bx3_inputs) - 1u;
    return (l.bx3_presplit & all) == all ? 1u : 2u; // the split pass, unless nothing is left to it
}

// Grow the split-float GEMM's workspace to what the largest of the planned
// launches needs (launches on the context's stream run one after the other and
// share it).
hipError_t ensure_bx3_workspace(tm_hip_ctx *ctx, const std::vector<Launch> &plan) {
    size_t xs = 0, partial = 0;
    for (const Launch &l : plan) {
        if (l.single == nullptr && (l.key.variant == V_BF16X3 || l.key.variant == V_MMA_SPLIT)) {
            xs = l.bx3_xs_bytes > xs ? (size_t)l.bx3_xs_bytes : xs;
            partial = l.bx3_partial_floats * 4u > partial ? (size_t)(l.bx3_partial_floats * 4u) : partial;
        }
    }
    auto grow = [&](void **buf, size_t *have, size_t need) -> hipError_t {
        if (need <= *have) {
            return hipSuccess;
        }
        need += need / 4u; // some room, so that a slightly larger chunk does not allocate again
        void *fresh = nullptr;
        hipError_t e = hipMalloc(&fresh, need);
        if (e != hipSuccess) {
            return e;
        }
        if (*buf != nullptr) {
            ctx->bx3_retired.push_back(*buf);
        }
        *buf = fresh;
        *have = need;
        return hipSuccess;
    };
    hipError_t e = grow((void **)&ctx->ws.xs, &ctx->ws.xs_bytes, xs);
    if (e == hipSuccess) {
        e = grow((void **)&ctx->ws.partials, &ctx->ws.partial_bytes, partial);
    }
    return e;
}

// The kernel of every matrix-core product (OP_MMA) of a sequence, decided per
// launch: consecutive products that do not depend on each other will share
// launches, and whether the ones that could run on the bf16 matrix cores do is
// decided on their sums (products of up to 32, up to 64 and of more tokens form
// three pools, each with the one tile q8::bx3_launch_tile gives it). The rest take the f32
// kernels. Entries of other operations are left unset.
std::vector<GemvKey> assign_mma_keys(tm_hip_ctx *ctx, const std::vector<Op> &ops) {
    std::vector<GemvKey> keys(ops.size());
    std::vector<size_t> run;
    uint64_t epoch = ++ctx->plan_epoch;
    auto close = [&]() {
        if (run.empty()) {
            return;
        }
        for (size_t i : run) {
            keys[i] = mma_f32_key(ops[i]);
        }
        for (uint32_t batch_class = 0; batch_class < 3; ++batch_class) {
            std::vector<size_t> pool;
            std::vector<q8::Bx3Shape3> shapes;
            for (size_t i : run) {
                const Op &op = ops[i];
                const uint32_t cls = op.batch <= 32u ? 0u : op.batch <= 64u ? 1u : 2u;
                if (bx3_admissible(op) && cls == batch_class) {
                    pool.push_back(i);
                    shapes.push_back(q8::Bx3Shape3{op.rows, op.cols, op.batch});
                }
            }
            const uint32_t tile = q8::bx3_launch_tile(shapes.data(), (int)shapes.size());
            if (tile == 0u) {
                continue;
            }
            for (size_t i : pool) {
                if (bx3_fits(ops[i], tile)) {
                    keys[i] = bx3_key(tile);
                }
            }
        }
        // The products left to the f32 matrix cores choose their token tile
        // together as well (q8::pick_mma_config: it depends on how many output
        // tiles the launch has). Those that could share a launch: the first
        // one's layout, alignment and K split.
        std::vector<size_t> f32_pool;
        std::vector<q8::MmaProduct> f32_shapes;
        for (size_t i : run) {
            const GemvKey &k = keys[i];
            if (k.variant != V_MMA || ops[i].batch <= 32u) {
                continue;
            }
            if (!f32_pool.empty()) {
                const GemvKey &first = keys[f32_pool.front()];
                if (k.packed != first.packed || k.flag != first.flag || k.p2 != first.p2) {
                    continue;
                }
            }
            f32_pool.push_back(i);
            f32_shapes.push_back(q8::MmaProduct{nullptr, nullptr, nullptr, ops[i].rows, ops[i].cols,
                                                ops[i].batch});
        }
        if (f32_pool.size() > 1) {
            const q8::MmaConfig c = q8::pick_mma_config(f32_shapes.data(), (int)f32_shapes.size());
            for (size_t i : f32_pool) {
                keys[i].p0 = (uint8_t)c.tmw;
            }
        }
        run.clear();
        epoch = ++ctx->plan_epoch;
    };
    for (size_t i = 0; i < ops.size(); ++i) {
        const Op &op = ops[i];
        if (op.kind != OP_MMA) {
            close();
            continue;
        }
        // the planner's own rule for sharing a launch (plan_launches below)
        const bool conflict = op.a[2]->read_epoch == epoch || op.a[2]->write_epoch == epoch ||
                              op.a[1]->write_epoch == epoch || op.a[0]->write_epoch == epoch;
        if (conflict || (int)run.size() == q8::MMA_MAX_DESCS) {
            close();
        }
        run.push_back(i);
        op.a[0]->read_epoch = epoch;
        op.a[1]->read_epoch = epoch;
        op.a[2]->write_epoch = epoch;
    }
    close();
    return keys;
}

// The K chunks of a bf16-matrix-core launch, decided for the launch as a whole
// once its list is known, and what it then needs of the workspace.
void cut_bx3_launch(Launch &l, uint64_t max_partial_floats = kBx3MaxPartialFloats) {
    if (l.single != nullptr || l.key.variant != V_BF16X3) {
        return;
    }
    q8::Bx3Shape3 shapes[q8::BX3_MAX_DESCS];
    uint32_t chunks[q8::BX3_MAX_DESCS];
    const int n = (int)l.list.size();
    for (int i = 0; i < n; ++i) {
        shapes[i] = q8::Bx3Shape3{l.list[i]->rows, l.list[i]->cols, l.list[i]->batch};
    }
    const uint32_t tile = l.key.p0 * 64u;
    q8::Bx3Tail tail;
    q8::bx3_plan_launch(shapes, n, tile, chunks, &tail);
    l.bx3_chunks.clear();
    l.bx3_tail = q8::Bx3Tail{};
    l.bx3_split_tiles = 0;
    l.bx3_partial_floats = 0;
    for (int i = 0; i < n; ++i) {
        const q8::Bx3Plan p = q8::bx3_plan_chunked(shapes[i].rows, shapes[i].cols, shapes[i].batch, tile,
                                                  chunks[i]);
        l.bx3_chunks.push_back((uint8_t)p.chunks);
        l.bx3_split_tiles += p.split_tiles;
        l.bx3_partial_floats += p.partial_floats;
    }
    if (tail.row_tiles != 0u) {
        // (the tail's product has its K whole, so nothing of it is counted above;
        // a tail that would not fit the workspace is left out)
        const q8::Bx3Shape3 &sh = shapes[tail.product];
        const uint32_t head = q8::bx3_head_rows(sh.rows, tail.row_tiles);
        const q8::Bx3Plan p = q8::bx3_plan_chunked(sh.rows - head, sh.cols, sh.batch, tile, tail.chunks);
        if (l.bx3_split_tiles + p.split_tiles <= q8::BX3_MAX_SPLIT_TILES &&
            l.bx3_partial_floats + p.partial_floats <= max_partial_floats) {
            l.bx3_tail = tail;
            l.bx3_tail.chunks = p.chunks;
            l.bx3_split_tiles += p.split_tiles;
            l.bx3_partial_floats += p.partial_floats;
        }
    }
}

// A bf16-matrix-core launch reads its activations in split form, which a pass
// of its own makes first: a dependent launch of about 5 us. Where the launch
// right before it is the RMSNorm or gated activation that writes those
// activations (the norm before q/k/v and before gate/up, the activation before
// the down projection), that operator writes the split form too, into the
// place in the workspace where the product launch expects it, and the input
// drops out of the split pass. Both launches are neighbours on one stream, so
// nothing else touches the workspace in between.
// plan[at] has just become a V_MMA_SPLIT launch. If it is the gate and the up
// projection of a gated unit, plan[at + 1] the gated activation over exactly their
// outputs and plan[at + 2] a launch of the same kind over exactly the activation's
// result (the down projection), the activation moves into the pair's launch, which
// then writes the projections, the activation and its split form (behind its own
// input's in the workspace): a layer's feed-forward half is three launches instead
// of four, every result with the same bits.
bool gated_pair_fusable(const std::vector<Launch> &plan, size_t at) {
    if (at + 2 >= plan.size()) {
        return false;
    }
    const Launch &pair = plan[at];
    const Launch &actl = plan[at + 1];
    const Launch &down = plan[at + 2];
    if (pair.list.size() != 2 || actl.single == nullptr || actl.update != nullptr || actl.split_xs_off >= 0 ||
        down.single != nullptr || down.key.variant != V_MMA || !down.key.packed) {
        return false;
    }
    const Op &act = *actl.single;
    if (act.kind != OP_SILU_MUL && act.kind != OP_GELU_MUL) {
        return false;
    }
    const Op *pg = pair.list[0], *pu = pair.list[1];
    const Alloc *out = act.a[2];
    const bool shapes = pg->rows == pu->rows && pg->cols == pu->cols && pg->y_off == 0 && pu->y_off == 0 &&
                        act.extra == (uint64_t)pg->rows * pg->batch && pg->rows % 32u == 0u;
    const bool wiring = pg->a[2] == act.a[0] && pu->a[2] == act.a[1] && pg->a[2] != pu->a[2] &&
                        out != pu->a[2] && out != pg->a[0] && out != pu->a[0];
    if (!shapes || !wiring) {
        return false;
    }
    for (const Op *op : down.list) {
        const bool whole = op->a[1] == out && op->x_off == 0 &&
                           (uint64_t)op->batch * op->cols == act.extra && op->cols == pg->rows;
        if (!whole || !same_input(*down.list[0], *op) || (uint64_t)op->batch * op->cols * 6u >= (1ull << 32) ||
            op->a[2] == out || op->a[2] == pg->a[2] || op->a[2] == pu->a[2]) {
            return false;
        }
    }
    return true;
}

void fuse_gated_pair(std::vector<Launch> &plan, size_t at) {
    if (!gated_pair_fusable(plan, at)) {
        return;
    }
    Launch &pair = plan[at];
    Launch &down = plan[at + 2];
    const Op &act = *plan[at + 1].single;
    pair.glu[0] = &act;
    pair.split_xs_off = (int64_t)pair.bx3_xs_bytes; // behind the pair's own input
    pair.split_cols = down.list[0]->cols;
    down.key.variant = V_MMA_SPLIT;
    down.bx3_inputs = 1;
    down.bx3_presplit = 1u;
    down.xs_in_off = pair.bx3_xs_bytes;
    down.bx3_xs_bytes = down.xs_in_off + bx3_xs_bytes_of(*down.list[0]);
    pair.bx3_xs_bytes = down.bx3_xs_bytes;
    plan.erase(plan.begin() + (ptrdiff_t)(at + 1));
}

void fuse_split_passes(std::vector<Launch> &plan) {
    for (size_t j = 1; j < plan.size(); ++j) {
        Launch &cons = plan[j];
        Launch &prod = plan[j - 1];
        if (cons.single != nullptr || prod.single == nullptr) {
            continue;
        }
        const Op &p = *prod.single;
        if (p.kind != OP_RMSNORM && p.kind != OP_SILU_MUL && p.kind != OP_GELU_MUL) {
            continue;
        }
        auto written_whole_by = [&](const Op &op) { // `op` reads exactly what `p` writes
            const bool whole = op.a[1] == p.a[2] && op.x_off == 0;
            const bool shape = p.kind == OP_RMSNORM ? op.batch == p.rows && op.cols == p.cols
                                                    : (uint64_t)op.batch * op.cols == p.extra;
            return whole && shape;
        };
        // (a gated pair on the staged kernel's 64-token tile, up to 256 tokens: with the
        // activation in its launch the small tiles are ahead; gate, up, silu_mul of the
        // 0.6B layer at 256 tokens 23.3 + 5.6 us staged)
        const bool staged_pair = cons.key.variant == V_BF16X3 && cons.key.p0 == 1 && cons.list.size() == 2 &&
                                 cons.list[0]->batch <= 256u && cons.list[0]->cols >= 512u &&
                                 cons.bx3_tail.row_tiles == 0u && gated_pair_fusable(plan, j);
        if (((cons.key.variant == V_MMA && cons.key.packed) || staged_pair) && prod.split_xs_off < 0) {
            // Products left to the f32 matrix cores (too few work units for the
            // staged kernel), all over the one input that `p` writes: with that
            // input in split form the same tiles run on the bf16 matrix cores
            // (gemm_mma_kernel<..., XP>), exact products in the place of f32 ones
            // and 20-30 % less time at every size measured (at 128 tokens: 4096 x 1024
            // 11.8 us against 16.4, 6144 x 1024 17.2 against 24.0, 1024 x 3072 12.1
            // against 15.2). Without the operator in front a split pass of 5 us
            // would have to make the split form: then the f32 kernel stays.
            bool all = true;
            for (const Op *op : cons.list) {
                all = all && written_whole_by(*op) && same_input(*cons.list[0], *op) &&
                      (uint64_t)op->batch * op->cols * 6u < (1ull << 32);
            }
            if (all) {
                cons.key.variant = V_MMA_SPLIT;
                cons.key.p0 = cons.key.p1 = cons.key.p2 = 0; // (the launcher picks the tiles)
                cons.bx3_chunks.clear();
                cons.bx3_split_tiles = 0;
                cons.bx3_partial_floats = 0;
                cons.bx3_inputs = 1;
                cons.bx3_presplit = 1u;
                cons.xs_in_off = 0;
                cons.bx3_xs_bytes = bx3_xs_bytes_of(*cons.list[0]);
                prod.split_xs_off = 0;
                prod.split_cols = cons.list[0]->cols;
                fuse_gated_pair(plan, j);
                continue;
            }
        }
        if (cons.key.variant != V_BF16X3) {
            continue;
        }
        // the launch's distinct inputs in list order, as launch_bx3_list lays them out
        const Op *input_of[q8::SPLIT_MAX_DESCS];
        int n_in = 0;
        size_t off = 0;
        for (const Op *op : cons.list) {
            int at = 0;
            while (at < n_in && !same_input(*input_of[at], *op)) {
                ++at;
            }
            if (at < n_in) {
                continue;
            }
            if (n_in == q8::SPLIT_MAX_DESCS) {
                break;
            }
            input_of[n_in] = op;
            if (written_whole_by(*op) && prod.split_xs_off < 0) {
                prod.split_xs_off = (int64_t)off;
                prod.split_cols = op->cols;
                cons.bx3_presplit |= 1u << n_in;
            }
            off += bx3_xs_bytes_of(*op);
            ++n_in;
        }
    }
}

// A launch of the token-split vector kernel whose products all came through the
// MFMA entry point (tolerance-qualified: free to take another kernel) at 9 to 16
// tokens, with 32 M weights and more between them, goes to the bf16 path instead,
// where up to 32 tokens means 32-token tiles behind a split pass
// (q8::bx3_small_batch_tiles): each product alone was too small for
// q8::mma_small_batch_on_tiles, together they are not (forty 2B-class matrices at 16
// tokens: 381 us on the vector kernel, about 210 there). Launches with operators fused
// in stay as they are.
void promote_small_batch_lists(std::vector<Launch> &plan) {
    for (Launch &l : plan) {
        if (l.single != nullptr || l.key.kind != OP_GEMV_LIST || l.key.variant != V_SPLIT || !l.key.packed ||
            l.norm != nullptr || l.per_token || l.list.empty() || l.list.size() > (size_t)q8::BX3_MAX_DESCS) {
            continue;
        }
        bool ok = true;
        q8::Bx3Shape3 shapes[q8::BX3_MAX_DESCS];
        const Op *input_of[q8::SPLIT_MAX_DESCS];
        int n = 0, n_in = 0;
        uint64_t xs_bytes = 0;
        for (size_t i = 0; i < l.list.size() && ok; ++i) {
            const Op &op = *l.list[i];
            Op as_mma = op;
            as_mma.kind = OP_MMA;
            ok = strcmp(op.what, "q8_0_gemm_mma") == 0 && op.batch >= 9u && op.batch <= 16u &&
                 l.residual[i] == nullptr && l.glu[i] == nullptr && bx3_admissible(as_mma) &&
                 bx3_fits(as_mma, 64u);
            shapes[n++] = q8::Bx3Shape3{op.rows, op.cols, op.batch};
            int at = 0;
            while (at < n_in && !same_input(*input_of[at], op)) {
                ++at;
            }
            if (at == n_in) {
                if (n_in == q8::SPLIT_MAX_DESCS) {
                    ok = false;
                    break;
                }
                input_of[n_in++] = &op;
                xs_bytes += bx3_xs_bytes_of(op);
            }
        }
        if (!ok || q8::bx3_launch_tile(shapes, n) != 64u) {
            continue;
        }
        l.key = bx3_key(64u);
        l.bx3_inputs = n_in;
        l.bx3_xs_bytes = xs_bytes;
        l.bx3_presplit = 0;
        l.descs = (uint32_t)n;
    }
}

// Plan the launches of a sequence of recorded operations. Consecutive
// list-kernel products that neither read nor overwrite each other's outputs
// share one launch; everything else launches on its own, in order.
std::vector<Launch> plan_launches(tm_hip_ctx *ctx, const std::vector<Op> &ops) {
    std::vector<Launch> plan;
    const std::vector<GemvKey> mma_keys = assign_mma_keys(ctx, ops);
    Launch cur;
    // Open prefill launches set aside while a product of another kernel is
    // listed (see below); closed together with `cur`.
    std::vector<Launch> parked;
    // Hazards are tracked per allocation with an epoch stamp, so planning a
    // step of n products costs O(n), not O(n^2).
    uint64_t epoch = ++ctx->plan_epoch;
    auto flush = [&]() {
        for (Launch &l : parked) {
            plan.push_back(std::move(l));
        }
        parked.clear();
        if (cur.norm != nullptr) {
            bool used = false;
            for (bool b : cur.normed) {
                used = used || b;
            }
            if (!used) { // nothing took the norm in: it launches on its own, first
                Launch one;
                one.single = cur.norm;
                plan.push_back(std::move(one));
                cur.norm = nullptr;
                // a few tokens stay one descriptor each only for a fusion that needs it
                bool other = false;
                for (size_t i = 0; i < cur.list.size(); ++i) {
                    other = other || cur.glu[i] != nullptr;
                }
                cur.per_token = cur.per_token && other;
            }
        }
        if (!cur.list.empty()) {
            plan.push_back(std::move(cur));
        }
        cur = Launch();
        epoch = ++ctx->plan_epoch;
    };
    for (size_t op_index = 0; op_index < ops.size(); ++op_index) {
        const Op &op = ops[op_index];
        if (op.kind == OP_GEMV_LIST || op.kind == OP_MMA || op.kind == OP_I8 ||
            op.kind == OP_F16_GEMM) {
            const GemvKey key = op.kind == OP_MMA ? mma_keys[op_index] : gemv_key(op);
            const int cap = key.kind == OP_MMA  ? q8::MMA_MAX_DESCS
                            : key.kind == OP_I8 ? q8::I8_MAX_DESCS
                                                : q8::GEMV_MAX_DESCS;
            // While a fused RMSNorm is pending only the decode kernel's
            // products may join its launch; the ones that read the norm's
            // whole output as their activations take it in without it going
            // through memory.
            const bool decode_kind = key.fusable();
            // (Not into a large product: the kernel variant with the fused forms
            // runs three waves per SIMD where the plain one runs four, which
            // costs a vocabulary projection three times the launch it saves:
            // 151936 x 1024 36.8 us with the norm inside against 24.5 + 3.9.)
            const bool large = (uint64_t)op.rows * op.cols > (16ull << 20);
            const bool normed = cur.norm != nullptr && decode_kind && !large &&
                                op.a[1] == cur.norm->a[2] && op.x_off == 0 &&
                                op.cols == cur.norm->cols && op.batch == cur.norm->rows;
            if ((cur.norm != nullptr && (!decode_kind || large)) || (cur.per_token && large)) {
                flush(); // (a large product does not go a token at a time either)
            }
            // a[0] = w (read), a[1] = x (read), a[2] = y (written), a[3] =
            // optional second output: the product joins the open launch
            // unless an output of it was read or written there, or one of
            // its inputs was written there.
            bool conflict = op.a[2]->read_epoch == epoch || op.a[2]->write_epoch == epoch ||
                            (!normed && op.a[1]->write_epoch == epoch) ||
                            op.a[0]->write_epoch == epoch;
            if (op.a[3] != nullptr) {
                conflict = conflict || op.a[3]->read_epoch == epoch || op.a[3]->write_epoch == epoch;
            }
            // The prefill products of a layer alternate between kernels (f32 and
            // bf16 matrix cores, tile shapes). As long as nothing depends on
            // anything since the last closed launch, each kernel keeps one
            // open launch: the open one is set aside, not closed, when a
            // product of another kernel arrives, and taken up again later.
            if (key.kind == OP_MMA && !conflict && cur.norm == nullptr && !cur.list.empty() &&
                cur.key.kind == OP_MMA && !(key == cur.key)) {
                parked.push_back(std::move(cur));
                cur = Launch();
                for (size_t i = 0; i < parked.size(); ++i) {
                    if (parked[i].key == key) {
                        cur = std::move(parked[i]);
                        parked.erase(parked.begin() + (long)i);
                        break;
                    }
                }
            }
            const bool open = !cur.list.empty() || cur.norm != nullptr;
            bool new_input = true;
            if (key.variant == V_BF16X3 && !cur.list.empty() && key == cur.key) {
                for (const Op *other : cur.list) {
                    new_input = new_input && !same_input(*other, op);
                }
                // the launch's share of the workspace stays within its limits
                const q8::Bx3Plan mine = bx3_plan_bound(op, key.p0 * 64u);
                conflict = conflict ||
                           cur.bx3_split_tiles + mine.split_tiles > q8::BX3_MAX_SPLIT_TILES ||
                           cur.bx3_partial_floats + mine.partial_floats > kBx3MaxPartialFloats ||
                           (new_input && cur.bx3_inputs == q8::SPLIT_MAX_DESCS);
            }
            // descriptors of this product (behind a pending norm, or in a launch
            // with a fusion already, a few tokens take one each)
            const bool each_token = key.few_tokens() && (cur.per_token || cur.norm != nullptr);
            const uint32_t need = each_token ? op.batch : split_token_groups(key, op.batch);
            if (open && (conflict || (!cur.list.empty() && !(key == cur.key)) ||
                         (int)(cur.descs + need) > cap)) {
                flush();
                new_input = true;
            }
            if (key.variant == V_BF16X3) {
                const q8::Bx3Plan mine = bx3_plan_bound(op, key.p0 * 64u);
                cur.bx3_split_tiles += mine.split_tiles;
                cur.bx3_partial_floats += mine.partial_floats;
                if (new_input) {
                    cur.bx3_inputs += 1;
                    cur.bx3_xs_bytes += bx3_xs_bytes_of(op);
                }
            }
            const bool takes_norm = normed && cur.norm != nullptr; // still pending after a flush?
            cur.key = key;
            cur.per_token = cur.per_token || (key.few_tokens() && cur.norm != nullptr);
            cur.descs += cur.per_token ? op.batch : split_token_groups(key, op.batch);
            cur.token_descs += op.batch;
            cur.list.push_back(&op);
            cur.residual.push_back(nullptr);
            cur.glu.push_back(nullptr);
            cur.normed.push_back(takes_norm);
            op.a[0]->read_epoch = epoch;
            op.a[1]->read_epoch = epoch;
            op.a[2]->write_epoch = epoch;
            if (op.a[3] != nullptr) {
                op.a[3]->write_epoch = epoch;
            }
        } else if (op.kind == OP_RMSNORM && op.rows <= 4u && op.cols >= 1024u &&
                   ((op.cols & 1023u) == 0u || (op.cols & 1023u) == 128u) && op.a[0] != op.a[2]) {
            // One row (or the few of a speculative step) in front of its
            // consumers (the norm before q/k/v, before gate/up, before the
            // vocabulary projection): held back and fused into the launch of
            // the products that read it, if any follow.
            flush();
            cur.norm = &op;
            op.a[0]->read_epoch = epoch;
            op.a[1]->read_epoch = epoch;
            op.a[2]->write_epoch = epoch;
        } else {
            // A residual update  h += alpha * t  right behind the one-token
            // product that wrote t rides in that product's epilogue (same
            // multiply-then-add per element), which saves a dependent launch:
            // t = a[0] must be exactly the product's whole output, and h must
            // be untouched by everything else in the open launch.
            // A gated activation right behind the gate and up projections it
            // consumes (same activations, same shape, decode kernel): both
            // rows of a pair are computed by one wave, which applies the
            // activation itself. `out` may be the gate buffer (in place).
            // With up to four tokens all of this holds per token: the launch
            // then takes a descriptor per product and token (Launch::per_token),
            // if they fit the kernel's list.
            const bool few_fit = cur.key.few_tokens() &&
                                 cur.token_descs <= (uint32_t)q8::GEMV_MAX_DESCS;
            if ((op.kind == OP_SILU_MUL || op.kind == OP_GELU_MUL) && cur.list.size() >= 2 &&
                (cur.key.decode() || few_fit)) {
                const size_t n = cur.list.size();
                const Op *pg = cur.list[n - 2], *pu = cur.list[n - 1];
                Alloc *out = op.a[2];
                const bool shapes = pg->batch == pu->batch && pg->a[1] == pu->a[1] &&
                                    pg->x_off == pu->x_off && pg->rows == pu->rows &&
                                    pg->cols == pu->cols && pg->cols >= 1024u &&
                                    ((pg->cols & 1023u) == 0u || (pg->cols & 1023u) == 128u) &&
                                    pg->y_off == 0 && pu->y_off == 0 &&
                                    op.extra == (uint64_t)pg->rows * pg->batch;
                const bool wiring = pg->a[2] == op.a[0] && pu->a[2] == op.a[1] &&
                                    pg->a[2] != pu->a[2] && out != pu->a[2];
                // (a few tokens: not with large products, which would then be read
                // once per token; the same bound as for the norm)
                const bool fits = !few_fit || (uint64_t)pg->rows * pg->cols <= (16ull << 20);
                const bool free_entries = fits && cur.residual[n - 2] == nullptr &&
                                          cur.residual[n - 1] == nullptr &&
                                          cur.glu[n - 2] == nullptr && cur.glu[n - 1] == nullptr &&
                                          (n < 3 || cur.glu[n - 3] == nullptr) &&
                                          cur.normed[n - 2] == cur.normed[n - 1];
                const bool out_free = out == pg->a[2] ||
                                      (out->read_epoch != epoch && out->write_epoch != epoch);
                if (shapes && wiring && free_entries && out_free) {
                    cur.glu[n - 2] = &op;
                    out->write_epoch = epoch;
                    if (few_fit) {
                        cur.per_token = true;
                        cur.descs = cur.token_descs;
                    }
                    continue;
                }
            }
            if (op.kind == OP_AXPY && !cur.list.empty() && cur.key.kind == OP_GEMV_LIST) {
                const Op *prod = cur.list.back();
                Alloc *h = op.a[1];
                const size_t n = cur.list.size();
                const bool in_pair = cur.glu[n - 1] != nullptr || (n >= 2 && cur.glu[n - 2] != nullptr);
                // (the token-split kernel has the same epilogue: any batch it takes;
                // which of the two kernels a few tokens run on is decided at the launch)
                const bool split = cur.key.variant == V_SPLIT;
                if (!in_pair && cur.residual.back() == nullptr && (prod->batch == 1 || split) &&
                    prod->a[2] == op.a[0] &&
                    prod->y_off == 0 && (uint64_t)prod->rows * prod->batch == op.extra &&
                    h != op.a[0] &&
                    h->read_epoch != epoch && h->write_epoch != epoch) {
                    cur.residual.back() = &op;
                    h->write_epoch = epoch;
                    continue;
                }
            }
            flush();
            // h += alpha * t, then the norm of h (the end of one block of a layer
            // and the start of the next, at prefill sizes): the norm does the
            // update on its way, one launch instead of two. The update must be
            // the launch right before, over exactly the norm's input.
            if (op.kind == OP_RMSNORM && !plan.empty() && plan.back().single != nullptr &&
                plan.back().single->kind == OP_AXPY && plan.back().update == nullptr) {
                const Op &up = *plan.back().single;
                if (up.a[1] == op.a[0] && (uint64_t)op.rows * op.cols == up.extra &&
                    up.a[0] != op.a[0] && up.a[0] != op.a[2] && op.a[1] != op.a[0]) {
                    plan.back().single = &op;
                    plan.back().update = &up;
                    continue;
                }
            }
            Launch one;
            one.single = &op;
            plan.push_back(std::move(one));
        }
    }
    flush();
    promote_small_batch_lists(plan);
    for (Launch &l : plan) {
        cut_bx3_launch(l);
    }
    fuse_split_passes(plan);
    return plan;
}

// One planned launch on the stream (`ws`: the context's grown workspace).
hipError_t issue_launch(tm_hip_ctx *ctx, hipEvent_t stop, const Launch &l) {
    if (l.single == nullptr) {
        return tmdev::launch_list(ctx->stream, stop, l, ctx->ws);
    }
    if (l.split_xs_off >= 0) {
        return tmdev::launch_single(ctx->stream, stop, *l.single,
                                    (uint16_t *)(ctx->ws.xs + l.split_xs_off), l.split_cols, l.update);
    }
    return tmdev::launch_single(ctx->stream, stop, *l.single, nullptr, 0, l.update);
}

// Issue the launches; the last one carries the commit's stop event.
hipError_t issue_ops(tm_hip_ctx *ctx, const std::vector<Op> &ops, hipEvent_t stop,
                     bool *stop_attached) {
    const std::vector<Launch> plan = plan_launches(ctx, ops);
    *stop_attached = false;
    hipError_t ws = ensure_bx3_workspace(ctx, plan);
    if (ws != hipSuccess) {
        return ws;
    }
    for (size_t i = 0; i < plan.size(); ++i) {
        const bool last = i + 1 == plan.size();
        const hipEvent_t ev = last ? stop : nullptr;
        const Launch &l = plan[i];
        hipError_t e = issue_launch(ctx, ev, l);
        if (e != hipSuccess) {
            return e;
        }
        ctx->launches.fetch_add(kernel_launches_of(l), std::memory_order_relaxed);
        if (last) {
            *stop_attached = true;
        }
    }
    return hipSuccess;
}

// Submit one commit: start event, the work `issue` puts on the stream, stop
// event, leases on `keep` until the stop event has been reached. `issue`
// receives the stop event and reports whether its last launch carries it.
template <typename Issue>
int commit_work(tm_hip_ctx *ctx, std::vector<Alloc *> keep, const char *label, const char *what,
                Issue issue, char *err, size_t cap) {
    Commit c;
    bool fresh_start = true;
    {
        std::lock_guard<std::mutex> g(ctx->q_mu);
        if (!ctx->pending.empty() && !ctx->pending.back().stop_lent &&
            hipEventQuery(ctx->pending.back().stop) == hipErrorNotReady) {
            c.start = ctx->pending.back().stop;
            ctx->pending.back().stop_lent = true;
            fresh_start = false;
        } else {
            c.start = take_event(ctx);
        }
        c.stop = take_event(ctx);
    }
    if (c.start == nullptr || c.stop == nullptr) {
        return fail(err, cap, TM_HIP_ERR_INTERNAL, "%s: event creation failed", what);
    }
    c.keep = std::move(keep);
    for (Alloc *a : c.keep) {
        a->refs.fetch_add(1, std::memory_order_relaxed);
        c.leased += a->len;
    }
    // Allocations still used by launches of the allocation-free entry point go
    // with this commit: it completes after them. Their bytes are in the ledger
    // already, and their references pass on as they are.
    const uint64_t adopted = ctx->noalloc_leased;
    c.keep.insert(c.keep.end(), ctx->noalloc_keep.begin(), ctx->noalloc_keep.end());
    ctx->noalloc_keep.clear();
    ctx->noalloc_leased = 0;
    if (ctx->profiling.load(std::memory_order_relaxed)) {
        snprintf(c.label, sizeof c.label, "%s", label);
    }
    hipError_t e = fresh_start ? hipEventRecord(c.start, ctx->stream) : hipSuccess;
    bool stop_attached = false;
    if (e == hipSuccess) {
        e = issue(c.stop, &stop_attached);
    }
    if (!stop_attached) { // an empty group, a replayed step, or a launch that failed
        hipError_t e2 = hipEventRecord(c.stop, ctx->stream);
        if (e == hipSuccess) {
            e = e2;
        }
    }
    c.seq = ctx->committed.fetch_add(1, std::memory_order_relaxed) + 1;
    ctx->leased.fetch_add(c.leased, std::memory_order_relaxed);
    c.leased += adopted;
    {
        std::lock_guard<std::mutex> g(ctx->q_mu);
        ctx->pending.push_back(std::move(c));
    }
    settle(ctx);
    if (e != hipSuccess) {
        return hip_fail(err, cap, what, e);
    }
    return TM_HIP_OK;
}

// Every allocation the operations touch, once each.
std::vector<Alloc *> allocs_of(tm_hip_ctx *ctx, const std::vector<Op> &ops) {
    std::vector<Alloc *> keep;
    const uint64_t keep_epoch = ++ctx->plan_epoch;
    keep.reserve(ops.size() * 3);
    for (const Op &op : ops) {
        for (int i = 0; i < op.n_alloc; ++i) {
            Alloc *a = op.a[i];
            if (a != nullptr && a->keep_epoch != keep_epoch) {
                a->keep_epoch = keep_epoch;
                keep.push_back(a);
            }
        }
    }
    return keep;
}

int commit_ops(tm_hip_ctx *ctx, const std::vector<Op> &ops, const char *label, const char *what,
               char *err, size_t cap) {
    return commit_work(
        ctx, allocs_of(ctx, ops), label, what,
        [&](hipEvent_t stop, bool *stop_attached) {
            return issue_ops(ctx, ops, stop, stop_attached);
        },
        err, cap);
}

// Either appends to the open group or commits on its own. The profile label
// is only formatted when profiling is on (it is off on the hot path).
int submit(tm_hip_ctx *ctx, Op &op, const char *what, char *err, size_t cap) {
    op.what = what;
    if (ctx->group_active) {
        ops_hold(op);
        ctx->group_ops.push_back(op);
        return TM_HIP_OK;
    }
    char label[kProfileName];
    label[0] = '\0';
    if (ctx->profiling.load(std::memory_order_relaxed)) {
        if (op.shape_label) {
            snprintf(label, sizeof label, "%s:%ux%u", what, op.rows, op.cols);
        } else {
            snprintf(label, sizeof label, "%s", what);
        }
    }
    std::vector<Op> one(1, op);
    return commit_ops(ctx, one, label, what, err, cap);
}

struct DeviceProbe {
    int available = 0;
    int device = -1;
    char info[256];
};

const DeviceProbe &probe() {
    static DeviceProbe p = [] {
        DeviceProbe r;
        int n = 0;
        if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
            (void)hipGetLastError();
            snprintf(r.info, sizeof r.info, "no HIP device available");
            return r;
        }
        for (int i = 0; i < n; ++i) {
            hipDeviceProp_t prop;
            if (hipGetDeviceProperties(&prop, i) != hipSuccess) {
                continue;
            }
            if (strncmp(prop.gcnArchName, "gfx950", 6) == 0) {
                r.available = 1;
                r.device = i;
                snprintf(r.info, sizeof r.info, "%s %s (%d CUs, %llu MiB device memory)", prop.name,
                         prop.gcnArchName, prop.multiProcessorCount,
                         (unsigned long long)(prop.totalGlobalMem / (1024ull * 1024ull)));
                return r;
            }
        }
        snprintf(r.info, sizeof r.info, "no HIP device of architecture gfx950 (%d other device%s)", n,
                 n == 1 ? "" : "s");
        return r;
    }();
    return p;
}

// Shared argument checks of the three products
// (native/metal/tm_metal.m:968-980, :1279-1290).
int check_product(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *x, tm_hip_buffer *y,
                  uint32_t rows, uint32_t cols, uint32_t batch, uint32_t max_batch, uint32_t x_off,
                  uint32_t y_off, char *err, size_t cap, const char *what) {
    if (check_ctx(ctx, err, cap, what) != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (rows == 0 || cols == 0 || (cols % 32u) != 0u || batch == 0 || batch > max_batch) {
        return fail(err, cap, TM_HIP_ERR_UNSUPPORTED,
                    "%s: rows %u, cols %u (a positive multiple of 32), batch %u (1..=%u)", what,
                    rows, cols, batch, max_batch);
    }
    const size_t w_need = (size_t)rows * ((size_t)cols / 32u) * 34u;
    const size_t x_need = ((size_t)x_off + (size_t)batch * cols) * 4u;
    const size_t y_need = ((size_t)y_off + (size_t)batch * rows) * 4u;
    tm_hip_buffer *bufs[3] = {w, x, y};
    const size_t needs[3] = {w_need, x_need, y_need};
    static const char *const suffix[3] = {"weights", "x", "y"};
    for (int i = 0; i < 3; ++i) {
        const tm_hip_buffer *b = bufs[i];
        if (b == nullptr || b->owner != ctx || needs[i] == 0 || b->len < needs[i]) {
            char name[64]; // only the refusal path formats the operand name
            snprintf(name, sizeof name, "%s.%s", what, suffix[i]);
            return check_buffer(ctx, bufs[i], needs[i], err, cap, name);
        }
    }
    if (w->alloc->packed && (w->alloc->prows != rows || w->alloc->pcols != cols)) {
        return fail(err, cap, TM_HIP_ERR_UNSUPPORTED,
                    "%s: weights were sealed as %ux%u but the call names %ux%u", what,
                    w->alloc->prows, w->alloc->pcols, rows, cols);
    }
    if (x->alloc->packed || y->alloc->packed) {
        return fail(err, cap, TM_HIP_ERR_UNSUPPORTED, "%s: x/y must not be sealed weight buffers",
                    what);
    }
    return TM_HIP_OK;
}

// The operation tm_hip_q8_0_gemm_mma records for a product.
Op mma_op(tm_hip_buffer *w, tm_hip_buffer *x, tm_hip_buffer *y, uint32_t rows, uint32_t cols,
          uint32_t batch, uint32_t x_off, uint32_t y_off) {
    Op op;
    // Below this batch a 32-token MFMA tile is mostly padding and the vector
    // kernels (GEMV arithmetic, which is within any tolerance of itself) are
    // faster: 1 token -> the decode kernel, 2..16 -> the token-split kernel.
    // (A large product is the exception: from 5 or 9 tokens it takes the 32-token
    // tiles on the bf16 matrix cores, q8::mma_small_batch_on_tiles.)
    const bool small = w->alloc->packed && (batch == 1 || (batch <= 16 && cols >= 1024u));
    op.kind = small ? OP_GEMV_LIST : OP_MMA;
    op.a[0] = w->alloc;
    op.a[1] = x->alloc;
    op.a[2] = y->alloc;
    op.n_alloc = 3;
    op.writes_mask = 4;
    op.rows = rows;
    op.cols = cols;
    op.batch = batch;
    op.x_off = x_off;
    op.y_off = y_off;
    op.packed = w->alloc->packed;
    op.what = "q8_0_gemm_mma";
    if (small && q8::mma_small_batch_on_tiles(rows, cols, batch)) {
        op.kind = OP_MMA;
        if (!bx3_admissible(op) || !bx3_fits(op, 64u)) {
            op.kind = OP_GEMV_LIST;
        }
    }
    return op;
}

// The stream must be idle with respect to the step's replays.
void step_dispose(tm_hip_step *step) {
    (void)hipGraphExecDestroy(step->exec);
    (void)hipGraphDestroy(step->graph);
    for (Alloc *a : step->keep) {
        alloc_release(a);
    }
    step->owner = nullptr;
    delete step;
}

} // namespace

// ================================================================ ABI =====

extern "C" {

int tm_hip_available(void) { return probe().available; }

const char *tm_hip_runtime_info(void) { return probe().info; }

tm_hip_ctx *tm_hip_create(char *err, size_t err_cap) {
    const DeviceProbe &p = probe();
    if (!p.available) {
        fail(err, err_cap, TM_HIP_ERR_NO_DEVICE, "%s", p.info);
        return nullptr;
    }
    hipError_t e = hipSetDevice(p.device);
    if (e != hipSuccess) {
        hip_fail(err, err_cap, "set device", e);
        return nullptr;
    }
    tm_hip_ctx *ctx = new (std::nothrow) tm_hip_ctx();
    if (ctx == nullptr) {
        fail(err, err_cap, TM_HIP_ERR_INTERNAL, "context allocation failed");
        return nullptr;
    }
    ctx->device = p.device;
    e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
    if (e == hipSuccess) {
        e = hipStreamCreateWithFlags(&ctx->copy_stream, hipStreamNonBlocking);
    }
    if (e != hipSuccess) {
        hip_fail(err, err_cap, "stream creation", e);
        tm_hip_destroy(ctx);
        return nullptr;
    }
    e = hipMalloc((void **)&ctx->ws.mma_queue, 256);
    if (e == hipSuccess) {
        e = hipMemset(ctx->ws.mma_queue, 0, 256);
    }
    if (e == hipSuccess) {
        e = hipMalloc((void **)&ctx->ws.mma_partials, q8::MMA_SHARED_PARTIAL_FLOATS * sizeof(float));
    }
    if (e == hipSuccess) {
        e = hipMalloc((void **)&ctx->ws.arrivals, q8::BX3_MAX_SPLIT_TILES * sizeof(uint32_t));
    }
    if (e == hipSuccess) {
        e = hipMemset(ctx->ws.arrivals, 0, q8::BX3_MAX_SPLIT_TILES * sizeof(uint32_t));
    }
    if (e != hipSuccess) {
        hip_fail(err, err_cap, "device-side counters", e);
        tm_hip_destroy(ctx);
        return nullptr;
    }
    // The static workspace of the entry point that allocates nothing: this
    // device's address of the array, asked here, with the device current; and
    // the device's event that orders the contexts' calls on it.
    uint8_t *fixed = nullptr;
    e = ctx->device >= 0 && ctx->device < kMaxDevices
            ? tmdev::scratch_on_current_device(ctx->device, &fixed)
            : hipErrorInvalidDevice;
    if (e == hipSuccess) {
        std::lock_guard<std::mutex> g(g_scratch_mu);
        if (g_scratch_event[ctx->device] == nullptr) {
            e = hipEventCreateWithFlags(&g_scratch_event[ctx->device], hipEventDisableTiming);
            if (e != hipSuccess) {
                g_scratch_event[ctx->device] = nullptr;
            }
        }
    }
    if (e != hipSuccess) {
        fail(err, err_cap, TM_HIP_ERR_SOURCE, "static workspace of this device is missing: %s",
             hipGetErrorString(e));
        tm_hip_destroy(ctx);
        return nullptr;
    }
    ctx->fixed.mma_queue = (uint32_t *)(fixed + kScratchQueueOff);
    ctx->fixed.arrivals = (uint32_t *)(fixed + kScratchArrivalsOff);
    ctx->fixed.xs = fixed + kScratchXsOff;
    ctx->fixed.xs_bytes = kScratchXsBytes;
    ctx->fixed.partials = (float *)(fixed + kScratchPartialOff);
    ctx->fixed.partial_bytes = kScratchPartialBytes;
    ctx->fixed.mma_partials = ctx->fixed.partials; // (a call runs one kernel family or the other)
    ctx->noalloc_keep.reserve(kNoallocKeepCap);
    // Fail at creation, not at first use, when the device code is missing.
    e = tmdev::kernels_present();
    if (e != hipSuccess) {
        fail(err, err_cap, TM_HIP_ERR_SOURCE, "kernels for this device are missing: %s",
             hipGetErrorString(e));
        tm_hip_destroy(ctx);
        return nullptr;
    }
    return ctx;
}

void tm_hip_destroy(tm_hip_ctx *ctx) {
    if (ctx == nullptr) {
        return;
    }
    if (ctx->group_active) {
        ops_drop(ctx->group_ops);
        ctx->group_active = false;
    }
    if (ctx->stream != nullptr) {
        (void)hipStreamSynchronize(ctx->stream);
    }
    settle(ctx);
    for (tm_hip_step *step : ctx->steps) { // recorded steps the caller never freed
        step_dispose(step);
    }
    ctx->steps.clear();
    {
        std::lock_guard<std::mutex> g(ctx->q_mu);
        for (Commit &c : ctx->pending) { // only after a device error
            for (Alloc *a : c.keep) {
                alloc_release(a);
            }
            (void)hipEventDestroy(c.start);
            if (!c.stop_lent) {
                (void)hipEventDestroy(c.stop);
            }
        }
        ctx->pending.clear();
        measure_retired(ctx); // hands the retired commits' events back to the pool
        for (hipEvent_t e : ctx->event_pool) {
            (void)hipEventDestroy(e);
        }
        ctx->event_pool.clear();
    }
    noalloc_release(ctx);
    {
        // (its stream is idle: no other context has anything left to wait for)
        std::lock_guard<std::mutex> g(g_scratch_mu);
        if (ctx->device >= 0 && ctx->device < kMaxDevices && g_scratch_last[ctx->device] == ctx) {
            g_scratch_last[ctx->device] = nullptr;
        }
    }
    for (void *p : {(void *)ctx->ws.mma_queue, (void *)ctx->ws.mma_partials,
                    (void *)ctx->ws.arrivals, (void *)ctx->ws.xs, (void *)ctx->ws.partials}) {
        if (p != nullptr) {
            (void)hipFree(p);
        }
    }
    for (void *p : ctx->bx3_retired) {
        (void)hipFree(p);
    }
    if (ctx->copy_stream != nullptr) {
        (void)hipStreamDestroy(ctx->copy_stream);
    }
    if (ctx->stream != nullptr) {
        (void)hipStreamDestroy(ctx->stream);
    }
    delete ctx;
}

tm_hip_buffer *tm_hip_buffer_new(tm_hip_ctx *ctx, size_t bytes, int shared, char *err,
                                 size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, "buffer_new") != TM_HIP_OK) {
        return nullptr;
    }
    if (bytes == 0) {
        fail(err, err_cap, TM_HIP_ERR_BOUNDS, "buffer_new: zero-length allocation");
        return nullptr;
    }
    void *ptr = nullptr;
    hipError_t e = hipMalloc(&ptr, bytes);
    if (e != hipSuccess || ptr == nullptr) {
        (void)hipGetLastError();
        fail(err, err_cap, TM_HIP_ERR_ALLOC, "buffer_new: allocation of %zu bytes failed (%s)",
             bytes, hipGetErrorString(e));
        return nullptr;
    }
    ctx->loose_work = true;
    e = hipMemsetAsync(ptr, 0, bytes, ctx->stream);
    if (e != hipSuccess) {
        (void)hipFree(ptr);
        hip_fail(err, err_cap, "buffer_new: zero fill", e);
        return nullptr;
    }
    Alloc *a = new (std::nothrow) Alloc();
    tm_hip_buffer *h = new (std::nothrow) tm_hip_buffer();
    if (a == nullptr || h == nullptr) {
        (void)hipStreamSynchronize(ctx->stream);
        (void)hipFree(ptr);
        delete a;
        delete h;
        fail(err, err_cap, TM_HIP_ERR_ALLOC, "buffer_new: handle allocation failed");
        return nullptr;
    }
    a->ptr = ptr;
    a->len = bytes;
    h->owner = ctx;
    h->alloc = a;
    h->len = bytes;
    h->shared = shared ? 1 : 0;
    ctx->allocated.fetch_add(bytes, std::memory_order_relaxed);
    return h;
}

void tm_hip_buffer_free(tm_hip_ctx *ctx, tm_hip_buffer *buffer) {
    if (ctx == nullptr || buffer == nullptr) {
        return;
    }
    if (buffer->owner != ctx) {
        fprintf(stderr, "tm_hip: buffer_free from a different context refused\n");
        return;
    }
    ctx->allocated.fetch_sub(buffer->len, std::memory_order_relaxed);
    Alloc *a = buffer->alloc;
    buffer->alloc = nullptr;
    buffer->owner = nullptr;
    delete buffer;
    settle(ctx);
    if (a->refs.load(std::memory_order_acquire) == 1) {
        // No commit leases it, but the zero fill of buffer_new or a host copy
        // may still be queued on the stream.
        (void)hipStreamSynchronize(ctx->stream);
        settle(ctx);
    }
    alloc_release(a);
}

size_t tm_hip_buffer_len(const tm_hip_ctx *ctx, const tm_hip_buffer *buffer) {
    if (ctx == nullptr || buffer == nullptr || buffer->owner != ctx) {
        return 0;
    }
    return buffer->len;
}

int tm_hip_buffer_zero(tm_hip_ctx *ctx, tm_hip_buffer *buffer, size_t off, size_t len, char *err,
                       size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, "buffer_zero") != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (buffer == nullptr || buffer->owner != ctx) {
        return fail(err, err_cap, TM_HIP_ERR_BOUNDS, "buffer_zero: foreign buffer");
    }
    if (len == 0) {
        return fail(err, err_cap, TM_HIP_ERR_BOUNDS, "buffer_zero: zero length");
    }
    if (off > buffer->len || len > buffer->len - off) {
        return fail(err, err_cap, TM_HIP_ERR_BOUNDS, "buffer_zero: range outside the buffer");
    }
    if (buffer->alloc->packed) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "buffer_zero: buffer holds sealed Q8_0 weights");
    }
    ctx->loose_work = true;
    hipError_t e = hipMemsetAsync((uint8_t *)buffer->alloc->ptr + off, 0, len, ctx->stream);
    if (e != hipSuccess) {
        return hip_fail(err, err_cap, "buffer_zero", e);
    }
    return TM_HIP_OK;
}

static int host_copy(tm_hip_ctx *ctx, tm_hip_buffer *buffer, size_t off, void *host, size_t len,
                     int to_device, char *err, size_t err_cap, const char *what) {
    if (check_ctx(ctx, err, err_cap, what) != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (buffer == nullptr || buffer->owner != ctx) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "%s: buffer does not belong to this context", what);
    }
    if (len == 0 || off > buffer->len || len > buffer->len - off) {
        return fail(err, err_cap, TM_HIP_ERR_BOUNDS, "%s: range %zu..%zu outside buffer", what, off,
                    off + len);
    }
    if (host == nullptr) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED, "%s: null host pointer", what);
    }
    if (!buffer->shared) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED, "%s: private buffers have no host copy",
                    what);
    }
    if (buffer->alloc->packed) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "%s: buffer holds sealed Q8_0 weights (device layout)", what);
    }
    if (ctx->group_active) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "%s: close the open dispatch group first", what);
    }
    int rc = wait_pending(ctx, err, err_cap);
    if (rc != TM_HIP_OK) {
        return rc;
    }
    uint8_t *dev = (uint8_t *)buffer->alloc->ptr + off;
    hipError_t e = to_device ? hipMemcpyAsync(dev, host, len, hipMemcpyHostToDevice, ctx->stream)
                             : hipMemcpyAsync(host, dev, len, hipMemcpyDeviceToHost, ctx->stream);
    if (e == hipSuccess) {
        e = hipStreamSynchronize(ctx->stream);
    }
    if (e != hipSuccess) {
        return hip_fail(err, err_cap, what, e);
    }
    return TM_HIP_OK;
}

int tm_hip_upload(tm_hip_ctx *ctx, tm_hip_buffer *dst, size_t off, const void *src, size_t len,
                  char *err, size_t err_cap) {
    return host_copy(ctx, dst, off, (void *)src, len, 1, err, err_cap, "upload");
}

int tm_hip_download(tm_hip_ctx *ctx, tm_hip_buffer *src, size_t off, void *dst, size_t len,
                    char *err, size_t err_cap) {
    return host_copy(ctx, src, off, dst, len, 0, err, err_cap, "download");
}

int tm_hip_download_after(tm_hip_ctx *ctx, tm_hip_buffer *src, size_t off, void *dst, size_t len,
                          uint64_t completed_target, char *err, size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, "download_after") != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (src == nullptr || src->owner != ctx) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "download_after: buffer does not belong to this context");
    }
    if (len == 0 || off > src->len || len > src->len - off) {
        return fail(err, err_cap, TM_HIP_ERR_BOUNDS, "download_after: range %zu..%zu outside buffer",
                    off, off + len);
    }
    if (dst == nullptr) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED, "download_after: null host pointer");
    }
    if (!src->shared || src->alloc->packed) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "download_after: buffer has no host copy");
    }
    if (completed_target > ctx->committed.load(std::memory_order_relaxed)) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "download_after: target is beyond the committed dispatches");
    }
    // Commits complete in stream order; wait for the target only.
    for (;;) {
        settle(ctx);
        if (ctx->completed.load(std::memory_order_acquire) >= completed_target) {
            break;
        }
        usleep(20);
    }
    std::lock_guard<std::mutex> g(ctx->copy_mu);
    hipError_t e = hipMemcpyAsync(dst, (const uint8_t *)src->alloc->ptr + off, len,
                                  hipMemcpyDeviceToHost, ctx->copy_stream);
    if (e == hipSuccess) {
        e = hipStreamSynchronize(ctx->copy_stream);
    }
    if (e != hipSuccess) {
        return hip_fail(err, err_cap, "download_after", e);
    }
    return TM_HIP_OK;
}

int tm_hip_copy_f32(tm_hip_ctx *ctx, tm_hip_buffer *src, uint32_t src_off, tm_hip_buffer *dst,
                    uint32_t dst_off, uint32_t n, char *err, size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, "copy_f32") != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (n == 0) {
        return fail(err, err_cap, TM_HIP_ERR_BOUNDS, "copy_f32: zero-length copy");
    }
    int rc;
    if ((rc = check_buffer(ctx, src, ((size_t)src_off + n) * 4u, err, err_cap, "copy_f32.src")) !=
            TM_HIP_OK ||
        (rc = check_buffer(ctx, dst, ((size_t)dst_off + n) * 4u, err, err_cap, "copy_f32.dst")) !=
            TM_HIP_OK) {
        return rc;
    }
    if (src->alloc->packed || dst->alloc->packed) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED, "copy_f32: sealed weight buffer");
    }
    Op op;
    op.kind = OP_COPY;
    op.a[0] = src->alloc;
    op.a[1] = dst->alloc;
    op.n_alloc = 2;
    op.writes_mask = 2;
    op.x_off = src_off;
    op.y_off = dst_off;
    op.extra = n;
    return submit(ctx, op, "copy_f32", err, err_cap);
}

int tm_hip_xor_checksum_u32(tm_hip_ctx *ctx, tm_hip_buffer *src, uint32_t src_off, uint32_t n,
                            tm_hip_buffer *partial, char *err, size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, "xor_checksum_u32") != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (n == 0) {
        return fail(err, err_cap, TM_HIP_ERR_BOUNDS, "xor_checksum_u32: zero length");
    }
    if ((src_off & 3u) != 0u) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "xor_checksum_u32: src_off %u is not a multiple of 4 words (16 bytes)", src_off);
    }
    int rc;
    if ((rc = check_buffer(ctx, src, ((size_t)src_off + n) * 4u, err, err_cap,
                           "xor_checksum_u32.src")) != TM_HIP_OK ||
        (rc = check_buffer(ctx, partial, TM_HIP_CHECKSUM_PARTIAL_BYTES, err, err_cap,
                           "xor_checksum_u32.partial")) != TM_HIP_OK) {
        return rc;
    }
    if (partial->alloc->packed) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "xor_checksum_u32: partial is a sealed weight buffer");
    }
    if (partial->alloc == src->alloc) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "xor_checksum_u32: partial must not be the buffer that is read");
    }
    Op op;
    op.kind = OP_CHECKSUM;
    op.a[0] = src->alloc;
    op.a[1] = partial->alloc;
    op.n_alloc = 2;
    op.writes_mask = 2;
    op.x_off = src_off;
    op.extra = n;
    return submit(ctx, op, "xor_checksum_u32", err, err_cap);
}

// ---- the small f32 operators either side of a product ----------------------

namespace {

// x -> y over n elements (f32, or binary16 on the side a cast names) with one scalar
// (native/metal/tm_metal.m:770-810).
int submit_1d(tm_hip_ctx *ctx, OpKind kind, tm_hip_buffer *a, tm_hip_buffer *b, float scalar,
              uint32_t n, char *err, size_t cap, const char *what) {
    const size_t a_elem = kind == OP_CAST_F16_F32 ? 2u : 4u;
    const size_t b_elem = kind == OP_CAST_F32_F16 ? 2u : 4u;
    if (check_ctx(ctx, err, cap, what) != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (n == 0) {
        return fail(err, cap, TM_HIP_ERR_BOUNDS, "%s: zero length", what);
    }
    int rc;
    if ((rc = check_buffer(ctx, a, (size_t)n * a_elem, err, cap, what)) != TM_HIP_OK ||
        (rc = check_buffer(ctx, b, (size_t)n * b_elem, err, cap, what)) != TM_HIP_OK) {
        return rc;
    }
    if (a->alloc->packed || b->alloc->packed) {
        return fail(err, cap, TM_HIP_ERR_UNSUPPORTED, "%s: sealed weight buffer", what);
    }
    Op op;
    op.kind = kind;
    op.a[0] = a->alloc;
    op.a[1] = b->alloc;
    op.n_alloc = 2;
    op.writes_mask = 2;
    op.extra = n;
    op.scalar = scalar;
    return submit(ctx, op, what, err, cap);
}

// out[i] = f(gate[i]) * up[i] (native/metal/tm_metal.m:1143-1177).
int submit_glu(tm_hip_ctx *ctx, OpKind kind, tm_hip_buffer *gate, tm_hip_buffer *up,
               tm_hip_buffer *out, uint32_t n, char *err, size_t cap, const char *what) {
    if (check_ctx(ctx, err, cap, what) != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (n == 0) {
        return fail(err, cap, TM_HIP_ERR_BOUNDS, "%s: zero length", what);
    }
    tm_hip_buffer *bufs[3] = {gate, up, out};
    static const char *const names[3] = {"gate", "up", "out"};
    for (int i = 0; i < 3; ++i) {
        char name[64];
        snprintf(name, sizeof name, "%s.%s", what, names[i]);
        const int rc = check_buffer(ctx, bufs[i], (size_t)n * 4u, err, cap, name);
        if (rc != TM_HIP_OK) {
            return rc;
        }
        if (bufs[i]->alloc->packed) {
            return fail(err, cap, TM_HIP_ERR_UNSUPPORTED, "%s: sealed weight buffer", name);
        }
    }
    Op op;
    op.kind = kind;
    op.a[0] = gate->alloc;
    op.a[1] = up->alloc;
    op.a[2] = out->alloc;
    op.n_alloc = 3;
    op.writes_mask = 4;
    op.extra = n;
    return submit(ctx, op, what, err, cap);
}

} // namespace

int tm_hip_f32_scale(tm_hip_ctx *ctx, tm_hip_buffer *x, tm_hip_buffer *y, float factor, uint32_t n,
                     char *err, size_t err_cap) {
    return submit_1d(ctx, OP_SCALE, x, y, factor, n, err, err_cap, "f32_scale");
}

int tm_hip_f32_axpy(tm_hip_ctx *ctx, tm_hip_buffer *a, tm_hip_buffer *y, float alpha, uint32_t n,
                    char *err, size_t err_cap) {
    return submit_1d(ctx, OP_AXPY, a, y, alpha, n, err, err_cap, "f32_axpy");
}

int tm_hip_cast_f16_f32(tm_hip_ctx *ctx, tm_hip_buffer *x, tm_hip_buffer *y, uint32_t n, char *err,
                        size_t err_cap) {
    return submit_1d(ctx, OP_CAST_F16_F32, x, y, 0.0f, n, err, err_cap, "cast_f16_f32");
}

int tm_hip_cast_f32_f16(tm_hip_ctx *ctx, tm_hip_buffer *x, tm_hip_buffer *y, uint32_t n, char *err,
                        size_t err_cap) {
    return submit_1d(ctx, OP_CAST_F32_F16, x, y, 0.0f, n, err, err_cap, "cast_f32_f16");
}

int tm_hip_silu_mul_f32(tm_hip_ctx *ctx, tm_hip_buffer *gate, tm_hip_buffer *up, tm_hip_buffer *out,
                        uint32_t n, char *err, size_t err_cap) {
    return submit_glu(ctx, OP_SILU_MUL, gate, up, out, n, err, err_cap, "silu_mul");
}

int tm_hip_gelu_tanh_mul_f32(tm_hip_ctx *ctx, tm_hip_buffer *gate, tm_hip_buffer *up,
                             tm_hip_buffer *out, uint32_t n, char *err, size_t err_cap) {
    return submit_glu(ctx, OP_GELU_MUL, gate, up, out, n, err, err_cap, "gelu_tanh_mul");
}

int tm_hip_rmsnorm_f32(tm_hip_ctx *ctx, tm_hip_buffer *x, tm_hip_buffer *weight, tm_hip_buffer *y,
                       uint32_t rows, uint32_t cols, float eps, char *err, size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, "rmsnorm") != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (rows == 0 || cols == 0) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED, "rmsnorm: zero shape");
    }
    const size_t x_need = (size_t)rows * cols * 4u;
    int rc;
    if ((rc = check_buffer(ctx, x, x_need, err, err_cap, "rmsnorm.x")) != TM_HIP_OK ||
        (rc = check_buffer(ctx, weight, (size_t)cols * 4u, err, err_cap, "rmsnorm.weight")) !=
            TM_HIP_OK ||
        (rc = check_buffer(ctx, y, x_need, err, err_cap, "rmsnorm.y")) != TM_HIP_OK) {
        return rc;
    }
    if (x->alloc->packed || weight->alloc->packed || y->alloc->packed) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED, "rmsnorm: sealed weight buffer");
    }
    Op op;
    op.kind = OP_RMSNORM;
    op.a[0] = x->alloc;
    op.a[1] = weight->alloc;
    op.a[2] = y->alloc;
    op.n_alloc = 3;
    op.writes_mask = 4;
    op.rows = rows;
    op.cols = cols;
    op.scalar = eps;
    return submit(ctx, op, "rmsnorm", err, err_cap);
}

int tm_hip_argmax_f32(tm_hip_ctx *ctx, tm_hip_buffer *x, uint32_t n, tm_hip_buffer *partial,
                      tm_hip_buffer *out, uint32_t out_index, char *err, size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, "argmax_f32") != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (n == 0) {
        return fail(err, err_cap, TM_HIP_ERR_BOUNDS, "argmax_f32: empty input");
    }
    int rc;
    if ((rc = check_buffer(ctx, x, (size_t)n * 4u, err, err_cap, "argmax_f32.x")) != TM_HIP_OK ||
        (rc = check_buffer(ctx, partial, q8::ARGMAX_PARTIAL_BYTES, err, err_cap,
                           "argmax_f32.partial")) != TM_HIP_OK ||
        (rc = check_buffer(ctx, out, ((size_t)out_index + 1u) * 4u, err, err_cap,
                           "argmax_f32.out")) != TM_HIP_OK) {
        return rc;
    }
    if (x->alloc->packed || partial->alloc->packed || out->alloc->packed) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED, "argmax_f32: sealed weight buffer");
    }
    Op op;
    op.kind = OP_ARGMAX;
    op.a[0] = x->alloc;
    op.a[1] = partial->alloc;
    op.a[2] = out->alloc;
    op.n_alloc = 3;
    op.writes_mask = 6;
    op.extra = n;
    op.y_off = out_index;
    return submit(ctx, op, "argmax_f32", err, err_cap);
}

int tm_hip_begin_group(tm_hip_ctx *ctx, char *err, size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, "begin_group") != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (ctx->group_active) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "begin_group: a dispatch group is already open");
    }
    ctx->group_ops.clear();
    ctx->group_active = true;
    return TM_HIP_OK;
}

int tm_hip_end_group(tm_hip_ctx *ctx, char *err, size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, "end_group") != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (!ctx->group_active) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED, "end_group: no dispatch group is open");
    }
    ctx->group_active = false;
    std::vector<Op> ops;
    ops.swap(ctx->group_ops);
    // An empty group still commits once, like an empty command buffer.
    const int rc = commit_ops(ctx, ops, "group", "group", err, err_cap);
    ops_drop(ops); // the commit holds its own leases now
    return rc;
}

int tm_hip_end_group_recorded(tm_hip_ctx *ctx, tm_hip_step **out, char *err, size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, "end_group_recorded") != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (out == nullptr) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED, "end_group_recorded: null result pointer");
    }
    *out = nullptr;
    if (!ctx->group_active) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "end_group_recorded: no dispatch group is open");
    }
    ctx->group_active = false;
    std::vector<Op> ops;
    ops.swap(ctx->group_ops);
    // The group's references go on every way out; a recorded step takes its own.
    struct DropOnExit {
        std::vector<Op> &ops;
        ~DropOnExit() { ops_drop(ops); }
    } drop_on_exit{ops};
    if (ops.empty()) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "end_group_recorded: the group holds no operation");
    }
    tm_hip_step *step = new (std::nothrow) tm_hip_step();
    if (step == nullptr) {
        return fail(err, err_cap, TM_HIP_ERR_ALLOC, "end_group_recorded: handle allocation failed");
    }
    step->owner = ctx;
    step->operators = (uint32_t)ops.size();
    const std::vector<Launch> plan = plan_launches(ctx, ops);
    hipError_t e = ensure_bx3_workspace(ctx, plan); // allocates: before the stream records
    if (e != hipSuccess) {
        delete step;
        return hip_fail(err, err_cap, "end_group_recorded: workspace", e);
    }
    // (No other context may put its ordering event on this stream while it
    // records: see tm_hip_q8_0_gemm_mma_noalloc.)
    std::lock_guard<std::mutex> scratch_guard(g_scratch_mu);
    // Relaxed mode: the launchers may query occupancy while the stream records.
    e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed);
    if (e != hipSuccess) {
        delete step;
        return hip_fail(err, err_cap, "end_group_recorded: begin capture", e);
    }
    hipError_t launch_err = hipSuccess;
    for (const Launch &l : plan) {
        launch_err = issue_launch(ctx, nullptr, l);
        if (launch_err != hipSuccess) {
            break;
        }
    }
    e = hipStreamEndCapture(ctx->stream, &step->graph);
    if (launch_err != hipSuccess || e != hipSuccess || step->graph == nullptr) {
        (void)hipGetLastError();
        if (step->graph != nullptr) {
            (void)hipGraphDestroy(step->graph);
        }
        delete step;
        return hip_fail(err, err_cap, "end_group_recorded: recording the launches",
                        launch_err != hipSuccess ? launch_err : e);
    }
    e = hipGraphInstantiate(&step->exec, step->graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        (void)hipGraphDestroy(step->graph);
        delete step;
        return hip_fail(err, err_cap, "end_group_recorded: graph instantiation", e);
    }
    step->launches = 0;
    for (const Launch &l : plan) {
        step->launches += kernel_launches_of(l);
    }
    step->keep = allocs_of(ctx, ops);
    for (Alloc *a : step->keep) {
        a->refs.fetch_add(1, std::memory_order_relaxed);
    }
    ctx->steps.push_back(step);
    *out = step;
    return TM_HIP_OK;
}

int tm_hip_step_run(tm_hip_ctx *ctx, tm_hip_step *step, char *err, size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, "step_run") != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (step == nullptr || step->owner != ctx) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "step_run: step does not belong to this context (different context or null)");
    }
    if (ctx->group_active) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "step_run: a dispatch group is open; end or abort it first");
    }
    const int rc = commit_work(
        ctx, step->keep, "step", "step_run",
        [&](hipEvent_t, bool *stop_attached) {
            *stop_attached = false;
            return hipGraphLaunch(step->exec, ctx->stream);
        },
        err, err_cap);
    if (rc == TM_HIP_OK) {
        ctx->launches.fetch_add(step->launches, std::memory_order_relaxed);
    }
    return rc;
}

uint32_t tm_hip_step_launches(const tm_hip_ctx *ctx, const tm_hip_step *step) {
    if (ctx == nullptr || step == nullptr || step->owner != ctx) {
        return 0;
    }
    return step->launches;
}

void tm_hip_step_free(tm_hip_ctx *ctx, tm_hip_step *step) {
    if (ctx == nullptr || step == nullptr) {
        return;
    }
    if (step->owner != ctx) {
        fprintf(stderr, "tm_hip: step_free from a different context refused\n");
        return;
    }
    // Replays still queued read the graph's kernel arguments and the buffers.
    (void)hipStreamSynchronize(ctx->stream);
    settle(ctx);
    for (size_t i = 0; i < ctx->steps.size(); ++i) {
        if (ctx->steps[i] == step) {
            ctx->steps.erase(ctx->steps.begin() + (long)i);
            break;
        }
    }
    step_dispose(step);
}

int tm_hip_abort_group(tm_hip_ctx *ctx, char *err, size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, "abort_group") != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (!ctx->group_active) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED, "abort_group: no dispatch group is open");
    }
    ops_drop(ctx->group_ops);
    ctx->group_active = false;
    return TM_HIP_OK;
}

int tm_hip_fence(tm_hip_ctx *ctx, char *err, size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, "fence") != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (ctx->group_active) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "fence: a dispatch group is open; end or abort it first");
    }
    return wait_pending(ctx, err, err_cap);
}

// ---------------------------------------------------------- products -----

static int product_list(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *x, tm_hip_buffer *y,
                        uint32_t rows, uint32_t cols, uint32_t batch, uint32_t x_off,
                        uint32_t y_off, const char *what, char *err, size_t err_cap) {
    Op op;
    op.kind = OP_GEMV_LIST;
    op.a[0] = w->alloc;
    op.a[1] = x->alloc;
    op.a[2] = y->alloc;
    op.n_alloc = 3;
    op.writes_mask = 4;
    op.rows = rows;
    op.cols = cols;
    op.batch = batch;
    op.x_off = x_off;
    op.y_off = y_off;
    op.packed = w->alloc->packed;
    op.shape_label = true; // native/metal/tm_metal.m:1008-1015
    return submit(ctx, op, what, err, err_cap);
}

int tm_hip_q8_0_gemv(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *x, tm_hip_buffer *y,
                     uint32_t rows, uint32_t cols, char *err, size_t err_cap) {
    int rc = check_product(ctx, w, x, y, rows, cols, 1, 1, 0, 0, err, err_cap, "q8_0_gemv");
    if (rc != TM_HIP_OK) {
        return rc;
    }
    return product_list(ctx, w, x, y, rows, cols, 1, 0, 0, "q8_0_gemv", err, err_cap);
}

int tm_hip_q8_0_gemm(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *x, tm_hip_buffer *y,
                     uint32_t rows, uint32_t cols, uint32_t batch, uint32_t x_off, uint32_t y_off,
                     char *err, size_t err_cap) {
    int rc = check_product(ctx, w, x, y, rows, cols, batch, TM_HIP_GEMM_MAX_BATCH, x_off, y_off, err,
                           err_cap, "q8_0_gemm");
    if (rc != TM_HIP_OK) {
        return rc;
    }
    return product_list(ctx, w, x, y, rows, cols, batch, x_off, y_off, "q8_0_gemm", err, err_cap);
}

int tm_hip_q8_0_gemm_mma(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *x, tm_hip_buffer *y,
                         uint32_t rows, uint32_t cols, uint32_t batch, uint32_t x_off,
                         uint32_t y_off, char *err, size_t err_cap) {
    int rc = check_product(ctx, w, x, y, rows, cols, batch, TM_HIP_GEMM_MMA_MAX_BATCH, x_off, y_off,
                           err, err_cap, "q8_0_gemm_mma");
    if (rc != TM_HIP_OK) {
        return rc;
    }
    Op op = mma_op(w, x, y, rows, cols, batch, x_off, y_off);
    return submit(ctx, op, "q8_0_gemm_mma", err, err_cap);
}

int tm_hip_q8_0_gemm_mma_noalloc(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *x,
                                 tm_hip_buffer *y, uint32_t rows, uint32_t cols, uint32_t batch,
                                 uint32_t x_off, uint32_t y_off, char *err, size_t err_cap) {
    const char *what = "q8_0_gemm_mma_noalloc";
    int rc = check_product(ctx, w, x, y, rows, cols, batch, TM_HIP_GEMM_MMA_MAX_BATCH, x_off, y_off,
                           err, err_cap, what);
    if (rc != TM_HIP_OK) {
        return rc;
    }
    if (ctx->group_active) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "%s: launches at once, not into the open dispatch group; close the group first",
                    what);
    }
    const Op op = mma_op(w, x, y, rows, cols, batch, x_off, y_off);
    Launch launch;
    launch.key = gemv_key(op);
    launch.list.push_back(&op);
    launch.residual.push_back(nullptr);
    launch.glu.push_back(nullptr);
    launch.normed.push_back(false);
    bool counters = launch.key.kind == OP_MMA; // the work-queue form of the f32 kernel may run
    if (launch.key.variant == V_BF16X3) {
        cut_bx3_launch(launch, ctx->fixed.partial_bytes / 4u); // (a tail only if the static array holds it)
        launch.bx3_xs_bytes = bx3_xs_bytes_of(op);
        launch.bx3_inputs = 1;
        if (launch.bx3_xs_bytes > ctx->fixed.xs_bytes ||
            launch.bx3_partial_floats * 4u > ctx->fixed.partial_bytes) {
            return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                        "%s: %u tokens x %u columns on %u rows need %llu bytes of split activations "
                        "and %llu bytes of partial tiles, the static workspace holds %zu and %zu; "
                        "use q8_0_gemm_mma, or fewer tokens per call",
                        what, batch, cols, rows, (unsigned long long)launch.bx3_xs_bytes,
                        (unsigned long long)(launch.bx3_partial_floats * 4u), ctx->fixed.xs_bytes,
                        ctx->fixed.partial_bytes);
        }
        counters = launch.bx3_split_tiles > 0;
    }
    if (ctx->noalloc_keep.size() + 3u > kNoallocKeepCap) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "%s: %zu buffers of earlier calls are still held; commit other work or call "
                    "fence first",
                    what, ctx->noalloc_keep.size());
    }
    // The array is this GPU's, not this context's: behind another context's calls
    // this one's launches wait for that context's stream first.
    std::lock_guard<std::mutex> scratch_guard(g_scratch_mu);
    if (g_scratch_last[ctx->device] != nullptr && g_scratch_last[ctx->device] != ctx) {
        hipError_t e = hipEventRecord(g_scratch_event[ctx->device], g_scratch_last[ctx->device]->stream);
        if (e == hipSuccess) {
            e = hipStreamWaitEvent(ctx->stream, g_scratch_event[ctx->device], 0);
        }
        if (e != hipSuccess) {
            return hip_fail(err, err_cap, "q8_0_gemm_mma_noalloc: ordering behind another context", e);
        }
    }
    g_scratch_last[ctx->device] = ctx;
    ctx->loose_work = true; // launched outside any commit: a fence asks the runtime
    // Held until the next commit adopts them or a fence has passed them (the list
    // has its capacity from tm_hip_create on).
    for (int i = 0; i < 3; ++i) {
        op.a[i]->refs.fetch_add(1, std::memory_order_relaxed);
        ctx->noalloc_keep.push_back(op.a[i]);
        ctx->noalloc_leased += op.a[i]->len;
        ctx->leased.fetch_add(op.a[i]->len, std::memory_order_relaxed);
    }
    if (counters) {
        // The array keeps what the last call left in it, and every call on this
        // GPU shares it: the counters start from zero whatever came before. A
        // fill kernel, not a memset, so that a caller may record the call.
        const hipError_t e = tmdev::zero_words(ctx->stream, (uint32_t *)ctx->fixed.mma_queue,
                                               (uint32_t)kScratchCounterDwords);
        if (e != hipSuccess) {
            return hip_fail(err, err_cap, what, e);
        }
        ctx->launches.fetch_add(1, std::memory_order_relaxed);
    }
    const hipError_t e = tmdev::launch_list(ctx->stream, nullptr, launch, ctx->fixed);
    if (e != hipSuccess) {
        return hip_fail(err, err_cap, what, e);
    }
    ctx->launches.fetch_add(kernel_launches_of(launch), std::memory_order_relaxed);
    return TM_HIP_OK;
}

int tm_hip_q8_0_row_f32(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *out, uint32_t row,
                        uint32_t cols, uint32_t out_off, char *err, size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, "q8_0_row") != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (cols == 0 || (cols % 32u) != 0u) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "q8_0_row: cols must be a positive multiple of 32");
    }
    const size_t w_need = ((size_t)row + 1u) * ((size_t)cols / 32u) * 34u;
    int rc;
    if ((rc = check_buffer(ctx, w, w_need, err, err_cap, "q8_0_row.weights")) != TM_HIP_OK ||
        (rc = check_buffer(ctx, out, ((size_t)out_off + cols) * 4u, err, err_cap, "q8_0_row.out")) !=
            TM_HIP_OK) {
        return rc;
    }
    if (w->alloc->packed && w->alloc->pcols != cols) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "q8_0_row: weights were sealed with cols %u but the call names %u",
                    w->alloc->pcols, cols);
    }
    if (out->alloc->packed) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED, "q8_0_row: out is a sealed weight buffer");
    }
    Op op;
    op.kind = OP_ROW;
    op.a[0] = w->alloc;
    op.a[1] = out->alloc;
    op.n_alloc = 2;
    op.writes_mask = 2;
    op.rows = w->alloc->packed ? w->alloc->prows : row + 1u;
    op.cols = cols;
    op.extra = row;
    op.y_off = out_off;
    op.packed = w->alloc->packed;
    return submit(ctx, op, "q8_0_row", err, err_cap);
}

int tm_hip_row_indirect_f32(tm_hip_ctx *ctx, tm_hip_buffer *w, uint32_t type_id, uint32_t rows,
                            uint32_t cols, tm_hip_buffer *ids, uint32_t slot, tm_hip_buffer *out,
                            char *err, size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, "row_indirect") != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    // native/metal/tm_metal.m:874-885: Q8_0 (type 8) or F16 (type 1)
    const bool f16 = type_id == 1u && cols > 0;
    if (!f16 && !(type_id == 8u && cols > 0 && (cols % 32u) == 0u)) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "row_indirect: type %u with cols %u is unsupported (Q8_0, type 8, with cols a "
                    "positive multiple of 32, or F16, type 1)",
                    type_id, cols);
    }
    const size_t w_need = f16 ? (size_t)rows * (size_t)cols * 2u
                              : (size_t)rows * ((size_t)cols / 32u) * 34u;
    if (rows == 0) {
        return fail(err, err_cap, TM_HIP_ERR_BOUNDS, "row_indirect: zero rows");
    }
    int rc;
    if ((rc = check_buffer(ctx, w, w_need, err, err_cap, "row_indirect.weights")) != TM_HIP_OK ||
        (rc = check_buffer(ctx, ids, ((size_t)slot + 1u) * 4u, err, err_cap, "row_indirect.ids")) !=
            TM_HIP_OK ||
        (rc = check_buffer(ctx, out, (size_t)cols * 4u, err, err_cap, "row_indirect.out")) !=
            TM_HIP_OK) {
        return rc;
    }
    if (f16 && w->alloc->packed) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "row_indirect: type 1 (F16) names a sealed Q8_0 weight buffer");
    }
    if (w->alloc->packed && (w->alloc->prows != rows || w->alloc->pcols != cols)) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "row_indirect: weights were sealed as %ux%u but the call names %ux%u",
                    w->alloc->prows, w->alloc->pcols, rows, cols);
    }
    if (ids->alloc->packed || out->alloc->packed) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED, "row_indirect: sealed weight buffer");
    }
    Op op;
    op.kind = f16 ? OP_F16_ROW_INDIRECT : OP_ROW_INDIRECT;
    op.a[0] = w->alloc;
    op.a[1] = out->alloc;
    op.a[2] = ids->alloc;
    op.n_alloc = 3;
    op.writes_mask = 2;
    op.rows = rows;
    op.cols = cols;
    op.extra = slot;
    op.packed = w->alloc->packed;
    return submit(ctx, op, "row_indirect", err, err_cap);
}

// ------------------------------------------------- F16 weight twins ------

// native/metal/tm_metal.m:1279-1290 (shape, then bounds) with w_need of :1349.
static int f16_product(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *x, tm_hip_buffer *y,
                       uint32_t rows, uint32_t cols, uint32_t batch, uint32_t x_off,
                       uint32_t y_off, const char *what, char *err, size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, what) != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (rows == 0 || cols == 0 || batch == 0 || batch > q8::F16_GEMM_MAX_BATCH) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED, "%s: rows %u, cols %u, batch %u (1..=%u)",
                    what, rows, cols, batch, q8::F16_GEMM_MAX_BATCH);
    }
    const size_t needs[3] = {(size_t)rows * (size_t)cols * 2u,
                             ((size_t)x_off + (size_t)batch * cols) * 4u,
                             ((size_t)y_off + (size_t)batch * rows) * 4u};
    tm_hip_buffer *bufs[3] = {w, x, y};
    static const char *const suffix[3] = {"weights", "x", "y"};
    for (int i = 0; i < 3; ++i) {
        char name[64];
        snprintf(name, sizeof name, "%s.%s", what, suffix[i]);
        const int rc = check_buffer(ctx, bufs[i], needs[i], err, err_cap, name);
        if (rc != TM_HIP_OK) {
            return rc;
        }
        if (bufs[i]->alloc->packed) {
            return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED, "%s is a sealed Q8_0 weight buffer",
                        name);
        }
    }
    Op op;
    op.kind = OP_F16_GEMM;
    op.a[0] = w->alloc;
    op.a[1] = x->alloc;
    op.a[2] = y->alloc;
    op.n_alloc = 3;
    op.writes_mask = 4;
    op.rows = rows;
    op.cols = cols;
    op.batch = batch;
    op.x_off = x_off;
    op.y_off = y_off;
    op.shape_label = true;
    return submit(ctx, op, what, err, err_cap);
}

int tm_hip_f16_gemv(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *x, tm_hip_buffer *y,
                    uint32_t rows, uint32_t cols, char *err, size_t err_cap) {
    return f16_product(ctx, w, x, y, rows, cols, 1, 0, 0, "f16_gemv", err, err_cap);
}

int tm_hip_f16_gemm(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *x, tm_hip_buffer *y,
                    uint32_t rows, uint32_t cols, uint32_t batch, uint32_t x_off, uint32_t y_off,
                    char *err, size_t err_cap) {
    return f16_product(ctx, w, x, y, rows, cols, batch, x_off, y_off, "f16_gemm", err, err_cap);
}

int tm_hip_f16_row_f32(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *out, uint32_t row,
                       uint32_t cols, uint32_t out_off, char *err, size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, "f16_row") != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (cols == 0) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED, "f16_row: zero cols");
    }
    int rc;
    if ((rc = check_buffer(ctx, w, ((size_t)row + 1u) * (size_t)cols * 2u, err, err_cap,
                           "f16_row.weights")) != TM_HIP_OK ||
        (rc = check_buffer(ctx, out, ((size_t)out_off + cols) * 4u, err, err_cap, "f16_row.out")) !=
            TM_HIP_OK) {
        return rc;
    }
    if (w->alloc->packed || out->alloc->packed) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED, "f16_row: sealed Q8_0 weight buffer");
    }
    Op op;
    op.kind = OP_F16_ROW;
    op.a[0] = w->alloc;
    op.a[1] = out->alloc;
    op.n_alloc = 2;
    op.writes_mask = 2;
    op.cols = cols;
    op.extra = row;
    op.y_off = out_off;
    return submit(ctx, op, "f16_row", err, err_cap);
}

// ---------------------------------------------------------- additions ----

int tm_hip_q8_0_pack(tm_hip_ctx *ctx, tm_hip_buffer *w, uint32_t rows, uint32_t cols, char *err,
                     size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, "q8_0_pack") != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (rows == 0 || cols == 0 || (cols % 32u) != 0u) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "q8_0_pack: rows %u, cols %u (cols must be a positive multiple of 32)", rows,
                    cols);
    }
    const size_t need = (size_t)rows * ((size_t)cols / 32u) * 34u;
    int rc = check_buffer(ctx, w, need, err, err_cap, "q8_0_pack.weights");
    if (rc != TM_HIP_OK) {
        return rc;
    }
    if (w->alloc->packed) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED, "q8_0_pack: buffer is already sealed");
    }
    if (ctx->group_active) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "q8_0_pack: close the open dispatch group first");
    }
    void *ptr = nullptr;
    hipError_t e = hipMalloc(&ptr, w->len);
    if (e != hipSuccess || ptr == nullptr) {
        (void)hipGetLastError();
        return fail(err, err_cap, TM_HIP_ERR_ALLOC,
                    "q8_0_pack: allocation of %zu bytes for the sealed copy failed (%s)", w->len,
                    hipGetErrorString(e));
    }
    Alloc *fresh = new (std::nothrow) Alloc();
    if (fresh == nullptr) {
        (void)hipFree(ptr);
        return fail(err, err_cap, TM_HIP_ERR_ALLOC, "q8_0_pack: handle allocation failed");
    }
    fresh->ptr = ptr;
    fresh->len = w->len;
    fresh->packed = true;
    fresh->prows = rows;
    fresh->pcols = cols;
    if (w->len > need) {
        ctx->loose_work = true;
        e = hipMemcpyAsync((uint8_t *)ptr + need, (const uint8_t *)w->alloc->ptr + need,
                           w->len - need, hipMemcpyDeviceToDevice, ctx->stream);
        if (e != hipSuccess) {
            alloc_release(fresh);
            return hip_fail(err, err_cap, "q8_0_pack: tail copy", e);
        }
    }
    Op op;
    op.kind = OP_PACK;
    op.a[0] = w->alloc;
    op.a[1] = fresh;
    op.n_alloc = 2;
    op.writes_mask = 2;
    op.rows = rows;
    op.cols = cols;
    op.what = "q8_0_pack";
    std::vector<Op> one(1, op);
    rc = commit_ops(ctx, one, "q8_0_pack", "q8_0_pack", err, err_cap);
    // The handle now names the sealed copy; the raw bytes stay leased by the
    // commit above until the pack kernel has read them.
    Alloc *old = w->alloc;
    w->alloc = fresh;
    alloc_release(old);
    return rc;
}

int tm_hip_q8_0_quantize_act(tm_hip_ctx *ctx, tm_hip_buffer *x, tm_hip_buffer *xq, uint32_t cols,
                             uint32_t batch, uint32_t x_off, char *err, size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, "q8_0_quantize_act") != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (cols == 0 || (cols % 32u) != 0u || batch == 0 || batch > TM_HIP_GEMM_I8_MAX_BATCH) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "q8_0_quantize_act: cols %u (a positive multiple of 32), batch %u (1..=%u)", cols,
                    batch, TM_HIP_GEMM_I8_MAX_BATCH);
    }
    const size_t x_need = ((size_t)x_off + (size_t)batch * cols) * 4u;
    const size_t q_need = q8::xq_bytes(cols, batch);
    int rc;
    if ((rc = check_buffer(ctx, x, x_need, err, err_cap, "q8_0_quantize_act.x")) != TM_HIP_OK ||
        (rc = check_buffer(ctx, xq, q_need, err, err_cap, "q8_0_quantize_act.xq")) != TM_HIP_OK) {
        return rc;
    }
    if (x->alloc->packed || xq->alloc->packed) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED, "q8_0_quantize_act: sealed weight buffer");
    }
    Op op;
    op.kind = OP_QUANT;
    op.a[0] = x->alloc;
    op.a[1] = xq->alloc;
    op.n_alloc = 2;
    op.writes_mask = 2;
    op.cols = cols;
    op.batch = batch;
    op.x_off = x_off;
    return submit(ctx, op, "q8_0_quantize_act", err, err_cap);
}

// `fused_tail`: the declared fast variant (tm_hip_q8_0_gemm_i8_fma).
static int gemm_i8_submit(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *xq, tm_hip_buffer *y,
                          tm_hip_buffer *sumi, uint32_t rows, uint32_t cols, uint32_t batch,
                          uint32_t y_off, bool fused_tail, char *err, size_t err_cap) {
    if (check_ctx(ctx, err, err_cap, "q8_0_gemm_i8") != TM_HIP_OK) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    if (rows == 0 || cols == 0 || (cols % 32u) != 0u || batch == 0 ||
        batch > TM_HIP_GEMM_I8_MAX_BATCH) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "q8_0_gemm_i8: rows %u, cols %u (a positive multiple of 32), batch %u (1..=%u)",
                    rows, cols, batch, TM_HIP_GEMM_I8_MAX_BATCH);
    }
    const size_t blocks = cols / 32u;
    const size_t w_need = (size_t)rows * blocks * 34u;
    const size_t q_need = q8::xq_bytes(cols, batch);
    const size_t y_need = ((size_t)y_off + (size_t)batch * rows) * 4u;
    int rc;
    if ((rc = check_buffer(ctx, w, w_need, err, err_cap, "q8_0_gemm_i8.weights")) != TM_HIP_OK ||
        (rc = check_buffer(ctx, xq, q_need, err, err_cap, "q8_0_gemm_i8.xq")) != TM_HIP_OK ||
        (rc = check_buffer(ctx, y, y_need, err, err_cap, "q8_0_gemm_i8.y")) != TM_HIP_OK) {
        return rc;
    }
    if (sumi != nullptr &&
        (rc = check_buffer(ctx, sumi, (size_t)batch * rows * blocks * 4u, err, err_cap,
                           "q8_0_gemm_i8.sumi")) != TM_HIP_OK) {
        return rc;
    }
    if (w->alloc->packed && (w->alloc->prows != rows || w->alloc->pcols != cols)) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED,
                    "q8_0_gemm_i8: weights were sealed as %ux%u but the call names %ux%u",
                    w->alloc->prows, w->alloc->pcols, rows, cols);
    }
    if (xq->alloc->packed || y->alloc->packed || (sumi != nullptr && sumi->alloc->packed)) {
        return fail(err, err_cap, TM_HIP_ERR_UNSUPPORTED, "q8_0_gemm_i8: sealed weight buffer");
    }
    Op op;
    op.kind = OP_I8;
    op.a[0] = w->alloc;
    op.a[1] = xq->alloc;
    op.a[2] = y->alloc;
    op.a[3] = sumi != nullptr ? sumi->alloc : nullptr;
    op.n_alloc = 4;
    op.writes_mask = 4 | 8;
    op.rows = rows;
    op.cols = cols;
    op.batch = batch;
    op.y_off = y_off;
    op.packed = w->alloc->packed;
    op.extra = fused_tail ? 1u : 0u;
    return submit(ctx, op, fused_tail ? "q8_0_gemm_i8_fma" : "q8_0_gemm_i8", err, err_cap);
}

int tm_hip_q8_0_gemm_i8(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *xq, tm_hip_buffer *y,
                        tm_hip_buffer *sumi, uint32_t rows, uint32_t cols, uint32_t batch,
                        uint32_t y_off, char *err, size_t err_cap) {
    return gemm_i8_submit(ctx, w, xq, y, sumi, rows, cols, batch, y_off, false, err, err_cap);
}

int tm_hip_q8_0_gemm_i8_fma(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *xq, tm_hip_buffer *y,
                            uint32_t rows, uint32_t cols, uint32_t batch, uint32_t y_off, char *err,
                            size_t err_cap) {
    return gemm_i8_submit(ctx, w, xq, y, nullptr, rows, cols, batch, y_off, true, err, err_cap);
}

// -------------------------------------------------------- measurement ----

uint64_t tm_hip_committed_dispatches(const tm_hip_ctx *ctx) {
    return ctx == nullptr ? 0 : ctx->committed.load(std::memory_order_relaxed);
}

uint64_t tm_hip_completed_dispatches(const tm_hip_ctx *ctx) {
    if (ctx == nullptr) {
        return 0;
    }
    settle(const_cast<tm_hip_ctx *>(ctx));
    return ctx->completed.load(std::memory_order_acquire);
}

double tm_hip_last_gpu_ms(const tm_hip_ctx *ctx) {
    if (ctx == nullptr) {
        return 0.0;
    }
    settle_and_measure(const_cast<tm_hip_ctx *>(ctx));
    return (double)ctx->last_gpu_nanos.load(std::memory_order_relaxed) / 1e6;
}

uint64_t tm_hip_gpu_nanos_total(const tm_hip_ctx *ctx) {
    if (ctx == nullptr) {
        return 0;
    }
    settle_and_measure(const_cast<tm_hip_ctx *>(ctx));
    return ctx->gpu_nanos_total.load(std::memory_order_relaxed);
}

uint64_t tm_hip_kernel_launches(const tm_hip_ctx *ctx) {
    return ctx == nullptr ? 0 : ctx->launches.load(std::memory_order_relaxed);
}

int tm_hip_profile_set(tm_hip_ctx *ctx, int enabled) {
    if (ctx == nullptr) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    settle(ctx);
    std::lock_guard<std::mutex> g(ctx->q_mu);
    measure_retired(ctx); // commits so far are accounted under the old setting
    ctx->profile_used = 0;
    ctx->profiling.store(enabled ? 1 : 0, std::memory_order_relaxed);
    return TM_HIP_OK;
}

int tm_hip_profile_read(tm_hip_ctx *ctx, uint32_t index, char *name, size_t name_cap,
                        uint64_t *nanos, uint64_t *count) {
    if (ctx == nullptr) {
        return 0;
    }
    settle(ctx);
    std::lock_guard<std::mutex> g(ctx->q_mu);
    measure_retired(ctx);
    if (index >= ctx->profile_used) {
        return 0;
    }
    if (name != nullptr && name_cap > 0) {
        snprintf(name, name_cap, "%s", ctx->profile[index].name);
    }
    if (nanos != nullptr) {
        *nanos = ctx->profile[index].nanos;
    }
    if (count != nullptr) {
        *count = ctx->profile[index].count;
    }
    return 1;
}

int tm_hip_commit_log_set(tm_hip_ctx *ctx, int enabled) {
    if (ctx == nullptr) {
        return TM_HIP_ERR_UNSUPPORTED;
    }
    settle(ctx);
    std::lock_guard<std::mutex> g(ctx->q_mu);
    measure_retired(ctx); // commits so far stay out of (or go into) the log as it was
    ctx->commit_log_on = enabled != 0;
    ctx->commit_log.clear();
    return TM_HIP_OK;
}

size_t tm_hip_commit_log_read(tm_hip_ctx *ctx, uint64_t *nanos, size_t cap) {
    if (ctx == nullptr || nanos == nullptr) {
        return 0;
    }
    settle(ctx);
    std::lock_guard<std::mutex> g(ctx->q_mu);
    measure_retired(ctx);
    size_t n = 0;
    while (n < cap && !ctx->commit_log.empty()) {
        nanos[n++] = ctx->commit_log.front();
        ctx->commit_log.pop_front();
    }
    return n;
}

uint64_t tm_hip_allocated_bytes(const tm_hip_ctx *ctx) {
    return ctx == nullptr ? 0 : ctx->allocated.load(std::memory_order_relaxed);
}

uint64_t tm_hip_in_flight_bytes(const tm_hip_ctx *ctx) {
    if (ctx == nullptr) {
        return 0;
    }
    settle(const_cast<tm_hip_ctx *>(ctx));
    return ctx->leased.load(std::memory_order_relaxed);
}

} // extern "C"

