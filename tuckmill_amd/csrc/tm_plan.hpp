// What the dispatch planner and the kernel launchers of libtm_hip share: device
// allocations, recorded operations, the key that names a kernel instantiation,
// a planned launch and the workspace layout. Plain C++ (no HIP types, no device
// code): tm_hip.cpp (host logic) and tm_launch.cpp (HIP launchers) include it,
// and so does the CPU build of the host logic that the tests run under
// sanitizers against a recording stand-in for the launchers.
#pragma once

#include <atomic>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <type_traits>

#include "q8_plan.hpp"
#include "tm_hip.h"

namespace tmh {

// Workspace of tm_hip_q8_0_gemm_mma_noalloc, the entry point that allocates
// nothing: device memory that exists from the moment the library is loaded, one
// copy per GPU, held until the process ends. Layout (byte offsets):
//   [0, 256)                 the two counters of the work-queue MFMA kernel
//   [256, 256 + 64 KiB)      arrival counters of the bf16 GEMM's K chunks
//   [128 KiB, +20 MiB)       split activations (6 bytes per activation element)
//   [128 KiB + 20 MiB, end)  partial tiles of products whose K is cut into chunks
constexpr size_t kScratchBytes = TM_HIP_NOALLOC_WORKSPACE_BYTES;
constexpr size_t kScratchQueueOff = 0;
constexpr size_t kScratchArrivalsOff = 256;
constexpr size_t kScratchCounterDwords = 64u + q8::BX3_MAX_SPLIT_TILES;
constexpr size_t kScratchXsOff = 128u << 10;
constexpr size_t kScratchXsBytes = TM_HIP_NOALLOC_XS_BYTES;
constexpr size_t kScratchPartialOff = kScratchXsOff + kScratchXsBytes;
constexpr size_t kScratchPartialBytes = kScratchBytes - kScratchPartialOff;
static_assert(kScratchArrivalsOff + q8::BX3_MAX_SPLIT_TILES * 4u <= kScratchXsOff, "counters");
static_assert(q8::MMA_SHARED_PARTIAL_FLOATS * 4u <= kScratchPartialBytes, "f32 partial tiles");
static_assert(q8::MMA_SHARED_MAX_TILES <= q8::BX3_MAX_SPLIT_TILES, "f32 arrival counters");
static_assert(q8::CHECKSUM_GROUPS * 4u == TM_HIP_CHECKSUM_PARTIAL_BYTES, "checksum partial words");

// Device memory the kernels use beyond a product's own buffers.
struct Workspace {
    uint32_t *mma_queue = nullptr; // two counters of the work-queue MFMA kernel, zero between launches
    // An f32 MFMA launch with few output tiles shares each tile between
    // workgroups (q8::mma_shared_parts): room for their partial tiles; the
    // arrival counters are the first of `arrivals` below.
    float *mma_partials = nullptr;
    // The bf16 split-float GEMM: split activations, partial tiles of products
    // whose K is cut into chunks, their arrival counters (zero between launches).
    uint8_t *xs = nullptr;
    size_t xs_bytes = 0;
    float *partials = nullptr;
    size_t partial_bytes = 0;
    uint32_t *arrivals = nullptr;
};

struct Alloc {
    void *ptr = nullptr;
    size_t len = 0;
    std::atomic<int> refs{1};
    bool packed = false;
    uint32_t prows = 0, pcols = 0;
    // Launch planning (under the caller's serialization): the planning epoch
    // in which this allocation was last read / written by a listed product.
    uint64_t read_epoch = 0, write_epoch = 0, keep_epoch = 0;
};

enum OpKind {
    OP_GEMV_LIST, OP_MMA, OP_ROW, OP_ROW_INDIRECT, OP_COPY, OP_PACK, OP_QUANT, OP_I8,
    OP_SCALE, OP_AXPY, OP_SILU_MUL, OP_GELU_MUL, OP_RMSNORM, OP_ARGMAX,
    OP_F16_GEMM, OP_F16_ROW, OP_F16_ROW_INDIRECT, OP_CAST_F16_F32, OP_CAST_F32_F16,
    OP_CHECKSUM
};

struct Op {
    OpKind kind;
    Alloc *a[4] = {nullptr, nullptr, nullptr, nullptr}; // a[0..] buffers touched; see writes_mask
    int n_alloc = 0;
    unsigned writes_mask = 0; // bit i: a[i] is written
    uint32_t rows = 0, cols = 0, batch = 0, x_off = 0, y_off = 0, extra = 0;
    float scalar = 0.0f;       // factor / alpha / eps of the small f32 operators
    bool packed = false;
    bool shape_label = false;  // profile label carries "<rows>x<cols>"
    const char *what = "";     // static operator name
};

// Which kernel family and instantiation a recorded product launches with.
// Products that may share a launch agree on the whole key.
enum Variant : uint8_t {
    V_DECODE,     // gemv_list_kernel, one token per pass (the streaming decode kernel)
    V_GENERAL,    // gemv_list_kernel, four tokens per pass (raw layout / narrow small batches)
    V_SPLIT,      // gemm_split_list_kernel: p0 = waves, p1 = tokens per wave, p2 = column tail
    V_MMA,        // f32 MFMA GEMM: p0 = tmw, p1 = tnw, p2 = K split
    V_BF16X3,     // prefill GEMM on the bf16 matrix cores, activations split in three:
                  // p0 = tokens per tile / 64
    V_MMA_SPLIT,  // the f32 kernel's tiles on the bf16 matrix cores, fed with the split form that
                  // the operator right before the launch has written (fuse_split_passes)
    V_I8_TILE,    // register-fed int8 MFMA GEMM: p0 = tile configuration
    V_I8_STREAM,  // int8 streaming kernel: p0 = tokens per pass
    V_I8_LDS,     // LDS-staged int8 MFMA GEMM: p0 = workgroup shape (q8::i8_lds_shape),
                  // p1 = 1: the term goes into the sum fused (tm_hip_q8_0_gemm_i8_fma)
    V_F16         // F16-weight list kernel: p0 = tokens per sweep, flag = every row 16-byte aligned
};

struct GemvKey {
    OpKind kind = OP_GEMV_LIST; // OP_GEMV_LIST, OP_MMA, OP_I8 or OP_F16_GEMM
    Variant variant = V_DECODE;
    uint8_t p0 = 0, p1 = 0, p2 = 0;
    bool packed = false;
    bool flag = false; // GEMV / MFMA f32: activations 16-byte aligned; int8: block dots are written out
    bool operator==(const GemvKey &o) const {
        return kind == o.kind && variant == o.variant && p0 == o.p0 && p1 == o.p1 && p2 == o.p2 &&
               packed == o.packed && flag == o.flag;
    }
    // one token, sealed weights, aligned activations: the kernel the planner's fusions target
    bool decode() const { return kind == OP_GEMV_LIST && variant == V_DECODE && packed && flag; }
    // up to four tokens through the exact small-batch product, sealed weights,
    // aligned activations: with a fusion such a launch goes to the one-token
    // kernel, a descriptor per product and token
    bool few_tokens() const {
        return kind == OP_GEMV_LIST && variant == V_SPLIT && packed && flag && p0 == 1;
    }
    bool fusable() const { return decode() || few_tokens(); }
};

// A vector of trivially copyable elements whose first N live inside the object:
// a launch of a few products (every launch of the entry point that allocates
// nothing has one) never touches the heap; longer lists spill to it.
template <typename T, size_t N> class InlineVec {
    static_assert(std::is_trivially_copyable<T>::value, "elements are copied with memcpy");

  public:
    InlineVec() = default;
    InlineVec(const InlineVec &o) { assign(o); }
    InlineVec(InlineVec &&o) noexcept { steal(o); }
    InlineVec &operator=(const InlineVec &o) {
        if (this != &o) {
            clear();
            assign(o);
        }
        return *this;
    }
    InlineVec &operator=(InlineVec &&o) noexcept {
        if (this != &o) {
            release();
            steal(o);
        }
        return *this;
    }
    ~InlineVec() { release(); }
    size_t size() const { return n_; }
    bool empty() const { return n_ == 0; }
    void clear() { n_ = 0; }
    T &operator[](size_t i) { return data()[i]; }
    const T &operator[](size_t i) const { return data()[i]; }
    T &back() { return data()[n_ - 1]; }
    const T &back() const { return data()[n_ - 1]; }
    T *begin() { return data(); }
    T *end() { return data() + n_; }
    const T *begin() const { return data(); }
    const T *end() const { return data() + n_; }
    void push_back(const T &v) {
        if (n_ == cap_) {
            grow();
        }
        data()[n_++] = v;
    }

  private:
    T *data() { return heap_ != nullptr ? heap_ : inline_; }
    const T *data() const { return heap_ != nullptr ? heap_ : inline_; }
    void grow() {
        const size_t cap = cap_ * 2;
        T *fresh = new T[cap];
        memcpy(fresh, data(), n_ * sizeof(T));
        delete[] heap_;
        heap_ = fresh;
        cap_ = cap;
    }
    void assign(const InlineVec &o) {
        for (const T &v : o) {
            push_back(v);
        }
    }
    void steal(InlineVec &o) {
        n_ = o.n_;
        if (o.heap_ != nullptr) {
            heap_ = o.heap_;
            cap_ = o.cap_;
            o.heap_ = nullptr;
            o.cap_ = N;
        } else {
            heap_ = nullptr;
            cap_ = N;
            memcpy(inline_, o.inline_, o.n_ * sizeof(T));
        }
        o.n_ = 0;
    }
    void release() {
        delete[] heap_;
        heap_ = nullptr;
        cap_ = N;
        n_ = 0;
    }
    T inline_[N];
    T *heap_ = nullptr;
    size_t n_ = 0, cap_ = N;
};

using OpList = InlineVec<const Op *, 4>;

// One kernel launch of a commit: a list of products, or a single operation.
struct Launch {
    OpList list;     // empty: `single`
    OpList residual; // per list entry: an axpy fused into it, or null
    OpList glu;      // per list entry: this product and the next are the gate
                     // and up projections of this fused gated activation
    InlineVec<uint8_t, 4> normed; // per list entry: reads the fused RMSNorm's output
    const Op *norm = nullptr;         // an RMSNorm fused in front of the flagged entries
    GemvKey key{};
    const Op *single = nullptr;
    // V_BF16X3: what the listed products need of the context's workspace (while
    // the launch is open, the most they can need; exact once cut_bx3_launch has
    // decided the K chunks of every product, `bx3_chunks`, per list entry)
    uint64_t bx3_split_tiles = 0, bx3_partial_floats = 0, bx3_xs_bytes = 0;
    InlineVec<uint8_t, 4> bx3_chunks;
    // the rows that one of the products gives up to a tail segment with chunks of
    // its own (q8::bx3_plan_launch); row_tiles == 0: none
    q8::Bx3Tail bx3_tail{};
    int bx3_inputs = 0;
    uint32_t descs = 0; // descriptors the listed products take (token groups count one each)
    uint32_t token_descs = 0; // the same at one descriptor per product and token
    // A launch of GemvKey::few_tokens products with a fused norm or gated
    // activation in it: it runs on the one-token kernel (which has those forms),
    // one descriptor per product and token.
    bool per_token = false;
    // V_BF16X3: bit i set = the launch's i-th distinct input (in list order)
    // arrives split already, written by the launch just before this one
    // (V_MMA_SPLIT: its one input always does).
    uint32_t bx3_presplit = 0;
    // V_MMA_SPLIT: byte offset in the split workspace of the launch's input.
    uint64_t xs_in_off = 0;
    // An RMSNorm or gated activation on its own (or a V_MMA_SPLIT launch with the
    // gated activation fused in, glu[0]) whose result is the next launch's input:
    // byte offset in the split workspace where it writes the split form as well,
    // or -1.
    int64_t split_xs_off = -1;
    uint32_t split_cols = 0; // the row length that result is cut by
    // An RMSNorm on its own: the residual update of its input that it does first.
    const Op *update = nullptr;
};

// Two products read the same activations (and can share their split form).
inline bool same_input(const Op &a, const Op &b) {
    return a.a[1] == b.a[1] && a.x_off == b.x_off && a.batch == b.batch && a.cols == b.cols;
}
inline size_t bx3_xs_bytes_of(const Op &op) { return ((size_t)op.batch * op.cols * 6u + 255u) & ~(size_t)255u; }

// Descriptors a product takes in a list launch: one, or for the token-split
// kernel as many groups of waves x tokens-per-wave tokens as its batch needs.
inline uint32_t split_token_groups(const GemvKey &key, uint32_t batch) {
    if (key.variant != V_SPLIT) {
        return 1u;
    }
    const uint32_t group_tokens = (uint32_t)key.p0 * key.p1;
    return (batch + group_tokens - 1u) / group_tokens;
}

} // namespace tmh
