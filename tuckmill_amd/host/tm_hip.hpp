// tm_hip.hpp — typed C++ handles over the tm_hip_* C ABI.
//
// The reference wraps its Metal ABI in Rust RAII types
// (crates/metal/src/lib.rs: MetalContext :755-, MetalBuffer :2480-2650) and
// builds the projection abstraction `Matrix` on them
// (crates/tuckcore/src/engine/metal.rs:106-226). This header is the same
// surface for the HIP ABI, for hosts written in C++: same method names,
// argument meaning and error mapping. Header-only; link against libtm_hip.so.
#pragma once

#include <algorithm>
#include <cstdint>
#include <cstring>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "tm_hip.h"

namespace tuckmill_hip {

constexpr size_t ERR_CAP = 512;               // crates/metal/src/lib.rs:32
constexpr uint32_t GEMM_MAX_BATCH = TM_HIP_GEMM_MAX_BATCH;
constexpr uint32_t GEMM_MMA_MAX_BATCH = TM_HIP_GEMM_MMA_MAX_BATCH;
constexpr uint32_t GEMM_I8_MAX_BATCH = TM_HIP_GEMM_I8_MAX_BATCH;
constexpr uint32_t PREFILL_BATCH = 128;        // crates/tuckcore/src/engine/metal.rs:25
constexpr size_t STAGING_CHUNK_BYTES = 4u << 20; // crates/tuckcore/src/qwen35_gpu.rs:1176

enum class ErrorCode {
    InvalidRequest, Unavailable, Internal, UnsupportedQuantization, InvalidArtifact,
    UnsupportedArchitecture
};

class TuckmillError : public std::runtime_error {
  public:
    TuckmillError(ErrorCode code, const std::string &message, int abi_code = 0)
        : std::runtime_error(message), code_(code), abi_code_(abi_code) {}
    ErrorCode code() const { return code_; }
    int abi_code() const { return abi_code_; }

  private:
    ErrorCode code_;
    int abi_code_;
};

// crates/metal/src/lib.rs:732-745
inline TuckmillError hip_error(int code, const char *text, const char *what) {
    ErrorCode c = ErrorCode::Internal;
    if (code == TM_HIP_ERR_BOUNDS || code == TM_HIP_ERR_UNSUPPORTED) {
        c = ErrorCode::InvalidRequest;
    } else if (code == TM_HIP_ERR_NO_DEVICE || code == TM_HIP_ERR_ALLOC) {
        c = ErrorCode::Unavailable;
    }
    return TuckmillError(c, std::string("hip ") + what + ": " + text, code);
}

struct Probe {
    bool available;
    std::string info;
};

inline Probe probe() { return Probe{tm_hip_available() != 0, tm_hip_runtime_info()}; }

// ---- kernel selection (crates/tuckcore/src/kernels.rs:36-113) ---------------
//
// `--kernels hip` next to auto / scalar / neon / metal. A forced selection never
// falls back silently: `hip` on a machine without a usable gfx950 device is a
// typed refusal at load, like `metal` off macOS and `neon` off aarch64.
enum class ResolvedKernels { Scalar, Neon, Metal, Hip };

inline const char *as_str(ResolvedKernels k) {
    switch (k) {
    case ResolvedKernels::Scalar: return "scalar";
    case ResolvedKernels::Neon: return "neon";
    case ResolvedKernels::Metal: return "metal";
    case ResolvedKernels::Hip: return "hip";
    }
    return "scalar";
}

inline ResolvedKernels default_kernels_for_target() {
#if defined(__aarch64__)
    return ResolvedKernels::Neon;
#else
    return ResolvedKernels::Scalar;
#endif
}

class KernelSelection {
  public:
    enum Kind { Auto, Scalar, Neon, Metal, Hip };
    KernelSelection(Kind kind = Auto) : kind_(kind) {}
    Kind kind() const { return kind_; }
    bool operator==(const KernelSelection &o) const { return kind_ == o.kind_; }

    // kernels.rs:46-54, with the new arm. `ok` is false for an unknown name.
    static KernelSelection parse(const std::string &s, bool *ok) {
        *ok = true;
        if (s == "auto") return Auto;
        if (s == "scalar") return Scalar;
        if (s == "neon") return Neon;
        if (s == "metal") return Metal;
        if (s == "hip") return Hip;
        *ok = false;
        return Auto;
    }

    // kernels.rs:58-86. `device` answers whether a HIP device is usable (the
    // library's probe by default; tests pass their own).
    ResolvedKernels resolve(Probe device = probe()) const {
        switch (kind_) {
        case Scalar: return ResolvedKernels::Scalar;
        case Auto: return default_kernels_for_target(); // never a GPU path unasked
        case Metal:
#if defined(__APPLE__)
            return ResolvedKernels::Metal;
#else
            throw TuckmillError(ErrorCode::Unavailable,
                                "the Metal kernel implementation requires macOS; select --kernels "
                                "auto, hip, neon, or scalar on this machine");
#endif
        case Neon:
#if defined(__aarch64__)
            return ResolvedKernels::Neon;
#else
            throw TuckmillError(ErrorCode::InvalidRequest,
                                "the NEON kernel implementation requires an aarch64 target; select "
                                "--kernels auto or --kernels scalar on this machine");
#endif
        case Hip:
            if (!device.available) {
                throw TuckmillError(ErrorCode::Unavailable,
                                    "the HIP kernel implementation requires a gfx950 device (" +
                                        device.info + "); select --kernels auto or scalar on this machine",
                                    TM_HIP_ERR_NO_DEVICE);
            }
            return ResolvedKernels::Hip;
        }
        return ResolvedKernels::Scalar;
    }

  private:
    Kind kind_;
};

// ---- numerical profile (crates/tuckcore/src/forward.rs:284-311) -------------
enum class NumericalProfile { OracleF32, LlamaCpu };

inline bool parse_numerical_profile(const std::string &s, NumericalProfile *out) {
    if (s == "oracle-f32") {
        *out = NumericalProfile::OracleF32;
        return true;
    }
    if (s == "llama-cpu") {
        *out = NumericalProfile::LlamaCpu;
        return true;
    }
    return false;
}

inline const char *as_str(NumericalProfile p) {
    return p == NumericalProfile::OracleF32 ? "oracle-f32" : "llama-cpu";
}

// The load-time checks of crates/tuckcore/src/executor.rs:294-314 with a device
// mode that covers Metal and HIP: a prefill batch only means something on a
// device path; the Metal path implements oracle-f32 only (typed refusal, never
// a silent substitution), the HIP path also implements llama-cpu for Q8_0
// weights (activations quantized per 32, int8 block dots).
inline void check_engine_options(ResolvedKernels kernels, NumericalProfile profile,
                                 bool prefill_batch_given) {
    const bool device_mode = kernels == ResolvedKernels::Metal || kernels == ResolvedKernels::Hip;
    if (!device_mode && prefill_batch_given) {
        throw TuckmillError(ErrorCode::InvalidRequest,
                            "prefill_batch applies only to the device kernel paths (metal, hip); the "
                            "resolved CPU kernels execute single-token steps and must not silently "
                            "ignore it");
    }
    if (kernels == ResolvedKernels::Metal && profile != NumericalProfile::OracleF32) {
        throw TuckmillError(ErrorCode::UnsupportedArchitecture,
                            "the Metal path implements the oracle-f32 numerical profile only; select "
                            "--numerical-profile oracle-f32, or --kernels hip for llama-cpu on a GPU");
    }
}

struct ContextInner {
    tm_hip_ctx *raw = nullptr;
    std::mutex lock; // one ABI call at a time, crates/metal/src/lib.rs:695-708
    bool owned = true;
    ~ContextInner() {
        if (raw != nullptr && owned) {
            tm_hip_destroy(raw);
        }
    }
};

class HipContext;

class HipBuffer {
  public:
    HipBuffer() = default;
    HipBuffer(std::shared_ptr<ContextInner> ctx, tm_hip_buffer *raw, bool owned = true)
        : ctx_(std::move(ctx)), raw_(raw), owned_(owned) {}
    HipBuffer(const HipBuffer &) = delete;
    HipBuffer &operator=(const HipBuffer &) = delete;
    HipBuffer(HipBuffer &&o) noexcept : ctx_(std::move(o.ctx_)), raw_(o.raw_), owned_(o.owned_) {
        o.raw_ = nullptr;
    }
    HipBuffer &operator=(HipBuffer &&o) noexcept {
        if (this != &o) {
            release();
            ctx_ = std::move(o.ctx_);
            raw_ = o.raw_;
            owned_ = o.owned_;
            o.raw_ = nullptr;
        }
        return *this;
    }
    ~HipBuffer() { release(); }

    tm_hip_buffer *raw() const { return raw_; }
    size_t len() const { return raw_ ? tm_hip_buffer_len(ctx_->raw, raw_) : 0; }
    bool is_empty() const { return len() == 0; }

    void zero(size_t offset, size_t length) const {
        call("buffer_zero", [&](char *e) {
            return tm_hip_buffer_zero(ctx_->raw, raw_, offset, length, e, ERR_CAP);
        });
    }
    void upload(size_t offset, const void *data, size_t length) const {
        call("upload", [&](char *e) {
            return tm_hip_upload(ctx_->raw, raw_, offset, data, length, e, ERR_CAP);
        });
    }
    void download(size_t offset, void *dst, size_t length) const {
        call("download", [&](char *e) {
            return tm_hip_download(ctx_->raw, raw_, offset, dst, length, e, ERR_CAP);
        });
    }
    // No lock: the wait must not block encoding of later work
    // (crates/metal/src/lib.rs:2618-2633).
    void download_after(size_t offset, void *dst, size_t length, uint64_t completed_target) const {
        char err[ERR_CAP] = {0};
        int code = tm_hip_download_after(ctx_->raw, raw_, offset, dst, length, completed_target, err,
                                         ERR_CAP);
        if (code != 0) {
            throw hip_error(code, err, "download_after");
        }
    }

  private:
    friend class HipContext;
    template <class F> void call(const char *what, F f) const {
        std::lock_guard<std::mutex> g(ctx_->lock);
        char err[ERR_CAP] = {0};
        int code = f(err);
        if (code != 0) {
            throw hip_error(code, err, what);
        }
    }
    void release() {
        if (raw_ != nullptr && owned_ && ctx_ && ctx_->raw != nullptr) {
            std::lock_guard<std::mutex> g(ctx_->lock);
            tm_hip_buffer_free(ctx_->raw, raw_);
        }
        raw_ = nullptr;
    }
    std::shared_ptr<ContextInner> ctx_;
    tm_hip_buffer *raw_ = nullptr;
    bool owned_ = true;
};

// A recorded dispatch group (tm_hip_end_group_recorded): replayed with run(),
// released with the last copy of the handle.
class RecordedStep {
  public:
    RecordedStep() = default;
    void run() const {
        std::lock_guard<std::mutex> g(state_->ctx->lock);
        char err[ERR_CAP] = {0};
        int code = tm_hip_step_run(state_->ctx->raw, state_->raw, err, ERR_CAP);
        if (code != 0) {
            throw hip_error(code, err, "step_run");
        }
    }
    uint32_t launches() const { return tm_hip_step_launches(state_->ctx->raw, state_->raw); }

  private:
    friend class HipContext;
    struct State {
        std::shared_ptr<ContextInner> ctx;
        tm_hip_step *raw = nullptr;
        ~State() {
            if (raw != nullptr && ctx && ctx->raw != nullptr) {
                std::lock_guard<std::mutex> g(ctx->lock);
                tm_hip_step_free(ctx->raw, raw);
            }
        }
    };
    std::shared_ptr<State> state_;
};

class HipContext {
  public:
    static HipContext open() {
        char err[ERR_CAP] = {0};
        tm_hip_ctx *raw = tm_hip_create(err, ERR_CAP);
        if (raw == nullptr) {
            throw hip_error(TM_HIP_ERR_NO_DEVICE, err, "create");
        }
        auto inner = std::make_shared<ContextInner>();
        inner->raw = raw;
        return HipContext(std::move(inner));
    }
    // Borrow a context created elsewhere (it is not destroyed here).
    static HipContext borrow(tm_hip_ctx *raw) {
        auto inner = std::make_shared<ContextInner>();
        inner->raw = raw;
        inner->owned = false;
        return HipContext(std::move(inner));
    }
    HipBuffer borrow_buffer(tm_hip_buffer *raw) const { return HipBuffer(inner_, raw, false); }

    HipBuffer buffer(size_t bytes, bool shared = true) const {
        if (bytes == 0) {
            throw TuckmillError(ErrorCode::InvalidRequest,
                                "zero-length HIP buffers are refused (allocation must be explicit)",
                                TM_HIP_ERR_BOUNDS);
        }
        std::lock_guard<std::mutex> g(inner_->lock);
        char err[ERR_CAP] = {0};
        tm_hip_buffer *raw = tm_hip_buffer_new(inner_->raw, bytes, shared ? 1 : 0, err, ERR_CAP);
        if (raw == nullptr) {
            throw hip_error(TM_HIP_ERR_ALLOC, err, "buffer");
        }
        return HipBuffer(inner_, raw);
    }

    void begin_group() const { operate("begin_group", [&](char *e) { return tm_hip_begin_group(raw(), e, ERR_CAP); }); }
    void end_group() const { operate("end_group", [&](char *e) { return tm_hip_end_group(raw(), e, ERR_CAP); }); }
    void abort_group() const { operate("abort_group", [&](char *e) { return tm_hip_abort_group(raw(), e, ERR_CAP); }); }
    void fence() const { operate("fence", [&](char *e) { return tm_hip_fence(raw(), e, ERR_CAP); }); }

    // Run `encode` inside one dispatch group; on any error the group is
    // discarded without committing (crates/tuckcore/src/qwen35_gpu.rs:66-85).
    template <class F> void grouped(F encode) const {
        begin_group();
        try {
            encode();
        } catch (...) {
            try {
                abort_group();
            } catch (...) {
            }
            throw;
        }
        end_group();
    }

    // Record `encode` as a replayable step instead of committing it.
    template <class F> RecordedStep recorded(F encode) const {
        begin_group();
        try {
            encode();
        } catch (...) {
            try {
                abort_group();
            } catch (...) {
            }
            throw;
        }
        tm_hip_step *raw_step = nullptr;
        operate("end_group_recorded",
                [&](char *e) { return tm_hip_end_group_recorded(raw(), &raw_step, e, ERR_CAP); });
        RecordedStep step;
        step.state_ = std::make_shared<RecordedStep::State>();
        step.state_->ctx = inner_;
        step.state_->raw = raw_step;
        return step;
    }

    void q8_0_gemv(const HipBuffer &w, const HipBuffer &x, const HipBuffer &y, uint32_t rows,
                   uint32_t cols) const {
        operate("q8_0_gemv", [&](char *e) {
            return tm_hip_q8_0_gemv(raw(), w.raw(), x.raw(), y.raw(), rows, cols, e, ERR_CAP);
        });
    }
    void q8_0_gemm(const HipBuffer &w, const HipBuffer &x, const HipBuffer &y, uint32_t rows,
                   uint32_t cols, uint32_t batch, uint32_t x_off, uint32_t y_off) const {
        operate("q8_0_gemm", [&](char *e) {
            return tm_hip_q8_0_gemm(raw(), w.raw(), x.raw(), y.raw(), rows, cols, batch, x_off, y_off,
                                    e, ERR_CAP);
        });
    }
    void q8_0_gemm_mma(const HipBuffer &w, const HipBuffer &x, const HipBuffer &y, uint32_t rows,
                       uint32_t cols, uint32_t batch, uint32_t x_off, uint32_t y_off) const {
        operate("q8_0_gemm_mma", [&](char *e) {
            return tm_hip_q8_0_gemm_mma(raw(), w.raw(), x.raw(), y.raw(), rows, cols, batch, x_off,
                                        y_off, e, ERR_CAP);
        });
    }
    // q8_0_gemm_mma out of the library's static device workspace: allocates
    // nothing on the device, launches at once, is not a commit.
    void q8_0_gemm_mma_noalloc(const HipBuffer &w, const HipBuffer &x, const HipBuffer &y,
                               uint32_t rows, uint32_t cols, uint32_t batch, uint32_t x_off,
                               uint32_t y_off) const {
        operate("q8_0_gemm_mma_noalloc", [&](char *e) {
            return tm_hip_q8_0_gemm_mma_noalloc(raw(), w.raw(), x.raw(), y.raw(), rows, cols, batch,
                                                x_off, y_off, e, ERR_CAP);
        });
    }
    void q8_0_row(const HipBuffer &w, const HipBuffer &out, uint32_t row, uint32_t cols,
                  uint32_t out_off) const {
        operate("q8_0_row", [&](char *e) {
            return tm_hip_q8_0_row_f32(raw(), w.raw(), out.raw(), row, cols, out_off, e, ERR_CAP);
        });
    }
    void f16_gemv(const HipBuffer &w, const HipBuffer &x, const HipBuffer &y, uint32_t rows,
                  uint32_t cols) const {
        operate("f16_gemv", [&](char *e) {
            return tm_hip_f16_gemv(raw(), w.raw(), x.raw(), y.raw(), rows, cols, e, ERR_CAP);
        });
    }
    void f16_gemm(const HipBuffer &w, const HipBuffer &x, const HipBuffer &y, uint32_t rows,
                  uint32_t cols, uint32_t batch, uint32_t x_off, uint32_t y_off) const {
        operate("f16_gemm", [&](char *e) {
            return tm_hip_f16_gemm(raw(), w.raw(), x.raw(), y.raw(), rows, cols, batch, x_off, y_off,
                                   e, ERR_CAP);
        });
    }
    void f16_row(const HipBuffer &w, const HipBuffer &out, uint32_t row, uint32_t cols,
                 uint32_t out_off) const {
        operate("f16_row", [&](char *e) {
            return tm_hip_f16_row_f32(raw(), w.raw(), out.raw(), row, cols, out_off, e, ERR_CAP);
        });
    }
    void row_indirect_f32(const HipBuffer &w, uint32_t type_id, uint32_t rows, uint32_t cols,
                          const HipBuffer &ids, uint32_t slot, const HipBuffer &out) const {
        operate("row_indirect", [&](char *e) {
            return tm_hip_row_indirect_f32(raw(), w.raw(), type_id, rows, cols, ids.raw(), slot,
                                           out.raw(), e, ERR_CAP);
        });
    }
    // The small f32 operators either side of a product
    // (crates/metal/src/lib.rs:1027-1060, :2244-2319).
    void f32_scale(const HipBuffer &x, const HipBuffer &y, float factor, uint32_t n) const {
        operate("f32_scale", [&](char *e) {
            return tm_hip_f32_scale(raw(), x.raw(), y.raw(), factor, n, e, ERR_CAP);
        });
    }
    // y = (f32) x over n binary16 elements / y = (half) x over n f32 elements
    // (crates/metal/src/lib.rs:1636-1662).
    void cast_f16_to_f32(const HipBuffer &x, const HipBuffer &y, uint32_t n) const {
        operate("cast_f16_f32", [&](char *e) {
            return tm_hip_cast_f16_f32(raw(), x.raw(), y.raw(), n, e, ERR_CAP);
        });
    }
    void cast_f32_to_f16(const HipBuffer &x, const HipBuffer &y, uint32_t n) const {
        operate("cast_f32_f16", [&](char *e) {
            return tm_hip_cast_f32_f16(raw(), x.raw(), y.raw(), n, e, ERR_CAP);
        });
    }
    void f32_axpy(const HipBuffer &a, const HipBuffer &y, float alpha, uint32_t n) const {
        operate("f32_axpy", [&](char *e) {
            return tm_hip_f32_axpy(raw(), a.raw(), y.raw(), alpha, n, e, ERR_CAP);
        });
    }
    void rmsnorm(const HipBuffer &x, const HipBuffer &weight, const HipBuffer &y, uint32_t rows,
                 uint32_t cols, float eps) const {
        operate("rmsnorm", [&](char *e) {
            return tm_hip_rmsnorm_f32(raw(), x.raw(), weight.raw(), y.raw(), rows, cols, eps, e,
                                      ERR_CAP);
        });
    }
    void silu_mul(const HipBuffer &gate, const HipBuffer &up, const HipBuffer &out,
                  uint32_t n) const {
        operate("silu_mul", [&](char *e) {
            return tm_hip_silu_mul_f32(raw(), gate.raw(), up.raw(), out.raw(), n, e, ERR_CAP);
        });
    }
    void gelu_tanh_mul(const HipBuffer &gate, const HipBuffer &up, const HipBuffer &out,
                       uint32_t n) const {
        operate("gelu_tanh_mul", [&](char *e) {
            return tm_hip_gelu_tanh_mul_f32(raw(), gate.raw(), up.raw(), out.raw(), n, e, ERR_CAP);
        });
    }
    void argmax_f32(const HipBuffer &x, uint32_t n, const HipBuffer &partial, const HipBuffer &out,
                    uint32_t out_index) const {
        operate("argmax_f32", [&](char *e) {
            return tm_hip_argmax_f32(raw(), x.raw(), n, partial.raw(), out.raw(), out_index, e,
                                     ERR_CAP);
        });
    }
    void q8_0_pack(const HipBuffer &w, uint32_t rows, uint32_t cols) const {
        operate("q8_0_pack",
                [&](char *e) { return tm_hip_q8_0_pack(raw(), w.raw(), rows, cols, e, ERR_CAP); });
    }
    void q8_0_quantize_act(const HipBuffer &x, const HipBuffer &xq, uint32_t cols, uint32_t batch,
                           uint32_t x_off) const {
        operate("q8_0_quantize_act", [&](char *e) {
            return tm_hip_q8_0_quantize_act(raw(), x.raw(), xq.raw(), cols, batch, x_off, e, ERR_CAP);
        });
    }
    void q8_0_gemm_i8(const HipBuffer &w, const HipBuffer &xq, const HipBuffer &y, uint32_t rows,
                      uint32_t cols, uint32_t batch, uint32_t y_off) const {
        operate("q8_0_gemm_i8", [&](char *e) {
            return tm_hip_q8_0_gemm_i8(raw(), w.raw(), xq.raw(), y.raw(), nullptr, rows, cols, batch,
                                       y_off, e, ERR_CAP);
        });
    }

    // The declared fast variant: exact block dots, each term fused into the sum.
    void q8_0_gemm_i8_fma(const HipBuffer &w, const HipBuffer &xq, const HipBuffer &y, uint32_t rows,
                          uint32_t cols, uint32_t batch, uint32_t y_off) const {
        operate("q8_0_gemm_i8_fma", [&](char *e) {
            return tm_hip_q8_0_gemm_i8_fma(raw(), w.raw(), xq.raw(), y.raw(), rows, cols, batch, y_off,
                                           e, ERR_CAP);
        });
    }

    uint64_t committed_dispatches() const { return tm_hip_committed_dispatches(raw()); }
    uint64_t completed_dispatches() const { return tm_hip_completed_dispatches(raw()); }
    double last_gpu_ms() const { return tm_hip_last_gpu_ms(raw()); }
    uint64_t gpu_nanos_total() const { return tm_hip_gpu_nanos_total(raw()); }
    uint64_t kernel_launches() const { return tm_hip_kernel_launches(raw()); }
    uint64_t allocated_bytes() const { return tm_hip_allocated_bytes(raw()); }
    uint64_t in_flight_bytes() const { return tm_hip_in_flight_bytes(raw()); }
    uint64_t live_gpu_bytes() const { return allocated_bytes() + in_flight_bytes(); }

    tm_hip_ctx *raw() const { return inner_->raw; }

  private:
    explicit HipContext(std::shared_ptr<ContextInner> inner) : inner_(std::move(inner)) {}
    template <class F> void operate(const char *what, F f) const {
        std::lock_guard<std::mutex> g(inner_->lock);
        char err[ERR_CAP];
        err[0] = '\0';
        int code = f(err);
        if (code != 0) {
            throw hip_error(code, err, what);
        }
    }
    std::shared_ptr<ContextInner> inner_;
};

// Bytes of a quantized-activation buffer (tm_hip_q8_0_quantize_act): batch * cols
// int8 quants, then (cols / 32) x (batch rounded up to 4) f32 scales.
inline size_t xq_bytes(uint32_t cols, uint32_t batch) {
    const size_t bpad = ((size_t)batch + 3u) & ~(size_t)3u;
    return (size_t)batch * cols + (size_t)(cols / 32u) * bpad * 4u;
}

// A device projection matrix (crates/tuckcore/src/engine/metal.rs:106-226) with
// the numerical profile its products run under
// (crates/tuckcore/src/forward.rs:606-645 switches per matvec):
//   oracle-f32  f32 activations, weights dequantized exactly (the default);
//   llama-cpu   Q8_0 weights: activations quantized per 32 on the device
//               (tensor.rs:184-206), int8 block dots, the f32 sum of
//               kernels.rs:206-221, bit for bit; the matrix owns the quantized
//               activation buffer and sizes it. F16 weights under llama-cpu
//               (activations rounded to f16, forward.rs:823-870) have no device
//               kernel here: a typed refusal at load, never a substitution.
class Matrix {
  public:
    static uint64_t plan(uint64_t in_dim, uint64_t out_dim, uint32_t type_id = 8) {
        return type_id == 1 ? out_dim * in_dim * 2u : out_dim * (in_dim / 32u) * 34u;
    }

    // Staged raw upload in 4 MiB slices (engine/metal.rs:138-147), then the
    // seal step that re-lays the weights out for coalesced device loads.
    static Matrix load(const HipContext &gpu, const uint8_t *raw, uint64_t in_dim, uint64_t out_dim,
                       uint32_t type_id = 8, bool seal = true,
                       NumericalProfile profile = NumericalProfile::OracleF32) {
        if (out_dim <= 1) {
            throw TuckmillError(ErrorCode::Internal, "1-D tensors use the f32 path");
        }
        if (type_id != 1 && type_id != 8) {
            throw TuckmillError(ErrorCode::UnsupportedQuantization,
                                "engine matrices must be F16 or Q8_0");
        }
        if (profile == NumericalProfile::LlamaCpu && type_id != 8) {
            throw TuckmillError(ErrorCode::UnsupportedArchitecture,
                                "the HIP path implements the llama-cpu numerical profile for Q8_0 "
                                "weights only; F16 weights run under oracle-f32",
                                TM_HIP_ERR_UNSUPPORTED);
        }
        const size_t total = (size_t)plan(in_dim, out_dim, type_id);
        Matrix m;
        m.buf = gpu.buffer(total, true);
        for (size_t off = 0; off < total;) {
            const size_t n = std::min(STAGING_CHUNK_BYTES, total - off);
            m.buf.upload(off, raw + off, n);
            off += n;
        }
        if (seal && type_id == 8) {
            gpu.q8_0_pack(m.buf, (uint32_t)out_dim, (uint32_t)in_dim);
        }
        m.type_id = type_id;
        m.in_dim = in_dim;
        m.out_dim = out_dim;
        m.profile = profile;
        return m;
    }

    void gemv(const HipContext &gpu, const HipBuffer &x, const HipBuffer &y) {
        if (profile == NumericalProfile::LlamaCpu) {
            gemm_llama_cpu(gpu, x, y, 1);
        } else if (type_id == 1) {
            gpu.f16_gemv(buf, x, y, (uint32_t)out_dim, (uint32_t)in_dim);
        } else {
            gpu.q8_0_gemv(buf, x, y, (uint32_t)out_dim, (uint32_t)in_dim);
        }
    }

    // engine/metal.rs:171-196: batch 1 and `exact` keep the GEMV's per-row
    // arithmetic in slices of GEMM_MAX_BATCH; other batches use the matrix cores.
    // Under llama-cpu every batch is exact already (the int8 products are
    // bit-identical to the CPU's whatever the batch).
    void gemm(const HipContext &gpu, const HipBuffer &x, const HipBuffer &y, uint32_t batch,
              bool exact) {
        const uint32_t rows = (uint32_t)out_dim, cols = (uint32_t)in_dim;
        if (profile == NumericalProfile::LlamaCpu) {
            gemm_llama_cpu(gpu, x, y, batch);
            return;
        }
        if (!exact && type_id == 8 && batch >= 2 && batch <= GEMM_MMA_MAX_BATCH) {
            gpu.q8_0_gemm_mma(buf, x, y, rows, cols, batch, 0, 0);
            return;
        }
        for (uint32_t t0 = 0; t0 < batch;) {
            const uint32_t n = std::min(batch - t0, GEMM_MAX_BATCH);
            if (type_id == 1) {
                gpu.f16_gemm(buf, x, y, rows, cols, n, t0 * cols, t0 * rows);
            } else {
                gpu.q8_0_gemm(buf, x, y, rows, cols, n, t0 * cols, t0 * rows);
            }
            t0 += n;
        }
    }

    void row_indirect(const HipContext &gpu, const HipBuffer &ids, uint32_t slot,
                      const HipBuffer &out) const {
        gpu.row_indirect_f32(buf, type_id, (uint32_t)out_dim, (uint32_t)in_dim, ids, slot, out);
    }

    void row_into(const HipContext &gpu, uint32_t row, const HipBuffer &out, uint32_t out_off) const {
        if (type_id == 1) {
            gpu.f16_row(buf, out, row, (uint32_t)in_dim, out_off);
        } else {
            gpu.q8_0_row(buf, out, row, (uint32_t)in_dim, out_off);
        }
    }

    HipBuffer buf;
    uint32_t type_id = 8;
    uint64_t in_dim = 0, out_dim = 0;
    NumericalProfile profile = NumericalProfile::OracleF32;
    // llama-cpu only, off unless the caller sets it: the int8 products take
    // tm_hip_q8_0_gemm_i8_fma (exact block dots, fused f32 tail: within 1e-5 of the
    // CPU's result instead of bit-identical to it, faster from 5 tokens).
    bool fused_i8_tail = false;

  private:
    // forward.rs:783-821 on the device: quantize the activations once per
    // product, then the int8 product, in slices of GEMM_I8_MAX_BATCH tokens. The
    // quantized-activation buffer grows to the largest slice seen and is kept (a
    // buffer that is replaced while a group still names it stays alive: the group
    // holds its memory).
    void gemm_llama_cpu(const HipContext &gpu, const HipBuffer &x, const HipBuffer &y,
                        uint32_t batch) {
        const uint32_t rows = (uint32_t)out_dim, cols = (uint32_t)in_dim;
        for (uint32_t t0 = 0; t0 < batch;) {
            const uint32_t n = std::min(batch - t0, GEMM_I8_MAX_BATCH);
            const size_t need = xq_bytes(cols, n);
            if (xq.len() < need) {
                xq = gpu.buffer(need, true);
            }
            gpu.q8_0_quantize_act(x, xq, cols, n, t0 * cols);
            if (fused_i8_tail) {
                gpu.q8_0_gemm_i8_fma(buf, xq, y, rows, cols, n, t0 * rows);
            } else {
                gpu.q8_0_gemm_i8(buf, xq, y, rows, cols, n, t0 * rows);
            }
            t0 += n;
        }
    }
    HipBuffer xq; // quantized activations of the llama-cpu profile
};

} // namespace tuckmill_hip
