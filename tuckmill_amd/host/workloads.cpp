// workloads.cpp — native step runner above the C ABI.
//
// A "step" is one pass of the hot path: a list of Q8_0 products issued the
// way the reference's engine issues a token step — one dispatch group per
// step (crates/tuckcore/src/engine/metal.rs:2462, qwen35_gpu.rs:66-85) — or
// one commit per product when `grouped` is 0; `grouped` 2 records the group
// once and replays it every step. The loop lives in native code so that the
// measured time is the library's, not an interpreter's.
#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <string>

#include "tm_hip.hpp"

using namespace tuckmill_hip;

extern "C" {

enum {
    TMH_GEMV = 0, TMH_GEMM = 1, TMH_GEMM_MMA = 2, TMH_GEMM_I8 = 3, TMH_QUANT = 4,
    // the operators either side of a product; `cols` is the element count:
    TMH_RMSNORM = 5,  // w = weight, x -> y, `rows` rows of `cols`
    TMH_SILU_MUL = 6, // w = gate, x = up -> y
    TMH_AXPY = 7,     // y += x (alpha = 1), w unused (pass y)
    TMH_ARGMAX = 8,   // x -> y[0], w = 512 bytes of scratch
    TMH_F16_GEMM = 9, // w holds rows*cols f16 values
    TMH_GELU_MUL = 10, // as TMH_SILU_MUL with ggml's tanh GELU
    TMH_GEMM_I8_FMA = 11 // as TMH_GEMM_I8 through the declared fast variant
};

struct tmh_product {
    tm_hip_buffer *w, *x, *y; // for TMH_GEMM_I8, x is the quantized activation buffer
    uint32_t rows, cols, batch, kind;
};

struct tmh_timing {
    double wall_ms;     // host clock around the timed steps, fence to fence
    double gpu_ms;      // sum of the commits' HIP-event times on the context's stream
    double host_ms;     // host time spent issuing the timed steps (before the final fence)
    uint64_t launches;  // kernel launches issued by the timed steps
    uint64_t commits;
    // GPU time per step from the commits' own events (a step's commits added up),
    // as order statistics over the timed steps: the robust figures beside the mean
    // gpu_ms / steps. Zero when a step's commits could not be told apart.
    double step_us_median, step_us_min, step_us_p10, step_us_p90;
};

struct Bound {
    HipBuffer w, x, y;
};

static void issue(const HipContext &gpu, const tmh_product *p, const std::vector<Bound> &b,
                  uint32_t n) {
    for (uint32_t i = 0; i < n; ++i) {
        const tmh_product &q = p[i];
        const HipBuffer &w = b[i].w, &x = b[i].x, &y = b[i].y;
        switch (q.kind) {
        case TMH_GEMV: gpu.q8_0_gemv(w, x, y, q.rows, q.cols); break;
        case TMH_GEMM: gpu.q8_0_gemm(w, x, y, q.rows, q.cols, q.batch, 0, 0); break;
        case TMH_GEMM_MMA: gpu.q8_0_gemm_mma(w, x, y, q.rows, q.cols, q.batch, 0, 0); break;
        case TMH_GEMM_I8: gpu.q8_0_gemm_i8(w, x, y, q.rows, q.cols, q.batch, 0); break;
        case TMH_GEMM_I8_FMA: gpu.q8_0_gemm_i8_fma(w, x, y, q.rows, q.cols, q.batch, 0); break;
        case TMH_QUANT: gpu.q8_0_quantize_act(x, y, q.cols, q.batch, 0); break;
        case TMH_RMSNORM: gpu.rmsnorm(x, w, y, q.rows, q.cols, 1e-6f); break;
        case TMH_SILU_MUL: gpu.silu_mul(w, x, y, q.cols); break;
        case TMH_GELU_MUL: gpu.gelu_tanh_mul(w, x, y, q.cols); break;
        case TMH_AXPY: gpu.f32_axpy(x, y, 1.0f, q.cols); break;
        case TMH_ARGMAX: gpu.argmax_f32(x, q.cols, w, y, 0); break;
        case TMH_F16_GEMM: gpu.f16_gemm(w, x, y, q.rows, q.cols, q.batch, 0, 0); break;
        default: throw TuckmillError(ErrorCode::InvalidRequest, "unknown product kind");
        }
    }
}

int tmh_run_steps(tm_hip_ctx *ctx, const tmh_product *products, uint32_t n, uint32_t warmup,
                  uint32_t steps, int grouped, tmh_timing *out, char *err, size_t err_cap) {
    try {
        HipContext gpu = HipContext::borrow(ctx);
        std::vector<Bound> bound;
        bound.reserve(n);
        for (uint32_t i = 0; i < n; ++i) {
            bound.push_back(Bound{gpu.borrow_buffer(products[i].w), gpu.borrow_buffer(products[i].x),
                                  gpu.borrow_buffer(products[i].y)});
        }
        RecordedStep recorded;
        if (grouped == 2) {
            recorded = gpu.recorded([&]() { issue(gpu, products, bound, n); });
        }
        auto one_step = [&]() {
            if (grouped == 2) {
                recorded.run();
            } else if (grouped) {
                gpu.grouped([&]() { issue(gpu, products, bound, n); });
            } else {
                issue(gpu, products, bound, n);
            }
        };
        for (uint32_t s = 0; s < warmup; ++s) {
            one_step();
        }
        gpu.fence();
        tm_hip_commit_log_set(ctx, 1);
        const uint64_t nanos0 = gpu.gpu_nanos_total();
        const uint64_t launches0 = gpu.kernel_launches();
        const uint64_t commits0 = gpu.committed_dispatches();
        const auto t0 = std::chrono::steady_clock::now();
        for (uint32_t s = 0; s < steps; ++s) {
            one_step();
        }
        const auto th = std::chrono::steady_clock::now();
        gpu.fence();
        const auto t1 = std::chrono::steady_clock::now();
        if (out != nullptr) {
            out->wall_ms = std::chrono::duration<double, std::milli>(t1 - t0).count();
            out->host_ms = std::chrono::duration<double, std::milli>(th - t0).count();
            out->gpu_ms = (double)(gpu.gpu_nanos_total() - nanos0) / 1e6;
            out->launches = gpu.kernel_launches() - launches0;
            out->commits = gpu.committed_dispatches() - commits0;
            out->step_us_median = out->step_us_min = out->step_us_p10 = out->step_us_p90 = 0.0;
            std::vector<uint64_t> log(TM_HIP_COMMIT_LOG_CAP);
            const size_t got = tm_hip_commit_log_read(ctx, log.data(), log.size());
            const uint64_t per_step = steps > 0 ? out->commits / steps : 0;
            if (steps > 0 && per_step > 0 && got == out->commits && per_step * steps == out->commits) {
                std::vector<double> us(steps, 0.0);
                for (size_t i = 0; i < got; ++i) {
                    us[i / per_step] += (double)log[i] / 1e3;
                }
                std::sort(us.begin(), us.end());
                out->step_us_min = us.front();
                out->step_us_median = steps % 2 ? us[steps / 2] : 0.5 * (us[steps / 2 - 1] + us[steps / 2]);
                out->step_us_p10 = us[(size_t)((steps - 1) * 0.1)];
                out->step_us_p90 = us[(size_t)((steps - 1) * 0.9)];
            }
        }
        tm_hip_commit_log_set(ctx, 0);
        return 0;
    } catch (const TuckmillError &e) {
        tm_hip_commit_log_set(ctx, 0);
        if (err != nullptr && err_cap > 0) {
            snprintf(err, err_cap, "%s", e.what());
        }
        return e.abi_code() != 0 ? e.abi_code() : TM_HIP_ERR_INTERNAL;
    }
}

// Self-check of the C++ handles (Matrix::load with its staged upload and
// seal, gemv, gemm slices, row lookup, ledger == plan) under a numerical
// profile ("oracle-f32" or "llama-cpu"). Returns 0 and the outputs for the
// caller to compare with its oracle.
int tmh_matrix_roundtrip_profile(const uint8_t *raw, uint32_t rows, uint32_t cols, uint32_t type_id,
                                 const char *profile_name, const float *x, uint32_t batch, int exact,
                                 float *y_out, float *row_out, uint32_t row, char *err,
                                 size_t err_cap) {
    try {
        NumericalProfile profile;
        if (!parse_numerical_profile(profile_name != nullptr ? profile_name : "", &profile)) {
            throw TuckmillError(ErrorCode::InvalidRequest,
                                std::string("unknown numerical profile '") +
                                    (profile_name != nullptr ? profile_name : "") +
                                    "' (oracle-f32, llama-cpu)",
                                TM_HIP_ERR_UNSUPPORTED);
        }
        HipContext gpu = HipContext::open();
        const uint64_t before = gpu.allocated_bytes();
        Matrix m = Matrix::load(gpu, raw, cols, rows, type_id, true, profile);
        if (gpu.allocated_bytes() - before != Matrix::plan(cols, rows, type_id)) {
            throw TuckmillError(ErrorCode::Internal, "allocation ledger differs from the plan");
        }
        HipBuffer xb = gpu.buffer((size_t)batch * cols * 4);
        HipBuffer yb = gpu.buffer((size_t)batch * rows * 4);
        HipBuffer ob = gpu.buffer((size_t)cols * 4);
        xb.upload(0, x, (size_t)batch * cols * 4);
        gpu.grouped([&]() {
            if (batch == 1) {
                m.gemv(gpu, xb, yb);
            } else {
                m.gemm(gpu, xb, yb, batch, exact != 0);
            }
            m.row_into(gpu, row, ob, 0);
        });
        yb.download(0, y_out, (size_t)batch * rows * 4);
        ob.download(0, row_out, (size_t)cols * 4);
        return 0;
    } catch (const TuckmillError &e) {
        if (err != nullptr && err_cap > 0) {
            snprintf(err, err_cap, "%s", e.what());
        }
        return e.abi_code() != 0 ? e.abi_code() : TM_HIP_ERR_INTERNAL;
    }
}

int tmh_matrix_roundtrip(const uint8_t *raw, uint32_t rows, uint32_t cols, const float *x,
                         uint32_t batch, int exact, float *y_out, float *row_out, uint32_t row,
                         char *err, size_t err_cap) {
    return tmh_matrix_roundtrip_profile(raw, rows, cols, 8, "oracle-f32", x, batch, exact, y_out,
                                        row_out, row, err, err_cap);
}

// The selection types through a C surface, for callers that test them without a
// GPU. Error classes: 0 ok, 1 unknown name, 2 InvalidRequest, 3 Unavailable,
// 4 UnsupportedArchitecture, 5 other.
static int error_class(const TuckmillError &e) {
    switch (e.code()) {
    case ErrorCode::InvalidRequest: return 2;
    case ErrorCode::Unavailable: return 3;
    case ErrorCode::UnsupportedArchitecture: return 4;
    default: return 5;
    }
}

// KernelSelection::parse(name).resolve() with `device_available` standing in
// for the probe (-1: ask the library); the resolved name goes to `resolved`.
int tmh_resolve_kernels(const char *name, int device_available, char *resolved, size_t cap,
                        char *err, size_t err_cap) {
    bool ok = false;
    const KernelSelection sel = KernelSelection::parse(name != nullptr ? name : "", &ok);
    if (!ok) {
        snprintf(err, err_cap, "unknown kernel selection '%s'", name != nullptr ? name : "");
        return 1;
    }
    try {
        const Probe device = device_available < 0
                                 ? probe()
                                 : Probe{device_available != 0, device_available != 0
                                                                    ? "test device"
                                                                    : "no HIP device available"};
        snprintf(resolved, cap, "%s", as_str(sel.resolve(device)));
        return 0;
    } catch (const TuckmillError &e) {
        snprintf(err, err_cap, "%s", e.what());
        return error_class(e);
    }
}

// check_engine_options(resolved kernels, profile, prefill batch given).
int tmh_check_engine_options(const char *kernels, const char *profile_name, int prefill_batch_given,
                             char *err, size_t err_cap) {
    ResolvedKernels k;
    const std::string ks = kernels != nullptr ? kernels : "";
    if (ks == "scalar") {
        k = ResolvedKernels::Scalar;
    } else if (ks == "neon") {
        k = ResolvedKernels::Neon;
    } else if (ks == "metal") {
        k = ResolvedKernels::Metal;
    } else if (ks == "hip") {
        k = ResolvedKernels::Hip;
    } else {
        snprintf(err, err_cap, "unknown resolved kernels '%s'", ks.c_str());
        return 1;
    }
    NumericalProfile profile;
    if (!parse_numerical_profile(profile_name != nullptr ? profile_name : "", &profile)) {
        snprintf(err, err_cap, "unknown numerical profile '%s'",
                 profile_name != nullptr ? profile_name : "");
        return 1;
    }
    try {
        check_engine_options(k, profile, prefill_batch_given != 0);
        snprintf(err, err_cap, "%s", as_str(profile));
        return 0;
    } catch (const TuckmillError &e) {
        snprintf(err, err_cap, "%s", e.what());
        return error_class(e);
    }
}

} // extern "C"
