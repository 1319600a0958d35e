/*
 * tm_hip.h — TuckCore <-> HIP narrow C ABI for the Q8_0 matrix-product path
 * on MI355X (gfx950).
 *
 * This is the HIP counterpart of the reference's Metal ABI
 * (native/metal/tm_metal.h): the same conventions, restricted to what the
 * Q8_0 decode GEMV / prefill GEMM / embedding-row path needs. Every entry
 * point names the reference declaration it stands in for.
 *
 * Conventions (native/metal/tm_metal.h:1-18, :32-40):
 *   - One context owns one device, one HIP stream and the loaded kernels.
 *   - Buffers are opaque handles with explicit lifetime, owned by exactly one
 *     context; every call checks ownership and length before any device work.
 *   - Dispatch is asynchronous; tm_hip_fence() waits for everything committed.
 *     Host copies are ordered after all committed work.
 *   - A context is used from one thread at a time (the caller serializes);
 *     the counters are atomic and tm_hip_download_after may be called without
 *     the caller's lock.
 *   - Operations return 0 or a negative TM_HIP_ERR_* code and write a
 *     NUL-terminated message into `err` (when non-NULL, `err_cap` bytes).
 *   - Dimensions are uint32_t; x/y offsets are in f32 ELEMENTS; X is
 *     [batch, cols] row-major, Y is [batch, rows] row-major (token-major).
 *
 * Q8_0 weights are `rows * cols/32` blocks of 34 bytes ([f16 d][i8 qs; 32],
 * little endian), rows contiguous, exactly as stored in GGUF. Every Q8_0
 * operation accepts a plain buffer holding those raw bytes. A buffer may
 * additionally be sealed with tm_hip_q8_0_pack(), which re-lays it out on
 * the device for coalesced loads; the same entry points then run their fast
 * kernels. Results do not depend on which layout a buffer is in.
 */
#ifndef TM_HIP_H
#define TM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tm_hip_ctx tm_hip_ctx;
typedef struct tm_hip_buffer tm_hip_buffer;

/* native/metal/tm_metal.h:32-40 */
enum {
    TM_HIP_OK = 0,
    TM_HIP_ERR_NO_DEVICE = -1,   /* no usable HIP device */
    TM_HIP_ERR_SOURCE = -2,      /* device code for this GPU is missing */
    TM_HIP_ERR_ALLOC = -3,       /* buffer allocation failed */
    TM_HIP_ERR_BOUNDS = -4,      /* size/range mismatch, zero length */
    TM_HIP_ERR_UNSUPPORTED = -5, /* invalid arguments / mode */
    TM_HIP_ERR_INTERNAL = -6     /* HIP runtime failure */
};

/* Largest batch of tm_hip_q8_0_gemm (native/metal/tm_metal.h:161-167;
 * crates/metal/src/lib.rs:28-30 GEMM_MAX_BATCH). */
#define TM_HIP_GEMM_MAX_BATCH 32u
/* Largest batch of tm_hip_q8_0_gemm_mma (native/metal/tm_metal.h:170). */
#define TM_HIP_GEMM_MMA_MAX_BATCH 512u
/* Largest batch of tm_hip_q8_0_gemm_i8 / tm_hip_q8_0_quantize_act. */
#define TM_HIP_GEMM_I8_MAX_BATCH 2048u

/* 1 when a gfx950 device is visible (native/metal/tm_metal.h:43). */
int tm_hip_available(void);

/* One-line runtime description; always a valid static string
 * (native/metal/tm_metal.h:47). */
const char *tm_hip_runtime_info(void);

/* Create a context on the current default device: stream, event pool and
 * kernels. Returns NULL and fills `err` on failure. The Metal counterpart
 * (native/metal/tm_metal.h:52) takes MSL source to compile; the HIP kernels
 * are compiled ahead of time into this library, so there is no source
 * argument. */
tm_hip_ctx *tm_hip_create(char *err, size_t err_cap);

/* Destroy the context after waiting for its work. Buffers created from it
 * must have been freed first (native/metal/tm_metal.h:56). */
void tm_hip_destroy(tm_hip_ctx *ctx);

/* Allocate `bytes` (> 0) of device memory. `shared` buffers accept host
 * copies; private (shared == 0) buffers refuse them, as on Metal. New
 * buffers read as zero (native/metal/tm_metal.h:61-62). */
tm_hip_buffer *tm_hip_buffer_new(tm_hip_ctx *ctx, size_t bytes, int shared, char *err,
                                 size_t err_cap);

/* Release a handle. Device memory that committed work still uses stays
 * alive (and counted by tm_hip_in_flight_bytes) until that work completes
 * (native/metal/tm_metal.h:66; lease rule native/metal/tm_metal.m:167-224). */
void tm_hip_buffer_free(tm_hip_ctx *ctx, tm_hip_buffer *buffer);

/* Length in bytes, 0 for an invalid handle (native/metal/tm_metal.h:73). */
size_t tm_hip_buffer_len(const tm_hip_ctx *ctx, const tm_hip_buffer *buffer);

/* Zero `len` bytes at byte offset `off` on the device, ordered with the
 * context's other work (native/metal/tm_metal.h:78-79). */
int tm_hip_buffer_zero(tm_hip_ctx *ctx, tm_hip_buffer *buffer, size_t off, size_t len,
                       char *err, size_t err_cap);

/* Host <-> device copies (shared buffers only). Both wait for every
 * committed dispatch first and are refused while a group is open
 * (native/metal/tm_metal.h:82-85; copy contract native/metal/tm_metal.m:569-609).
 * Sealed (packed) weight buffers refuse them. */
int tm_hip_upload(tm_hip_ctx *ctx, tm_hip_buffer *dst, size_t off, const void *src, size_t len,
                  char *err, size_t err_cap);
int tm_hip_download(tm_hip_ctx *ctx, tm_hip_buffer *src, size_t off, void *dst, size_t len,
                    char *err, size_t err_cap);

/* Copy a range once the first `completed_target` commits have completed,
 * without waiting for later work (native/metal/tm_metal.h:295-300). */
int tm_hip_download_after(tm_hip_ctx *ctx, tm_hip_buffer *src, size_t off, void *dst,
                          size_t len, uint64_t completed_target, char *err, size_t err_cap);

/* dst[dst_off + i] = src[src_off + i], i < n, f32 elements, bit-exact;
 * usable inside a group (native/metal/tm_metal.h:108-113). */
int tm_hip_copy_f32(tm_hip_ctx *ctx, tm_hip_buffer *src, uint32_t src_off, tm_hip_buffer *dst,
                    uint32_t dst_off, uint32_t n, char *err, size_t err_cap);

/* ---- the small f32 operators either side of a product ----------------------
 * All are usable inside a dispatch group; a zero length is refused with
 * TM_HIP_ERR_BOUNDS (rmsnorm: a zero shape with TM_HIP_ERR_UNSUPPORTED), as in
 * the reference host code (native/metal/tm_metal.m:770-810, :1096-1177). */

/* y[i] = x[i] * factor, i < n (native/metal/tm_metal.h:88-90). */
int tm_hip_f32_scale(tm_hip_ctx *ctx, tm_hip_buffer *x, tm_hip_buffer *y, float factor, uint32_t n,
                     char *err, size_t err_cap);

/* y[i] = (float)x[i], i < n, x in IEEE binary16 (n * 2 bytes), exact
 * (native/metal/tm_metal.h:118-120). */
int tm_hip_cast_f16_f32(tm_hip_ctx *ctx, tm_hip_buffer *x, tm_hip_buffer *y, uint32_t n, char *err,
                        size_t err_cap);

/* y[i] = (half)x[i], i < n, y in IEEE binary16 (n * 2 bytes): round to nearest
 * even, overflow to infinity, a NaN stays a NaN (native/metal/tm_metal.h:122-124). */
int tm_hip_cast_f32_f16(tm_hip_ctx *ctx, tm_hip_buffer *x, tm_hip_buffer *y, uint32_t n, char *err,
                        size_t err_cap);

/* y[i] = y[i] + alpha * a[i], i < n: multiply, then add, unfused
 * (native/metal/tm_metal.h:115-116). */
int tm_hip_f32_axpy(tm_hip_ctx *ctx, tm_hip_buffer *a, tm_hip_buffer *y, float alpha, uint32_t n,
                    char *err, size_t err_cap);

/* y[row] = x[row] / sqrt(mean(x[row]^2) + eps) * weight for `rows` rows of
 * `cols`; in place (x == y) is allowed (native/metal/tm_metal.h:147-149,
 * crates/tuckcore/src/forward.rs:911-927). */
int tm_hip_rmsnorm_f32(tm_hip_ctx *ctx, tm_hip_buffer *x, tm_hip_buffer *weight, tm_hip_buffer *y,
                       uint32_t rows, uint32_t cols, float eps, char *err, size_t err_cap);

/* out[i] = silu(gate[i]) * up[i], silu(g) = g / (1 + exp(-g))
 * (native/metal/tm_metal.h:189-191, crates/tuckcore/src/forward.rs:906-908). */
int tm_hip_silu_mul_f32(tm_hip_ctx *ctx, tm_hip_buffer *gate, tm_hip_buffer *up, tm_hip_buffer *out,
                        uint32_t n, char *err, size_t err_cap);

/* out[i] = gelu_tanh(gate[i]) * up[i], ggml's tanh form
 * (native/metal/tm_metal.h:193-195, native/metal/kernels.metal:382-396). */
int tm_hip_gelu_tanh_mul_f32(tm_hip_ctx *ctx, tm_hip_buffer *gate, tm_hip_buffer *up,
                             tm_hip_buffer *out, uint32_t n, char *err, size_t err_cap);

/* Greedy argmax of x[0..n) into out[out_index] (u32), the CPU rule: NaN
 * skipped, largest value wins, ties to the lowest index, 0xFFFFFFFF when every
 * entry is NaN. `partial` is TM_HIP_ARGMAX_PARTIAL_BYTES of scratch
 * (native/metal/tm_metal.h:92-98, crates/backend/src/sampling.rs:66-83). The
 * result can feed tm_hip_row_indirect_f32 inside the same group. */
#define TM_HIP_ARGMAX_NONE 0xFFFFFFFFu
#define TM_HIP_ARGMAX_PARTIAL_BYTES 512
int tm_hip_argmax_f32(tm_hip_ctx *ctx, tm_hip_buffer *x, uint32_t n, tm_hip_buffer *partial,
                      tm_hip_buffer *out, uint32_t out_index, char *err, size_t err_cap);

/* Grouped encoding: operations between begin and end are submitted as ONE
 * commit at end_group; abort_group discards them unsubmitted. Copies and
 * fence require no open group (native/metal/tm_metal.h:125-135). Inside a
 * group, consecutive Q8_0 products whose buffers do not depend on each
 * other are executed by a single kernel launch. */
int tm_hip_begin_group(tm_hip_ctx *ctx, char *err, size_t err_cap);
int tm_hip_end_group(tm_hip_ctx *ctx, char *err, size_t err_cap);
int tm_hip_abort_group(tm_hip_ctx *ctx, char *err, size_t err_cap);

/* A recorded group. The reference encodes the same operators on the same
 * buffers again for every generated token (one command buffer per token:
 * crates/tuckcore/src/qwen35_gpu.rs:71-77 around the per-layer calls of
 * crates/tuckcore/src/engine/metal.rs:496-511, :1125-1131); Metal command
 * buffers cannot be resubmitted, HIP graphs can. end_group_recorded closes the
 * open group like end_group but, instead of committing it, keeps its planned
 * launches as a replayable step (nothing runs yet); every step_run is one
 * commit that executes them again on the current contents of the same buffers,
 * with the results end_group would give. The step holds a reference on every
 * buffer it touches until step_free (freeing a buffer handle earlier is
 * allowed; the memory lives on), and on the weight bytes as they were laid out
 * when it was recorded: seal weights before recording. A group that holds no
 * operation cannot be recorded. step_free waits for queued replays. */
typedef struct tm_hip_step tm_hip_step;
int tm_hip_end_group_recorded(tm_hip_ctx *ctx, tm_hip_step **out, char *err, size_t err_cap);
int tm_hip_step_run(tm_hip_ctx *ctx, tm_hip_step *step, char *err, size_t err_cap);
uint32_t tm_hip_step_launches(const tm_hip_ctx *ctx, const tm_hip_step *step);
void tm_hip_step_free(tm_hip_ctx *ctx, tm_hip_step *step);

/* Block until every commit has completed; refused while a group is open
 * (native/metal/tm_metal.h:289-291). */
int tm_hip_fence(tm_hip_ctx *ctx, char *err, size_t err_cap);

/* ---- the Q8_0 products ---- */

/* y[r] = dot(dequant_q8_0(w_row_r), x), r < rows. `cols` a positive multiple
 * of 32; x holds cols f32, y rows f32 (native/metal/tm_metal.h:196-202;
 * validation native/metal/tm_metal.m:962-980). */
int tm_hip_q8_0_gemv(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *x, tm_hip_buffer *y,
                     uint32_t rows, uint32_t cols, char *err, size_t err_cap);

/* Y[b, :] = W . X[b, :], b < batch (1..=TM_HIP_GEMM_MAX_BATCH), with the
 * GEMV's per-token arithmetic: batch = 1 is bit-identical to
 * tm_hip_q8_0_gemv, and every token's row equals the GEMV of that token
 * (native/metal/tm_metal.h:161-167). */
int tm_hip_q8_0_gemm(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *x, tm_hip_buffer *y,
                     uint32_t rows, uint32_t cols, uint32_t batch, uint32_t x_off,
                     uint32_t y_off, char *err, size_t err_cap);

/* Same contract for batch 1..=TM_HIP_GEMM_MMA_MAX_BATCH on the MFMA matrix
 * cores: every product q*x is exact (f32 operand tiles with W dequantized
 * exactly as d*q; or, from 17 tokens over sealed weights, bf16 tiles with
 * every activation split into three exact bf16 pieces). Summation order
 * differs from the GEMV: tolerance-qualified, not bit-identical
 * (native/metal/tm_metal.h:172-178). Which of the two forms runs, and how K is
 * cut, is decided per launch from the products that share it (independent
 * products of one dispatch group): the same group gives the same bits every
 * time, on every replay of a recorded step too, but a product's last bits may
 * differ between groupings. The bf16 form keeps a workspace in the context
 * (6 bytes per activation element plus partial tiles), grown on first use and
 * freed with the context. */
int tm_hip_q8_0_gemm_mma(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *x, tm_hip_buffer *y,
                         uint32_t rows, uint32_t cols, uint32_t batch, uint32_t x_off,
                         uint32_t y_off, char *err, size_t err_cap);

/* tm_hip_q8_0_gemm_mma for callers that cannot allocate device memory: code
 * under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc. No counterpart in the reference. Same arguments, refusals, kernels
 * and results as tm_hip_q8_0_gemm_mma (bit for bit), with these differences:
 *   - Nothing is allocated or freed on the device, in this call or later because
 *     of it: the workspace of the large-product form lies in a static device
 *     array of TM_HIP_NOALLOC_WORKSPACE_BYTES that every GPU the library runs on
 *     holds from load to process exit. A product whose split activations
 *     (6 bytes x batch x cols, at most TM_HIP_NOALLOC_XS_BYTES) or partial tiles
 *     do not fit is refused with TM_HIP_ERR_UNSUPPORTED and a message that says
 *     what it needs; tm_hip_q8_0_gemm_mma takes it.
 *   - The kernels are launched at once on the context's stream, in order with
 *     everything committed before and after; the call is not a commit (no
 *     events, not counted by committed_dispatches) and is refused while a
 *     dispatch group is open. tm_hip_fence and host copies wait for it like for
 *     any other work.
 *   - w, x and y stay leased (visible in tm_hip_in_flight_bytes, safe to free)
 *     until the next commit of the context completes or a fence has passed;
 *     after TM_HIP_NOALLOC_MAX_PENDING calls without either, the call is refused.
 *   - All calls on one GPU share the one array, which keeps the last call's
 *     contents (what must start at zero is cleared by the call itself). One
 *     context orders its own calls; calls from different contexts of one process
 *     are ordered by the library (a call that follows another context's makes
 *     its stream wait for that context's stream first, under a process-wide
 *     lock held for the duration of the call), so they may come from different
 *     threads without a fence between them. The call allocates nothing on the
 *     host either. Two PROCESSES each hold their own copy of the array. */
#define TM_HIP_NOALLOC_WORKSPACE_BYTES (64u << 20)
#define TM_HIP_NOALLOC_XS_BYTES (20u << 20)
#define TM_HIP_NOALLOC_MAX_PENDING 1024u
int tm_hip_q8_0_gemm_mma_noalloc(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *x,
                                 tm_hip_buffer *y, uint32_t rows, uint32_t cols, uint32_t batch,
                                 uint32_t x_off, uint32_t y_off, char *err, size_t err_cap);

/* out[out_off + i] = d * q of row `row`, i < cols; exact
 * (native/metal/tm_metal.h:137-139). */
int tm_hip_q8_0_row_f32(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *out, uint32_t row,
                        uint32_t cols, uint32_t out_off, char *err, size_t err_cap);

/* out[i] = row ids[slot] of `w` dequantized to f32; an id >= rows writes
 * zeros. type_id 8 is Q8_0 (cols a multiple of 32), type_id 1 is F16
 * (native/metal/tm_metal.h:100-106, native/metal/tm_metal.m:874-885). */
int tm_hip_row_indirect_f32(tm_hip_ctx *ctx, tm_hip_buffer *w, uint32_t type_id, uint32_t rows,
                            uint32_t cols, tm_hip_buffer *ids, uint32_t slot, tm_hip_buffer *out,
                            char *err, size_t err_cap);

/* ---- F16 weight twins of the products ---- */

/* y[r] = dot(f32(w_row_r), x); `w` holds rows*cols f16 values, any cols > 0
 * (native/metal/tm_metal.h:141-144). */
int tm_hip_f16_gemv(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *x, tm_hip_buffer *y,
                    uint32_t rows, uint32_t cols, char *err, size_t err_cap);

/* The contract of tm_hip_q8_0_gemm on F16 weights: batch 1..=32, offsets in
 * f32 elements, token b bit-identical to the GEMV on x[b]
 * (native/metal/tm_metal.h:179-181, native/metal/kernels.metal:638-668). */
int tm_hip_f16_gemm(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *x, tm_hip_buffer *y,
                    uint32_t rows, uint32_t cols, uint32_t batch, uint32_t x_off, uint32_t y_off,
                    char *err, size_t err_cap);

/* out[out_off + i] = f32(w[row][i]), i < cols; exact
 * (native/metal/tm_metal.h:155-157). */
int tm_hip_f16_row_f32(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *out, uint32_t row,
                       uint32_t cols, uint32_t out_off, char *err, size_t err_cap);

/* ---- additions with no Metal counterpart ---- */

/* Seal `w` (which holds the raw GGUF bytes of a rows x cols Q8_0 matrix) in
 * the device layout: all int8 quants first ([rows][cols], 16-byte pieces
 * aligned), then all f16 scales ([rows][cols/32]) — the same byte count, so
 * the allocation ledger is unchanged. Called once after the staged upload
 * that crates/tuckcore/src/engine/metal.rs:138-147 performs. After sealing,
 * host copies and buffer_zero on `w` are refused, and Q8_0 operations must
 * name the same rows/cols. No counterpart in the reference: Apple's unified
 * memory has no use for it. */
int tm_hip_q8_0_pack(tm_hip_ctx *ctx, tm_hip_buffer *w, uint32_t rows, uint32_t cols, char *err,
                     size_t err_cap);

/* Quantize `batch` rows of `cols` f32 activations (at element offset x_off
 * of `x`) to Q8_0 with the rule of crates/tuckcore/src/tensor.rs:184-206.
 * `xq` receives batch*cols int8 quants (token-major) followed by the f32
 * scales (each the f32 value of the f16-rounded scale) stored block-major as
 * [cols/32][bpad], bpad = batch rounded up to a multiple of 4; entries of
 * the padding tokens are not written. Bytes needed:
 * batch*cols + (cols/32)*bpad*4. Device form of the `llama-cpu` numerical
 * profile's first step (crates/tuckcore/src/forward.rs:783-793). */
int tm_hip_q8_0_quantize_act(tm_hip_ctx *ctx, tm_hip_buffer *x, tm_hip_buffer *xq, uint32_t cols,
                             uint32_t batch, uint32_t x_off, char *err, size_t err_cap);

/* Y[b, r] = sum over blocks of (d_w * d_x[b]) * (i32 block dot), the
 * arithmetic of crates/tuckcore/src/kernels.rs:206-221, with `xq` produced
 * by tm_hip_q8_0_quantize_act. The i32 block dots are exact; batch
 * 1..=TM_HIP_GEMM_I8_MAX_BATCH. When `sumi` is non-NULL it receives the raw
 * block dots as int32 [batch, rows, cols/32] (verification aid). */
int tm_hip_q8_0_gemm_i8(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *xq, tm_hip_buffer *y,
                        tm_hip_buffer *sumi, uint32_t rows, uint32_t cols, uint32_t batch,
                        uint32_t y_off, char *err, size_t err_cap);

/* tm_hip_q8_0_gemm_i8 with a declared, faster tail: the same exact i32 block
 * dots and the same scale product d_w * d_x, but each block's term enters the
 * sum with one fused multiply-add, acc = fma(d_w * d_x, (float)sumi, acc),
 * where crates/tuckcore/src/kernels.rs:206-221 rounds the product and then the
 * sum. One rounding fewer per block: the f32 result is within the 1e-5
 * (normalised) tolerance of the CPU's, not bit-identical to it. Never chosen by
 * the library on its own: a caller that wants the CPU's bits calls
 * tm_hip_q8_0_gemm_i8. Batches that the bit-exact kernels serve at the speed of
 * the weight stream (up to 4 tokens, or weights as uploaded) take those kernels
 * and their bits. No counterpart in the reference. */
int tm_hip_q8_0_gemm_i8_fma(tm_hip_ctx *ctx, tm_hip_buffer *w, tm_hip_buffer *xq, tm_hip_buffer *y,
                            uint32_t rows, uint32_t cols, uint32_t batch, uint32_t y_off, char *err,
                            size_t err_cap);

/* ---- measurement surface (native/metal/tm_metal.h:293-325) ---- */

/* XOR of the n 32-bit words at word offset src_off (a multiple of 4) of `src`,
 * left as TM_HIP_CHECKSUM_PARTIAL_BYTES / 4 partial words in `partial` whose
 * XOR is the result (any buffer contents, sealed weights included: the bytes
 * are read as they lie on the device). Usable inside a group. The kernel only
 * reads (non-temporal 16-byte loads, a wave's tile 8 KiB like the decode
 * GEMV's) and writes 8 KiB whatever n is: over a gibibyte it measures the
 * sustained HBM read bandwidth the streaming kernels are set against, and it
 * checks an upload without a download. No counterpart in the reference. */
#define TM_HIP_CHECKSUM_PARTIAL_BYTES 8192u
int tm_hip_xor_checksum_u32(tm_hip_ctx *ctx, tm_hip_buffer *src, uint32_t src_off, uint32_t n,
                            tm_hip_buffer *partial, char *err, size_t err_cap);

uint64_t tm_hip_committed_dispatches(const tm_hip_ctx *ctx);
uint64_t tm_hip_completed_dispatches(const tm_hip_ctx *ctx);
/* GPU milliseconds of the most recently completed commit (HIP events on the
 * context's stream). */
double tm_hip_last_gpu_ms(const tm_hip_ctx *ctx);
/* Cumulative GPU nanoseconds over every completed commit. */
uint64_t tm_hip_gpu_nanos_total(const tm_hip_ctx *ctx);
/* Number of kernel launches issued so far (a group may issue fewer launches
 * than it holds operations). */
uint64_t tm_hip_kernel_launches(const tm_hip_ctx *ctx);
/* Opt-in per-operator GPU time table; labels carry the shape
 * ("q8_0_gemv:3072x1024"), a group is attributed to "group". */
int tm_hip_profile_set(tm_hip_ctx *ctx, int enabled);
int tm_hip_profile_read(tm_hip_ctx *ctx, uint32_t index, char *name, size_t name_cap,
                        uint64_t *nanos, uint64_t *count);
/* Per-commit GPU times, for benchmarks that report a robust statistic the way
 * the reference's isolated timings do (crates/metal/src/tests.rs:1057-1066,
 * benchmarks/tools/ggml-mul-mat.c:69-75). While enabled, every commit that
 * completes appends its GPU nanoseconds (the value last_gpu_ms reports for it)
 * to a log kept by the context; the log holds the most recent
 * TM_HIP_COMMIT_LOG_CAP entries. read copies up to `cap` entries in completion
 * order into `nanos`, removes them and returns their number. set(…, 0) stops
 * logging and clears the log. No counterpart in the reference. */
#define TM_HIP_COMMIT_LOG_CAP 65536u
int tm_hip_commit_log_set(tm_hip_ctx *ctx, int enabled);
size_t tm_hip_commit_log_read(tm_hip_ctx *ctx, uint64_t *nanos, size_t cap);
/* Live bytes in handles of this context. */
uint64_t tm_hip_allocated_bytes(const tm_hip_ctx *ctx);
/* Bytes leased by commits that have not completed yet. */
uint64_t tm_hip_in_flight_bytes(const tm_hip_ctx *ctx);

#ifdef __cplusplus
}
#endif

#endif /* TM_HIP_H */
