/*
 * q8_oracle.h — CPU restatement of TuckCore's scalar Q8_0 path.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing in the product library links, loads or
 * calls this file; it exists so that tests (and the CPU-baseline leg of the
 * benchmark) can check the HIP kernels against the reference's arithmetic.
 *
 * Every function names the reference lines it follows (paths relative to the
 * reference checkout). The translation unit must be compiled with
 * `-O2 -ffp-contract=off -fno-fast-math`: Rust never fuses a*b+c and never
 * reassociates, and the restatement must not either.
 */
#ifndef Q8_ORACLE_H
#define Q8_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define Q8O_BLOCK_ELEMS 32
#define Q8O_BLOCK_BYTES 34

/* crates/tuckcore/src/tensor.rs:12-28 */
float q8o_f16_to_f32(uint16_t bits);
/* crates/tuckcore/src/tensor.rs:145-178 (NaN input encodes as +/-inf: the
 * `exp >= 0x1f` branch at :150-153 does not keep the NaN payload). */
uint16_t q8o_f32_to_f16_bits(float value);

/* The two functions above over n elements (crates/metal/src/tests.rs:257-305 checks the
 * device casts against them element by element). */
void q8o_f16_to_f32_n(const uint16_t *bits, size_t n, float *out);
void q8o_f32_to_f16_bits_n(const float *values, size_t n, uint16_t *out);

/* crates/tuckcore/src/tensor.rs:94-104: out[i] = d * q for `blocks` blocks. */
void q8o_dequant_q8_0(const uint8_t *bytes, size_t blocks, float *out);

/* crates/tuckcore/src/tensor.rs:184-206. `n` must be a multiple of 32.
 * qs receives n int8 values, d receives n/32 f32 scales (each the f32 value
 * of the f16-rounded scale). */
void q8o_quantize_row_q8_0(const float *x, size_t n, int8_t *qs, float *d);

/* crates/tuckcore/src/kernels.rs:139-149. 0 when the row is a positive
 * multiple of 34 bytes and x_len == blocks*32; -1 malformed row
 * (InvalidArtifact), -2 activation length mismatch (Internal). */
int q8o_validate_q8_0_row(size_t row_bytes, size_t x_len);
/* crates/tuckcore/src/kernels.rs:153-165; same codes. */
int q8o_validate_q8_0_q8_0(size_t row_bytes, size_t x_qs_blocks, size_t x_d_len);

/* crates/tuckcore/src/kernels.rs:186-204 (scalar::dot_q8_0_x_f32). */
float q8o_dot_q8_0_x_f32(const uint8_t *row, size_t blocks, const float *x);
/* crates/tuckcore/src/kernels.rs:206-221 (scalar::dot_q8_0_q8_0). When
 * `sumi_out` is non-NULL it receives the `blocks` exact i32 block dots. */
float q8o_dot_q8_0_q8_0(const uint8_t *row, size_t blocks, const int8_t *x_qs,
                        const float *x_d, int32_t *sumi_out);

/* F16 weight rows (the reference's F16 twins of the Q8_0 products).
 * crates/tuckcore/src/kernels.rs:167-178: 0 when the row is a positive even
 * number of bytes and x_len == row_bytes / 2; -1 malformed row, -2 length. */
int q8o_validate_f16_row(size_t row_bytes, size_t x_len);
/* crates/tuckcore/src/kernels.rs:223-232 (scalar::dot_f16_x_f32):
 * acc += f16_to_f32(w[i]) * x[i], sequential from 0.0, unfused. */
float q8o_dot_f16_x_f32(const uint8_t *row, size_t elems, const float *x);
/* y[b*rows + r] = dot_f16_x_f32(row r, x[b]) (the row loop of
 * forward.rs:703-735 over F16 rows; native/metal/kernels.metal:296-315,
 * :638-668 state the same contract for the device). */
void q8o_gemm_f16_f32(const uint8_t *w, size_t rows, size_t cols, const float *x, size_t batch,
                      float *y);

/* Row loop of crates/tuckcore/src/forward.rs:703-735 (matvec_fused):
 * y[r] = dot_q8_0_x_f32(row r, x). `threads` > 1 partitions rows (rows are
 * independent, so the output is bit-identical for every thread count). */
void q8o_gemv_q8_0_f32(const uint8_t *w, size_t rows, size_t cols, const float *x,
                       float *y, int threads);
/* Row loop of crates/tuckcore/src/forward.rs:783-821 (matvec_q8_0_llama_cpu):
 * quantize x once, then dot_q8_0_q8_0 per row. */
void q8o_gemv_q8_0_q8_0(const uint8_t *w, size_t rows, size_t cols, const float *x,
                        float *y, int threads);
/* GEMM = one GEMV per token: X [batch, cols], Y [batch, rows], both
 * row-major (token-major), as native/metal/kernels.metal:473 stores them. */
void q8o_gemm_q8_0_f32(const uint8_t *w, size_t rows, size_t cols, const float *x,
                       size_t batch, float *y, int threads);
void q8o_gemm_q8_0_q8_0(const uint8_t *w, size_t rows, size_t cols, const float *x,
                        size_t batch, float *y, int threads);

/* The other order the reference uses in its GPU operator tests:
 * acc += d*q*x element by element, crates/metal/src/tests.rs:100-116. */
void q8o_gemv_q8_0_f32_dequant_first(const uint8_t *w, size_t rows, size_t cols,
                                     const float *x, float *y);
/* f64 evaluation of the same sum (error-budget reference, not a reference
 * function). */
void q8o_gemv_q8_0_f64(const uint8_t *w, size_t rows, size_t cols, const float *x,
                       double *y);

/* ---- generators held by the reference's own tests ---- */

/* xorshift64* stream, crates/metal/src/tests.rs:30-40. */
uint64_t q8o_rng_next(uint64_t *state);
/* crates/metal/src/tests.rs:119-149. out holds rows*(cols/32)*34 bytes. */
void q8o_boundary_weights(size_t rows, size_t cols, uint64_t seed, uint8_t *out);
/* crates/metal/src/tests.rs:151-162. */
void q8o_boundary_input(size_t n, uint64_t seed, float *out);
/* crates/tuckcore/src/kernels.rs:434-443 (Rng::next_f32). */
float q8o_krng_next_f32(uint64_t *state, float scale);
/* crates/tuckcore/src/kernels.rs:445-456 (random_q8_0_row). */
void q8o_random_q8_0_row(uint64_t *state, size_t blocks, uint8_t *out);


/* ---- the small f32 operators either side of a product --------------------
 * rmsnorm: crates/tuckcore/src/forward.rs:917-927; silu_mul: forward.rs:906-908;
 * gelu_tanh_mul: native/metal/kernels.metal:382-396; axpy / scale:
 * kernels.metal:14-36; argmax: crates/backend/src/sampling.rs:69-83. */
void q8o_rmsnorm(const float *x, const float *w, size_t n, float eps, float *y);
void q8o_silu_mul(const float *gate, const float *up, size_t n, float *out);
void q8o_gelu_tanh_mul(const float *gate, const float *up, size_t n, float *out);
void q8o_axpy(const float *a, float alpha, size_t n, float *y);
void q8o_scale(const float *x, float factor, size_t n, float *y);
uint32_t q8o_argmax(const float *x, size_t n);

#ifdef __cplusplus
}
#endif

#endif /* Q8_ORACLE_H */
