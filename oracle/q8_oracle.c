/*
 * q8_oracle.c — CPU restatement of TuckCore's scalar Q8_0 path.
 *
 * TEST INFRASTRUCTURE ONLY (see q8_oracle.h). Build with
 *   gcc -O2 -ffp-contract=off -fno-fast-math -fopenmp -shared -fPIC
 * so that no multiply-add is fused and no sum is reassociated.
 *
 * Pinning status (which known answers fix each function is listed next to
 * it; the tests that apply them live in tests/test_oracle_*.py):
 *   f16_to_f32, f32_to_f16_bits, dequant, quantize_row_q8_0,
 *   dot_q8_0_x_f32, dot_q8_0_q8_0, dot_f16_x_f32, the generators: pinned.
 *   No function here is "parity unpinned".
 */
#include "q8_oracle.h"

#include <math.h>
#include <string.h>

/* ------------------------------------------------------------------ f16 -- */

/* crates/tuckcore/src/tensor.rs:12-28. Pinned by the known values at
 * tensor.rs:264-272 and by an exhaustive comparison against the compiler's
 * _Float16 -> float conversion over all 65536 encodings. */
float q8o_f16_to_f32(uint16_t bits) {
    unsigned sign = (bits >> 15) & 1u;
    unsigned exp = (bits >> 10) & 0x1fu;
    unsigned mant = bits & 0x3ffu;
    float value;
    if (exp == 0 && mant == 0) {
        value = 0.0f;
    } else if (exp == 0) {
        value = (float)mant * 0x1p-24f;
    } else if (exp == 31 && mant == 0) {
        value = INFINITY;
    } else if (exp == 31) {
        value = NAN;
    } else {
        value = (1.0f + (float)mant / 1024.0f) * ldexpf(1.0f, (int)exp - 15);
    }
    return sign ? -value : value;
}

/* crates/tuckcore/src/tensor.rs:145-178. Pinned by tensor.rs:358-370 and
 * crates/metal/src/tests.rs:257-275, and by comparison against the
 * compiler's (_Float16) rounding on every f16 value, every midpoint between
 * neighbouring f16 values and a dense sample of finite f32. */
uint16_t q8o_f32_to_f16_bits(float value) {
    uint32_t bits;
    memcpy(&bits, &value, sizeof bits);
    uint16_t sign = (uint16_t)((bits >> 16) & 0x8000u);
    int32_t exp = (int32_t)((bits >> 23) & 0xffu) - 127 + 15;
    uint32_t mant = bits & 0x7fffffu;
    if (exp >= 0x1f) {
        return (uint16_t)(sign | 0x7c00u);
    }
    if (exp <= 0) {
        if (exp < -10) {
            return sign;
        }
        uint32_t m = mant | 0x800000u;
        uint32_t shift = (uint32_t)(14 - exp);
        uint32_t half = (m >> shift) & 0x3ffu;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1u);
        uint32_t round_up = (rem > halfway || (rem == halfway && (half & 1u) == 1u)) ? 1u : 0u;
        half += round_up;
        return (uint16_t)(sign | (uint16_t)half);
    }
    uint32_t rounded = mant + 0x0fffu + ((mant >> 13) & 1u);
    if (rounded & 0x800000u) {
        exp += 1;
        if (exp >= 0x1f) {
            return (uint16_t)(sign | 0x7c00u);
        }
        return (uint16_t)(sign | (uint16_t)((uint32_t)exp << 10));
    }
    return (uint16_t)(sign | (uint16_t)((uint32_t)exp << 10) | (uint16_t)(rounded >> 13));
}

/* The two conversions over arrays (the checker of the device cast operators,
 * crates/metal/src/tests.rs:257-305): element by element through the functions above. */
void q8o_f16_to_f32_n(const uint16_t *bits, size_t n, float *out) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) {
        out[i] = q8o_f16_to_f32(bits[i]);
    }
}

void q8o_f32_to_f16_bits_n(const float *values, size_t n, uint16_t *out) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; ++i) {
        out[i] = q8o_f32_to_f16_bits(values[i]);
    }
}

static inline uint16_t read_u16_le(const uint8_t *p) {
    return (uint16_t)((uint16_t)p[0] | ((uint16_t)p[1] << 8));
}

/* crates/tuckcore/src/tensor.rs:94-104. Pinned by tensor.rs:302-314 and the
 * fixture closed form of crates/manifest/src/testing.rs:679-691. */
void q8o_dequant_q8_0(const uint8_t *bytes, size_t blocks, float *out) {
    for (size_t b = 0; b < blocks; ++b) {
        const uint8_t *block = bytes + b * Q8O_BLOCK_BYTES;
        float d = q8o_f16_to_f32(read_u16_le(block));
        for (int q = 0; q < 32; ++q) {
            out[b * 32 + (size_t)q] = d * (float)(int8_t)block[2 + q];
        }
    }
}

/* ------------------------------------------------------------ quantizer -- */

/* crates/tuckcore/src/tensor.rs:184-206. Pinned by tensor.rs:373-392 and by
 * invariants (|q| <= 127, zero block -> d = 0 and q = 0, |x - d*q| <= d/2,
 * agreement with an independent float64 evaluation of the same rule). */
void q8o_quantize_row_q8_0(const float *x, size_t n, int8_t *qs, float *d_out) {
    size_t blocks = n / 32;
    for (size_t b = 0; b < blocks; ++b) {
        const float *chunk = x + b * 32;
        float amax = 0.0f;
        for (int i = 0; i < 32; ++i) {
            /* f32::max returns the other operand when one is NaN. */
            amax = fmaxf(amax, fabsf(chunk[i]));
        }
        float d = amax / 127.0f;
        float id = (d != 0.0f) ? 1.0f / d : 0.0f;
        float d_f16 = q8o_f16_to_f32(q8o_f32_to_f16_bits(d));
        for (int i = 0; i < 32; ++i) {
            float r = nearbyintf(chunk[i] * id); /* round_ties_even */
            int8_t q;
            if (isnan(r)) {
                q = 0; /* `NaN as i8` is 0 in Rust */
            } else {
                if (r < -127.0f) r = -127.0f;
                if (r > 127.0f) r = 127.0f;
                q = (int8_t)r;
            }
            qs[b * 32 + (size_t)i] = q;
        }
        d_out[b] = d_f16;
    }
}

/* ----------------------------------------------------------- validation -- */

/* crates/tuckcore/src/kernels.rs:139-149 */
int q8o_validate_q8_0_row(size_t row_bytes, size_t x_len) {
    if (row_bytes == 0 || row_bytes % Q8O_BLOCK_BYTES != 0) {
        return -1;
    }
    size_t blocks = row_bytes / Q8O_BLOCK_BYTES;
    if (x_len != blocks * 32) {
        return -2;
    }
    return 0;
}

/* crates/tuckcore/src/kernels.rs:167-178 */
int q8o_validate_f16_row(size_t row_bytes, size_t x_len) {
    if (row_bytes == 0 || row_bytes % 2 != 0) {
        return -1;
    }
    if (x_len != row_bytes / 2) {
        return -2;
    }
    return 0;
}

/* crates/tuckcore/src/kernels.rs:223-232. Pinned by the zero row
 * (kernels.rs:596-598), the error cases (kernels.rs:583-586), exact integer
 * cases (small integers are exact in f16 and their products and sums in f32),
 * an order-sensitive case that only the sequential sum from 0.0 satisfies,
 * and a float64 evaluation within the rounding bound. */
float q8o_dot_f16_x_f32(const uint8_t *row, size_t elems, const float *x) {
    float acc = 0.0f;
    for (size_t i = 0; i < elems; ++i) {
        float w = q8o_f16_to_f32(read_u16_le(row + 2 * i));
        float p = w * x[i];
        acc += p;
    }
    return acc;
}

void q8o_gemm_f16_f32(const uint8_t *w, size_t rows, size_t cols, const float *x, size_t batch,
                      float *y) {
    for (size_t b = 0; b < batch; ++b) {
        for (size_t r = 0; r < rows; ++r) {
            y[b * rows + r] = q8o_dot_f16_x_f32(w + r * cols * 2, cols, x + b * cols);
        }
    }
}

/* crates/tuckcore/src/kernels.rs:153-165 */
int q8o_validate_q8_0_q8_0(size_t row_bytes, size_t x_qs_blocks, size_t x_d_len) {
    if (row_bytes == 0 || row_bytes % Q8O_BLOCK_BYTES != 0) {
        return -1;
    }
    size_t blocks = row_bytes / Q8O_BLOCK_BYTES;
    if (x_qs_blocks != blocks || x_d_len != blocks) {
        return -2;
    }
    return 0;
}

/* ----------------------------------------------------------------- dots -- */

/* crates/tuckcore/src/kernels.rs:186-204: block_sum sequential from 0.0,
 * then acc += d * block_sum, sequential over blocks. Pinned by the ones case
 * (crates/metal/src/tests.rs:310-330), zeros (kernels.rs:590-599), integer
 * closed forms that are exact in f32, an f64 error bound, and a crafted case
 * on which this order and the dequantize-first order differ in the last bit. */
float q8o_dot_q8_0_x_f32(const uint8_t *row, size_t blocks, const float *x) {
    float acc = 0.0f;
    for (size_t b = 0; b < blocks; ++b) {
        const uint8_t *block = row + b * Q8O_BLOCK_BYTES;
        const float *xb = x + b * 32;
        float d = q8o_f16_to_f32(read_u16_le(block));
        float block_sum = 0.0f;
        for (int q = 0; q < 32; ++q) {
            float w = (float)(int8_t)block[2 + q];
            block_sum += w * xb[q];
        }
        acc += d * block_sum;
    }
    return acc;
}

/* crates/tuckcore/src/kernels.rs:206-221. The i32 block dot is exact; pinned
 * against an i64 brute force including the extremes q_w = -128, q_x = +-127. */
float q8o_dot_q8_0_q8_0(const uint8_t *row, size_t blocks, const int8_t *x_qs,
                        const float *x_d, int32_t *sumi_out) {
    float acc = 0.0f;
    for (size_t b = 0; b < blocks; ++b) {
        const uint8_t *block = row + b * Q8O_BLOCK_BYTES;
        const int8_t *qx = x_qs + b * 32;
        float d_w = q8o_f16_to_f32(read_u16_le(block));
        int32_t sumi = 0;
        for (int q = 0; q < 32; ++q) {
            sumi += (int32_t)(int8_t)block[2 + q] * (int32_t)qx[q];
        }
        if (sumi_out) {
            sumi_out[b] = sumi;
        }
        acc += (d_w * x_d[b]) * (float)sumi;
    }
    return acc;
}

/* ------------------------------------------------------------ row loops -- */

/* crates/tuckcore/src/forward.rs:703-735 */
void q8o_gemv_q8_0_f32(const uint8_t *w, size_t rows, size_t cols, const float *x,
                       float *y, int threads) {
    size_t blocks = cols / 32;
    size_t row_bytes = blocks * Q8O_BLOCK_BYTES;
    if (threads < 1) threads = 1;
#pragma omp parallel for schedule(static) num_threads(threads) if (threads > 1)
    for (long long r = 0; r < (long long)rows; ++r) {
        y[r] = q8o_dot_q8_0_x_f32(w + (size_t)r * row_bytes, blocks, x);
    }
}

/* crates/tuckcore/src/forward.rs:783-821 */
void q8o_gemv_q8_0_q8_0(const uint8_t *w, size_t rows, size_t cols, const float *x,
                        float *y, int threads) {
    size_t blocks = cols / 32;
    size_t row_bytes = blocks * Q8O_BLOCK_BYTES;
    int8_t qs[cols];
    float d[blocks];
    q8o_quantize_row_q8_0(x, cols, qs, d);
    if (threads < 1) threads = 1;
#pragma omp parallel for schedule(static) num_threads(threads) if (threads > 1)
    for (long long r = 0; r < (long long)rows; ++r) {
        y[r] = q8o_dot_q8_0_q8_0(w + (size_t)r * row_bytes, blocks, qs, d, NULL);
    }
}

void q8o_gemm_q8_0_f32(const uint8_t *w, size_t rows, size_t cols, const float *x,
                       size_t batch, float *y, int threads) {
    for (size_t b = 0; b < batch; ++b) {
        q8o_gemv_q8_0_f32(w, rows, cols, x + b * cols, y + b * rows, threads);
    }
}

void q8o_gemm_q8_0_q8_0(const uint8_t *w, size_t rows, size_t cols, const float *x,
                        size_t batch, float *y, int threads) {
    for (size_t b = 0; b < batch; ++b) {
        q8o_gemv_q8_0_q8_0(w, rows, cols, x + b * cols, y + b * rows, threads);
    }
}

/* crates/metal/src/tests.rs:100-116: acc += d * q * x, one element at a time
 * (Rust evaluates `d * q * xv` left to right: (d*q)*xv). */
void q8o_gemv_q8_0_f32_dequant_first(const uint8_t *w, size_t rows, size_t cols,
                                     const float *x, float *y) {
    size_t blocks = cols / 32;
    for (size_t r = 0; r < rows; ++r) {
        float acc = 0.0f;
        for (size_t b = 0; b < blocks; ++b) {
            const uint8_t *block = w + (r * blocks + b) * Q8O_BLOCK_BYTES;
            float d = q8o_f16_to_f32(read_u16_le(block));
            for (int l = 0; l < 32; ++l) {
                float q = (float)(int8_t)block[2 + l];
                float dq = d * q;
                acc += dq * x[b * 32 + (size_t)l];
            }
        }
        y[r] = acc;
    }
}

void q8o_gemv_q8_0_f64(const uint8_t *w, size_t rows, size_t cols, const float *x,
                       double *y) {
    size_t blocks = cols / 32;
    for (size_t r = 0; r < rows; ++r) {
        double acc = 0.0;
        for (size_t b = 0; b < blocks; ++b) {
            const uint8_t *block = w + (r * blocks + b) * Q8O_BLOCK_BYTES;
            double d = (double)q8o_f16_to_f32(read_u16_le(block));
            double bs = 0.0;
            for (int l = 0; l < 32; ++l) {
                bs += (double)(int8_t)block[2 + l] * (double)x[b * 32 + (size_t)l];
            }
            acc += d * bs;
        }
        y[r] = acc;
    }
}

/* ----------------------------------------------------------- generators -- */

/* crates/metal/src/tests.rs:30-40. Pinned against an independent
 * arbitrary-precision evaluation of xorshift64* in the tests. */
uint64_t q8o_rng_next(uint64_t *state) {
    uint64_t x = *state;
    x ^= x >> 12;
    x ^= x << 25;
    x ^= x >> 27;
    *state = x;
    return x * 0x2545F4914F6CDD1DULL;
}

/* crates/metal/src/tests.rs:119-149 */
void q8o_boundary_weights(size_t rows, size_t cols, uint64_t seed, uint8_t *out) {
    static const float scales[10] = {
        1.0f, -0.5f, 0x1p-12f, 65504.0f, -65504.0f, 5.96e-8f, 0.0f, -0.0f, 448.0f, 6e-5f,
    };
    size_t blocks = cols / 32;
    uint64_t rng = seed;
    uint8_t *p = out;
    for (size_t i = 0; i < rows * blocks; ++i) {
        float scale = scales[q8o_rng_next(&rng) % 10u];
        uint16_t h = q8o_f32_to_f16_bits(scale);
        *p++ = (uint8_t)(h & 0xff);
        *p++ = (uint8_t)(h >> 8);
        for (int l = 0; l < 32; ++l) {
            /* The match scrutinee draws once; the default arm draws again. */
            uint64_t sel = q8o_rng_next(&rng) % 8u;
            int8_t q;
            if (sel == 0) {
                q = -128;
            } else if (sel == 1) {
                q = 127;
            } else if (sel == 2) {
                q = 0;
            } else {
                q = (int8_t)(uint8_t)(q8o_rng_next(&rng) % 256u);
            }
            *p++ = (uint8_t)q;
        }
    }
}

/* crates/metal/src/tests.rs:151-162 */
void q8o_boundary_input(size_t n, uint64_t seed, float *out) {
    uint64_t rng = seed;
    for (size_t i = 0; i < n; ++i) {
        switch (i % 7) {
        case 0: out[i] = 0.0f; break;
        case 1: out[i] = -1.0f; break;
        case 2: out[i] = 1e3f; break;
        case 3: out[i] = -1e3f; break;
        default:
            out[i] = ((float)(q8o_rng_next(&rng) % 20001u) - 10000.0f) / 1000.0f;
            break;
        }
    }
}

/* crates/tuckcore/src/kernels.rs:434-443 */
float q8o_krng_next_f32(uint64_t *state, float scale) {
    uint64_t s = *state;
    s ^= s >> 12;
    s ^= s << 25;
    s ^= s >> 27;
    *state = s;
    float u = (float)((s * 0x2545F4914F6CDD1DULL) >> 40);
    return ((u / (float)(1ull << 24)) * 2.0f - 1.0f) * scale;
}

/* crates/tuckcore/src/kernels.rs:445-456 */
void q8o_random_q8_0_row(uint64_t *state, size_t blocks, uint8_t *out) {
    uint8_t *p = out;
    for (size_t b = 0; b < blocks; ++b) {
        float d = fabsf(q8o_krng_next_f32(state, 0.05f)) + 1e-4f;
        uint16_t h = q8o_f32_to_f16_bits(d);
        *p++ = (uint8_t)(h & 0xff);
        *p++ = (uint8_t)(h >> 8);
        for (int i = 0; i < 32; ++i) {
            float r = roundf(q8o_krng_next_f32(state, 127.0f)); /* f32::round: half away */
            if (r < -127.0f) r = -127.0f;
            if (r > 127.0f) r = 127.0f;
            *p++ = (uint8_t)(int8_t)r;
        }
    }
}

/* ---- the small f32 operators either side of a product -------------------- */

/* crates/tuckcore/src/forward.rs:917-927: sequential f32 sum of squares,
 * inv = 1 / sqrt(ss / n + eps), y = (x * inv) * w. */
void q8o_rmsnorm(const float *x, const float *w, size_t n, float eps, float *y) {
    float ss = 0.0f;
    for (size_t i = 0; i < n; ++i) {
        ss += x[i] * x[i];
    }
    const float inv = 1.0f / sqrtf(ss / (float)n + eps);
    for (size_t i = 0; i < n; ++i) {
        y[i] = x[i] * inv * w[i];
    }
}

/* crates/tuckcore/src/forward.rs:906-908 and the gate of
 * crates/metal/src/tests.rs:648: (g / (1 + exp(-g))) * up. */
void q8o_silu_mul(const float *gate, const float *up, size_t n, float *out) {
    for (size_t i = 0; i < n; ++i) {
        const float g = gate[i];
        out[i] = (g / (1.0f + expf(-g))) * up[i];
    }
}

/* native/metal/kernels.metal:382-396 (no CPU twin in the reference): ggml's
 * tanh GELU, 0.5 x (1 + tanh(sqrt(2/pi) x (1 + 0.044715 x^2))) * up. */
void q8o_gelu_tanh_mul(const float *gate, const float *up, size_t n, float *out) {
    for (size_t i = 0; i < n; ++i) {
        const float x = gate[i];
        const float inner = 0.7978845608028654f * x * (1.0f + 0.044715f * x * x);
        out[i] = 0.5f * x * (1.0f + tanhf(inner)) * up[i];
    }
}

/* native/metal/kernels.metal:26-36: y += alpha * a (multiply, then add). */
void q8o_axpy(const float *a, float alpha, size_t n, float *y) {
    for (size_t i = 0; i < n; ++i) {
        const float p = alpha * a[i];
        y[i] = y[i] + p;
    }
}

/* native/metal/kernels.metal:14-24 */
void q8o_scale(const float *x, float factor, size_t n, float *y) {
    for (size_t i = 0; i < n; ++i) {
        y[i] = x[i] * factor;
    }
}

/* crates/backend/src/sampling.rs:69-83: NaN skipped, strict >, so ties go to
 * the lowest index; 0xFFFFFFFF when every entry is NaN
 * (crates/metal/src/tests.rs:1257-1270). */
uint32_t q8o_argmax(const float *x, size_t n) {
    int have = 0;
    size_t bi = 0;
    float bv = 0.0f;
    for (size_t i = 0; i < n; ++i) {
        const float v = x[i];
        if (v != v) {
            continue;
        }
        if (!have || v > bv) {
            have = 1;
            bi = i;
            bv = v;
        }
    }
    return have ? (uint32_t)bi : 0xFFFFFFFFu;
}
