// Shared device helpers for the Q8_0 kernels (gfx950, wave64).
//
// Two weight layouts are understood everywhere:
//   RAW    — GGUF bytes: blocks of 34 bytes ([f16 d][i8 qs; 32]), rows
//            contiguous (crates/manifest/src/ggml.rs:47).
//   PACKED — the sealed device layout: int8 quants [rows][cols] first, then
//            f16 scales [rows][cols/32]; same total byte count.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include "q8_plan.hpp"

// Launch with an optional stop event attached to the dispatch itself: the
// event completes with the kernel and costs no extra packet on the stream
// (a separate hipEventRecord after each launch measured +3 us per launch).
// Without an event it is the plain launch, the form stream capture records.
#define Q8_LAUNCH(kernel, grid, block, lds, stream, stop_event, ...)                              \
    do {                                                                                          \
        if ((stop_event) == nullptr) {                                                            \
            hipLaunchKernelGGL(kernel, grid, block, lds, stream, __VA_ARGS__);                    \
        } else {                                                                                  \
            hipExtLaunchKernelGGL(kernel, grid, block, lds, stream, nullptr, stop_event, 0,       \
                                  __VA_ARGS__);                                                   \
        }                                                                                         \
    } while (0)

namespace q8 {

constexpr int WAVE = 64;

enum Layout : int { RAW = 0, PACKED = 1 };

// binary16 -> binary32. v_cvt_f32_f16 is exact for every encoding, subnormals
// included: kernels run with FP16 denormals enabled (the HSA default mode).
__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

// An f32 as the exact sum of three bf16 numbers: its 24-bit significand cut into
// 8 + 8 + 8 bits (h = trunc(x), m = trunc(x - h), l = x - h - m; both
// subtractions are exact). An infinity or NaN goes into h whole, m = l = 0.
__device__ __forceinline__ void split3_bf16(float x, uint32_t &h, uint32_t &m, uint32_t &l) {
    const uint32_t xb = __builtin_bit_cast(uint32_t, x);
    const bool finite = (xb & 0x7f800000u) != 0x7f800000u;
    // (a NaN whose payload sits in the low 16 bits only must stay a NaN)
    const uint32_t hb = finite ? xb & 0xffff0000u : xb | ((xb & 0xffffu) ? 0x00400000u : 0u);
    const float r1 = finite ? x - __builtin_bit_cast(float, hb) : 0.0f; // exact
    const uint32_t mb = __builtin_bit_cast(uint32_t, r1) & 0xffff0000u;
    const float r2 = r1 - __builtin_bit_cast(float, mb); // exact, at most 8 significant bits
    h = hb >> 16;
    m = mb >> 16;
    l = __builtin_bit_cast(uint32_t, r2) >> 16;
}

// act(g) * u of the gated activations fused into product kernels: silu (kind 0) or
// ggml's tanh GELU (kind 1), the expressions of silu_mul_kernel / gelu_tanh_mul_kernel.
__device__ __forceinline__ float glu_act(float g, float u, uint32_t kind) {
    if (kind == 0u) {
        const float s = g / (1.0f + expf(-g));
        return s * u;
    }
    const float inner = 0.7978845608028654f * g * (1.0f + 0.044715f * g * g);
    return 0.5f * g * (1.0f + tanhf(inner)) * u;
}

// Where the pieces of element (token t, column k) of a [batch][cols] matrix live
// in its split form [cols / 32][3][batch][32] (bf16 units): the h piece at the
// returned index, m and l each batch * 32 further on.
__device__ __forceinline__ size_t split_index(uint32_t batch, uint32_t t, uint32_t k) {
    return ((size_t)(k >> 5) * 3u * batch + t) * 32u + (k & 31u);
}

// One element into the split form (for the operators that write a matrix product's
// activations and its split form in one pass).
__device__ __forceinline__ void split_store(uint16_t *xs, uint32_t batch, uint32_t t, uint32_t k,
                                            float v) {
    uint32_t h, m, l;
    split3_bf16(v, h, m, l);
    uint16_t *dst = xs + split_index(batch, t, k);
    const size_t piece = (size_t)batch * 32u;
    dst[0] = (uint16_t)h;
    dst[piece] = (uint16_t)m;
    dst[2u * piece] = (uint16_t)l;
}

// binary32 -> binary16 bits with the rounding of
// crates/tuckcore/src/tensor.rs:145-178: round to nearest even, overflow and
// NaN both become +-inf, magnitudes below 2^-25 become +-0.
__device__ __forceinline__ uint32_t f32_to_f16_bits(float value) {
    uint32_t bits = __float_as_uint(value);
    uint32_t sign = (bits >> 16) & 0x8000u;
    int32_t exp = (int32_t)((bits >> 23) & 0xffu) - 127 + 15;
    uint32_t mant = bits & 0x7fffffu;
    if (exp >= 0x1f) {
        return sign | 0x7c00u;
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
        if (rem > halfway || (rem == halfway && (half & 1u))) {
            half += 1u;
        }
        return sign | half;
    }
    uint32_t rounded = mant + 0x0fffu + ((mant >> 13) & 1u);
    if (rounded & 0x800000u) {
        exp += 1;
        if (exp >= 0x1f) {
            return sign | 0x7c00u;
        }
        return sign | ((uint32_t)exp << 10);
    }
    return sign | ((uint32_t)exp << 10) | (rounded >> 13);
}

// Signed byte `i` (0..3) of a dword as float.
__device__ __forceinline__ float sbyte_to_float(uint32_t w, int i) {
    return (float)(int)(int8_t)(w >> (8 * i));
}

// ---- streaming loads ------------------------------------------------------
//
// Weights of a GEMV are read exactly once per launch. Loading them with the
// non-temporal hint keeps them from displacing reusable lines (activations,
// other kernels' data) in the L2 / Infinity Cache and is measurably faster
// for pure streaming on MI355X (6.8 TB/s against 6.2 TB/s with plain loads
// over the same 633 MB).
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

// 8 signed bytes (two dwords) -> 8 bf16: the conversion to f32 is exact and
// its upper half is the bf16.
__device__ __forceinline__ bf16x8_t sbytes_to_bf16x8(uint32_t lo, uint32_t hi) {
    uint32_t p[4];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const uint32_t f0 = __builtin_bit_cast(uint32_t, sbyte_to_float(lo, 2 * i));
        const uint32_t f1 = __builtin_bit_cast(uint32_t, sbyte_to_float(lo, 2 * i + 1));
        p[i] = __builtin_amdgcn_perm(f1, f0, 0x07060302u);
        const uint32_t g0 = __builtin_bit_cast(uint32_t, sbyte_to_float(hi, 2 * i));
        const uint32_t g1 = __builtin_bit_cast(uint32_t, sbyte_to_float(hi, 2 * i + 1));
        p[2 + i] = __builtin_amdgcn_perm(g1, g0, 0x07060302u);
    }
    const u32x4 v = {p[0], p[1], p[2], p[3]};
    return __builtin_bit_cast(bf16x8_t, v);
}


template <bool NT, class T> __device__ __forceinline__ T load_maybe_nt(const T *p) {
    if constexpr (NT) {
        return __builtin_nontemporal_load(p);
    } else {
        return *p;
    }
}

// ---- weight views -------------------------------------------------------

template <int L> struct WView;

template <> struct WView<PACKED> {
    const uint8_t *q;   // [rows][cols] int8
    const uint16_t *s;  // [rows][blocks] f16 bits
    uint32_t cols, blocks;
    __device__ __forceinline__ WView(const uint8_t *base, uint32_t rows, uint32_t cols_)
        : q(base), s((const uint16_t *)(base + (size_t)rows * cols_)), cols(cols_),
          blocks(cols_ / 32u) {}
    // NB consecutive quants of `row` starting at column `col` (col % NB == 0,
    // the piece lies inside one block) into NB/4 dwords (low bytes first).
    template <int NB, bool NT = false>
    __device__ __forceinline__ void load_quants(uint32_t row, uint32_t col, uint32_t *out) const {
        const uint8_t *p = q + (size_t)row * cols + col;
        if constexpr (NB == 16) {
            const u32x4 v = load_maybe_nt<NT>((const u32x4 *)p);
            out[0] = v.x; out[1] = v.y; out[2] = v.z; out[3] = v.w;
        } else if constexpr (NB == 8) {
            const u32x2 v = load_maybe_nt<NT>((const u32x2 *)p);
            out[0] = v.x; out[1] = v.y;
        } else if constexpr (NB == 4) {
            out[0] = load_maybe_nt<NT>((const uint32_t *)p);
        } else if constexpr (NB == 2) {
            out[0] = load_maybe_nt<NT>((const uint16_t *)p);
        } else {
            out[0] = load_maybe_nt<NT>(p);
        }
    }
    template <bool NT = false>
    __device__ __forceinline__ uint32_t scale_bits(uint32_t row, uint32_t block) const {
        return load_maybe_nt<NT>(s + (size_t)row * blocks + block);
    }
};

template <> struct WView<RAW> {
    const uint8_t *base;
    uint32_t blocks;
    size_t row_bytes;
    __device__ __forceinline__ WView(const uint8_t *base_, uint32_t /*rows*/, uint32_t cols_)
        : base(base_), blocks(cols_ / 32u), row_bytes((size_t)(cols_ / 32u) * 34u) {}
    template <int NB, bool NT = false>
    __device__ __forceinline__ void load_quants(uint32_t row, uint32_t col, uint32_t *out) const {
        // 34-byte blocks leave the quants only 2-byte aligned.
        const uint8_t *p = base + (size_t)row * row_bytes + (size_t)(col >> 5) * 34u + 2u + (col & 31u);
        if constexpr (NB >= 2) {
            const uint16_t *h = (const uint16_t *)p;
#pragma unroll
            for (int i = 0; i < NB / 4; ++i) {
                out[i] = (uint32_t)h[2 * i] | ((uint32_t)h[2 * i + 1] << 16);
            }
            if constexpr (NB == 2) {
                out[0] = h[0];
            }
        } else {
            out[0] = *p;
        }
    }
    template <bool NT = false>
    __device__ __forceinline__ uint32_t scale_bits(uint32_t row, uint32_t block) const {
        return *(const uint16_t *)(base + (size_t)row * row_bytes + (size_t)block * 34u);
    }
};

// Sum over the 64 lanes of a wave; every lane returns the same bits. The
// pairing (xor 32, 16, 8, 4, 2, 1) is fixed: all kernels that must agree
// bit for bit reduce through this one function.
__device__ __forceinline__ float wave_sum(float v) {
    v += __shfl_xor(v, 32, WAVE);
    v += __shfl_xor(v, 16, WAVE);
    v += __shfl_xor(v, 8, WAVE);
    v += __shfl_xor(v, 4, WAVE);
    v += __shfl_xor(v, 2, WAVE);
    v += __shfl_xor(v, 1, WAVE);
    return v;
}

} // namespace q8
