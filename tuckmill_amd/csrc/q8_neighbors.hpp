// The small f32 operators either side of a Q8_0 product in a decode or prefill
// step: RMSNorm before the projections, the gated activations and the residual
// update after them, greedy argmax after the vocabulary projection.
// Reference kernels: native/metal/kernels.metal:14-36 (scale, axpy), :142-226
// (argmax), :341-362 (rmsnorm), :382-406 (gelu_tanh_mul, silu_mul); CPU
// definitions: crates/tuckcore/src/forward.rs:906-927,
// crates/backend/src/sampling.rs:69-83.
//
// All of them move a few KB to a few hundred KB: on this part they are bound by
// launch latency, not by HBM, so each is one plain kernel (argmax: two) meant to
// be recorded inside a dispatch group.
#pragma once

#include "q8_gemv.hpp"

namespace q8 {

// The element-wise kernels walk n elements in strides of the whole grid: one
// step for every size in practice, and no limit from the 2^32 threads a launch
// may hold (the host caps the grid, tm_hip.cpp::strided_blocks_of).

// y[i] = x[i] * factor
__global__ __launch_bounds__(256) void scale_kernel(const float *x, float *y, float factor,
                                                    uint32_t n) {
    for (uint64_t i = blockIdx.x * 256u + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256u) {
        y[i] = x[i] * factor;
    }
}

// y[i] = y[i] + alpha * a[i]   (multiply, then add: no contraction)
__global__ __launch_bounds__(256) void axpy_kernel(const float *a, float *y, float alpha,
                                                   uint32_t n) {
    for (uint64_t i = blockIdx.x * 256u + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256u) {
        const float p = __fmul_rn(alpha, a[i]);
        y[i] = __fadd_rn(y[i], p);
    }
}

// y[i] = (float)x[i], x in IEEE binary16: exact for every encoding (a NaN stays a
// NaN of the same sign). Eight elements per lane while eight are left (16 bytes in,
// 32 out), single elements behind them.
__global__ __launch_bounds__(256) void cast_f16_f32_kernel(const uint16_t *x, float *y, uint32_t n) {
    const uint32_t i = (blockIdx.x * 256u + threadIdx.x) * 8u;
    if (i < n && n - i >= 8u) {
        const u32x4 v = *(const u32x4 *)(x + i);
        f32x4 lo, hi;
        lo[0] = f16_bits_to_f32(v[0] & 0xffffu);
        lo[1] = f16_bits_to_f32(v[0] >> 16);
        lo[2] = f16_bits_to_f32(v[1] & 0xffffu);
        lo[3] = f16_bits_to_f32(v[1] >> 16);
        hi[0] = f16_bits_to_f32(v[2] & 0xffffu);
        hi[1] = f16_bits_to_f32(v[2] >> 16);
        hi[2] = f16_bits_to_f32(v[3] & 0xffffu);
        hi[3] = f16_bits_to_f32(v[3] >> 16);
        *(f32x4 *)(y + i) = lo;
        *(f32x4 *)(y + i + 4u) = hi;
    } else {
        for (uint32_t k = i; k < n; ++k) {
            y[k] = f16_bits_to_f32(x[k]);
        }
    }
}

// binary32 -> binary16 for the cast operator: round to nearest even, overflow to
// infinity, magnitudes below 2^-25 to a signed zero - the rounding of
// crates/tuckcore/src/tensor.rs:145-178 on every number - and a NaN to the quiet
// NaN of its sign, as a conversion in hardware gives (native/metal/kernels.metal:50-58;
// tensor.rs:150-153 would make it an infinity).
__device__ __forceinline__ uint32_t cast_to_f16_bits(float v) {
    const uint32_t bits = __float_as_uint(v);
    if ((bits & 0x7fffffffu) > 0x7f800000u) {
        return ((bits >> 16) & 0x8000u) | 0x7e00u;
    }
    return f32_to_f16_bits(v);
}

// y[i] = (half)x[i]. Eight elements per lane while eight are left.
__global__ __launch_bounds__(256) void cast_f32_f16_kernel(const float *x, uint16_t *y, uint32_t n) {
    const uint32_t i = (blockIdx.x * 256u + threadIdx.x) * 8u;
    if (i < n && n - i >= 8u) {
        const f32x4 lo = *(const f32x4 *)(x + i);
        const f32x4 hi = *(const f32x4 *)(x + i + 4u);
        u32x4 v;
        v[0] = cast_to_f16_bits(lo[0]) | (cast_to_f16_bits(lo[1]) << 16);
        v[1] = cast_to_f16_bits(lo[2]) | (cast_to_f16_bits(lo[3]) << 16);
        v[2] = cast_to_f16_bits(hi[0]) | (cast_to_f16_bits(hi[1]) << 16);
        v[3] = cast_to_f16_bits(hi[2]) | (cast_to_f16_bits(hi[3]) << 16);
        *(u32x4 *)(y + i) = v;
    } else {
        for (uint32_t k = i; k < n; ++k) {
            y[k] = (uint16_t)cast_to_f16_bits(x[k]);
        }
    }
}

// The three operators below can write, next to their f32 result, its split form
// for the bf16 matrix cores (q8_gemm_bf16x3.hpp) when the product that reads
// the result follows directly: `xs` non-null, the result taken as a
// [n / cols][cols] matrix. That saves the product's own split pass, a dependent
// launch of about 5 us.

// out[i] = silu(gate[i]) * up[i],  silu(g) = g / (1 + exp(-g))
__global__ __launch_bounds__(256) void silu_mul_kernel(const float *gate, const float *up,
                                                       float *out, uint32_t n, uint16_t *xs,
                                                       uint32_t cols) {
    for (uint64_t e = blockIdx.x * 256u + threadIdx.x; e < n; e += (uint64_t)gridDim.x * 256u) {
        const uint32_t i = (uint32_t)e;
        const float g = gate[i];
        const float s = g / (1.0f + expf(-g));
        const float v = s * up[i];
        out[i] = v;
        if (xs != nullptr) {
            split_store(xs, n / cols, i / cols, i % cols, v);
        }
    }
}

// out[i] = gelu_tanh(gate[i]) * up[i], ggml's tanh form
// 0.5 x (1 + tanh(sqrt(2/pi) x (1 + 0.044715 x^2))), evaluated in the order of
// kernels.metal:391-395.
__global__ __launch_bounds__(256) void gelu_tanh_mul_kernel(const float *gate, const float *up,
                                                            float *out, uint32_t n, uint16_t *xs,
                                                            uint32_t cols) {
    for (uint64_t e = blockIdx.x * 256u + threadIdx.x; e < n; e += (uint64_t)gridDim.x * 256u) {
        const uint32_t i = (uint32_t)e;
        const float x = gate[i];
        const float inner = 0.7978845608028654f * x * (1.0f + 0.044715f * x * x);
        const float v = 0.5f * x * (1.0f + tanhf(inner)) * up[i];
        out[i] = v;
        if (xs != nullptr) {
            split_store(xs, n / cols, i / cols, i % cols, v);
        }
    }
}

// One wave per row (RMSNORM_ROWS rows per workgroup: one, so that the few hundred
// rows of a prefill chunk spread over the whole chip): y = (x * inv) * w with
// inv = 1 / sqrt(mean(x^2) + eps). The sum of squares is q8::row_sumsq's: fixed
// order, not the CPU's sequential one, hence tolerance-qualified like the
// reference's own GPU kernel; the GEMV kernel's fused form computes the same
// bits. In place (x == y) is safe: a lane rereads only what it writes itself.

// `add` non-null: the residual update x += alpha * add of the same rows comes
// first (axpy_kernel's operations: multiply, then add; x is written back), for
// the pair "h += alpha * t; xn = rmsnorm(h)" between two layers' products. Every
// lane then updates, squares and normalises its own elements only (row_sumsq's
// runs of 16), so the row never passes from one lane to another through memory.
__global__ __launch_bounds__(64 * RMSNORM_ROWS) void rmsnorm_kernel(float *x, const float *weight,
                                                                    float *y, uint32_t rows,
                                                                    uint32_t cols, float eps,
                                                                    uint16_t *xs, const float *add,
                                                                    float alpha) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t row = blockIdx.x * RMSNORM_ROWS + (threadIdx.x >> 6);
    if (row >= rows) {
        return;
    }
    float *xr = x + (size_t)row * cols;
    float *yr = y + (size_t)row * cols;
    const bool vec = (cols & 3u) == 0u && ((((uintptr_t)x) | ((uintptr_t)y) | ((uintptr_t)weight) |
                                            ((uintptr_t)add)) & 15u) == 0u;
    if (add != nullptr && vec && cols <= 1024u) {
        // One run of 16 per lane: the updated values stay in registers for the sum
        // of squares (row_sumsq's order: the lane's elements in turn, then
        // q8::wave_sum) and for the normalisation.
        const float *ar = add + (size_t)row * cols;
        const uint32_t e0 = lane * 16u;
        const uint32_t mine = e0 >= cols ? 0u : (cols - e0 < 16u ? cols - e0 : 16u); // a multiple of 4
        float hv[16];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if ((uint32_t)(4 * q) < mine) {
                const float4 h = *(const float4 *)(xr + e0 + 4 * q);
                const float4 t = *(const float4 *)(ar + e0 + 4 * q);
                hv[4 * q] = __fadd_rn(h.x, __fmul_rn(alpha, t.x));
                hv[4 * q + 1] = __fadd_rn(h.y, __fmul_rn(alpha, t.y));
                hv[4 * q + 2] = __fadd_rn(h.z, __fmul_rn(alpha, t.z));
                hv[4 * q + 3] = __fadd_rn(h.w, __fmul_rn(alpha, t.w));
                *(float4 *)(xr + e0 + 4 * q) = make_float4(hv[4 * q], hv[4 * q + 1], hv[4 * q + 2], hv[4 * q + 3]);
            } else {
                hv[4 * q] = hv[4 * q + 1] = hv[4 * q + 2] = hv[4 * q + 3] = 0.0f;
            }
        }
        float acc = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            if ((uint32_t)i < mine) {
                acc += hv[i] * hv[i];
            }
        }
        const float inv = 1.0f / sqrtf(wave_sum(acc) / (float)cols + eps);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if ((uint32_t)(4 * q) < mine) {
                const uint32_t e = e0 + 4u * q;
                const float4 wv = *(const float4 *)(weight + e);
                const float4 v = make_float4(hv[4 * q] * inv * wv.x, hv[4 * q + 1] * inv * wv.y,
                                             hv[4 * q + 2] * inv * wv.z, hv[4 * q + 3] * inv * wv.w);
                *(float4 *)(yr + e) = v;
                if (xs != nullptr) {
                    const float in[4] = {v.x, v.y, v.z, v.w};
                    uint32_t h[4], m[4], l[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        split3_bf16(in[i], h[i], m[i], l[i]);
                    }
                    uint16_t *dst = xs + split_index(rows, row, e);
                    const size_t piece = (size_t)rows * 32u;
                    *(uint2 *)dst = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
                    *(uint2 *)(dst + piece) = make_uint2(m[0] | (m[1] << 16), m[2] | (m[3] << 16));
                    *(uint2 *)(dst + 2u * piece) = make_uint2(l[0] | (l[1] << 16), l[2] | (l[3] << 16));
                }
            }
        }
        return;
    }
    if (add != nullptr) {
        const float *ar = add + (size_t)row * cols;
        for (uint32_t e0 = lane * 16u; e0 < cols; e0 += 1024u) {
            const uint32_t e1 = e0 + 16u < cols ? e0 + 16u : cols;
            if (vec) {
                for (uint32_t e = e0; e < e1; e += 4u) {
                    const float4 h = *(const float4 *)(xr + e);
                    const float4 t = *(const float4 *)(ar + e);
                    *(float4 *)(xr + e) = make_float4(
                        __fadd_rn(h.x, __fmul_rn(alpha, t.x)), __fadd_rn(h.y, __fmul_rn(alpha, t.y)),
                        __fadd_rn(h.z, __fmul_rn(alpha, t.z)), __fadd_rn(h.w, __fmul_rn(alpha, t.w)));
                }
            } else {
                for (uint32_t e = e0; e < e1; ++e) {
                    xr[e] = __fadd_rn(xr[e], __fmul_rn(alpha, ar[e]));
                }
            }
        }
    }
    const float sumsq = vec ? row_sumsq<true>(xr, cols, lane) : row_sumsq<false>(xr, cols, lane);
    const float inv = 1.0f / sqrtf(sumsq / (float)cols + eps);
    // elements e .. e+3 of the row: normalise, store, split
    auto four_of = [&](uint32_t e, const float4 xv, const float4 wv) {
        const float4 v = make_float4(xv.x * inv * wv.x, xv.y * inv * wv.y, xv.z * inv * wv.z,
                                     xv.w * inv * wv.w);
        *(float4 *)(yr + e) = v;
        if (xs != nullptr) {
            const float in[4] = {v.x, v.y, v.z, v.w};
            uint32_t h[4], m[4], l[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                split3_bf16(in[i], h[i], m[i], l[i]);
            }
            uint16_t *dst = xs + split_index(rows, row, e); // the four share a block of 32
            const size_t piece = (size_t)rows * 32u;
            *(uint2 *)dst = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
            *(uint2 *)(dst + piece) = make_uint2(m[0] | (m[1] << 16), m[2] | (m[3] << 16));
            *(uint2 *)(dst + 2u * piece) = make_uint2(l[0] | (l[1] << 16), l[2] | (l[3] << 16));
        }
    };
    auto four = [&](uint32_t e) {
        four_of(e, *(const float4 *)(xr + e), *(const float4 *)(weight + e));
    };
    if (add != nullptr) {
        for (uint32_t e0 = lane * 16u; e0 < cols; e0 += 1024u) {
            const uint32_t e1 = e0 + 16u < cols ? e0 + 16u : cols;
            if (vec) {
                for (uint32_t e = e0; e < e1; e += 4u) {
                    four(e);
                }
            } else {
                for (uint32_t e = e0; e < e1; ++e) {
                    const float v = xr[e] * inv * weight[e];
                    yr[e] = v;
                    if (xs != nullptr) {
                        split_store(xs, rows, row, e, v);
                    }
                }
            }
        }
        return;
    }
    if (vec) {
        // four consecutive elements per lane, a wave's 1 KiB in one piece; the
        // loads of four such pieces are requested together (a lane reads and
        // writes its own elements only, in place too)
        for (uint32_t e = lane * 4u; e < cols; e += 1024u) {
            float4 xv[4], wv[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t ee = e + 256u * (uint32_t)j;
                if (ee < cols) {
                    xv[j] = *(const float4 *)(xr + ee);
                    wv[j] = *(const float4 *)(weight + ee);
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t ee = e + 256u * (uint32_t)j;
                if (ee < cols) {
                    four_of(ee, xv[j], wv[j]);
                }
            }
        }
        return;
    }
    for (uint32_t e = lane; e < cols; e += 64u) {
        const float v = xr[e] * inv * weight[e];
        yr[e] = v;
        if (xs != nullptr) {
            split_store(xs, rows, row, e, v);
        }
    }
}

// Greedy argmax, the CPU rule: NaN entries are skipped, the largest value
// wins, ties go to the lowest index; ARGMAX_NONE when every entry is NaN.
// "a is better than b" is a strict total order on (value, index) pairs, so any
// reduction tree returns the sequential scan's answer.
constexpr uint32_t ARGMAX_NONE = 0xffffffffu;

__device__ __forceinline__ bool argmax_better(float av, uint32_t ai, float bv, uint32_t bi) {
    if (ai == ARGMAX_NONE) {
        return false;
    }
    if (bi == ARGMAX_NONE) {
        return true;
    }
    return av > bv || (av == bv && ai < bi);
}

__device__ __forceinline__ void argmax_workgroup(float &v, uint32_t &i, float *tv, uint32_t *ti) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(v, off, WAVE);
        const uint32_t oi = (uint32_t)__shfl_xor((int)i, off, WAVE);
        if (argmax_better(ov, oi, v, i)) {
            v = ov;
            i = oi;
        }
    }
    const uint32_t wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63u) == 0u) {
        tv[wave] = v;
        ti[wave] = i;
    }
    __syncthreads();
    v = tv[0];
    i = ti[0];
#pragma unroll
    for (int w = 1; w < 4; ++w) {
        if (argmax_better(tv[w], ti[w], v, i)) {
            v = tv[w];
            i = ti[w];
        }
    }
}

__global__ __launch_bounds__(256) void argmax_partial_kernel(const float *x, float *part_v,
                                                             uint32_t *part_i, uint32_t n) {
    __shared__ float tv[4];
    __shared__ uint32_t ti[4];
    float v = -__builtin_inff();
    uint32_t i = ARGMAX_NONE;
    // (the rule is a total order on (value, index): any partition of the elements
    // gives the same winner; four per lane and step, so that a vocabulary takes
    // three or four dependent loads per lane, not sixteen)
    const uint32_t n4 = n & ~3u;
    for (uint32_t k = (blockIdx.x * 256u + threadIdx.x) * 4u; k < n4; k += ARGMAX_GROUPS * 1024u) {
        const f32x4 q = *(const f32x4 *)(x + k);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float xv = q[e];
            if (xv == xv && argmax_better(xv, k + (uint32_t)e, v, i)) {
                v = xv;
                i = k + (uint32_t)e;
            }
        }
    }
    if (blockIdx.x == 0u && threadIdx.x < n - n4) {
        const uint32_t k = n4 + threadIdx.x;
        const float xv = x[k];
        if (xv == xv && argmax_better(xv, k, v, i)) {
            v = xv;
            i = k;
        }
    }
    argmax_workgroup(v, i, tv, ti);
    if (threadIdx.x == 0u) {
        part_v[blockIdx.x] = v;
        part_i[blockIdx.x] = i;
    }
}

__global__ __launch_bounds__(256) void argmax_final_kernel(const float *part_v,
                                                           const uint32_t *part_i, uint32_t *out,
                                                           uint32_t out_index) {
    __shared__ float tv[4];
    __shared__ uint32_t ti[4];
    float v = threadIdx.x < ARGMAX_GROUPS ? part_v[threadIdx.x] : -__builtin_inff();
    uint32_t i = threadIdx.x < ARGMAX_GROUPS ? part_i[threadIdx.x] : ARGMAX_NONE;
    argmax_workgroup(v, i, tv, ti);
    if (threadIdx.x == 0u) {
        out[out_index] = i;
    }
}

} // namespace q8
