// F16-weight twins of the Q8_0 products: y[b][r] = sum_i f32(w[r][i]) * x[b][i]
// for 1 <= batch <= 32 (native/metal/kernels.metal:296-315 tm_f16_gemv,
// :638-668 tm_f16_gemm), single-row conversion (:409-419) and the indirect row
// lookup (:257-269). They serve F16-weight artifacts (model fixtures, F16 twins
// of quantized tensors), not the headline decode path, but are HBM-bound just
// the same: 2 bytes per weight, streamed once per group of TB tokens (up to 8).
//
// Summation order (fixed; tolerance-qualified against the CPU's sequential sum
// like the reference's own kernel): a lane owns 8 consecutive columns of every
// 512-column chunk, adds their unfused products w*x in column order onto its
// accumulator, chunk after chunk; the 64 lane sums go through q8::reduce_store's
// butterfly. Token b of a batch gets exactly the arithmetic of a one-token
// call on x[b], so the batched form is bit-identical to the GEMV, as the
// reference states for its pair. Any cols > 0 is accepted: rows whose length
// is not a multiple of 8 are not 16-byte aligned and take the element loop.
#pragma once

#include "q8_gemv.hpp"

namespace q8 {

typedef float f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

__device__ __forceinline__ float f16_lo(uint32_t v) { return f16_bits_to_f32(v & 0xffffu); }
__device__ __forceinline__ float f16_hi(uint32_t v) { return f16_bits_to_f32(v >> 16); }

// VEC: cols % 8 == 0 for every product of the launch (16-byte loads of 8
// halves per lane). Like the Q8_0 kernels it is a list kernel: independent
// products of a dispatch group share one launch, a wave finds its product by
// its tile number. A wave owns `rows_per_tile` rows (a multiple of 8), 8 rows
// per pass, TB tokens per sweep over its rows; the weights of the next
// (pass, chunk) step are requested before the current one is used.
template <int TB, bool VEC>
__global__ __launch_bounds__(256) void f16_gemm_list_kernel(const GemvArgs args) {
    constexpr int R = 8;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t tile = blockIdx.x * 4u + wave;
    if (tile >= args.total_tiles) {
        return;
    }
    uint32_t lo = 0, hi = args.n;
    while (hi - lo > 1u) {
        const uint32_t mid = (lo + hi) >> 1;
        if (args.d[mid].tile_begin <= tile) {
            lo = mid;
        } else {
            hi = mid;
        }
    }
    const GemvDesc &d = args.d[lo];
    const uint16_t *__restrict__ w = (const uint16_t *)d.w;
    const float *__restrict__ x = d.x;
    float *__restrict__ y = d.y;
    const uint32_t rows = d.rows, cols = d.cols, batch = d.batch;
    const uint32_t row_first = (tile - d.tile_begin) * d.rows_per_tile;
    const uint32_t row_end = rows - row_first < d.rows_per_tile ? rows : row_first + d.rows_per_tile;
    const uint32_t nchunks = (cols + 511u) >> 9;
    const uint32_t passes = (row_end - row_first + R - 1) / R;
    const uint32_t nsteps = passes * nchunks;

    auto load_step = [&](uint32_t p, uint32_t c, u32x4 (&q)[R]) {
        uint32_t col = (c << 9) + lane * 8u;
        if (col >= cols) {
            col = 0; // lanes past the row's end read valid memory and use nothing of it
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            uint32_t row = row_first + p * R + r;
            if (row >= row_end) {
                row = row_end - 1u;
            }
            const uint16_t *src = w + (size_t)row * cols + col;
            if constexpr (VEC) {
                q[r] = __builtin_nontemporal_load((const u32x4 *)src);
            } else {
                // up to 8 elements, the last chunk of a row may hold fewer
                uint32_t h[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const uint32_t ci = (c << 9) + lane * 8u + i;
                    h[i] = ci < cols ? (uint32_t)w[(size_t)row * cols + ci] : 0u;
                }
                q[r] = u32x4{h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16),
                             h[6] | (h[7] << 16)};
            }
        }
    };

    for (uint32_t t0 = 0; t0 < batch; t0 += TB) {
        uint32_t tok[TB];
#pragma unroll
        for (int t = 0; t < TB; ++t) {
            tok[t] = (t0 + t < batch) ? t0 + t : batch - 1u;
        }
        u32x4 q[R];
        load_step(0, 0, q);
        float acc[TB][R];
        uint32_t p = 0, c = 0;
        for (uint32_t step = 0; step < nsteps; ++step) {
            uint32_t cn = c + 1u, pn = p;
            if (cn == nchunks) {
                cn = 0;
                pn = p + 1u;
            }
            u32x4 qn[R];
            if (step + 1u < nsteps) {
                load_step(pn, cn, qn);
            }
            if (c == 0u) {
#pragma unroll
                for (int t = 0; t < TB; ++t) {
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        acc[t][r] = 0.0f;
                    }
                }
            }
            const uint32_t col = (c << 9) + lane * 8u;
            // elements of this lane's slice that exist (8 everywhere but at a row's end)
            const uint32_t live = col >= cols ? 0u : (cols - col < 8u ? cols - col : 8u);
            if (live != 0u) {
                float xv[TB][8];
#pragma unroll
                for (int t = 0; t < TB; ++t) {
                    const float *xp = x + (size_t)tok[t] * cols + col;
                    if (VEC || live == 8u) {
                        const f32x4_a4 a = *(const f32x4_a4 *)xp;
                        const f32x4_a4 b = *(const f32x4_a4 *)(xp + 4);
                        xv[t][0] = a.x; xv[t][1] = a.y; xv[t][2] = a.z; xv[t][3] = a.w;
                        xv[t][4] = b.x; xv[t][5] = b.y; xv[t][6] = b.z; xv[t][7] = b.w;
                    } else {
#pragma unroll
                        for (int i = 0; i < 8; ++i) {
                            xv[t][i] = (uint32_t)i < live ? xp[i] : 0.0f;
                        }
                    }
                }
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const uint32_t qr[4] = {q[r].x, q[r].y, q[r].z, q[r].w};
                    float wf[8];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        wf[2 * i] = f16_lo(qr[i]);
                        wf[2 * i + 1] = f16_hi(qr[i]);
                    }
#pragma unroll
                    for (int t = 0; t < TB; ++t) {
                        float a = acc[t][r];
#pragma unroll
                        for (int i = 0; i < 8; ++i) {
                            if (VEC || (uint32_t)i < live) {
                                a = __fadd_rn(a, __fmul_rn(wf[i], xv[t][i]));
                            }
                        }
                        acc[t][r] = a;
                    }
                }
            }
            if (cn == 0u) {
                const uint32_t r0 = row_first + p * R;
#pragma unroll
                for (int t = 0; t < TB; ++t) {
                    reduce_store<R>(acc[t], y + (size_t)tok[t] * rows, r0, row_end, lane,
                                    t0 + t < batch);
                }
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                q[r] = qn[r];
            }
            p = pn;
            c = cn;
        }
    }
}

// out[out_off + i] = f32(w[row][i])
__global__ __launch_bounds__(256) void f16_row_kernel(const uint16_t *__restrict__ w,
                                                      float *__restrict__ out, uint32_t cols,
                                                      uint32_t row, uint32_t out_off) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < cols) {
        out[(size_t)out_off + i] = f16_bits_to_f32(w[(size_t)row * cols + i]);
    }
}

// Row index read from device memory; an index past the table writes zeros.
__global__ __launch_bounds__(256) void f16_row_indirect_kernel(const uint16_t *__restrict__ w,
                                                               float *__restrict__ out,
                                                               const uint32_t *__restrict__ ids,
                                                               uint32_t slot, uint32_t rows,
                                                               uint32_t cols) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= cols) {
        return;
    }
    const uint32_t row = ids[slot];
    out[i] = row < rows ? f16_bits_to_f32(w[(size_t)row * cols + i]) : 0.0f;
}

// About 16 KiB of weights per wave, at least one pass of 8 rows; a matrix that
// would give fewer than 1024 tiles gets one-pass tiles so that it still spreads.
inline uint32_t f16_rows_per_tile(uint32_t rows, uint32_t cols) {
    uint32_t rpt = (uint32_t)(16384u / ((uint64_t)cols * 2u)) & ~7u;
    if (rpt < 8u) {
        rpt = 8u;
    }
    if (rpt > 64u) {
        rpt = 64u;
    }
    if ((rows + rpt - 1u) / rpt < 1024u) {
        rpt = 8u;
    }
    return rpt;
}

struct F16Product {
    const uint16_t *w;
    const float *x;
    float *y;
    uint32_t rows, cols, batch;
};

template <int TB, bool VEC>
inline hipError_t launch_f16_list_cfg(hipStream_t stream, hipEvent_t stop, const F16Product *prods,
                                      int n) {
    GemvArgs args; // only the used descriptors are written
    args.n = (uint32_t)n;
    args.pad = 0;
    args.norm_eps = 0.0f;
    args.norm_h = nullptr;
    args.norm_w = nullptr;
    args.norm_out = nullptr;
    uint64_t tiles = 0;
    for (int i = 0; i < n; ++i) {
        GemvDesc &d = args.d[i];
        d.w = (const uint8_t *)prods[i].w;
        d.x = prods[i].x;
        d.y = prods[i].y;
        d.rows = prods[i].rows;
        d.cols = prods[i].cols;
        d.batch = prods[i].batch;
        d.tile_begin = (uint32_t)tiles;
        d.rows_per_tile = f16_rows_per_tile(prods[i].rows, prods[i].cols);
        d.pad = 0;
        d.res = nullptr;
        d.alpha = 0.0f;
        d.pad2 = 0;
        tiles += (prods[i].rows + d.rows_per_tile - 1u) / d.rows_per_tile;
    }
    if (tiles == 0 || tiles > 0xffffffffull) {
        return hipErrorInvalidValue;
    }
    args.total_tiles = (uint32_t)tiles;
    Q8_LAUNCH((f16_gemm_list_kernel<TB, VEC>), dim3((unsigned)((tiles + 3u) / 4u)), dim3(256), 0,
              stream, stop, args);
    return hipGetLastError();
}

// Every product of the list has f16_tokens(batch) == tb; vec: all cols % 8 == 0.
inline hipError_t launch_f16_list(hipStream_t stream, hipEvent_t stop, int tb, bool vec,
                                  const F16Product *prods, int n) {
    if (n <= 0 || n > GEMV_MAX_DESCS) {
        return hipErrorInvalidValue;
    }
    for (int i = 0; i < n; ++i) {
        if (prods[i].rows == 0 || prods[i].cols == 0 || prods[i].batch == 0 ||
            prods[i].batch > F16_GEMM_MAX_BATCH || (vec && (prods[i].cols & 7u) != 0u)) {
            return hipErrorInvalidValue;
        }
    }
    switch (tb) {
    case 1:
        return vec ? launch_f16_list_cfg<1, true>(stream, stop, prods, n)
                   : launch_f16_list_cfg<1, false>(stream, stop, prods, n);
    case 2:
        return vec ? launch_f16_list_cfg<2, true>(stream, stop, prods, n)
                   : launch_f16_list_cfg<2, false>(stream, stop, prods, n);
    case 4:
        return vec ? launch_f16_list_cfg<4, true>(stream, stop, prods, n)
                   : launch_f16_list_cfg<4, false>(stream, stop, prods, n);
    case 8:
        return vec ? launch_f16_list_cfg<8, true>(stream, stop, prods, n)
                   : launch_f16_list_cfg<8, false>(stream, stop, prods, n);
    default:
        return hipErrorInvalidValue;
    }
}

} // namespace q8
