// Q8_0 matrix-vector / small-batch matrix-matrix kernel (bandwidth-bound).
//
// One launch runs a LIST of products (a decode step issues ~200 of them, most
// far too small to fill 256 CUs alone). A wave owns `rows_per_tile` consecutive
// rows of one product and walks them R rows at a time:
//
//   columns are cut into chunks of 1024 (16 quants per lane, one 16-byte load
//   per lane per row = 1 KiB contiguous per wave), then a tail of 512/256/128/
//   64/32 columns (8/4/2/1/1 quants per lane). A lane's piece always lies in
//   one Q8_0 block, so   acc += d_block * (sum of q*x over the piece)
//   with the sum taken left to right in fused multiply-adds. The 64 lane
//   partials are reduced by q8::wave_sum.
//
// Per-(row, token) arithmetic depends only on `cols`, never on R, TB,
// rows_per_tile, the layout or which other products share the launch: this is
// what makes gemm(batch = 1) bit-identical to gemv, and every token of the
// small-batch gemm bit-identical to its own gemv
// (contract: native/metal/tm_metal.h:161-164).
#pragma once

#include "q8_common.hpp"

namespace q8 {

struct GemvDesc {
    const uint8_t *w;
    const float *x;        // x_off already applied
    float *y;              // y_off already applied
    uint32_t rows, cols;
    uint32_t batch;
    uint32_t tile_begin;   // index of this product's first tile in the launch
    uint32_t rows_per_tile;
    uint32_t pad;
};

// The list travels in the kernel-argument segment (read through the scalar
// cache): 256 * 48 + 16 = 12304 bytes, enough for a whole decode step of a
// 28-layer model (197 products) in one launch.
constexpr int GEMV_MAX_DESCS = 256;

struct GemvArgs {
    uint32_t n;
    uint32_t total_tiles;
    uint32_t pad[2];
    GemvDesc d[GEMV_MAX_DESCS];
};

template <int NB, bool XA>
__device__ __forceinline__ void load_x(const float *p, float *out) {
    if constexpr (XA && NB >= 4) {
#pragma unroll
        for (int i = 0; i < NB / 4; ++i) {
            float4 v = ((const float4 *)p)[i];
            out[4 * i] = v.x; out[4 * i + 1] = v.y; out[4 * i + 2] = v.z; out[4 * i + 3] = v.w;
        }
    } else if constexpr (XA && NB == 2) {
        float2 v = *(const float2 *)p;
        out[0] = v.x; out[1] = v.y;
    } else {
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            out[i] = p[i];
        }
    }
}

template <int NB>
__device__ __forceinline__ float piece_dot(const uint32_t *q, const float *x) {
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        s = __builtin_fmaf(sbyte_to_float(q[i / 4], i % 4), x[i], s);
    }
    return s;
}

// One chunk of 64*NB columns starting at `col0`, for R rows and TB tokens.
// `active` is false only for the upper half-wave of a trailing 32-column
// chunk; inactive lanes still execute (on clamped addresses) and add 0.
template <int L, int R, int TB, int NB, bool XA, bool NT>
__device__ __forceinline__ void chunk(const WView<L> &wv, const float *x, uint32_t cols,
                                      const uint32_t (&row)[R], const uint32_t (&tok)[TB],
                                      uint32_t col0, uint32_t lane, bool active,
                                      float (&acc)[R][TB]) {
    const uint32_t col = col0 + (active ? lane * NB : 0u);
    constexpr int ND = NB >= 4 ? NB / 4 : 1;
    uint32_t q[R][ND];
    uint32_t sb[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        wv.template load_quants<NB, NT>(row[r], col, q[r]);
        sb[r] = wv.scale_bits(row[r], col >> 5);
    }
#pragma unroll
    for (int t = 0; t < TB; ++t) {
        float xv[NB];
        load_x<NB, XA>(x + (size_t)tok[t] * cols + col, xv);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float d = active ? f16_bits_to_f32(sb[r]) : 0.0f;
            const float s = active ? piece_dot<NB>(q[r], xv) : 0.0f;
            acc[r][t] = __builtin_fmaf(d, s, acc[r][t]);
        }
    }
}

// Sums R per-lane partials over the wave and stores row r0 + r (token `t`).
// For R == 8 the xor-butterfly halves the number of live values at each of
// its first three steps (lanes with bit 5/4/3 set carry rows +4/+2/+1), so 10
// shuffles serve 8 rows; every addition has the same two operands as in
// q8::wave_sum, hence the same bits.
template <int R>
__device__ __forceinline__ void reduce_store(const float (&acc)[R], float *y, uint32_t r0,
                                             uint32_t row_end, uint32_t lane, bool token_ok) {
    if constexpr (R == 8) {
        float a4[4], a2[2];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float keep = (lane & 32u) ? acc[i + 4] : acc[i];
            const float send = (lane & 32u) ? acc[i] : acc[i + 4];
            a4[i] = keep + __shfl_xor(send, 32, WAVE);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const float keep = (lane & 16u) ? a4[i + 2] : a4[i];
            const float send = (lane & 16u) ? a4[i] : a4[i + 2];
            a2[i] = keep + __shfl_xor(send, 16, WAVE);
        }
        const float keep = (lane & 8u) ? a2[1] : a2[0];
        const float send = (lane & 8u) ? a2[0] : a2[1];
        float a1 = keep + __shfl_xor(send, 8, WAVE);
        a1 += __shfl_xor(a1, 4, WAVE);
        a1 += __shfl_xor(a1, 2, WAVE);
        a1 += __shfl_xor(a1, 1, WAVE);
        const uint32_t r = ((lane >> 5) & 1u) * 4u + ((lane >> 4) & 1u) * 2u + ((lane >> 3) & 1u);
        if ((lane & 7u) == 0u && r0 + r < row_end && token_ok) {
            y[r0 + r] = a1;
        }
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float total = wave_sum(acc[r]);
            if (lane == 0u && r0 + r < row_end && token_ok) {
                y[r0 + r] = total;
            }
        }
    }
}

template <int L, int R, int TB, bool XA>
__global__ __launch_bounds__(256) void gemv_list_kernel(const GemvArgs args) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t tile = blockIdx.x * 4u + wave;
    if (tile >= args.total_tiles) {
        return;
    }
    // Locate the product that owns this tile (tile_begin is increasing).
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
    const uint32_t rows = d.rows, cols = d.cols, batch = d.batch;
    const WView<L> wv(d.w, rows, cols);
    const float *x = d.x;
    float *y = d.y;
    const uint32_t row_first = (tile - d.tile_begin) * d.rows_per_tile;
    uint32_t row_end = row_first + d.rows_per_tile;
    if (row_end > rows) {
        row_end = rows;
    }
    const uint32_t full = cols >> 10;
    const uint32_t tail0 = full << 10;
    // With one pass over the tokens every quant is read once: stream it. (The
    // f16 scales stay on plain loads: neighbouring rows share their cache
    // lines.) The multi-token form re-reads the tile per token group: keep it
    // cached.
    constexpr bool NT = TB == 1;

    if constexpr (TB == 1 && L == PACKED) {
        if ((cols & 1023u) == 0u) {
            // Whole 1024-column chunks only (every Qwen3 projection): the
            // (row pass, chunk) steps form one software-pipelined sequence in
            // which the 8 weight loads of step s+1 are in flight while step s
            // is multiplied. With a single chunk this lane's 16 activations
            // stay in registers for the whole tile. Same per-row arithmetic
            // as the general path below: chunks in order, acc from 0.
            const uint32_t nchunk = cols >> 10;
            const uint32_t nsteps = ((row_end - row_first + R - 1) / R) * nchunk;
            float xv[16];
            if (nchunk == 1u) {
                load_x<16, XA>(x + lane * 16u, xv);
            }
            uint32_t q[R][4], sb[R];
            auto load_step = [&](uint32_t r0, uint32_t c, uint32_t (&qq)[R][4], uint32_t (&ss)[R]) {
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const uint32_t row = (r0 + r < row_end) ? r0 + r : row_end - 1u;
                    wv.template load_quants<16, true>(row, (c << 10) + lane * 16u, qq[r]);
                    ss[r] = wv.scale_bits(row, (c << 5) + (lane >> 1));
                }
            };
            uint32_t r0 = row_first, c = 0;
            load_step(r0, c, q, sb);
            float acc[R];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                acc[r] = 0.0f;
            }
            for (uint32_t step = 0; step < nsteps; ++step) {
                if (nchunk > 1u) {
                    load_x<16, XA>(x + (c << 10) + lane * 16u, xv);
                }
                uint32_t cn = c + 1u, rn = r0;
                if (cn == nchunk) {
                    cn = 0;
                    rn = r0 + R;
                }
                uint32_t qn[R][4], sn[R];
                if (step + 1u < nsteps) {
                    load_step(rn, cn, qn, sn);
                }
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    acc[r] = __builtin_fmaf(f16_bits_to_f32(sb[r]), piece_dot<16>(q[r], xv), acc[r]);
                }
                if (cn == 0u) {
                    reduce_store<R>(acc, y, r0, row_end, lane, true);
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        acc[r] = 0.0f;
                    }
                }
#pragma unroll
                for (int r = 0; r < R; ++r) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        q[r][i] = qn[r][i];
                    }
                    sb[r] = sn[r];
                }
                c = cn;
                r0 = rn;
            }
            return;
        }
    }

    for (uint32_t t0 = 0; t0 < batch; t0 += TB) {
        uint32_t tok[TB];
#pragma unroll
        for (int t = 0; t < TB; ++t) {
            tok[t] = (t0 + t < batch) ? t0 + t : batch - 1u;
        }
        for (uint32_t r0 = row_first; r0 < row_end; r0 += R) {
            uint32_t row[R];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                row[r] = (r0 + r < row_end) ? r0 + r : row_end - 1u;
            }
            float acc[R][TB];
#pragma unroll
            for (int r = 0; r < R; ++r) {
#pragma unroll
                for (int t = 0; t < TB; ++t) {
                    acc[r][t] = 0.0f;
                }
            }
            for (uint32_t c = 0; c < full; ++c) {
                chunk<L, R, TB, 16, XA, NT>(wv, x, cols, row, tok, c << 10, lane, true, acc);
            }
            uint32_t col0 = tail0;
            if (cols & 512u) {
                chunk<L, R, TB, 8, XA, NT>(wv, x, cols, row, tok, col0, lane, true, acc);
                col0 += 512u;
            }
            if (cols & 256u) {
                chunk<L, R, TB, 4, XA, NT>(wv, x, cols, row, tok, col0, lane, true, acc);
                col0 += 256u;
            }
            if (cols & 128u) {
                chunk<L, R, TB, 2, XA, NT>(wv, x, cols, row, tok, col0, lane, true, acc);
                col0 += 128u;
            }
            if (cols & 64u) {
                chunk<L, R, TB, 1, XA, NT>(wv, x, cols, row, tok, col0, lane, true, acc);
                col0 += 64u;
            }
            if (cols & 32u) {
                chunk<L, R, TB, 1, XA, NT>(wv, x, cols, row, tok, col0, lane, lane < 32u, acc);
            }
#pragma unroll
            for (int t = 0; t < TB; ++t) {
                float col_acc[R];
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    col_acc[r] = acc[r][t];
                }
                reduce_store<R>(col_acc, y + (size_t)(t0 + t) * rows, r0, row_end, lane,
                                t0 + t < batch);
            }
        }
    }
}

} // namespace q8
