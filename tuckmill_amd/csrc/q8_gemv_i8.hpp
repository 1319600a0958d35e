// The int8-activation profile at decode-sized batches (1 <= batch <= 16, sealed
// weights): a bandwidth-bound streaming kernel instead of the MFMA tile kernel.
// It is the fastest form up to 4 tokens; from 5 the LDS-staged MFMA kernel
// (q8_gemm_i8_lds.hpp) takes over unless the caller asks for the block dots.
//
// Reference arithmetic (crates/tuckcore/src/kernels.rs:206-221) per row:
//     for each block in order:  sum += (d_w * d_x) * (float)sumi
// sumi is an integer (any evaluation order is exact: v_dot4_i32_i8 over a
// lane's 16 quants, two lanes per block), but the f32 sum over blocks is a
// strictly ordered chain, which does not reduce over lanes the way the f32
// GEMV's partials do. So the kernel works in two phases per 1024-column chunk:
//
//   A  lanes across columns (the GEMV's coalesced weight stream, 8 rows per
//      pass, loads one pass ahead): every lane pair produces its block's term
//      (d_w * d_x) * sumi and parks it in the wave's LDS slice, [row][block];
//   B  lanes across (token, row): each lane walks its row's 32 terms in block
//      order with plain f32 additions, continuing the sum it carries from the
//      previous chunk.
//
// Both multiplications and the addition are unfused, as in the reference, so
// the result is the reference's bit for bit. A wave owns up to 64 / TB rows of
// one product for TB tokens; products of a dispatch group share one launch.
#pragma once

#include "q8_gemm_i8.hpp"

namespace q8 {

constexpr int GI8_STRIDE = 36; // floats per [row] of the term buffer: 32 blocks + 4 of padding
                               // (row-strided 16-byte reads then spread over all banks)

template <int TB> struct Gi8Shape {
    static constexpr int max_rows = TB >= 8 ? 8 : (TB >= 4 ? 16 : 32); // rows per wave tile;
                                                                        // max_rows * TB <= 64
};

template <int TB, bool SUMI>
__global__ __launch_bounds__(256) void gemv_i8_list_kernel(const I8Args args) {
    constexpr int R = 8;
    constexpr int RTM = Gi8Shape<TB>::max_rows;
    __shared__ __attribute__((aligned(16))) float terms_all[4][TB * RTM * GI8_STRIDE];
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
    const I8Desc &d = args.d[lo];
    const uint32_t rows = d.rows, cols = d.cols, batch = d.batch;
    const uint32_t rpt = d.tiles_t; // rows per tile for this kernel (a multiple of 8, <= RTM)
    const uint32_t row_first = (tile - d.tile_begin) * rpt;
    uint32_t row_end = row_first + rpt;
    if (row_end > rows) {
        row_end = rows;
    }
    const uint32_t blocks = cols >> 5;
    const uint32_t bpad = xq_bpad(batch);
    const WView<PACKED> wv(d.w, rows, cols);
    const uint8_t *xqs = d.xq;
    const float *xd = (const float *)(d.xq + (size_t)batch * cols);
    float *terms = terms_all[wave];

    const uint32_t nchunks = (cols + 1023u) >> 10;
    const uint32_t passes = (row_end - row_first + R - 1) / R;
    const uint32_t nsteps = nchunks * passes;
    const bool even = (lane & 1u) == 0u;
    // phase B: this lane's (token, row) pair
    const uint32_t b_tok = lane / RTM, b_row = lane % RTM;
    const bool b_live = b_tok < (uint32_t)TB && row_first + b_row < row_end;

    for (uint32_t t0 = 0; t0 < batch; t0 += TB) {
        uint32_t tok[TB];
#pragma unroll
        for (int t = 0; t < TB; ++t) {
            tok[t] = (t0 + t < batch) ? t0 + t : batch - 1u;
        }
        auto load_pass = [&](uint32_t c, uint32_t p, uint32_t (&qq)[R][4], uint32_t (&ss)[R]) {
            uint32_t col = (c << 10) + lane * 16u;
            if (col >= cols) {
                col = 0; // lanes past the last block read valid memory and contribute nothing
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                uint32_t row = row_first + p * R + r;
                if (row >= row_end) {
                    row = row_end - 1u;
                }
                wv.template load_quants<16, true>(row, col, qq[r]);
                ss[r] = wv.scale_bits(row, col >> 5);
            }
        };
        uint32_t q[R][4], sb[R];
        load_pass(0, 0, q, sb);
        uint32_t c = 0, p = 0;
        uint32_t xq[TB][4];
        float dx[TB];
        float sum = 0.0f; // phase B's running row sum
        for (uint32_t step = 0; step < nsteps; ++step) {
            const uint32_t col_raw = (c << 10) + lane * 16u;
            const bool active = col_raw < cols;
            const uint32_t col = active ? col_raw : 0u;
            if (p == 0u) {
#pragma unroll
                for (int t = 0; t < TB; ++t) {
                    const u32x4 v = *(const u32x4 *)(xqs + (size_t)tok[t] * cols + col);
                    xq[t][0] = v.x; xq[t][1] = v.y; xq[t][2] = v.z; xq[t][3] = v.w;
                    dx[t] = xd[(size_t)(col >> 5) * bpad + tok[t]];
                }
            }
            uint32_t pn = p + 1u, cn = c;
            if (pn == passes) {
                pn = 0;
                cn = c + 1u;
            }
            uint32_t qn[R][4], sn[R];
            if (step + 1u < nsteps) {
                load_pass(cn, pn, qn, sn);
            }
            // phase A for the 8 rows of this pass
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const float dw = f16_bits_to_f32(sb[r]);
#pragma unroll
                for (int t = 0; t < TB; ++t) {
                    int s = 0;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        s = __builtin_amdgcn_sdot4((int)q[r][i], (int)xq[t][i], s, false);
                    }
                    s += __shfl_xor(s, 1, WAVE); // the other half of the block
                    const float term = __fmul_rn(__fmul_rn(dw, dx[t]), (float)s);
                    if (active && even) {
                        terms[(t * RTM + (int)(p * R) + r) * GI8_STRIDE + (lane >> 1)] = term;
                        if constexpr (SUMI) {
                            const uint32_t row = row_first + p * R + r;
                            if (row < row_end && t0 + t < batch) {
                                d.sumi[((size_t)(t0 + t) * rows + row) * blocks + (col >> 5)] = s;
                            }
                        }
                    }
                }
            }
            if (pn == 0u) {
                // phase B: the chunk's terms of this lane's row, in block order
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                const uint32_t nblk = blocks - (c << 5) < 32u ? blocks - (c << 5) : 32u;
                if (b_live) {
                    const float4 *src = (const float4 *)(terms + (b_tok * RTM + b_row) * GI8_STRIDE);
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        const float4 v = src[k];
                        if (4u * k + 0u < nblk) sum = __fadd_rn(sum, v.x);
                        if (4u * k + 1u < nblk) sum = __fadd_rn(sum, v.y);
                        if (4u * k + 2u < nblk) sum = __fadd_rn(sum, v.z);
                        if (4u * k + 3u < nblk) sum = __fadd_rn(sum, v.w);
                    }
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    q[r][i] = qn[r][i];
                }
                sb[r] = sn[r];
            }
            p = pn;
            c = cn;
        }
        if (b_live && t0 + b_tok < batch) {
            d.y[(size_t)(t0 + b_tok) * rows + row_first + b_row] = sum;
        }
    }
}

// Rows per wave tile: as many as the shape allows, fewer for a matrix that
// would otherwise give fewer than 512 tiles.
template <int TB> inline uint32_t gi8_rows_per_tile(uint32_t rows) {
    uint32_t rpt = (uint32_t)Gi8Shape<TB>::max_rows;
    while (rpt > 8u && (rows + rpt - 1u) / rpt < 512u) {
        rpt >>= 1;
    }
    return rpt;
}

template <int TB, bool SUMI>
inline hipError_t launch_gemv_i8_cfg(hipStream_t stream, hipEvent_t stop, const I8Product *prods,
                                     int n) {
    I8Args args;
    args.n = (uint32_t)n;
    uint64_t tiles = 0;
    for (int i = 0; i < n; ++i) {
        I8Desc &d = args.d[i];
        d.w = prods[i].w;
        d.xq = prods[i].xq;
        d.y = prods[i].y;
        d.sumi = prods[i].sumi;
        d.rows = prods[i].rows;
        d.cols = prods[i].cols;
        d.batch = prods[i].batch;
        d.tile_begin = (uint32_t)tiles;
        d.tiles_t = gi8_rows_per_tile<TB>(prods[i].rows);
        d.pad = 0;
        tiles += (prods[i].rows + d.tiles_t - 1u) / d.tiles_t;
    }
    args.total_tiles = (uint32_t)tiles;
    args.chunk_wgs = 1;
    args.pad = 0;
    Q8_LAUNCH((gemv_i8_list_kernel<TB, SUMI>), dim3((unsigned)((tiles + 3u) / 4u)), dim3(256), 0,
              stream, stop, args);
    return hipGetLastError();
}

// Sealed weights only; tb is gemv_i8_tokens(batch) of every product in the list.
inline hipError_t launch_gemv_i8_list(hipStream_t stream, hipEvent_t stop, bool sumi, int tb,
                                      const I8Product *prods, int n) {
    if (n <= 0 || n > I8_MAX_DESCS) {
        return hipErrorInvalidValue;
    }
    switch (tb) {
    case 1:
        return sumi ? launch_gemv_i8_cfg<1, true>(stream, stop, prods, n)
                    : launch_gemv_i8_cfg<1, false>(stream, stop, prods, n);
    case 2:
        return sumi ? launch_gemv_i8_cfg<2, true>(stream, stop, prods, n)
                    : launch_gemv_i8_cfg<2, false>(stream, stop, prods, n);
    case 4:
        return sumi ? launch_gemv_i8_cfg<4, true>(stream, stop, prods, n)
                    : launch_gemv_i8_cfg<4, false>(stream, stop, prods, n);
    case 8:
        return sumi ? launch_gemv_i8_cfg<8, true>(stream, stop, prods, n)
                    : launch_gemv_i8_cfg<8, false>(stream, stop, prods, n);
    default:
        return hipErrorInvalidValue;
    }
}

} // namespace q8
