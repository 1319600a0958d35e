// The int8-activation profile: activations quantized to Q8_0 on the device,
// then int8 x int8 -> i32 block dots on the MFMA matrix cores.
//
// Reference arithmetic (crates/tuckcore/src/kernels.rs:206-221):
//     sumi  = sum_{l<32} q_w[l] * q_x[l]                 (i32, exact)
//     acc  += (d_w * d_x[blk]) * (float)sumi             (f32, blocks in order)
// v_mfma_i32_16x16x32_i8 has K = 32 = one Q8_0 block, so one MFMA yields the
// exact sumi of a 16-token x 16-row tile for one block. Each output element
// then applies the two multiplications and the addition above, unfused and
// in block order, so the f32 result is the reference's bit for bit as well.
#pragma once

#include "q8_common.hpp"

namespace q8 {

typedef int intx4 __attribute__((ext_vector_type(4)));

// Activation quantizer, crates/tuckcore/src/tensor.rs:184-206: per block of
// 32, d = amax/127, id = 1/d (0 when d == 0), q = clamp(rte(x*id), +-127),
// stored scale = f32 value of the f16 rounding of d. One half-wave per block.
__global__ __launch_bounds__(256) void quantize_act_kernel(const float *__restrict__ x,
                                                           uint8_t *__restrict__ xq, uint32_t cols,
                                                           uint32_t batch) {
    const uint32_t blocks = cols >> 5;
    const size_t nblocks = (size_t)batch * blocks;
    const size_t b = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) >> 5;
    const uint32_t l = threadIdx.x & 31u;
    const bool live = b < nblocks;
    const size_t bb = live ? b : nblocks - 1u;
    const float v = x[bb * 32u + l];
    float amax = __builtin_fabsf(v);
    // f32::max semantics (a NaN operand is ignored); xor masks below 32 stay
    // inside the half-wave that owns the block.
    if (amax != amax) {
        amax = 0.0f;
    }
#pragma unroll
    for (int m = 16; m >= 1; m >>= 1) {
        const float o = __shfl_xor(amax, m, WAVE);
        amax = __builtin_fmaxf(amax, o);
    }
    const float d = amax / 127.0f;
    const float id = (d != 0.0f) ? 1.0f / d : 0.0f;
    float r = __builtin_rintf(v * id);
    int q;
    if (r != r) {
        q = 0;
    } else {
        r = r < -127.0f ? -127.0f : r;
        r = r > 127.0f ? 127.0f : r;
        q = (int)r;
    }
    if (live) {
        xq[bb * 32u + l] = (uint8_t)(int8_t)q;
        if (l == 0u) {
            float *scales = (float *)(xq + (size_t)batch * cols);
            const uint32_t token = (uint32_t)(bb / blocks), blk = (uint32_t)(bb % blocks);
            scales[(size_t)blk * xq_bpad(batch) + token] = f16_bits_to_f32(f32_to_f16_bits(d));
        }
    }
}

inline hipError_t launch_quantize_act(hipStream_t stream, hipEvent_t stop, const float *x,
                                      uint8_t *xq, uint32_t cols, uint32_t batch) {
    const size_t nblocks = (size_t)batch * (cols / 32u);
    const unsigned groups = (unsigned)((nblocks * 32u + 255u) / 256u);
    Q8_LAUNCH(quantize_act_kernel, dim3(groups), dim3(256), 0, stream, stop, x, xq, cols, batch);
    return hipGetLastError();
}

struct I8Desc {
    const uint8_t *w;
    const uint8_t *xq;
    float *y;            // y_off already applied
    int32_t *sumi;       // optional [batch][rows][blocks]
    uint32_t rows, cols, batch;
    uint32_t tile_begin; // first output tile of this product in the launch
    uint32_t tiles_t;    // token tiles per row tile
    uint32_t pad;
};

struct I8Args {
    uint32_t n;
    uint32_t total_tiles;
    uint32_t chunk_wgs;
    uint32_t pad;
    I8Desc d[I8_MAX_DESCS];
};

template <int TM, int TN> struct I8Raw {
    long a[TM], b[TN];
    float4 dx[TM];
    uint32_t dwb[TN];
};

// One wave owns a TM*16-token x TN*16-row tile and walks the blocks in order,
// one block ahead with its loads. MFMA operand layout (16x16x32 i8): lane
// (i = lane % 16, g = lane / 16) supplies the 8 bytes k = 8g..8g+7 of token i
// (A) and of weight row i (B); result register v holds (token 4g + v, row i).
// A launch runs a list of products; tiles are numbered token-tile fastest and
// whole row-tiles are dealt to the XCDs in turn (one L2 per weight tile).
template <int L, int TM, int TN, bool SUMI>
__global__ __launch_bounds__(256) void gemm_i8_kernel(const I8Args args) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    uint32_t gidx = blockIdx.x;
    {
        const uint32_t cw = args.chunk_wgs;
        const uint32_t span = 8u * cw;
        const uint32_t g_full = (gridDim.x / span) * span;
        if (gidx < g_full) {
            const uint32_t xcd = gidx & 7u, j = gidx >> 3;
            gidx = ((j / cw) * 8u + xcd) * cw + (j % cw);
        }
    }
    const uint32_t tile = gidx * 4u + wave;
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
    const uint32_t local = tile - d.tile_begin;
    const uint32_t tn = local / d.tiles_t, tt = local % d.tiles_t;
    const uint32_t t0 = tt * (16u * TM), n0 = tn * (16u * TN);
    const uint32_t i16 = lane & 15u, g = lane >> 4;
    const uint32_t blocks = cols >> 5;
    const uint32_t bpad = xq_bpad(batch);
    const WView<L> wv(d.w, rows, cols);
    const int8_t *xqs = (const int8_t *)d.xq;
    const float *xd = (const float *)(d.xq + (size_t)batch * cols);
    float *y = d.y;

    uint32_t wrow[TN], atok[TM], tgrp[TM];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const uint32_t r = n0 + 16u * j + i16;
        wrow[j] = r < rows ? r : rows - 1u;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const uint32_t t = t0 + 16u * i + i16;
        atok[i] = t < batch ? t : batch - 1u;
        const uint32_t tg = t0 + 16u * i + 4u * g; // first of the 4 tokens this lane rescales
        tgrp[i] = tg + 4u <= bpad ? tg : bpad - 4u;
    }

    float acc[TM][TN][4];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                acc[i][j][v] = 0.0f;
            }
        }
    }

    auto load_block = [&](uint32_t kb, I8Raw<TM, TN> &raw) {
        const uint32_t col = (kb << 5) + (g << 3);
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            uint32_t q[2];
            wv.template load_quants<8>(wrow[j], col, q);
            raw.b[j] = (long)(((uint64_t)q[1] << 32) | q[0]);
            raw.dwb[j] = wv.scale_bits(wrow[j], kb);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const uint2 qa = *(const uint2 *)(xqs + (size_t)atok[i] * cols + col);
            raw.a[i] = (long)(((uint64_t)qa.y << 32) | qa.x);
            raw.dx[i] = *(const float4 *)(xd + (size_t)kb * bpad + tgrp[i]);
        }
    };

    I8Raw<TM, TN> cur;
    load_block(0, cur);
    for (uint32_t kb = 0; kb < blocks; ++kb) {
        I8Raw<TM, TN> nxt;
        if (kb + 1u < blocks) {
            load_block(kb + 1u, nxt);
        }
        float dw[TN];
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            dw[j] = f16_bits_to_f32(cur.dwb[j]);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const float dxv[4] = {cur.dx[i].x, cur.dx[i].y, cur.dx[i].z, cur.dx[i].w};
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const intx4 z = {0, 0, 0, 0};
                const intx4 s = __builtin_amdgcn_mfma_i32_16x16x32_i8(cur.a[i], cur.b[j], z, 0, 0, 0);
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    // (d_w * d_x) * sumi, then the add: unfused, block order
                    const float scale = __fmul_rn(dw[j], dxv[v]);
                    const float term = __fmul_rn(scale, (float)s[v]);
                    acc[i][j][v] = __fadd_rn(acc[i][j][v], term);
                    if constexpr (SUMI) {
                        const uint32_t t = t0 + 16u * i + 4u * g + v;
                        const uint32_t n = n0 + 16u * j + i16;
                        if (t < batch && n < rows) {
                            d.sumi[((size_t)t * rows + n) * blocks + kb] = s[v];
                        }
                    }
                }
            }
        }
        cur = nxt;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const uint32_t t = t0 + 16u * i + 4u * g + v;
                const uint32_t n = n0 + 16u * j + i16;
                if (t < batch && n < rows) {
                    y[(size_t)t * rows + n] = acc[i][j][v];
                }
            }
        }
    }
}

struct I8Product {
    const uint8_t *w;
    const uint8_t *xq;
    float *y;
    int32_t *sumi;
    uint32_t rows, cols, batch;
};

template <int L, int TM, int TN, bool SUMI>
inline hipError_t launch_i8_cfg(hipStream_t stream, hipEvent_t stop, const I8Product *prods, int n) {
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
        d.tiles_t = (prods[i].batch + 16u * TM - 1) / (16u * TM);
        d.pad = 0;
        tiles += (uint64_t)d.tiles_t * ((prods[i].rows + 16u * TN - 1) / (16u * TN));
    }
    args.total_tiles = (uint32_t)tiles;
    args.chunk_wgs = args.d[0].tiles_t >= 4u ? args.d[0].tiles_t / 4u : 1u;
    args.pad = 0;
    Q8_LAUNCH((gemm_i8_kernel<L, TM, TN, SUMI>), dim3((unsigned)((tiles + 3u) / 4u)), dim3(256), 0,
              stream, stop, args);
    return hipGetLastError();
}

template <int L, bool SUMI>
inline hipError_t launch_i8_layout(hipStream_t stream, hipEvent_t stop, int cfg,
                                   const I8Product *prods, int n) {
    switch (cfg) {
    case 0: return launch_i8_cfg<L, 1, 4, SUMI>(stream, stop, prods, n);
    case 1: return launch_i8_cfg<L, 2, 2, SUMI>(stream, stop, prods, n);
    case 2: return launch_i8_cfg<L, 4, 2, SUMI>(stream, stop, prods, n);
    default: return launch_i8_cfg<L, 4, 4, SUMI>(stream, stop, prods, n);
    }
}

// All products of one call share the weight layout, the tile configuration and
// whether the verification output is written (the caller groups them so).
inline hipError_t launch_gemm_i8_list(hipStream_t stream, hipEvent_t stop, bool packed, bool sumi,
                                      int cfg, const I8Product *prods, int n) {
    if (n <= 0 || n > I8_MAX_DESCS) {
        return hipErrorInvalidValue;
    }
    if (packed) {
        return sumi ? launch_i8_layout<PACKED, true>(stream, stop, cfg, prods, n)
                    : launch_i8_layout<PACKED, false>(stream, stop, cfg, prods, n);
    }
    return sumi ? launch_i8_layout<RAW, true>(stream, stop, cfg, prods, n)
                : launch_i8_layout<RAW, false>(stream, stop, cfg, prods, n);
}

} // namespace q8
