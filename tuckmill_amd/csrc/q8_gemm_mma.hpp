// Q8_0 prefill GEMM on the MFMA matrix cores, f32 operand tiles.
//
//   Y[t][n] = sum_k X[t][k] * (d[n][k/32] * q[n][k])      t < batch, n < rows
//
// W is dequantized to f32 as d*q (exact: an 11-bit by 8-bit product fits the
// 24-bit significand), X stays f32, and v_mfma_f32_32x32x2_f32 accumulates in
// f32. Summation order differs from the GEMV, so the result is
// tolerance-qualified against it (contract: native/metal/tm_metal.h:172-175).
//
// Mapping. The MFMA's M index is the token, its N index the weight row, so a
// 32x32 accumulator tile stores 32 consecutive rows of one token as one
// 128-byte segment. A wave owns TMW x TNW such tiles. For one Q8_0 block
// (32 k-values) lane (i = lane % 32, h = lane / 32) loads the 16 quants
// k = 16h..16h+15 of weight row i and the matching 16 activations of token i;
// MFMA step j then multiplies k = j (lower half-wave) and k = 16 + j (upper
// half-wave), so one 16-byte weight load and four 16-byte activation loads
// feed 16 MFMAs per tile with no cross-lane traffic and no LDS.
//
// f32 MFMA is slow enough (64 cycles per 32x32x2 issue) that operand
// bandwidth is not the limit; filling all 1024 SIMDs is. Shapes with few
// output tiles therefore split K over the S waves of a workgroup slot and
// reduce through LDS in a fixed order (deterministic).
#pragma once

#include "q8_common.hpp"

namespace q8 {

typedef float floatx16 __attribute__((ext_vector_type(16)));

template <bool XA>
__device__ __forceinline__ void load_x16(const float *p, float (&out)[16]) {
    if constexpr (XA) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float4 v = ((const float4 *)p)[i];
            out[4 * i] = v.x; out[4 * i + 1] = v.y; out[4 * i + 2] = v.z; out[4 * i + 3] = v.w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            out[i] = p[i];
        }
    }
}

// Workgroup = 4 waves = P slots x S k-slices. Slot p of workgroup g owns
// output tile g*P + p; its S waves each take a contiguous share of the Q8_0
// blocks and wave s = 0 adds the partial tiles of s = 1..S-1 in that order.
template <int L, int TMW, int TNW, int S, bool XA>
__global__ __launch_bounds__(256) void gemm_mma_kernel(const uint8_t *__restrict__ w,
                                                       const float *__restrict__ x,
                                                       float *__restrict__ y, uint32_t rows,
                                                       uint32_t cols, uint32_t batch,
                                                       uint32_t tiles_t, uint32_t tiles_n) {
    constexpr int P = 4 / S;
    constexpr int TILE_FLOATS = TMW * TNW * 16 * WAVE;
    extern __shared__ float red[]; // [P][S-1][TILE_FLOATS]

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t p = wave / S, s = wave % S;
    const uint32_t idx = lane & 31u, half = lane >> 5;

    // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a
    // contiguous range of tiles so that a weight tile lives in one L2.
    uint32_t g = blockIdx.x;
    const uint32_t G = gridDim.x;
    if ((G & 7u) == 0u) {
        g = (g & 7u) * (G >> 3) + (g >> 3);
    }
    const uint32_t tile = g * P + p;
    const bool valid = tile < tiles_t * tiles_n;
    const uint32_t tn = valid ? tile / tiles_t : 0u;
    const uint32_t tt = valid ? tile % tiles_t : 0u;
    const uint32_t t0 = tt * (32u * TMW), n0 = tn * (32u * TNW);

    const WView<L> wv(w, rows, cols);
    const uint32_t blocks = cols >> 5;
    const uint32_t kb_begin = (uint32_t)(((uint64_t)blocks * s) / S);
    const uint32_t kb_end = (uint32_t)(((uint64_t)blocks * (s + 1u)) / S);

    uint32_t wrow[TNW], tok[TMW];
#pragma unroll
    for (int j = 0; j < TNW; ++j) {
        const uint32_t r = n0 + 32u * j + idx;
        wrow[j] = r < rows ? r : rows - 1u;
    }
#pragma unroll
    for (int i = 0; i < TMW; ++i) {
        const uint32_t t = t0 + 32u * i + idx;
        tok[i] = t < batch ? t : batch - 1u;
    }

    floatx16 acc[TMW][TNW];
#pragma unroll
    for (int i = 0; i < TMW; ++i) {
#pragma unroll
        for (int j = 0; j < TNW; ++j) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                acc[i][j][v] = 0.0f;
            }
        }
    }

    if (valid) {
        for (uint32_t kb = kb_begin; kb < kb_end; ++kb) {
            const uint32_t col = (kb << 5) + (half << 4);
            uint32_t q[TNW][4];
            uint32_t sb[TNW];
            float xv[TMW][16];
#pragma unroll
            for (int j = 0; j < TNW; ++j) {
                wv.template load_quants<16>(wrow[j], col, q[j]);
                sb[j] = wv.scale_bits(wrow[j], kb);
            }
#pragma unroll
            for (int i = 0; i < TMW; ++i) {
                load_x16<XA>(x + (size_t)tok[i] * cols + col, xv[i]);
            }
            float wf[TNW][16];
#pragma unroll
            for (int j = 0; j < TNW; ++j) {
                const float d = f16_bits_to_f32(sb[j]);
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    wf[j][e] = d * sbyte_to_float(q[j][e / 4], e % 4);
                }
            }
#pragma unroll
            for (int e = 0; e < 16; ++e) {
#pragma unroll
                for (int i = 0; i < TMW; ++i) {
#pragma unroll
                    for (int j = 0; j < TNW; ++j) {
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(xv[i][e], wf[j][e],
                                                                         acc[i][j], 0, 0, 0);
                    }
                }
            }
        }
    }

    if constexpr (S > 1) {
        if (s > 0u) {
            float *mine = red + ((size_t)p * (S - 1) + (s - 1u)) * TILE_FLOATS;
#pragma unroll
            for (int i = 0; i < TMW; ++i) {
#pragma unroll
                for (int j = 0; j < TNW; ++j) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        mine[((i * TNW + j) * 16 + v) * WAVE + lane] = acc[i][j][v];
                    }
                }
            }
        }
        __syncthreads();
        if (s > 0u) {
            return;
        }
        for (int o = 0; o < S - 1; ++o) {
            const float *other = red + ((size_t)p * (S - 1) + o) * TILE_FLOATS;
#pragma unroll
            for (int i = 0; i < TMW; ++i) {
#pragma unroll
                for (int j = 0; j < TNW; ++j) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        acc[i][j][v] += other[((i * TNW + j) * 16 + v) * WAVE + lane];
                    }
                }
            }
        }
    }
    if (!valid) {
        return;
    }
    // acc[v] of a 32x32 tile is (token 8*(v/4) + 4*half + v%4, row idx).
#pragma unroll
    for (int i = 0; i < TMW; ++i) {
#pragma unroll
        for (int j = 0; j < TNW; ++j) {
            const uint32_t n = n0 + 32u * j + idx;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t t = t0 + 32u * i + 8u * (v / 4) + 4u * half + (v % 4);
                if (t < batch && n < rows) {
                    y[(size_t)t * rows + n] = acc[i][j][v];
                }
            }
        }
    }
}

struct MmaConfig {
    int tmw, tnw, s;
};

// Pick the tile and K split that leave the fewest idle SIMD-rounds: the
// chip has 1024 SIMDs and one wave's MFMA stream occupies one of them.
inline MmaConfig pick_mma_config(uint32_t rows, uint32_t cols, uint32_t batch) {
    static const MmaConfig candidates[] = {
        {2, 2, 1}, {2, 1, 1}, {1, 1, 1}, {2, 2, 2}, {2, 1, 2}, {1, 1, 2}, {2, 1, 4}, {1, 1, 4},
    };
    const uint32_t blocks = cols / 32u;
    MmaConfig best = candidates[2];
    double best_cost = 1e300;
    for (const MmaConfig &c : candidates) {
        if ((uint32_t)c.s > blocks) {
            continue;
        }
        const uint64_t tiles = (uint64_t)((batch + 32u * c.tmw - 1) / (32u * c.tmw)) *
                               ((rows + 32u * c.tnw - 1) / (32u * c.tnw));
        const uint64_t waves = tiles * c.s;
        const uint64_t rounds = (waves + 1023u) / 1024u;
        // MFMA issues per wave, plus a charge for operand loads per issue
        // (small tiles reload more) and for the split-K reduction.
        const double mfma = (double)c.tmw * c.tnw * 16.0 * ((blocks + c.s - 1) / c.s);
        const double load_penalty = 1.0 + 0.10 * (1.0 / c.tmw + 1.0 / c.tnw);
        const double cost = rounds * (mfma * load_penalty) + (c.s > 1 ? 40.0 * c.tmw * c.tnw : 0.0);
        if (cost < best_cost) {
            best_cost = cost;
            best = c;
        }
    }
    return best;
}

template <int L, int TMW, int TNW, int S, bool XA>
inline hipError_t launch_mma_cfg(hipStream_t stream, const uint8_t *w, const float *x, float *y,
                                 uint32_t rows, uint32_t cols, uint32_t batch) {
    constexpr int P = 4 / S;
    const uint32_t tiles_t = (batch + 32u * TMW - 1) / (32u * TMW);
    const uint32_t tiles_n = (rows + 32u * TNW - 1) / (32u * TNW);
    const uint64_t tiles = (uint64_t)tiles_t * tiles_n;
    const uint32_t groups = (uint32_t)((tiles + P - 1) / P);
    const size_t lds = S > 1 ? (size_t)P * (S - 1) * TMW * TNW * 16 * WAVE * sizeof(float) : 0;
    hipLaunchKernelGGL((gemm_mma_kernel<L, TMW, TNW, S, XA>), dim3(groups), dim3(256), lds, stream,
                       w, x, y, rows, cols, batch, tiles_t, tiles_n);
    return hipGetLastError();
}

template <int L, bool XA>
inline hipError_t launch_mma_layout(hipStream_t stream, const uint8_t *w, const float *x, float *y,
                                    uint32_t rows, uint32_t cols, uint32_t batch) {
    const MmaConfig c = pick_mma_config(rows, cols, batch);
#define TM_MMA_CASE(A, B, C)                                                           \
    if (c.tmw == A && c.tnw == B && c.s == C) {                                        \
        return launch_mma_cfg<L, A, B, C, XA>(stream, w, x, y, rows, cols, batch);     \
    }
    TM_MMA_CASE(2, 2, 1)
    TM_MMA_CASE(2, 1, 1)
    TM_MMA_CASE(1, 1, 1)
    TM_MMA_CASE(2, 2, 2)
    TM_MMA_CASE(2, 1, 2)
    TM_MMA_CASE(1, 1, 2)
    TM_MMA_CASE(2, 1, 4)
    TM_MMA_CASE(1, 1, 4)
#undef TM_MMA_CASE
    return hipErrorInvalidValue;
}

inline hipError_t launch_gemm_mma(hipStream_t stream, bool packed, const uint8_t *w, const float *x,
                                  float *y, uint32_t rows, uint32_t cols, uint32_t batch) {
    const bool xa = ((uintptr_t)x % 16u) == 0;
    if (packed) {
        return xa ? launch_mma_layout<PACKED, true>(stream, w, x, y, rows, cols, batch)
                  : launch_mma_layout<PACKED, false>(stream, w, x, y, rows, cols, batch);
    }
    return xa ? launch_mma_layout<RAW, true>(stream, w, x, y, rows, cols, batch)
              : launch_mma_layout<RAW, false>(stream, w, x, y, rows, cols, batch);
}

} // namespace q8
