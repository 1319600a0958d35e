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
// xq layout: [batch][cols] int8, then [batch][cols/32] f32.
template <bool XA>
__global__ __launch_bounds__(256) void quantize_act_kernel(const float *__restrict__ x,
                                                           uint8_t *__restrict__ xq, uint32_t cols,
                                                           uint32_t batch) {
    const size_t nblocks = (size_t)batch * (cols >> 5);
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
            scales[bb] = f16_bits_to_f32(f32_to_f16_bits(d));
        }
    }
}

inline hipError_t launch_quantize_act(hipStream_t stream, hipEvent_t stop, const float *x,
                                      uint8_t *xq, uint32_t cols, uint32_t batch) {
    const size_t nblocks = (size_t)batch * (cols / 32u);
    const unsigned groups = (unsigned)((nblocks * 32u + 255u) / 256u);
    Q8_LAUNCH(quantize_act_kernel<true>, dim3(groups), dim3(256), 0, stream, stop, x, xq, cols,
              batch);
    return hipGetLastError();
}

// One wave owns a TM*16-token x TN*16-row tile and walks the blocks in order.
// MFMA operand layout (16x16x32 i8): lane (i = lane % 16, g = lane / 16)
// supplies the 8 bytes k = 8g..8g+7 of token i (A) and of weight row i (B);
// result register v holds (token 4g + v, row i).
template <int L, int TM, int TN>
__global__ __launch_bounds__(256) void gemm_i8_kernel(const uint8_t *__restrict__ w,
                                                      const uint8_t *__restrict__ xq,
                                                      float *__restrict__ y,
                                                      int32_t *__restrict__ sumi_out, uint32_t rows,
                                                      uint32_t cols, uint32_t batch,
                                                      uint32_t tiles_t, uint32_t tiles_n) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t tile = blockIdx.x * 4u + wave;
    if (tile >= tiles_t * tiles_n) {
        return;
    }
    const uint32_t tn = tile / tiles_t, tt = tile % tiles_t;
    const uint32_t t0 = tt * (16u * TM), n0 = tn * (16u * TN);
    const uint32_t i16 = lane & 15u, g = lane >> 4;
    const uint32_t blocks = cols >> 5;
    const WView<L> wv(w, rows, cols);
    const int8_t *xqs = (const int8_t *)xq;
    const float *xd = (const float *)(xq + (size_t)batch * cols);

    uint32_t wrow[TN], atok[TM];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const uint32_t r = n0 + 16u * j + i16;
        wrow[j] = r < rows ? r : rows - 1u;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const uint32_t t = t0 + 16u * i + i16;
        atok[i] = t < batch ? t : batch - 1u;
    }
    // tokens this lane produces results for: 16*i + 4g + v
    uint32_t otok[TM][4];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const uint32_t t = t0 + 16u * i + 4u * g + v;
            otok[i][v] = t < batch ? t : batch - 1u;
        }
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

    for (uint32_t kb = 0; kb < blocks; ++kb) {
        const uint32_t col = (kb << 5) + (g << 3);
        long a[TM], b[TN];
        float dw[TN], dx[TM][4];
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            uint32_t q[2];
            wv.template load_quants<8>(wrow[j], col, q);
            b[j] = (long)(((uint64_t)q[1] << 32) | q[0]);
            dw[j] = f16_bits_to_f32(wv.scale_bits(wrow[j], kb));
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const uint2 qa = *(const uint2 *)(xqs + (size_t)atok[i] * cols + col);
            a[i] = (long)(((uint64_t)qa.y << 32) | qa.x);
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                dx[i][v] = xd[(size_t)otok[i][v] * blocks + kb];
            }
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                intx4 z = {0, 0, 0, 0};
                const intx4 s = __builtin_amdgcn_mfma_i32_16x16x32_i8(a[i], b[j], z, 0, 0, 0);
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float scale = __fmul_rn(dw[j], dx[i][v]);
                    const float term = __fmul_rn(scale, (float)s[v]);
                    acc[i][j][v] = __fadd_rn(acc[i][j][v], term);
                    if (sumi_out != nullptr) {
                        const uint32_t t = t0 + 16u * i + 4u * g + v;
                        const uint32_t n = n0 + 16u * j + i16;
                        if (t < batch && n < rows) {
                            sumi_out[((size_t)t * rows + n) * blocks + kb] = s[v];
                        }
                    }
                }
            }
        }
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

template <int L, int TM, int TN>
inline hipError_t launch_i8_cfg(hipStream_t stream, hipEvent_t stop, const uint8_t *w,
                                const uint8_t *xq, float *y, int32_t *sumi, uint32_t rows,
                                uint32_t cols, uint32_t batch) {
    const uint32_t tiles_t = (batch + 16u * TM - 1) / (16u * TM);
    const uint32_t tiles_n = (rows + 16u * TN - 1) / (16u * TN);
    const uint64_t tiles = (uint64_t)tiles_t * tiles_n;
    Q8_LAUNCH((gemm_i8_kernel<L, TM, TN>), dim3((unsigned)((tiles + 3u) / 4u)), dim3(256), 0, stream,
              stop, w, xq, y, sumi, rows, cols, batch, tiles_t, tiles_n);
    return hipGetLastError();
}

inline hipError_t launch_gemm_i8(hipStream_t stream, hipEvent_t stop, bool packed, const uint8_t *w,
                                 const uint8_t *xq, float *y, int32_t *sumi, uint32_t rows,
                                 uint32_t cols, uint32_t batch) {
    if (batch <= 16u) {
        return packed ? launch_i8_cfg<PACKED, 1, 2>(stream, stop, w, xq, y, sumi, rows, cols, batch)
                      : launch_i8_cfg<RAW, 1, 2>(stream, stop, w, xq, y, sumi, rows, cols, batch);
    }
    return packed ? launch_i8_cfg<PACKED, 2, 2>(stream, stop, w, xq, y, sumi, rows, cols, batch)
                  : launch_i8_cfg<RAW, 2, 2>(stream, stop, w, xq, y, sumi, rows, cols, batch);
}

} // namespace q8
