// Small Q8_0 helpers: sealing (raw -> packed), single-row dequantization,
// f32 copy. None of them is performance critical.
#pragma once

#include "q8_common.hpp"

namespace q8 {

// One thread per Q8_0 block: 34 raw bytes -> 32 quant bytes + 1 scale.
__global__ __launch_bounds__(256) void pack_kernel(const uint8_t *__restrict__ raw,
                                                   uint8_t *__restrict__ packed, uint32_t rows,
                                                   uint32_t cols) {
    const size_t nblocks = (size_t)rows * (cols / 32u);
    const size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= nblocks) {
        return;
    }
    const uint16_t *src = (const uint16_t *)(raw + b * 34u); // 2-byte aligned
    uint32_t v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        v[i] = (uint32_t)src[1 + 2 * i] | ((uint32_t)src[2 + 2 * i] << 16);
    }
    uint4 *dst = (uint4 *)(packed + b * 32u);
    dst[0] = make_uint4(v[0], v[1], v[2], v[3]);
    dst[1] = make_uint4(v[4], v[5], v[6], v[7]);
    uint16_t *scales = (uint16_t *)(packed + (size_t)rows * cols);
    scales[b] = src[0];
}

// out[out_off + i] = d * q for row `row` (native/metal/kernels.metal:275-292
// computes the same product; it is exact in f32).
template <int L>
__global__ __launch_bounds__(256) void row_kernel(const uint8_t *__restrict__ w,
                                                  float *__restrict__ out, uint32_t rows,
                                                  uint32_t cols, uint32_t row, uint32_t out_off) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= cols) {
        return;
    }
    const WView<L> wv(w, rows, cols);
    uint32_t q;
    wv.template load_quants<1>(row, i, &q);
    out[(size_t)out_off + i] = f16_bits_to_f32(wv.scale_bits(row, i >> 5)) * sbyte_to_float(q, 0);
}

// Row index read from device memory; an index past the table writes zeros
// (native/metal/kernels.metal:235-255).
template <int L>
__global__ __launch_bounds__(256) void row_indirect_kernel(const uint8_t *__restrict__ w,
                                                           float *__restrict__ out,
                                                           const uint32_t *__restrict__ ids,
                                                           uint32_t slot, uint32_t rows,
                                                           uint32_t cols) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= cols) {
        return;
    }
    const uint32_t row = ids[slot];
    if (row >= rows) {
        out[i] = 0.0f;
        return;
    }
    const WView<L> wv(w, rows, cols);
    uint32_t q;
    wv.template load_quants<1>(row, i, &q);
    out[i] = f16_bits_to_f32(wv.scale_bits(row, i >> 5)) * sbyte_to_float(q, 0);
}

__global__ __launch_bounds__(256) void copy_f32_kernel(const float *src, float *dst,
                                                       uint32_t n) {
    for (uint64_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n;
         i += (uint64_t)gridDim.x * blockDim.x) {
        dst[i] = src[i];
    }
}

// Clears n dwords (counters that must read zero when the next kernel starts).
__global__ __launch_bounds__(256) void zero_u32_kernel(uint32_t *dst, uint32_t n) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        dst[i] = 0u;
    }
}

} // namespace q8
