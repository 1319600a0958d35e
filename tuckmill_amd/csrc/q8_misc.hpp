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

// XOR of n 32-bit words, read once with non-temporal 16-byte loads: a wave
// takes a tile of 8 KiB at a time, the shape in which the decode GEMV streams
// its weights (eight 1 KiB rows in flight per wave). It writes one word per
// workgroup, so what it measures is the read path alone: the sustained HBM
// read bandwidth that the streaming kernels can be set against. `src` is
// 16-byte aligned.

__global__ __launch_bounds__(256) void xor_checksum_kernel(const uint32_t *__restrict__ src,
                                                           uint32_t *__restrict__ partial,
                                                           uint32_t n) {
    const uint32_t lane = threadIdx.x & 63u, wave_in = threadIdx.x >> 6;
    const uint32_t pieces = n >> 2; // whole 16-byte pieces
    const uint32_t full_tiles = pieces >> 9; // 512 pieces = 8 KiB
    const uint32_t waves = gridDim.x * 4u;
    const u32x4 *base = (const u32x4 *)src;
    u32x4 acc = {0u, 0u, 0u, 0u};
    uint32_t tile = blockIdx.x * 4u + wave_in;
    for (; tile < full_tiles; tile += waves) {
        const u32x4 *p = base + (size_t)tile * 512u + lane;
        u32x4 v[8];
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            v[r] = __builtin_nontemporal_load(p + r * 64);
        }
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            acc ^= v[r];
        }
    }
    if (tile == full_tiles) { // the ragged last tile: piece by piece
#pragma unroll 1
        for (uint32_t i = (full_tiles << 9) + lane; i < pieces; i += 64u) {
            acc ^= base[i];
        }
        if (lane < (n & 3u)) { // and the last one to three words
            acc.x ^= src[(size_t)pieces * 4u + lane];
        }
    }
    uint32_t x = acc.x ^ acc.y ^ acc.z ^ acc.w;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        x ^= (uint32_t)__shfl_xor((int)x, off, 64);
    }
    __shared__ uint32_t per_wave[4];
    if (lane == 0u) {
        per_wave[wave_in] = x;
    }
    __syncthreads();
    if (threadIdx.x == 0u) {
        partial[blockIdx.x] = per_wave[0] ^ per_wave[1] ^ per_wave[2] ^ per_wave[3];
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
