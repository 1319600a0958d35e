// int8-activation GEMM for batches of five tokens and more over sealed weights:
// operand tiles staged through LDS.
//
// Same arithmetic as gemm_i8_kernel (q8_gemm_i8.hpp): one
// v_mfma_i32_16x16x32_i8 per Q8_0 block and 16x16 tile gives the exact sumi,
// each output then applies (d_w * d_x) * sumi and the addition unfused, in block
// order: bit-identical to crates/tuckcore/src/kernels.rs:206-221.
//
// What changes is how the operands arrive. The register-fed kernel lets every
// lane fetch 8 bytes of its own token / weight row per block: 16 cache lines
// per load instruction, a quarter of each used, re-fetched from L2 by every
// wave. Here a workgroup of WM x WN waves owns (WM*TM*16 tokens) x (WN*TN*16 rows)
// and walks K in stages of KS blocks; per stage every operand byte is fetched once
// per workgroup as whole 16-byte pieces of full rows (buffer_load ... lds, no
// registers held in flight), double-buffered. Pieces are stored XOR-swizzled
// (the fetching lane chooses which piece of its row it brings, its LDS slot is
// fixed by the instruction) so that the MFMA operand reads, 8 bytes per lane
// with 16 lanes on 16 different rows, touch every bank once.
//
// One fetch instruction moves 1 KiB: 64 / (2*KS) operand rows of 32*KS bytes each.
// How that kilobyte is spread over cache lines matters more than anything else
// when the batch is small and the kernel lives off the weight stream: with
// stages of 2 blocks an instruction touches 16 lines for 64 bytes each and the
// fetch runs at about a quarter of HBM speed; with 4 blocks it takes 8 whole
// lines (i8_lds_shape below picks the stage depth per batch).
#pragma once

#include "q8_gemm_i8.hpp"

namespace q8 {

template <int WM, int WN, int KS, int TM = 4, int TN = 4> struct I8LdsShape {
    static constexpr int tokens = WM * TM * 16, rows = WN * TN * 16;
    static constexpr int row_bytes = KS * 32;           // one operand row of a stage
    static constexpr int pieces = KS * 2;               // 16-byte pieces per operand row
    // operand rows per 256 bytes of LDS (rows of 256 bytes or more: one)
    static constexpr int rows_per_bankrow = pieces >= 16 ? 1 : 16 / pieces;
    static constexpr int a_bytes = tokens * row_bytes;
    static constexpr int b_bytes = rows * row_bytes;
    // [block][token] f32, rounded up to whole 1 KiB fetch instructions
    static constexpr int dx_bytes = (KS * tokens * 4 + 1023) / 1024 * 1024;
    static constexpr int dw_bytes = rows * KS * 4;       // [row][block] f16 bits, widened to 4 bytes
    static constexpr int stage_bytes = a_bytes + b_bytes + dx_bytes + dw_bytes;
};

// Which stored slot holds piece p of operand row r (and vice versa: the swizzle
// is an involution on the piece index).
template <int WM, int WN, int KS>
__device__ __forceinline__ uint32_t i8_swz(uint32_t r, uint32_t p) {
    using Sh = I8LdsShape<WM, WN, KS>; // the swizzle does not depend on the wave tile
    return p ^ ((r / Sh::rows_per_bankrow) % (Sh::pieces < 16 ? Sh::pieces : 16));
}

// FMA = false: the tail of crates/tuckcore/src/kernels.rs:206-221 operation for
// operation, (d_w * d_x) * sumi rounded, then the addition: the f32 result has the
// CPU's bits. FMA = true (the declared fast variant, tm_hip_q8_0_gemm_i8_fma): the
// same exact i32 block dots and the same scale product, but the term goes into
// the sum with one fused multiply-add (one rounding fewer per block, three vector
// operations per output and block instead of four): within 1e-5 of the CPU's
// result, not its bits.
template <int WM, int WN, int KS, int TM = 4, int TN = 4, bool FMA = false>
__global__ __launch_bounds__(WM * WN * 64, 2) void gemm_i8_lds_kernel(const I8Args args) {
    using Sh = I8LdsShape<WM, WN, KS, TM, TN>;
    constexpr int NW = WM * WN; // 16x16 tiles per wave: 16*TM tokens x 16*TN rows
    // two stage buffers as separate objects (reads of one provably do not alias
    // the fetch into the other)
    __shared__ __attribute__((aligned(16))) uint8_t stage_a[Sh::stage_bytes];
    __shared__ __attribute__((aligned(16))) uint8_t stage_b[Sh::stage_bytes];

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t wm = wave / WN, wn = wave % WN;
    const uint32_t i16 = lane & 15u, g = lane >> 4;

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
    const uint32_t tile = gidx; // one workgroup tile per workgroup
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
    const uint32_t t0 = (local % d.tiles_t) * Sh::tokens, n0 = (local / d.tiles_t) * Sh::rows;
    const uint32_t blocks = cols >> 5;
    const uint32_t bpad = xq_bpad(batch);
    const uint32_t nstages = (blocks + KS - 1) / KS;

    // Buffer descriptors: reads past the end of a region return zero instead
    // of faulting (the last stage of a row may extend past the row's end).
    const uint8_t *wq = d.w;
    const uint8_t *ws = d.w + (size_t)rows * cols;
    const uint8_t *xq = d.xq;
    const uint8_t *xs = d.xq + (size_t)batch * cols;
    const __amdgpu_buffer_rsrc_t rs_wq =
        __builtin_amdgcn_make_buffer_rsrc((void *)wq, 0, (uint32_t)((size_t)rows * cols), 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_ws = __builtin_amdgcn_make_buffer_rsrc(
        (void *)ws, 0, (uint32_t)((size_t)rows * blocks * 2u), 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_xq =
        __builtin_amdgcn_make_buffer_rsrc((void *)xq, 0, (uint32_t)((size_t)batch * cols), 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_xs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)xs, 0, (uint32_t)((size_t)blocks * bpad * 4u), 0x00020000);

    // One fetch instruction moves 64 pieces = 64 / pieces operand rows.
    constexpr int ROWS_PER_INSTR = 64 / Sh::pieces;
    const uint32_t f_row = lane / Sh::pieces, f_slot = lane % Sh::pieces;
    auto fetch = [&](uint32_t st, uint8_t *stage) {
        const uint32_t k0 = st * (KS * 32u);
        // activations: Sh::tokens rows of row_bytes
        for (uint32_t i = wave; i < (uint32_t)(Sh::tokens / ROWS_PER_INSTR); i += NW) {
            const uint32_t r = i * ROWS_PER_INSTR + f_row; // row within the tile
            uint32_t t = t0 + r;
            t = t < batch ? t : batch - 1u;
            const uint32_t piece = i8_swz<WM, WN, KS>(r, f_slot);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                rs_xq, (__attribute__((address_space(3))) void *)(stage + i * 1024u), 16,
                t * cols + k0 + piece * 16u, 0, 0, 0);
        }
        // weights
        for (uint32_t i = wave; i < (uint32_t)(Sh::rows / ROWS_PER_INSTR); i += NW) {
            const uint32_t r = i * ROWS_PER_INSTR + f_row;
            uint32_t n = n0 + r;
            n = n < rows ? n : rows - 1u;
            const uint32_t piece = i8_swz<WM, WN, KS>(r, f_slot);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                rs_wq, (__attribute__((address_space(3))) void *)(stage + Sh::a_bytes + i * 1024u),
                16, n * cols + k0 + piece * 16u, 0, 0, 0);
        }
        // activation scales: [block][token] f32, 4 tokens per lane
        for (uint32_t i = wave; i < (uint32_t)(Sh::dx_bytes / 1024); i += NW) {
            const uint32_t e = i * 256u + lane * 4u; // element index in [block][token]
            const uint32_t blk = e / Sh::tokens, tk = e % Sh::tokens;
            uint32_t t = t0 + tk;
            t = t + 4u <= bpad ? t : bpad - 4u;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                rs_xs,
                (__attribute__((address_space(3))) void *)(stage + Sh::a_bytes + Sh::b_bytes +
                                                           i * 1024u),
                16, ((st * KS + blk) * bpad + t) * 4u, 0, 0, 0);
        }
        // weight scales: f16 bits of [row][block], one per lane, widened to a dword each
        for (uint32_t i = wave; i < (uint32_t)(Sh::rows * KS / 64); i += NW) {
            const uint32_t e = i * 64u + lane;
            const uint32_t r = e / KS, blk = e % KS;
            uint32_t n = n0 + r;
            n = n < rows ? n : rows - 1u;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                rs_ws,
                (__attribute__((address_space(3))) void *)(stage + Sh::a_bytes + Sh::b_bytes +
                                                           Sh::dx_bytes + i * 256u),
                2, (n * blocks + st * KS + blk) * 2u, 0, 0, 0);
        }
    };

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

    auto compute = [&](uint32_t st, const uint8_t *stage) {
        const uint32_t nblk = blocks - st * KS < (uint32_t)KS ? blocks - st * KS : (uint32_t)KS;
        const uint8_t *sa = stage, *sb = stage + Sh::a_bytes;
        const float *sdx = (const float *)(stage + Sh::a_bytes + Sh::b_bytes);
        const uint32_t *sdw = (const uint32_t *)(stage + Sh::a_bytes + Sh::b_bytes + Sh::dx_bytes);
        for (uint32_t kb = 0; kb < nblk; ++kb) {
            const uint32_t p = kb * 2u + (g >> 1), half = (g & 1u) * 8u;
            long a[TM], b[TN];
            float4 dx[TM];
            float dw[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const uint32_t r = wm * (16u * TM) + 16u * i + i16;
                a[i] = *(const long *)(sa + r * Sh::row_bytes + i8_swz<WM, WN, KS>(r, p) * 16u + half);
                dx[i] = *(const float4 *)(sdx + kb * Sh::tokens + wm * (16u * TM) + 16u * i + 4u * g);
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const uint32_t r = wn * (16u * TN) + 16u * j + i16;
                b[j] = *(const long *)(sb + r * Sh::row_bytes + i8_swz<WM, WN, KS>(r, p) * 16u + half);
                dw[j] = f16_bits_to_f32(sdw[r * KS + kb] & 0xffffu);
            }
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const float dxv[4] = {dx[i].x, dx[i].y, dx[i].z, dx[i].w};
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const intx4 z = {0, 0, 0, 0};
                    const intx4 s = __builtin_amdgcn_mfma_i32_16x16x32_i8(a[i], b[j], z, 0, 0, 0);
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        // (d_w * d_x) * sumi, then the add: unfused, block order
                        const float scale = __fmul_rn(dw[j], dxv[v]);
                        if constexpr (FMA) {
                            acc[i][j][v] = __builtin_fmaf(scale, (float)s[v], acc[i][j][v]);
                        } else {
                            const float term = __fmul_rn(scale, (float)s[v]);
                            acc[i][j][v] = __fadd_rn(acc[i][j][v], term);
                        }
                    }
                }
            }
        }
    };

    // A wave fetches only its share of a stage and every wave reads all of it:
    // each wave waits for its own fetch (the only vector memory operations it
    // has in flight; the barrier alone does not wait for loads that land in
    // LDS), then all meet.
    auto landed = [&]() {
        __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8)); // vmcnt(0)
        __syncthreads();
    };
    fetch(0, stage_a);
    for (uint32_t st = 0; st < nstages; st += 2u) {
        landed(); // stage st is there for everyone; stage_b is free
        fetch(st + 1u < nstages ? st + 1u : st, stage_b);
        compute(st, stage_a);
        if (st + 1u < nstages) {
            landed();
            fetch(st + 2u < nstages ? st + 2u : st + 1u, stage_a);
            compute(st + 1u, stage_b);
        }
    }
    landed(); // no fetch may be in flight when the workgroup gives up its LDS

#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const uint32_t t = t0 + wm * (16u * TM) + 16u * i + 4u * g + v;
                const uint32_t n = n0 + wn * (16u * TN) + 16u * j + i16;
                if (t < batch && n < rows) {
                    d.y[(size_t)t * rows + n] = acc[i][j][v];
                }
            }
        }
    }
}

template <int WM, int WN, int KS, int TM = 4, int TN = 4, bool FMA = false>
inline hipError_t launch_i8_lds_cfg(hipStream_t stream, hipEvent_t stop, const I8Product *prods,
                                    int n) {
    using Sh = I8LdsShape<WM, WN, KS, TM, TN>;
    I8Args args;
    args.n = (uint32_t)n;
    uint64_t tiles = 0;
    for (int i = 0; i < n; ++i) {
        I8Desc &d = args.d[i];
        d.w = prods[i].w;
        d.xq = prods[i].xq;
        d.y = prods[i].y;
        d.sumi = nullptr;
        d.rows = prods[i].rows;
        d.cols = prods[i].cols;
        d.batch = prods[i].batch;
        d.tile_begin = (uint32_t)tiles;
        d.tiles_t = (prods[i].batch + Sh::tokens - 1) / Sh::tokens;
        d.pad = 0;
        tiles += (uint64_t)d.tiles_t * ((prods[i].rows + Sh::rows - 1) / Sh::rows);
    }
    args.total_tiles = (uint32_t)tiles;
    args.chunk_wgs = args.d[0].tiles_t;
    args.pad = 0;
    Q8_LAUNCH((gemm_i8_lds_kernel<WM, WN, KS, TM, TN, FMA>), dim3((unsigned)tiles),
              dim3(WM * WN * 64), 0, stream, stop, args);
    return hipGetLastError();
}

// Sealed weights, no verification output, every region below 4 GiB (32-bit
// buffer offsets): the caller checks these before choosing this kernel.
inline hipError_t launch_gemm_i8_lds_list(hipStream_t stream, hipEvent_t stop, int shape,
                                          const I8Product *prods, int n, bool fma = false) {
    if (n <= 0 || n > I8_MAX_DESCS) {
        return hipErrorInvalidValue;
    }
    if (fma) {
        switch (shape) {
        case 0: return launch_i8_lds_cfg<1, 4, 8, 1, 1, true>(stream, stop, prods, n);
        case 1: return launch_i8_lds_cfg<1, 4, 4, 2, 1, true>(stream, stop, prods, n);
        case 2: return launch_i8_lds_cfg<1, 4, 4, 3, 1, true>(stream, stop, prods, n);
        case 3: return launch_i8_lds_cfg<1, 4, 4, 4, 1, true>(stream, stop, prods, n);
        case 4: return launch_i8_lds_cfg<2, 2, 2, 4, 4, true>(stream, stop, prods, n);
        default: return hipErrorInvalidValue;
        }
    }
    switch (shape) {
    case 0: return launch_i8_lds_cfg<1, 4, 8, 1, 1>(stream, stop, prods, n);
    case 1: return launch_i8_lds_cfg<1, 4, 4, 2, 1>(stream, stop, prods, n);
    case 2: return launch_i8_lds_cfg<1, 4, 4, 3, 1>(stream, stop, prods, n);
    case 3: return launch_i8_lds_cfg<1, 4, 4, 4, 1>(stream, stop, prods, n);
    case 4: return launch_i8_lds_cfg<2, 2, 2, 4, 4>(stream, stop, prods, n);
    default: return hipErrorInvalidValue;
    }
}

} // namespace q8
