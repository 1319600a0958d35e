// Q8_0 prefill GEMM with f32 activations on the bf16 matrix cores, exact
// products ("split-float" form).
//
//   Y[t][n] = sum_b d[n][b] * sum_{k in block b} q[n][k] * X[t][k]
//
// The f32 MFMA kernel (q8_gemm_mma.hpp) is bound by the f32 matrix rate, which
// on this part equals the vector rate (157 TFLOP/s); bf16 MFMA is 16 times
// faster per instruction. An f32 activation is the exact sum of three bf16
// numbers (its 24-bit significand cut into 8 + 8 + 8 bits: h = trunc(x),
// m = trunc(x - h), l = x - h - m), a Q8_0 quant is exact in bf16, and an
// 8-bit by 8-bit product is exact in the MFMA's f32 accumulator. So
//     S = sum_k q*l + sum_k q*m + sum_k q*h        (three bf16 MFMAs per 16 k)
// accumulates, in f32, exactly the products q*x of one block, smallest pieces
// first, and  y += d * S  applies the block scale in f32 per output: no
// activation is rounded anywhere (unlike the int8-activation profile), only the
// order of the f32 additions differs from the CPU's, as for every MFMA kernel
// (contract: native/metal/tm_metal.h:172-175, tolerance-qualified).
// An infinite or NaN activation goes into the first piece whole (the other two
// are zero), so it reaches the outputs as it would through f32 products.
//
// Two kernels: split_act_list_kernel writes the three bf16 planes of every
// distinct X of a launch once; gemm_bf16x3_kernel is LDS-staged like the int8 GEMM
// (q8_gemm_i8_lds.hpp): a workgroup of WM x WN waves owns (WM*TM*32 tokens) x
// (WN*64 rows) of one K chunk (a tile whose K is cut into chunks is the sum of
// its chunks' partial tiles, added in chunk order by whichever chunk finishes
// last), walks K one Q8_0 block per stage, fetches every operand byte once per
// workgroup as 16-byte pieces straight into LDS (a ring of four stages,
// XOR-swizzled so that the operand reads are conflict-free) and each wave
// computes a (TM*32) x 64 tile as TM x 2 MFMA tiles of 32 x 32.
#pragma once

#include "q8_common.hpp"
#include "q8_gemm_mma.hpp"

namespace q8 {

typedef float floatx16_t __attribute__((ext_vector_type(16)));

// xs holds, per Q8_0 block kb and piece p (0 = h, 1 = m, 2 = l), the 32 bf16
// values of every token: [cols / 32][3][batch][32]. A workgroup's tokens of one
// block and piece are then one contiguous run, which its fetches read as whole
// cache lines.
struct SplitDesc {
    const float *x;   // [batch][cols], 16-byte aligned
    uint16_t *xs;
    uint32_t batch, cols;
    uint32_t wg_begin; // first workgroup of this input in the launch
    uint32_t pad;
};

struct SplitArgs {
    uint32_t n;
    uint32_t pad;
    SplitDesc d[SPLIT_MAX_DESCS];
};

// The distinct inputs of a launch's products, split once each (q/k/v and
// gate/up share theirs).
__global__ __launch_bounds__(256) void split_act_list_kernel(const SplitArgs args) {
    uint32_t which = 0;
    while (which + 1u < args.n && args.d[which + 1u].wg_begin <= blockIdx.x) {
        ++which;
    }
    const SplitDesc &d = args.d[which];
    const uint32_t batch = d.batch, cols = d.cols;
    const uint32_t i = ((blockIdx.x - d.wg_begin) * 256u + threadIdx.x) * 4u; // element of [batch][cols]
    if (i >= batch * cols) {
        return;
    }
    const uint32_t t = i / cols, k = i % cols; // cols is a multiple of 32: the 4 share a block
    const float4 v = *(const float4 *)(d.x + i);
    const float in[4] = {v.x, v.y, v.z, v.w};
    uint32_t h[4], m[4], l[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        split3_bf16(in[e], h[e], m[e], l[e]);
    }
    const size_t piece = (size_t)batch * 32u;
    uint16_t *dst = d.xs + split_index(batch, t, k);
    *(uint2 *)dst = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
    *(uint2 *)(dst + piece) = make_uint2(m[0] | (m[1] << 16), m[2] | (m[3] << 16));
    *(uint2 *)(dst + 2u * piece) = make_uint2(l[0] | (l[1] << 16), l[2] | (l[3] << 16));
}

struct Bx3Desc {
    const uint8_t *w;    // sealed weights
    const uint16_t *xs;  // the split activations of this product, [cols/32][3][batch][32] bf16
    float *y;            // y_off already applied
    uint32_t rows, cols, batch; // the whole matrix (rows: also the row stride of y)
    uint32_t row_begin, row_end; // the rows this descriptor computes (a product, or a segment of one)
    uint32_t tile_begin; // first work unit of this product in the launch
    uint32_t tiles_t;    // token tiles per row tile
    uint32_t chunks;     // K chunks per output tile (work units per tile)
    uint32_t chunk_blocks; // Q8_0 blocks per chunk
    uint32_t part_begin; // first arrival counter of this product (one per output tile)
    uint32_t part_tile;  // first partial tile of this product in `partials`
};

struct Bx3Args {
    uint32_t n;
    uint32_t total_tiles; // work units
    uint32_t chunk_wgs;
    uint32_t pad;
    float *partials;      // partial tiles [tile][chunk] of the products with chunks > 1
    uint32_t *arrivals;   // one counter per split tile, zero between launches
    Bx3Desc d[BX3_MAX_DESCS];
};

template <int WM, int WN, int TM> struct Bx3Shape {
    static constexpr int tokens = WM * TM * 32, rows = WN * 64;
    static constexpr int a_plane = tokens * 64;          // one plane: 32 bf16 = 64 bytes per token
    static constexpr int a_bytes = 3 * a_plane;
    static constexpr int b_bytes = rows * 32;            // 32 int8 per row
    static constexpr int dw_bytes = rows * 4;            // per row the dword that holds its f16 scale
    static constexpr int stage_bytes = a_bytes + b_bytes + dw_bytes;
};

// SEG: some descriptor of the launch covers a range of its product's rows only
// (a product with a tail segment, bx3_plan_launch). A separate instantiation:
// the two extra descriptor words in the plain kernel's addressing cost its
// hand-ordered loop 3-4 % (measured: 0.6B vocabulary at 512 tokens 505 -> 525 us).
template <int WM, int WN, int TM, int NS, bool SEG = false>
// (Two waves per SIMD, declared: with a register budget of 256 the compiler keeps
// the MFMA results in ordinary vector registers, which the rescale reads
// directly. With a single wave's budget it parked the small tile's results in
// accumulation registers and paid a v_accvgpr_read per result and block, 64 of
// the tile's 184 vector instructions per stage: 5-7 % slower.)
__global__ __launch_bounds__(WM * WN * 64, 2) void gemm_bf16x3_kernel(const Bx3Args args) {
    using Sh = Bx3Shape<WM, WN, TM>;
    constexpr int NW = WM * WN;
    constexpr int TN = 2; // a wave computes TM x 2 tiles of 32 x 32: 32*TM tokens x 64 rows
    // A ring of NS stage buffers. A buffer is refilled as soon as every wave has
    // taken what it needs of its block into registers (three quarters into the
    // block, see the main loop), so NS - 1 blocks are in flight or waiting while
    // one is being used (a fetch takes about three stages' worth of MFMAs to
    // arrive on the large tile, with one workgroup per CU; the small tile runs
    // two workgroups per CU with three buffers each).
    __shared__ __attribute__((aligned(16))) uint8_t stage_mem[NS][Sh::stage_bytes];

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t wm = wave / WN, wn = wave % WN;
    const uint32_t idx = lane & 31u, half = lane >> 5;

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
    const uint32_t tile = gidx; // one work unit (output tile x K chunk) per workgroup
    uint32_t lo = 0, hi = args.n;
    while (hi - lo > 1u) {
        const uint32_t mid = (lo + hi) >> 1;
        if (args.d[mid].tile_begin <= tile) {
            lo = mid;
        } else {
            hi = mid;
        }
    }
    const Bx3Desc &d = args.d[lo];
    const uint32_t rows = d.rows, cols = d.cols, batch = d.batch;
    const uint32_t unit = tile - d.tile_begin;
    const uint32_t chunks = d.chunks, chunk = unit % chunks, local = unit / chunks;
    const uint32_t t0 = (local % d.tiles_t) * Sh::tokens;
    // (SEG: rows of the tile at or beyond d.row_end, a segment's last tile, are
    // computed from the matrix's own rows there and not stored)
    const uint32_t n0 = (SEG ? d.row_begin : 0u) + (local / d.tiles_t) * Sh::rows;
    const uint32_t blocks = cols >> 5;
    const uint32_t kb_first = chunk * d.chunk_blocks;
    const uint32_t kb_last = kb_first + d.chunk_blocks < blocks ? kb_first + d.chunk_blocks : blocks;

    // Buffer descriptors (base, no stride, size in bytes, raw 32-bit format;
    // 32-bit offsets: the caller keeps every region below 4 GiB). Reads past a
    // region's end return zero instead of faulting.
    auto descriptor = [](const void *base, size_t bytes) {
        const uint64_t a = (uint64_t)(uintptr_t)base;
        const u32x4 r = {(uint32_t)a, (uint32_t)(a >> 32) & 0xffffu, (uint32_t)bytes, 0x00020000u};
        return r;
    };
    const u32x4 rs_wq = descriptor(d.w, (size_t)rows * cols);
    // (an odd number of scales ends inside the last dword: the two bytes behind
    // it are allocation slack, never a fault, and never used)
    const u32x4 rs_ws = descriptor(d.w + (size_t)rows * cols, (((size_t)rows * blocks + 1u) >> 1) * 4u);
    const u32x4 rs_x = descriptor(d.xs, (size_t)batch * cols * 6u);

    // The fetches are issued from inline assembly so that the compiler does not
    // order LDS reads after them itself: its bookkeeping for loads that land in
    // LDS waits for every such load in flight once a read cannot be matched to
    // one fetch, which would drain the ring at every stage. The kernel waits
    // by hand instead (`landed` below); there is no other vector memory
    // operation between the first fetch and the last wait.
    auto dma16 = [](const u32x4 &r, const uint8_t *lds, uint32_t lane_bytes, uint32_t block_bytes) {
        const uint32_t m = (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) uint8_t *)lds;
        asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                     :
                     : "s"(m), "v"(lane_bytes), "s"(r), "s"(block_bytes)
                     : "memory", "m0");
    };
    auto dma4 = [](const u32x4 &r, const uint8_t *lds, uint32_t lane_bytes) {
        const uint32_t m = (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) uint8_t *)lds;
        asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dword %1, %2, 0 offen lds"
                     :
                     : "s"(m), "v"(lane_bytes), "s"(r)
                     : "memory", "m0");
    };
    // What a lane fetches does not change from block to block except for the
    // block's byte offset, which rides in the instruction's scalar offset.
    constexpr int NA = 3 * Sh::tokens / 16 / NW, NB = Sh::rows / 32 / NW;
    uint32_t a_lane[NA], b_lane[NB], dw_first;
#pragma unroll
    for (int u = 0; u < NA; ++u) {
        const uint32_t i = wave + (uint32_t)(u * NW);
        const uint32_t pl = i / (Sh::tokens / 16), ri = i % (Sh::tokens / 16);
        const uint32_t r = ri * 16u + (lane >> 2);
        uint32_t t = t0 + r;
        t = t < batch ? t : batch - 1u;
        const uint32_t piece = (lane & 3u) ^ ((r >> 2) & 3u);
        a_lane[u] = ((pl * batch + t) * 32u + piece * 8u) * 2u;
    }
#pragma unroll
    for (int u = 0; u < NB; ++u) {
        const uint32_t i = wave + (uint32_t)(u * NW);
        const uint32_t r = i * 32u + (lane >> 1);
        uint32_t n = n0 + r;
        n = n < rows ? n : rows - 1u;
        const uint32_t piece = (lane & 1u) ^ ((r >> 3) & 1u);
        b_lane[u] = n * cols + piece * 16u;
    }
    {
        // Weight scales: per row the aligned dword that contains the f16 scale of
        // the block (element e = row * blocks + kb lives in dword e / 2, half
        // e % 2), one row per lane. Every wave issues one such fetch per block
        // (waves beyond rows / 64 repeat a piece: same bytes, same place).
        uint32_t n = n0 + (wave % (uint32_t)(Sh::rows / 64)) * 64u + lane;
        n = n < rows ? n : rows - 1u;
        dw_first = n * blocks;
    }
    const uint32_t a_block_bytes = __builtin_amdgcn_readfirstlane(batch * 192u);
    auto fetch = [&](uint32_t kb_in, uint8_t *stage) {
        // (fully unrolled: the number of fetch instructions per block is a
        // compile-time constant, which the wait counters below rely on)
        const uint32_t kb = __builtin_amdgcn_readfirstlane(kb_in); // scalar operand of the fetches
#pragma unroll
        for (int u = 0; u < NA; ++u) {
            dma16(rs_x, stage + (wave + (uint32_t)(u * NW)) * 1024u, a_lane[u], kb * a_block_bytes);
        }
#pragma unroll
        for (int u = 0; u < NB; ++u) {
            dma16(rs_wq, stage + Sh::a_bytes + (wave + (uint32_t)(u * NW)) * 1024u, b_lane[u], kb * 32u);
        }
        dma4(rs_ws, stage + Sh::a_bytes + Sh::b_bytes + (wave % (uint32_t)(Sh::rows / 64)) * 256u,
             ((dw_first + kb) >> 1) * 4u);
    };

    floatx16_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                acc[i][j][v] = 0.0f;
            }
        }
    }

    uint32_t row_odd[TN]; // parity of this lane's first scale element per row tile
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        uint32_t n = n0 + wn * 64u + 32u * j + idx;
        n = n < rows ? n : rows - 1u;
        row_odd[j] = (n * blocks) & 1u;
    }

    // MFMA step m takes from lane (idx, half) the 8 values k = 16*half + 8m + 0..7
    // of token / weight row idx (any assignment of a block's 32 k to the two
    // steps' lanes does, as long as both operands use it): a lane's 16 quants of
    // a weight row are then one 16-byte piece, read in one go.

    // Every wave issues the same number of fetch instructions per block, so
    // "all but the newest NS - 2 blocks have landed" is one counter value.
    constexpr int F = NA + NB + 1;
    static_assert((3 * Sh::tokens / 16) % NW == 0 && (Sh::rows / 32) % NW == 0, "uniform fetch");
    constexpr int IN_FLIGHT = (NS - 2) * F; // fetches of the newest NS - 2 blocks
    static_assert(IN_FLIGHT < 64, "vmcnt field");
    constexpr int WAIT_OLDEST_BLOCK =
        (IN_FLIGHT & 15) | ((IN_FLIGHT >> 4) << 14) | (7 << 4) | (15 << 8);
    auto landed = [&]() {
        // this wave's fetch of the block about to be used is complete ...
        __builtin_amdgcn_s_waitcnt(WAIT_OLDEST_BLOCK);
        // ... everybody's is, and everybody is done with the previous block's buffer
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    auto at = [&](uint32_t kb) { return kb < kb_last ? kb : kb_last - 1u; };
#pragma unroll
    for (int u = 0; u < NS - 1; ++u) {
        fetch(at(kb_first + (uint32_t)u), stage_mem[u]);
    }
    {
        // The instruction order of a block is written out (scheduling barriers pin
        // it). A wave's vector instructions hide under MFMAs only where they sit
        // between the MFMAs of its own instruction stream (measured with a
        // stand-alone co-issue loop: four independent vector instructions per
        // 32-cycle MFMA cost nothing there, while a wave that only issues MFMAs
        // keeps the SIMD's issue port and the partner wave's vector work waits),
        // so every MFMA is followed by a piece of the next weight rows'
        // conversion, a few rescale FMAs of the chain before it, or one of the
        // refill's fetch instructions.
        //
        // The loop is rotated by a quarter block, so that a wave's MFMAs run on
        // across block boundaries: the barrier that hands a block over sits
        // between the third and the fourth of a block's MFMA chains. By then a
        // wave holds everything it still needs of block k in registers, so behind
        // that barrier block k's buffer is refilled at once (one block more in
        // flight than the buffers would otherwise allow), and the first operands
        // of block k + 1 (the first token tile's planes, the first row tile's
        // weights) are read and converted under the fourth chain's MFMAs, into
        // the registers the first chains have just given up. The rescale of a
        // block's fourth chain rides in the next block's first. Together 2-3 %
        // faster than the compiler's own order of the plain loop (which issues
        // runs of eight and more MFMAs back to back and the conversions on their
        // own in front of them).
        static_assert(TM == 2 && TN == 2 && F <= 6, "written for 2 x 2 tiles per wave");
        const floatx16_t zero = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f,
                                 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        const uint32_t r0 = wn * 64u + idx, r1 = r0 + 32u, ta0 = wm * 64u + idx, ta1 = ta0 + 32u;
        auto load_a = [&](const uint8_t *stage, bf16x8_t (&a)[3][2], uint32_t r) {
#pragma unroll
            for (int pl = 0; pl < 3; ++pl) {
#pragma unroll
                for (int m = 0; m < 2; ++m) {
                    const uint32_t slot = (2u * half + (uint32_t)m) ^ ((r >> 2) & 3u);
                    a[pl][m] = *(const bf16x8_t *)(stage + pl * Sh::a_plane + r * 64u + slot * 16u);
                }
            }
        };
        auto rd_raw = [&](const uint8_t *stage, uint32_t r) {
            return *(const u32x4 *)(stage + Sh::a_bytes + r * 32u + (half ^ ((r >> 3) & 1u)) * 16u);
        };
        auto rd_pair = [&](const uint8_t *stage, uint32_t r) {
            return ((const uint32_t *)(stage + Sh::a_bytes + Sh::b_bytes))[r];
        };
        auto scale_of = [&](uint32_t pair, int j, uint32_t kb) {
            return f16_bits_to_f32(((row_odd[j] + kb) & 1u) ? pair >> 16 : pair & 0xffffu);
        };
        auto two = [](uint32_t w, int i) { // bytes 2i, 2i+1 of w as two bf16
            const uint32_t f0 = __builtin_bit_cast(uint32_t, sbyte_to_float(w, 2 * i));
            const uint32_t f1 = __builtin_bit_cast(uint32_t, sbyte_to_float(w, 2 * i + 1));
            return __builtin_amdgcn_perm(f1, f0, 0x07060302u);
        };
        auto pack = [](uint32_t p0, uint32_t p1, uint32_t p2, uint32_t p3) {
            const u32x4 v = {p0, p1, p2, p3};
            return __builtin_bit_cast(bf16x8_t, v);
        };
        auto fetch_piece = [&](int i, uint32_t kb_in, uint8_t *stage) { // the i-th of a block's F fetches
            const uint32_t kb = __builtin_amdgcn_readfirstlane(kb_in);
            if (i < NA) {
                dma16(rs_x, stage + (wave + (uint32_t)(i * NW)) * 1024u, a_lane[i < NA ? i : 0], kb * a_block_bytes);
            } else if (i < NA + NB) {
                dma16(rs_wq, stage + Sh::a_bytes + (wave + (uint32_t)((i - NA) * NW)) * 1024u,
                      b_lane[i < NA + NB && i >= NA ? i - NA : 0], kb * 32u);
            } else if (i == NA + NB) {
                dma4(rs_ws, stage + Sh::a_bytes + Sh::b_bytes + (wave % (uint32_t)(Sh::rows / 64)) * 256u,
                     ((dw_first + kb) >> 1) * 4u);
            }
        };
#define BX3_SB __builtin_amdgcn_sched_barrier(0)
#define BX3_MFMA(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0)
        auto fma4 = [](floatx16_t &into, const floatx16_t &prev, float dw, int g) {
#pragma unroll
            for (int v = 4 * g; v < 4 * g + 4; ++v) {
                into[v] = __builtin_fmaf(dw, prev[v], into[v]);
            }
        };
        // a chain of six MFMAs with the rescale of the chain before it in between
        auto chain = [&](const bf16x8_t (&a)[3][2], const bf16x8_t &bA, const bf16x8_t &bB,
                         const floatx16_t &prev, float prev_dw, floatx16_t &into) {
            floatx16_t t = BX3_MFMA(a[2][0], bA, zero);
            BX3_SB;
            t = BX3_MFMA(a[2][1], bB, t);
            BX3_SB;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                t = BX3_MFMA(a[1 - g / 2][g % 2], g % 2 ? bB : bA, t);
                fma4(into, prev, prev_dw, g);
                BX3_SB;
            }
            return t;
        };

        bf16x8_t a0[3][2], a1[3][2], b00, b01, b10, b11;
        u32x4 raw1;
        uint32_t pair1;
        float dw0, dw_last = 0.0f;
        floatx16_t t = zero; // a block's fourth chain, rescaled under the next block's first
        {
            landed();
            fetch(at(kb_first + (uint32_t)(NS - 1)), stage_mem[NS - 1]);
            load_a(stage_mem[0], a0, ta0);
            const u32x4 raw0 = rd_raw(stage_mem[0], r0);
            raw1 = rd_raw(stage_mem[0], r1);
            const uint32_t pair0 = rd_pair(stage_mem[0], r0);
            pair1 = rd_pair(stage_mem[0], r1);
            b00 = pack(two(raw0.x, 0), two(raw0.x, 1), two(raw0.y, 0), two(raw0.y, 1));
            b01 = pack(two(raw0.z, 0), two(raw0.z, 1), two(raw0.w, 0), two(raw0.w, 1));
            dw0 = scale_of(pair0, 0, kb_first);
            BX3_SB;
        }
        for (uint32_t kb = kb_first; kb < kb_last; kb += (uint32_t)NS) {
#pragma unroll
            for (int u = 0; u < NS; ++u) {
                const uint32_t k = kb + (uint32_t)u;
                if (k < kb_last) { // (uniform over the workgroup)
                    uint8_t *cur = stage_mem[u];
                    const uint8_t *nxt = stage_mem[(u + 1) % NS];
                    // chain (0, 0): the second token tile's planes are read, the second row
                    // tile's weights converted and the last block's fourth chain rescaled on the way
                    floatx16_t s = BX3_MFMA(a0[2][0], b00, zero);
                    load_a(cur, a1, ta1);
                    const uint32_t q0 = two(raw1.x, 0), q1 = two(raw1.x, 1);
                    BX3_SB;
                    s = BX3_MFMA(a0[2][1], b01, s);
                    const uint32_t q2 = two(raw1.y, 0), q3 = two(raw1.y, 1);
                    BX3_SB;
                    s = BX3_MFMA(a0[1][0], b00, s);
                    fma4(acc[1][1], t, dw_last, 0);
                    const uint32_t q4 = two(raw1.z, 0);
                    BX3_SB;
                    s = BX3_MFMA(a0[1][1], b01, s);
                    fma4(acc[1][1], t, dw_last, 1);
                    const uint32_t q5 = two(raw1.z, 1);
                    BX3_SB;
                    s = BX3_MFMA(a0[0][0], b00, s);
                    fma4(acc[1][1], t, dw_last, 2);
                    const uint32_t q6 = two(raw1.w, 0);
                    BX3_SB;
                    s = BX3_MFMA(a0[0][1], b01, s);
                    fma4(acc[1][1], t, dw_last, 3);
                    const uint32_t q7 = two(raw1.w, 1);
                    b10 = pack(q0, q1, q2, q3);
                    b11 = pack(q4, q5, q6, q7);
                    const float dw1 = scale_of(pair1, 1, k);
                    BX3_SB;
                    t = chain(a1, b00, b01, s, dw0, acc[0][0]); // chain (1, 0)
                    s = chain(a0, b10, b11, t, dw0, acc[1][0]);            // chain (0, 1)
                    if (k + 1u < kb_last) {
                        // block k + 1 has landed for everybody, and nobody reads block k's buffer again
                        landed();
                        load_a(nxt, a0, ta0);
                        const u32x4 raw0 = rd_raw(nxt, r0);
                        raw1 = rd_raw(nxt, r1);
                        const uint32_t pair0 = rd_pair(nxt, r0);
                        pair1 = rd_pair(nxt, r1);
                        const uint32_t refill = at(k + (uint32_t)NS);
                        BX3_SB;
                        // chain (1, 1)
                        t = BX3_MFMA(a1[2][0], b10, zero);
                        fetch_piece(0, refill, cur);
                        BX3_SB;
                        t = BX3_MFMA(a1[2][1], b11, t);
                        fetch_piece(1, refill, cur);
                        BX3_SB;
                        t = BX3_MFMA(a1[1][0], b10, t);
                        fetch_piece(2, refill, cur);
                        fma4(acc[0][1], s, dw1, 0);
                        const uint32_t p0 = two(raw0.x, 0), p1 = two(raw0.x, 1);
                        BX3_SB;
                        t = BX3_MFMA(a1[1][1], b11, t);
                        fetch_piece(3, refill, cur);
                        fma4(acc[0][1], s, dw1, 1);
                        const uint32_t p2 = two(raw0.y, 0), p3 = two(raw0.y, 1);
                        BX3_SB;
                        t = BX3_MFMA(a1[0][0], b10, t);
                        fetch_piece(4, refill, cur);
                        fma4(acc[0][1], s, dw1, 2);
                        const uint32_t p4 = two(raw0.z, 0), p5 = two(raw0.z, 1);
                        BX3_SB;
                        t = BX3_MFMA(a1[0][1], b11, t);
                        fetch_piece(5, refill, cur);
                        fma4(acc[0][1], s, dw1, 3);
                        const uint32_t p6 = two(raw0.w, 0), p7 = two(raw0.w, 1);
                        b00 = pack(p0, p1, p2, p3);
                        b01 = pack(p4, p5, p6, p7);
                        dw0 = scale_of(pair0, 0, k + 1u);
                        BX3_SB;
                    } else {
                        t = chain(a1, b10, b11, s, dw1, acc[0][1]); // chain (1, 1) of the last block
                    }
                    dw_last = dw1;
                }
            }
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            acc[1][1][v] = __builtin_fmaf(dw_last, t[v], acc[1][1][v]);
        }
#undef BX3_MFMA
#undef BX3_SB
    }
    __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8)); // vmcnt(0): every fetch has landed
    __syncthreads(); // ... before the workgroup gives up its LDS

    // A tile whose K is cut into chunks: every chunk's workgroup parks its
    // partial tile; the one that arrives last adds the partial tiles in chunk
    // order (whoever it is: the result does not depend on the order of arrival)
    // and stores the sum. The arrival counter goes back to zero for the next launch.
    if (chunks > 1u) {
        constexpr uint32_t TILE_FLOATS = (uint32_t)NW * TM * TN * 16u * 64u;
        const uint32_t slot = d.part_begin + local;
        const size_t first_tile = (size_t)d.part_tile + (size_t)local * chunks;
        float *mine = args.partials + (first_tile + chunk) * TILE_FLOATS +
                      (size_t)wave * (TM * TN * 16u * 64u) + lane;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    __hip_atomic_store(mine + ((i * TN + j) * 16 + v) * 64, acc[i][j][v], __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                }
            }
        }
        // The partial tiles go to memory and come back from it with device-scope
        // accesses that bypass this XCD's L2, so all it takes to publish them is
        // to wait for the stores before the arrival is counted: no fence, which
        // would write back and invalidate the whole L2 under the other
        // workgroups' feet (measured: 14336 x 4096 in four chunks 481 us with
        // fences).
        __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8)); // vmcnt(0)
        asm volatile("" ::: "memory");
        __shared__ uint32_t arrived;
        __syncthreads();
        if (threadIdx.x == 0u) {
            arrived = __hip_atomic_fetch_add(&args.arrivals[slot], 1u, __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (arrived != chunks - 1u) {
            return;
        }
        // (the loads below are issued after the count has come back; this keeps
        // the compiler from moving them above the branch)
        asm volatile("" ::: "memory");
        if (threadIdx.x == 0u) {
            __hip_atomic_store(&args.arrivals[slot], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        const float *first = args.partials + first_tile * TILE_FLOATS +
                             (size_t)wave * (TM * TN * 16u * 64u) + lane;
        for (uint32_t c = 0; c < chunks; ++c) {
            const float *part = first + (size_t)c * TILE_FLOATS;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
#pragma unroll
                for (int j = 0; j < TN; ++j) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const float pv = __hip_atomic_load(part + ((i * TN + j) * 16 + v) * 64,
                                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        acc[i][j][v] = c == 0u ? pv : acc[i][j][v] + pv;
                    }
                }
            }
        }
    }

    // acc[v] of a 32x32 tile is (token 8*(v/4) + 4*half + v%4, row idx).
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const uint32_t n = n0 + wn * 64u + 32u * j + idx;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t t = t0 + wm * (32u * TM) + 32u * i + 8u * (v / 4) + 4u * half + (v % 4);
                if (t < batch && n < (SEG ? d.row_end : rows)) {
                    d.y[(size_t)t * rows + n] = acc[i][j][v];
                }
            }
        }
    }
}

struct Bx3Product {
    const uint8_t *w;
    const uint16_t *xs;
    float *y;
    uint32_t rows, cols, batch;
    uint32_t chunks; // K chunks of this product, as bx3_plan_launch cut the launch
    // the rows to compute: the whole product (0, rows), or one of the two
    // segments of a product with a tail (bx3_plan_launch)
    uint32_t row_begin, row_end;
};

template <int WM, int WN, int TM, int NS>
inline hipError_t launch_bx3_cfg(hipStream_t stream, hipEvent_t stop, const Bx3Product *prods_in,
                                 int n, float *partials, uint32_t *arrivals) {
    using Sh = Bx3Shape<WM, WN, TM>;
    static_assert(Sh::rows == (int)BX3_TILE_ROWS, "tile");
    Bx3Args args;
    args.n = (uint32_t)n;
    args.partials = partials;
    args.arrivals = arrivals;
    // Longest work unit first (the order of the list changes no product's
    // result). A unit is an output tile x K chunk and lasts one stage per Q8_0
    // block of its chunk; the chip takes units in list order as workgroups
    // retire, so the long ones must not come last. Products whose K is cut into
    // chunks have the SHORT units: listed by K, the seven projections of a
    // Qwen3-0.6B layer at 512 tokens (160 units of 32 stages, 160 of 16) ran
    // the short ones first and finished after 48 stages; long ones first, 32.
    Bx3Product prods[BX3_MAX_DESCS];
    uint32_t unit_blocks[BX3_MAX_DESCS];
    for (int i = 0; i < n; ++i) {
        if (prods_in[i].row_begin >= prods_in[i].row_end || prods_in[i].row_end > prods_in[i].rows ||
            prods_in[i].row_begin % (uint32_t)Sh::rows != 0u) {
            return hipErrorInvalidValue;
        }
        const uint32_t mine = bx3_plan_chunked(prods_in[i].row_end - prods_in[i].row_begin, prods_in[i].cols,
                                               prods_in[i].batch, (uint32_t)Sh::tokens,
                                               prods_in[i].chunks).chunk_blocks;
        int at = i;
        while (at > 0 && (unit_blocks[at - 1] < mine ||
                          (unit_blocks[at - 1] == mine && prods[at - 1].cols < prods_in[i].cols))) {
            prods[at] = prods[at - 1];
            unit_blocks[at] = unit_blocks[at - 1];
            --at;
        }
        prods[at] = prods_in[i];
        unit_blocks[at] = mine;
    }
    uint64_t units = 0, split_tiles = 0, partial_tiles = 0;
    for (int i = 0; i < n; ++i) {
        Bx3Desc &d = args.d[i];
        d.w = prods[i].w;
        d.xs = prods[i].xs;
        d.y = prods[i].y;
        d.rows = prods[i].rows;
        d.row_begin = prods[i].row_begin;
        d.row_end = prods[i].row_end;
        d.cols = prods[i].cols;
        d.batch = prods[i].batch;
        d.tile_begin = (uint32_t)units;
        // K chunks as the launch was cut
        const uint32_t seg_rows = prods[i].row_end - prods[i].row_begin;
        const Bx3Plan plan = bx3_plan_chunked(seg_rows, prods[i].cols, prods[i].batch,
                                              (uint32_t)Sh::tokens, prods[i].chunks);
        d.tiles_t = (prods[i].batch + Sh::tokens - 1) / Sh::tokens;
        d.chunk_blocks = plan.chunk_blocks;
        d.chunks = plan.chunks;
        d.part_begin = (uint32_t)split_tiles;
        d.part_tile = (uint32_t)partial_tiles;
        const uint64_t tiles = (uint64_t)d.tiles_t * ((seg_rows + Sh::rows - 1) / Sh::rows);
        units += tiles * d.chunks;
        if (d.chunks > 1u) {
            split_tiles += tiles;
            partial_tiles += tiles * d.chunks;
        }
    }
    if (units == 0 || units > 0x7fffffffull || split_tiles > BX3_MAX_SPLIT_TILES ||
        (split_tiles > 0 && (partials == nullptr || arrivals == nullptr))) {
        return hipErrorInvalidValue;
    }
    args.total_tiles = (uint32_t)units;
    args.chunk_wgs = args.d[0].tiles_t * args.d[0].chunks;
    args.pad = 0;
    bool segments = false;
    for (int i = 0; i < n; ++i) {
        segments = segments || prods[i].row_begin != 0u || prods[i].row_end != prods[i].rows;
    }
    if (segments) {
        Q8_LAUNCH((gemm_bf16x3_kernel<WM, WN, TM, NS, true>), dim3((unsigned)units), dim3(WM * WN * 64), 0,
                  stream, stop, args);
    } else {
        Q8_LAUNCH((gemm_bf16x3_kernel<WM, WN, TM, NS, false>), dim3((unsigned)units), dim3(WM * WN * 64), 0,
                  stream, stop, args);
    }
    return hipGetLastError();
}

// Sealed weights, every region below 4 GiB (32-bit buffer offsets): the caller
// checks these before choosing this kernel; every product carries the chunk
// count bx3_plan_launch gave it. `partials` holds the sum of the products' partial_floats,
// `arrivals` BX3_MAX_SPLIT_TILES counters that are zero between launches (both
// may be null when no product's K is cut into chunks).
inline hipError_t launch_gemm_bf16x3_list(hipStream_t stream, hipEvent_t stop, uint32_t tile_tokens,
                                          const Bx3Product *prods, int n, float *partials,
                                          uint32_t *arrivals) {
    if (n <= 0 || n > BX3_MAX_DESCS) {
        return hipErrorInvalidValue;
    }
    switch (tile_tokens) {
    case 128: return launch_bx3_cfg<2, 4, 2, 4>(stream, stop, prods, n, partials, arrivals);
    case 64: return launch_bx3_cfg<1, 4, 2, 3>(stream, stop, prods, n, partials, arrivals);
    default: return hipErrorInvalidValue;
    }
}

struct SplitInput {
    const float *x;
    uint16_t *xs;
    uint32_t batch, cols;
};

// Every input: cols a positive multiple of 32, x 16-byte aligned, batch * cols below 2^30.
inline hipError_t launch_split_act_list(hipStream_t stream, const SplitInput *in, int n) {
    if (n <= 0 || n > SPLIT_MAX_DESCS) {
        return hipErrorInvalidValue;
    }
    SplitArgs args;
    args.n = (uint32_t)n;
    args.pad = 0;
    uint32_t wgs = 0;
    for (int i = 0; i < n; ++i) {
        if (in[i].batch == 0 || in[i].cols == 0 || (in[i].cols & 31u) != 0u ||
            (uint64_t)in[i].batch * in[i].cols >= (1ull << 30)) {
            return hipErrorInvalidValue;
        }
        args.d[i] = SplitDesc{in[i].x, in[i].xs, in[i].batch, in[i].cols, wgs, 0};
        wgs += (in[i].batch * in[i].cols / 4u + 255u) / 256u;
    }
    hipLaunchKernelGGL(split_act_list_kernel, dim3(wgs), dim3(256), 0, stream, args);
    return hipGetLastError();
}

} // namespace q8
