// Small-batch Q8_0 product with the GEMV's arithmetic (2 <= batch <= 32,
// cols >= 1024; sealed weights, or raw ones with cols a multiple of 1024): the exact / speculative-verify
// path (contract: native/metal/tm_metal.h:161-164,
// crates/tuckcore/src/engine/metal.rs:81-83).
//
// At these batch sizes the product is bound by f32 vector multiply-adds and by
// registers, not by HBM: a lane needs batch x 16 activations per weight piece.
// So the NW waves of a workgroup share one tile of rows and split the TOKENS:
// wave w owns tokens w*TW .. w*TW+TW-1. The weights of a step (8 rows x 1024
// columns) are fetched once per workgroup straight into LDS (buffer_load ...
// lds, 16 bytes per lane: no registers are held while the data is in flight),
// double-buffered, and every wave reads its lane's 16 quants of each row back
// with one ds_read_b128. A wave then keeps only 8 x TW accumulators and TW x 16
// activations in registers, and a weight byte is converted once per wave.
//
// Per-(row, token) arithmetic is exactly the decode kernel's (q8_gemv.hpp):
// the lane -> column mapping, the left-to-right fused multiply-adds over a
// lane's 16 quants, one fused multiply-add per block scale with chunks in
// ascending order, and the same butterfly; every token is bit-identical to its
// own GEMV.
#pragma once

#include "q8_gemv.hpp"

namespace q8 {

constexpr int SMALL_R = 8; // rows per step

// TAIL: some product of the launch has cols % 1024 != 0 (kept out of the
// common instantiation: the tail code costs registers even when it never runs).
// Two waves per SIMD are declared: left to itself the 8-token tail variant
// takes a single wave's budget (256 registers and 71 more parked in accumulation
// registers, one wave per SIMD); held to 256 it keeps 72 dwords per lane in
// scratch memory instead and is still 22 % faster on the Gemma FFN shapes at
// 17-32 tokens, because the second wave hides the first one's waits.
//
// L == RAW: weights as uploaded (34-byte blocks), cols a multiple of 64 (rows
// start dword aligned). A row's chunk is then 1088 bytes, fetched into LDS as 68
// 16-byte pieces (a second, four-lane fetch per row brings the last 64 bytes);
// a lane reads back the five aligned dwords that hold its 16 quants and moves
// the bytes into place, and the block's scale comes out of the same bytes
// (q8_gemv.hpp's stream_rows_raw has the details). The arithmetic is the sealed
// form's.
//
// R: rows per step, 8, or 4 for launches of few rows under a long K (a product
// of 4096 x 14336 has 512 workgroups of 8 rows on 256 CUs, each with one step
// of 8 KB on its way: with 4 rows a step it has 1024).
template <int L, int NW, int TW, bool XA, bool TAIL, int R = SMALL_R>
__global__ __launch_bounds__(NW * 64, 2) void gemm_split_list_kernel(const GemvArgs args) {
    static_assert(R == 8 || R == 4, "rows per step");
    static_assert(R % NW == 0, "every wave fetches whole rows of a step");
    constexpr uint32_t ROWB = L == PACKED ? 1024u : RAW_CHUNK_BYTES; // a staged row
    // One wave with two tokens (the big launches of a two-token step) is short of
    // bytes in flight, not of registers: with all 8 rows of a step in LDS, LDS
    // holds 10 workgroups per CU, 80 KB on their way at any time, where the
    // one-token kernel has 128 KB. Half of the rows of a step then travel
    // through registers instead (SR rows staged, R - SR loaded by the lanes
    // directly), which halves the workgroup's LDS and lets 16 of them run: 128 KB
    // on their way, 127 registers (2 B-class shapes, 535 MB at two tokens:
    // 113 -> 105 us). With four tokens per wave the same (6 rows staged, 163
    // registers, 96 KB) gains nothing measurable: that form waits for its
    // multiply-adds, and keeps all rows in LDS. The column-tail variant
    // would fall to two waves per SIMD.
    constexpr bool HYBRID = NW == 1 && TW == 2 && L == PACKED && !TAIL && R == 8;
    constexpr int SR = HYBRID ? R / 2 : R; // rows of a step that go through LDS
    constexpr int DR = HYBRID ? R - SR : 1; // rows of a step loaded directly (1: unused)
    // Two separate objects (not one array indexed by parity): the compiler then
    // sees that reads of one buffer cannot alias the fetch into the other and
    // does not wait for the prefetch before reading.
    __shared__ __attribute__((aligned(16))) uint8_t stage_a[SR * ROWB];
    __shared__ __attribute__((aligned(16))) uint8_t stage_b[SR * ROWB];
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t tile = blockIdx.x; // one tile per workgroup; the grid is exactly total_tiles
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
    const uint32_t nsteps = ((row_end - row_first + R - 1) / R) * full;

    uint32_t xoff[TW], tok[TW];
    bool tok_ok[TW];
#pragma unroll
    for (int t = 0; t < TW; ++t) {
        const uint32_t tk = wave * TW + t;
        tok_ok[t] = tk < batch;
        tok[t] = tok_ok[t] ? tk : batch - 1u;
        xoff[t] = tok[t] * cols + lane * 16u;
    }
    const bool has_tokens = wave * TW < batch; // wave-uniform

    // Wave w fetches rows 2w and 2w+1 of a step; lane l's 16 bytes land at
    // row * 1024 + l * 16 of the stage buffer. The fetch is a buffer load (not
    // a global one): the compiler's wait-count bookkeeping treats a global
    // load into LDS as a flat access and would make every later wait drain
    // the prefetch too. The descriptor covers the tile's quants only.
    const uint32_t row_stride = L == PACKED ? cols : (cols >> 5) * 34u; // bytes from row to row
    const uint8_t *tile_q;
    if constexpr (L == PACKED) {
        tile_q = wv.q + (size_t)row_first * row_stride;
    } else {
        tile_q = wv.base + (size_t)row_first * row_stride;
    }
    const size_t tile_len = (size_t)(row_end - row_first) * row_stride;
    const __amdgpu_buffer_rsrc_t tile_rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)tile_q, 0, tile_len > 0xffffffffull ? 0xffffffffu : (uint32_t)tile_len, 0x00020000);
    auto fetch = [&](uint32_t r0, uint32_t c, uint8_t *stage) {
#pragma unroll
        for (int i = 0; i < SR / NW; ++i) {
            const uint32_t r = wave * (SR / NW) + i;
            const uint32_t row = (r0 + r < row_end) ? r0 + r : row_end - 1u;
            const uint32_t base =
                __builtin_amdgcn_readfirstlane((row - row_first) * row_stride + c * ROWB);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                tile_rs, (__attribute__((address_space(3))) void *)(stage + r * ROWB), 16,
                lane * 16u, base, 0, 0);
            if constexpr (L == RAW) {
                if (lane < 4u) { // bytes 1024..1087 of the row's chunk
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(
                        tile_rs,
                        (__attribute__((address_space(3))) void *)(stage + r * ROWB + 1024u), 16,
                        lane * 16u + 1024u, base, 0, 0);
                }
            }
        }
    };
    // (the rows of a step that do not go through LDS: rows SR .. R-1)
    auto load_direct = [&](uint32_t r0, uint32_t c, uint32_t (&qq)[DR][4]) {
#pragma unroll
        for (int r = SR; r < R; ++r) {
            const uint32_t row = (r0 + r < row_end) ? r0 + r : row_end - 1u;
            wv.template load_quants<16, true>(row, (c << 10) + lane * 16u, qq[r - SR]);
        }
    };
    auto load_scales = [&](uint32_t r0, uint32_t c, uint32_t (&ss)[R]) {
        if constexpr (L == PACKED) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint32_t row = (r0 + r < row_end) ? r0 + r : row_end - 1u;
                ss[r] = wv.scale_bits(row, (c << 5) + (lane >> 1));
            }
        }
    };
    // raw layout: this lane's window in a staged row (see stream_rows_raw)
    const uint32_t raw_off = (lane >> 1) * 34u + (lane & 1u) * 16u;
    const bool raw_high = (raw_off & 2u) != 0u;
    const uint32_t raw_sel = raw_high ? 0x07060504u : 0x05040302u;

    uint32_t sb[R], sn[R];
    uint32_t qd[DR][4], qdn[DR][4]; // this step's and the next one's direct rows
    fetch(row_first, 0, stage_a);
    if constexpr (HYBRID) {
        load_direct(row_first, 0, qd);
    }
    load_scales(row_first, 0, sb);
    uint32_t r0 = row_first, c = 0;
    float acc[R][TW];
    auto do_step = [&](uint32_t step, uint8_t *cur, uint8_t *nxt) {
        // The fetch of this step has landed: each wave waits for its own part
        // (the barrier alone does not wait for loads that land in LDS; the
        // scale loads requested with them are as old and come back with them),
        // then all meet, and every wave has finished reading the other buffer.
        __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8)); // vmcnt(0)
        __syncthreads();
        uint32_t cn = c + 1u, rn = r0;
        if (cn == full) {
            cn = 0;
            rn = r0 + R;
        }
        // This step's activations are requested before the next step's
        // weights: the memory counter retires in order, and the multiplies
        // below must not wait for the prefetch.
        // This step's activations are requested before the next step's
        // weights: the memory counter retires in order, and the multiplies
        // below must not wait for the prefetch. (Requesting them a whole step
        // ahead was measured slower: the registers cost more than the wait.)
        float xv[TW][16];
#pragma unroll
        for (int t = 0; t < TW; ++t) {
            load_x<16, XA>(x + xoff[t] + (c << 10), xv[t]);
        }
        __builtin_amdgcn_sched_barrier(0); // keep the instruction scheduler from swapping the two
        // The prefetch is unconditional (the last step fetches its own data
        // again, into the buffer nobody reads any more): with a branch here the
        // wait for the activations above would have to cover both paths and
        // would drain the prefetch too.
        const bool last = step + 1u == nsteps;
        fetch(last ? r0 : rn, last ? c : cn, nxt);
        if constexpr (HYBRID) {
            load_direct(last ? r0 : rn, last ? c : cn, qdn);
        }
        load_scales(last ? r0 : rn, last ? c : cn, sn);
        if (has_tokens) {
            if (c == 0u) {
#pragma unroll
                for (int r = 0; r < R; ++r) {
#pragma unroll
                    for (int t = 0; t < TW; ++t) {
                        acc[r][t] = 0.0f;
                    }
                }
                // Column tail first, as in the decode kernel; these few pieces
                // come straight from global memory.
                if constexpr (TAIL) {
                  if (cols & 1023u) {
                    uint32_t row[R];
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        row[r] = (r0 + r < row_end) ? r0 + r : row_end - 1u;
                    }
                    uint32_t col0 = full << 10;
                    if (cols & 512u) {
                        chunk<L, R, TW, 8, XA, false>(wv, x, cols, row, tok, col0, lane, true, acc);
                        col0 += 512u;
                    }
                    if (cols & 256u) {
                        chunk<L, R, TW, 4, XA, false>(wv, x, cols, row, tok, col0, lane, true, acc);
                        col0 += 256u;
                    }
                    if (cols & 128u) {
                        chunk<L, R, TW, 2, XA, false>(wv, x, cols, row, tok, col0, lane, true, acc);
                        col0 += 128u;
                    }
                    if (cols & 64u) {
                        chunk<L, R, TW, 1, XA, false>(wv, x, cols, row, tok, col0, lane, true, acc);
                        col0 += 64u;
                    }
                    if (cols & 32u) {
                        chunk<L, R, TW, 1, XA, false>(wv, x, cols, row, tok, col0, lane,
                                                           lane < 32u, acc);
                    }
                  }
                }
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                uint32_t q[4];
                if constexpr (HYBRID) {
                    if (r >= SR) {
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            q[i] = qd[r - SR][i];
                        }
                    }
                }
                if constexpr (L == PACKED) {
                    if (r < SR) {
                        const uint4 qv = *(const uint4 *)(cur + r * ROWB + lane * 16u);
                        q[0] = qv.x;
                        q[1] = qv.y;
                        q[2] = qv.z;
                        q[3] = qv.w;
                    }
                } else {
                    const uint32_t *w = (const uint32_t *)(cur + r * ROWB + (raw_off & ~3u));
                    const uint32_t d0 = w[0], d1 = w[1], d2 = w[2], d3 = w[3], d4 = w[4];
                    q[0] = __builtin_amdgcn_perm(d1, d0, raw_sel);
                    q[1] = __builtin_amdgcn_perm(d2, d1, raw_sel);
                    q[2] = __builtin_amdgcn_perm(d3, d2, raw_sel);
                    q[3] = __builtin_amdgcn_perm(d4, d3, raw_sel);
                    const uint32_t own = raw_high ? d0 >> 16 : d0;
                    // quad_perm [0, 0, 2, 2]: odd lanes take their even neighbour's scale
                    sb[r] = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)own, 0xA0, 0xf, 0xf, false) &
                            0xffffu;
                }
                float qf[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    qf[i] = sbyte_to_float(q[i / 4], i % 4);
                }
                const float dsc = f16_bits_to_f32(sb[r]);
#pragma unroll
                for (int t = 0; t < TW; ++t) {
                    float s = 0.0f;
#pragma unroll
                    for (int i = 0; i < 16; ++i) {
                        s = __builtin_fmaf(qf[i], xv[t][i], s);
                    }
                    acc[r][t] = __builtin_fmaf(dsc, s, acc[r][t]);
                }
            }
            if (cn == 0u) {
#pragma unroll
                for (int t = 0; t < TW; ++t) {
                    float col_acc[R];
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        col_acc[r] = acc[r][t];
                    }
                    // (an optional residual update of the token's row rides along,
                    // as in the one-token kernel)
                    const size_t token_off = (size_t)(wave * TW + t) * rows;
                    reduce_store<R>(col_acc, y + token_off, r0, row_end, lane, tok_ok[t],
                                    d.res != nullptr ? d.res + token_off : nullptr, d.alpha);
                }
            }
        }
        if constexpr (L == PACKED) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                sb[r] = sn[r];
            }
        }
        if constexpr (HYBRID) {
#pragma unroll
            for (int r = 0; r < R - SR; ++r) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    qd[r][i] = qdn[r][i];
                }
            }
        }
        c = cn;
        r0 = rn;
    };
    for (uint32_t step = 0; step < nsteps; step += 2u) {
        do_step(step, stage_a, stage_b);
        if (step + 1u < nsteps) {
            do_step(step + 1u, stage_b, stage_a);
        }
    }
    // no fetch may still be in flight when the workgroup gives up its LDS
    __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8)); // vmcnt(0)
    __syncthreads();
}

} // namespace q8
