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
    // Optional fused residual update: res[r] += alpha * y[r] (row r of every
    // token of the descriptor, res laid out like y), multiply then add, exactly
    // what a separate axpy over y would compute.
    float *res;
    float alpha;
    uint32_t pad2;         // the row of the launch's fused RMSNorm that this descriptor reads
};

// Descriptor flag bits (GemvDesc::pad): the product's activations are the
// launch's fused RMSNorm output, and this product's first tile writes it out.
constexpr uint32_t GEMV_X_NORMED = 1u, GEMV_WRITES_NORM = 2u;
// This product and the next descriptor are the gate and up projections of a
// fused gated activation (see stream_rows_glu).
constexpr uint32_t GEMV_PAIR = 4u;

template <int ND> struct GemvArgsT {
    uint32_t n;
    uint32_t total_tiles;
    // At most one fused RMSNorm per launch (norm_w == nullptr: none):
    // n = h / sqrt(mean(h^2) + eps) * w over norm_cols elements, a multiple of
    // 1024; products flagged GEMV_X_NORMED read n without it going through
    // memory, one of them also stores it to norm_out. A few tokens (rows of
    // the norm) go as one descriptor per product and token, GemvDesc::pad2
    // saying which row; one descriptor per row stores it.
    float norm_eps;
    uint32_t pad;
    const float *norm_h;
    const float *norm_w;
    float *norm_out;
    GemvDesc d[ND];
};
using GemvArgs = GemvArgsT<GEMV_MAX_DESCS>;

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
                                             uint32_t row_end, uint32_t lane, bool token_ok,
                                             float *res = nullptr, float alpha = 0.0f) {
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
            if (res != nullptr) {
                res[r0 + r] = __fadd_rn(res[r0 + r], __fmul_rn(alpha, a1));
            }
        }
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float total = wave_sum(acc[r]);
            if (lane == 0u && r0 + r < row_end && token_ok) {
                y[r0 + r] = total;
                if (res != nullptr) {
                    res[r0 + r] = __fadd_rn(res[r0 + r], __fmul_rn(alpha, total));
                }
            }
        }
    }
}

// Where a lane's 16 activations of a chunk come from: memory, or the fused
// RMSNorm of the launch, (h * inv) * w with the operations of rmsnorm_kernel.
// (loadn: the N activations of a column-tail piece.)
struct PlainX {
    const float *x;
    template <bool XA>
    __device__ __forceinline__ void load16(uint32_t col, float (&out)[16]) const {
        load_x<16, XA>(x + col, out);
    }
    template <int N, bool XA>
    __device__ __forceinline__ void loadn(uint32_t col, float (&out)[N]) const {
        load_x<N, XA>(x + col, out);
    }
};
struct NormedX {
    const float *h, *w;
    float inv;
    template <bool XA>
    __device__ __forceinline__ void load16(uint32_t col, float (&out)[16]) const {
        loadn<16, XA>(col, out);
    }
    template <int N, bool XA>
    __device__ __forceinline__ void loadn(uint32_t col, float (&out)[N]) const {
        float hv[N], wv[N];
        load_x<N, true>(h + col, hv);
        load_x<N, true>(w + col, wv);
#pragma unroll
        for (int i = 0; i < N; ++i) {
            out[i] = hv[i] * inv * wv[i];
        }
    }
};

// Sum of squares of a row in the order every kernel that must agree uses: lane
// l adds its elements 1024*c + 16*l + i sequentially (c, then i, ascending;
// multiply, then add), the 64 partials go through q8::wave_sum.
// The loads of four chunks are requested before the first of them is added up
// (the additions keep their order): a row of 4096 waits for memory once, not
// four times, which every wave of a launch with a fused norm does before it
// streams anything. XA: h is 16-byte aligned.
template <bool XA = false>
__device__ __forceinline__ float row_sumsq(const float *h, uint32_t cols, uint32_t lane) {
    float acc = 0.0f;
    const uint32_t full = cols >> 10; // whole chunks: the same for every lane
    uint32_t c = 0;
    for (; c + 4u <= full; c += 4u) {
        float hv[4][16];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            load_x<16, XA>(h + ((c + (uint32_t)j) << 10) + lane * 16u, hv[j]);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                acc += hv[j][i] * hv[j][i];
            }
        }
    }
    for (; c < full; ++c) {
        float hv[16];
        load_x<16, XA>(h + (c << 10) + lane * 16u, hv);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            acc += hv[i] * hv[i];
        }
    }
    const uint32_t e0 = (full << 10) + lane * 16u; // the lane's run in the last, partial chunk
    if (e0 + 16u <= cols) {
        float hv[16];
        load_x<16, XA>(h + e0, hv);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            acc += hv[i] * hv[i];
        }
    } else {
        for (uint32_t e = e0; e < cols; ++e) {
            acc += h[e] * h[e];
        }
    }
    return wave_sum(acc);
}

// Which weight rows a pass of R accumulators covers: R consecutive rows of one
// matrix, or R/2 rows of a gate matrix followed by the same R/2 rows of an up
// matrix (the fused gated-activation form: both results of a row end up in one
// wave).
struct SingleRows {
    WView<PACKED> wv;
    static constexpr bool pair = false;
    template <int R>
    __device__ __forceinline__ void chunk(int r, uint32_t r0, uint32_t row_end, uint32_t c,
                                          uint32_t lane, uint32_t (&q)[4], uint32_t &sb) const {
        const uint32_t row = (r0 + r < row_end) ? r0 + r : row_end - 1u;
        wv.template load_quants<16, true>(row, (c << 10) + lane * 16u, q);
        sb = wv.scale_bits(row, (c << 5) + (lane >> 1));
    }
};
struct PairRows {
    WView<PACKED> gate, up;
    static constexpr bool pair = true;
    template <int R>
    __device__ __forceinline__ void chunk(int r, uint32_t r0, uint32_t row_end, uint32_t c,
                                          uint32_t lane, uint32_t (&q)[4], uint32_t &sb) const {
        const uint32_t j = (uint32_t)(r % (R / 2));
        const uint32_t row = (r0 + j < row_end) ? r0 + j : row_end - 1u;
        const WView<PACKED> &wv = r < R / 2 ? gate : up;
        wv.template load_quants<16, true>(row, (c << 10) + lane * 16u, q);
        sb = wv.scale_bits(row, (c << 5) + (lane >> 1));
    }
};

// The decode path: one token, sealed weights, at least one whole 1024-column
// chunk per row. TAILMASK = cols % 1024 selects the tail pieces at compile time
// (bit 512/256/128/64/32 -> a piece of 8/4/2/1/1 quants per lane).
//
// Per pass of R rows the arithmetic is: acc = 0; tail pieces in descending
// width; whole chunks in ascending order; reduce. The loads run one step ahead
// of the multiplies: while chunk c is multiplied the R weight loads of chunk
// c+1 are in flight, and during the last chunk of a pass the tail pieces and
// the first chunk of the next pass are. Tail pieces come first in a pass so
// that their registers are free again before the next prefetch is issued.
// With a single chunk per row this lane's activations never leave registers.
// `sink(acc, r0)` receives the R per-lane partial sums of a finished pass.
template <int R, bool XA, int TAILMASK, class XS, class ROWS, class SINK>
__device__ __forceinline__ void stream_rows_to(const ROWS rows_src, const XS xs, uint32_t cols,
                                               uint32_t row_first, uint32_t row_end, uint32_t lane,
                                               SINK sink) {
    constexpr uint32_t ADV = ROWS::pair ? R / 2 : R; // rows a pass advances by
    // the matrix row r of a pass comes from (the paired form: gate rows, then up rows)
    auto view_of = [&](int r) -> const WView<PACKED> & {
        if constexpr (ROWS::pair) {
            return r < R / 2 ? rows_src.gate : rows_src.up;
        } else {
            return rows_src.wv;
        }
    };
    auto row_of = [&](int r, uint32_t r0) {
        const uint32_t row = r0 + (ROWS::pair ? (uint32_t)(r % (R / 2)) : (uint32_t)r);
        return row < row_end ? row : row_end - 1u;
    };
    constexpr bool T8 = (TAILMASK & 512) != 0, T4 = (TAILMASK & 256) != 0;
    constexpr bool T2 = (TAILMASK & 128) != 0, T1 = (TAILMASK & 64) != 0;
    constexpr bool TH = (TAILMASK & 32) != 0;
    const uint32_t full = cols >> 10;
    const uint32_t c8 = full << 10;
    const uint32_t c4 = c8 + (T8 ? 512u : 0u);
    const uint32_t c2 = c4 + (T4 ? 256u : 0u);
    const uint32_t c1 = c2 + (T2 ? 128u : 0u);
    const uint32_t ch = c1 + (T1 ? 64u : 0u);
    const bool low = lane < 32u;

    // activations of the tail pieces: loop invariant, kept in registers
    float x8[8], x4[4], x2[2], x1[1], xh[1];
    if constexpr (T8) xs.template loadn<8, XA>(c8 + lane * 8u, x8);
    if constexpr (T4) xs.template loadn<4, XA>(c4 + lane * 4u, x4);
    if constexpr (T2) xs.template loadn<2, XA>(c2 + lane * 2u, x2);
    if constexpr (T1) xs.template loadn<1, XA>(c1 + lane, x1);
    if constexpr (TH) xs.template loadn<1, XA>(ch + (low ? lane : 0u), xh);
    float xv[16];
    if (full == 1u) {
        xs.template load16<XA>(lane * 16u, xv);
    }


    uint32_t q8[R][2], q4[R][1], q2[R][1], q1[R][1], qh[R][1];
    uint32_t s8[R], s4[R], s2[R], s1[R], sh[R];
    auto load_tails = [&](uint32_t r0) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const uint32_t row = row_of(r, r0);
            const WView<PACKED> &wv = view_of(r);
            if constexpr (T8) {
                wv.template load_quants<8, true>(row, c8 + lane * 8u, q8[r]);
                s8[r] = wv.scale_bits(row, (c8 + lane * 8u) >> 5);
            }
            if constexpr (T4) {
                wv.template load_quants<4, true>(row, c4 + lane * 4u, q4[r]);
                s4[r] = wv.scale_bits(row, (c4 + lane * 4u) >> 5);
            }
            if constexpr (T2) {
                wv.template load_quants<2, true>(row, c2 + lane * 2u, q2[r]);
                s2[r] = wv.scale_bits(row, (c2 + lane * 2u) >> 5);
            }
            if constexpr (T1) {
                wv.template load_quants<1, true>(row, c1 + lane, q1[r]);
                s1[r] = wv.scale_bits(row, (c1 + lane) >> 5);
            }
            if constexpr (TH) {
                wv.template load_quants<1, true>(row, ch + (low ? lane : 0u), qh[r]);
                sh[r] = wv.scale_bits(row, ch >> 5);
            }
        }
    };
    uint32_t q[R][4], sb[R];
    auto load_chunk = [&](uint32_t r0, uint32_t c, uint32_t (&qq)[R][4], uint32_t (&ss)[R]) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            rows_src.template chunk<R>(r, r0, row_end, c, lane, qq[r], ss[r]);
        }
    };

    // One flat sequence of (pass, chunk) steps; the tail pieces of a pass
    // travel with its first chunk.
    const uint32_t nsteps = ((row_end - row_first + ADV - 1) / ADV) * full;
    uint32_t r0 = row_first, c = 0;
    if constexpr (TAILMASK != 0) {
        load_tails(r0);
    }
    load_chunk(r0, 0, q, sb);
    float acc[R];
    for (uint32_t step = 0; step < nsteps; ++step) {
        if (c == 0u) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                float a = 0.0f;
                if constexpr (T8) a = __builtin_fmaf(f16_bits_to_f32(s8[r]), piece_dot<8>(q8[r], x8), a);
                if constexpr (T4) a = __builtin_fmaf(f16_bits_to_f32(s4[r]), piece_dot<4>(q4[r], x4), a);
                if constexpr (T2) a = __builtin_fmaf(f16_bits_to_f32(s2[r]), piece_dot<2>(q2[r], x2), a);
                if constexpr (T1) a = __builtin_fmaf(f16_bits_to_f32(s1[r]), piece_dot<1>(q1[r], x1), a);
                if constexpr (TH) {
                    const float d = low ? f16_bits_to_f32(sh[r]) : 0.0f;
                    const float sd = low ? piece_dot<1>(qh[r], xh) : 0.0f;
                    a = __builtin_fmaf(d, sd, a);
                }
                acc[r] = a;
            }
        }
        if (full > 1u) {
            xs.template load16<XA>((c << 10) + lane * 16u, xv);
        }
        uint32_t cn = c + 1u, rn = r0;
        if (cn == full) {
            cn = 0;
            rn = r0 + ADV;
        }
        uint32_t qn[R][4], sn[R];
        if (step + 1u < nsteps) {
            if constexpr (TAILMASK != 0) {
                if (cn == 0u) {
                    load_tails(rn); // the current pass consumed its tail pieces at c == 0
                }
            }
            load_chunk(rn, cn, qn, sn);
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            acc[r] = __builtin_fmaf(f16_bits_to_f32(sb[r]), piece_dot<16>(q[r], xv), acc[r]);
        }
        if (cn == 0u) {
            sink(acc, r0);
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
}

// One matrix: reduce each pass over the wave and store (plus the optional
// fused residual update).
template <int R, bool XA, int TAILMASK, class XS = PlainX>
__device__ __forceinline__ void stream_rows(const WView<PACKED> &wv, const XS xs, float *y,
                                            uint32_t cols, uint32_t row_first, uint32_t row_end,
                                            uint32_t lane, float *res, float alpha) {
    stream_rows_to<R, XA, TAILMASK>(SingleRows{wv}, xs, cols, row_first, row_end, lane,
                                    [&](const float (&acc)[R], uint32_t r0) {
                                        reduce_store<R>(acc, y, r0, row_end, lane, true, res, alpha);
                                    });
}

// stream_rows for rows of exactly one whole chunk (1024 columns, or 1152 with
// TAILMASK = 128) in tiles of at most R rows: the tile is a single step, so there
// is nothing to run ahead of, no loop, and no second set of weight registers to
// hold: every load of the tile is issued at once. Same arithmetic as stream_rows:
// the tail piece first, then the chunk. Measured on the 262144 x 1152 vocabulary:
// 47.2 -> 44.5 us (the kernel that carries this form instead of the pipelined one
// for such rows needs 120 registers instead of 164: four waves per SIMD, which
// is where the gain comes from). For rows of 1024 columns, whose kernel has four
// waves anyway, the same form is slower than the pipelined one run for a single
// step (Qwen3-0.6B decode step 95.4 -> 100.2 us): TAILMASK = 0 is not used.
template <int R, bool XA, int TAILMASK, class XS = PlainX>
__device__ __forceinline__ void stream_rows_once(const WView<PACKED> &wv, const XS xs, float *y,
                                                 uint32_t row_first, uint32_t row_end,
                                                 uint32_t lane, float *res, float alpha) {
    static_assert(TAILMASK == 0 || TAILMASK == 128, "one whole chunk, with or without a 128-column tail");
    constexpr bool T2 = TAILMASK == 128;
    float x2[2], xv[16];
    if constexpr (T2) xs.template loadn<2, XA>(1024u + lane * 2u, x2);
    xs.template load16<XA>(lane * 16u, xv);
    uint32_t q2[R][1], s2[R], q[R][4], sb[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const uint32_t row = row_first + (uint32_t)r < row_end ? row_first + (uint32_t)r : row_end - 1u;
        if constexpr (T2) {
            wv.template load_quants<2, true>(row, 1024u + lane * 2u, q2[r]);
            s2[r] = wv.scale_bits(row, (1024u + lane * 2u) >> 5);
        }
        wv.template load_quants<16, true>(row, lane * 16u, q[r]);
        sb[r] = wv.scale_bits(row, lane >> 1);
    }
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        float a = 0.0f;
        if constexpr (T2) a = __builtin_fmaf(f16_bits_to_f32(s2[r]), piece_dot<2>(q2[r], x2), a);
        acc[r] = __builtin_fmaf(f16_bits_to_f32(sb[r]), piece_dot<16>(q[r], xv), a);
    }
    reduce_store<R>(acc, y, row_first, row_end, lane, true, res, alpha);
}

// stream_rows for passes of few rows under a long K (a small product cut into
// short tiles, so that more waves share it): a step covers C chunks of the R
// rows instead of one, which keeps R x C kilobytes per wave in flight where the
// plain form would have R. Same arithmetic: a pass starts with its tail pieces
// and adds the chunks in ascending order; a last, shorter group of chunks
// repeats its last chunk's loads and leaves the surplus out of the sums.
template <int R, int C, bool XA, int TAILMASK, class XS = PlainX>
__device__ __forceinline__ void stream_rows_wide(const WView<PACKED> &wv, const XS xs, float *y,
                                                 uint32_t cols, uint32_t row_first,
                                                 uint32_t row_end, uint32_t lane, float *res,
                                                 float alpha) {
    constexpr bool T8 = (TAILMASK & 512) != 0, T4 = (TAILMASK & 256) != 0;
    constexpr bool T2 = (TAILMASK & 128) != 0;
    static_assert((TAILMASK & 127) == 0, "the column tails with a streaming path");
    const uint32_t full = cols >> 10;
    const uint32_t groups = (full + (uint32_t)C - 1u) / (uint32_t)C;
    const uint32_t c8 = full << 10;
    const uint32_t c4 = c8 + (T8 ? 512u : 0u);
    const uint32_t c2 = c4 + (T4 ? 256u : 0u);
    auto row_of = [&](int r, uint32_t r0) {
        return r0 + (uint32_t)r < row_end ? r0 + (uint32_t)r : row_end - 1u;
    };
    float x8[8], x4[4], x2[2];
    if constexpr (T8) xs.template loadn<8, XA>(c8 + lane * 8u, x8);
    if constexpr (T4) xs.template loadn<4, XA>(c4 + lane * 4u, x4);
    if constexpr (T2) xs.template loadn<2, XA>(c2 + lane * 2u, x2);
    uint32_t q8[R][2], q4[R][1], q2[R][1];
    uint32_t s8[R], s4[R], s2[R];
    auto load_tails = [&](uint32_t r0) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const uint32_t row = row_of(r, r0);
            if constexpr (T8) {
                wv.template load_quants<8, true>(row, c8 + lane * 8u, q8[r]);
                s8[r] = wv.scale_bits(row, (c8 + lane * 8u) >> 5);
            }
            if constexpr (T4) {
                wv.template load_quants<4, true>(row, c4 + lane * 4u, q4[r]);
                s4[r] = wv.scale_bits(row, (c4 + lane * 4u) >> 5);
            }
            if constexpr (T2) {
                wv.template load_quants<2, true>(row, c2 + lane * 2u, q2[r]);
                s2[r] = wv.scale_bits(row, (c2 + lane * 2u) >> 5);
            }
        }
    };
    auto load_group = [&](uint32_t r0, uint32_t g, uint32_t (&qq)[R][C][4], uint32_t (&ss)[R][C]) {
#pragma unroll
        for (int cc = 0; cc < C; ++cc) {
            const uint32_t want = g * (uint32_t)C + (uint32_t)cc;
            const uint32_t c = want < full ? want : full - 1u;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint32_t row = row_of(r, r0);
                wv.template load_quants<16, true>(row, (c << 10) + lane * 16u, qq[r][cc]);
                ss[r][cc] = wv.scale_bits(row, (c << 5) + (lane >> 1));
            }
        }
    };
    const uint32_t nsteps = ((row_end - row_first + R - 1) / R) * groups;
    uint32_t r0 = row_first, g = 0;
    uint32_t q[R][C][4], sb[R][C];
    if constexpr (TAILMASK != 0) {
        load_tails(r0);
    }
    load_group(r0, 0, q, sb);
    float acc[R];
    for (uint32_t step = 0; step < nsteps; ++step) {
        if (g == 0u) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                float a = 0.0f;
                if constexpr (T8) a = __builtin_fmaf(f16_bits_to_f32(s8[r]), piece_dot<8>(q8[r], x8), a);
                if constexpr (T4) a = __builtin_fmaf(f16_bits_to_f32(s4[r]), piece_dot<4>(q4[r], x4), a);
                if constexpr (T2) a = __builtin_fmaf(f16_bits_to_f32(s2[r]), piece_dot<2>(q2[r], x2), a);
                acc[r] = a;
            }
        }
        // this step's activations are requested before the next step's weights
        float xv[C][16];
#pragma unroll
        for (int cc = 0; cc < C; ++cc) {
            const uint32_t want = g * (uint32_t)C + (uint32_t)cc;
            const uint32_t c = want < full ? want : full - 1u;
            xs.template load16<XA>((c << 10) + lane * 16u, xv[cc]);
        }
        uint32_t gn = g + 1u, rn = r0;
        if (gn == groups) {
            gn = 0;
            rn = r0 + (uint32_t)R;
        }
        uint32_t qn[R][C][4], sn[R][C];
        if (step + 1u < nsteps) {
            if constexpr (TAILMASK != 0) {
                if (gn == 0u) {
                    load_tails(rn);
                }
            }
            load_group(rn, gn, qn, sn);
        }
#pragma unroll
        for (int cc = 0; cc < C; ++cc) {
            if (g * (uint32_t)C + (uint32_t)cc < full) {
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    acc[r] = __builtin_fmaf(f16_bits_to_f32(sb[r][cc]), piece_dot<16>(q[r][cc], xv[cc]),
                                            acc[r]);
                }
            }
        }
        if (gn == 0u) {
            reduce_store<R>(acc, y, r0, row_end, lane, true, res, alpha);
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
#pragma unroll
            for (int cc = 0; cc < C; ++cc) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    q[r][cc][i] = qn[r][cc][i];
                }
                sb[r][cc] = sn[r][cc];
            }
        }
        g = gn;
        r0 = rn;
    }
}

// One token over weights in the raw layout (34-byte blocks: f16 scale, 32
// quants), rows of whole 1024-column chunks. A lane's 16 quants start 2 or 18
// bytes into a block, at an even address: loaded from memory in that shape, a
// wave's 16-byte pieces straddle the aligned ones and the step runs at half the
// sealed layout's rate. Instead the wave streams the R x 1088 bytes of a step
// (R rows of one chunk; 1088 = 68 aligned 16-byte pieces) exactly like sealed
// quants - aligned, contiguous, non-temporal - parks them in its own piece of
// LDS, and every lane reads back the five aligned dwords that hold its quants
// and moves the bytes into place (even lanes find the block's scale in front of
// them; odd lanes take it from their neighbour). From there on the registers
// and the arithmetic are those of stream_rows. The loads of step s+1 are in
// flight while step s is multiplied.
constexpr uint32_t RAW_CHUNK_BYTES = 1088u; // 32 blocks of 34 bytes
typedef unsigned int u32x4_a8 __attribute__((ext_vector_type(4), aligned(8)));
// LDS a wave needs for it: R staged rows of a chunk, or (TAILS == 1) of a whole
// 1152-column row.
template <int R, int TAILS> constexpr uint32_t raw_stage_bytes() {
    return (uint32_t)R * (TAILS == 1 ? RAW_CHUNK_BYTES + 136u : RAW_CHUNK_BYTES);
}

// A lane's 2, 4 or 8 quants of a tail piece out of staged raw bytes: they start
// at the even byte `at`; the aligned dwords that hold them, bytes moved into place.
__device__ __forceinline__ uint32_t raw_sel(uint32_t at) {
    return (at & 2u) ? 0x05040302u : 0x03020100u;
}

// TAILMASK = cols % 1024: 0, or one of the two column tails with a path of their
// own. 768 (rows of 6912 columns: 16-byte aligned like rows of whole chunks): the
// tail's 24 blocks of each row are a step of their own in front of the chunks, as
// the arithmetic has the tail pieces first. 128 with a single chunk (rows of 1152
// columns, 1224 bytes: only 8-byte aligned, but R of them are contiguous and
// start aligned): a pass is staged whole, chunk and tail in one step.
template <int R, bool XA, int TAILMASK>
__device__ __forceinline__ void stream_rows_raw(const WView<RAW> &wv, const float *x, float *y,
                                                uint32_t cols, uint32_t row_first,
                                                uint32_t row_end, uint32_t lane, uint8_t *stage,
                                                float *res, float alpha) {
    static_assert(TAILMASK == 0 || TAILMASK == 128 || TAILMASK == 768, "column tails with a path");
    constexpr bool WHOLE = TAILMASK == 128; // a pass is one step over R whole rows
    constexpr bool TSEG = TAILMASK == 768;  // the tail blocks are a step of their own
    constexpr uint32_t TAILB = (uint32_t)TAILMASK / 32u * 34u;          // a row's tail bytes
    constexpr uint32_t ROWB = WHOLE ? RAW_CHUNK_BYTES + TAILB : RAW_CHUNK_BYTES; // a staged row
    constexpr uint32_t PIECES = (uint32_t)R * ROWB / 16u;               // 16-byte pieces of a step
    constexpr int NL = (int)((PIECES + 63u) / 64u);                     // loads per lane and step
    constexpr uint32_t ROW_PIECES = ROWB / 16u;
    constexpr uint32_t TROW_PIECES = TAILB / 16u;                       // (TSEG) 51
    constexpr uint32_t TPIECES = (uint32_t)R * TROW_PIECES;
    constexpr int NLT = TSEG ? (int)((TPIECES + 63u) / 64u) : 0;
    static_assert(!TSEG || TAILB % 16u == 0u, "tail rows are whole pieces");
    const uint32_t full = cols >> 10;
    const uint32_t row_bytes = (uint32_t)wv.row_bytes;
    // Piece g = i * 64 + lane of a step is piece g % ROW_PIECES of row
    // g / ROW_PIECES and is staged at byte 16 g; a last, partly filled round
    // of pieces is left to the lanes below PIECES % 64. Rows past the tile's
    // end repeat its last row. With rows staged whole a piece's place in the
    // stage is its offset in memory, and pieces that would reach past the last
    // row of the tile are its last 16 bytes instead (an odd number of 1224-byte
    // rows ends on an 8-byte boundary: such a piece is 8-byte aligned, in
    // memory and in the stage).
    auto piece_offset = [&](int i, uint32_t last) { // from the step's first byte
        const uint32_t g = (uint32_t)i * 64u + lane;
        if constexpr (WHOLE) {
            const uint32_t end = (last + 1u) * ROWB - 16u;
            return g * 16u < end ? g * 16u : end;
        } else {
            const uint32_t row = g / ROW_PIECES;
            return (row < last ? row : last) * row_bytes + (g % ROW_PIECES) * 16u;
        }
    };
    uint32_t poff[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        poff[i] = piece_offset(i, (uint32_t)R - 1u);
    }
    // seg -1: the tail step (TSEG only); 0 .. full-1: the chunks
    auto fetch = [&](uint32_t r0, int32_t seg, u32x4 (&p)[NL]) {
        const uint32_t last = row_end - 1u - r0;
        const uint8_t *row0 = wv.base + (size_t)r0 * wv.row_bytes;
        if constexpr (TSEG) {
            if (seg < 0) {
                const uint8_t *base = row0 + (size_t)full * RAW_CHUNK_BYTES;
#pragma unroll
                for (int i = 0; i < NLT; ++i) {
                    const uint32_t g = (uint32_t)i * 64u + lane;
                    const uint32_t row = g / TROW_PIECES;
                    const uint32_t o =
                        (row < last ? row : last) * row_bytes + (g % TROW_PIECES) * 16u;
                    if (i < NLT - 1 || lane < TPIECES % 64u || TPIECES % 64u == 0u) {
                        p[i] = __builtin_nontemporal_load((const u32x4 *)(base + o));
                    }
                }
                return;
            }
        }
        const uint8_t *base = row0 + (size_t)seg * RAW_CHUNK_BYTES;
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            const uint32_t o = last >= (uint32_t)R - 1u ? poff[i] : piece_offset(i, last);
            if (i < NL - 1 || lane < PIECES % 64u || PIECES % 64u == 0u) {
                if constexpr (WHOLE) {
                    p[i] = __builtin_nontemporal_load((const u32x4_a8 *)(base + o));
                } else {
                    p[i] = __builtin_nontemporal_load((const u32x4 *)(base + o));
                }
            }
        }
    };
    // where the pieces of a chunk step go in the stage
    auto stage_at = [&](int i, uint32_t last) {
        if constexpr (WHOLE) {
            return last >= (uint32_t)R - 1u ? poff[i] : piece_offset(i, last);
        } else {
            return (uint32_t)i * 1024u + lane * 16u;
        }
    };
    // this lane's window in a staged chunk: the aligned dword at or below the
    // block's first byte (even lanes) or its 17th (odd lanes)
    const uint32_t off = (lane >> 1) * 34u + (lane & 1u) * 16u;
    const bool high = (off & 2u) != 0u; // quants from dword 1 on, the scale in dword 0's upper half
    const uint32_t sel = high ? 0x07060504u : 0x05040302u;
    const uint8_t *window = stage + (off & ~3u);

    // the tail pieces' activations and places in a staged row (loop invariant)
    float x8[8], x4[4], x2[2];
    uint32_t s8_at = 0, q8_at = 0, s4_at = 0, q4_at = 0, s2_at = 0, q2_at = 0;
    if constexpr (TSEG) { // 512 columns as 8 quants per lane, then 256 as 4
        load_x<8, XA>(x + (full << 10) + lane * 8u, x8);
        load_x<4, XA>(x + (full << 10) + 512u + lane * 4u, x4);
        s8_at = (lane >> 2) * 34u;
        q8_at = s8_at + 2u + 8u * (lane & 3u);
        s4_at = (16u + (lane >> 3)) * 34u;
        q4_at = s4_at + 2u + 4u * (lane & 7u);
    }
    if constexpr (WHOLE) { // 128 columns as 2 quants per lane
        load_x<2, XA>(x + 1024u + lane * 2u, x2);
        s2_at = RAW_CHUNK_BYTES + (lane >> 4) * 34u;
        q2_at = s2_at + 2u + 2u * (lane & 15u);
    }

    float xv[16];
    if (full == 1u) {
        load_x<16, XA>(x + lane * 16u, xv);
    }
    constexpr int32_t SEG0 = TSEG ? -1 : 0;
    const uint32_t nsteps = ((row_end - row_first + R - 1) / R) * (full + (TSEG ? 1u : 0u));
    uint32_t r0 = row_first;
    int32_t seg = SEG0;
    u32x4 p[NL];
    fetch(r0, seg, p);
    float acc[R];
    for (uint32_t step = 0; step < nsteps; ++step) {
        __builtin_amdgcn_wave_barrier(); // the previous step's reads come first
        if (TSEG && seg < 0) {
#pragma unroll
            for (int i = 0; i < NLT; ++i) {
                if (i < NLT - 1 || lane < TPIECES % 64u || TPIECES % 64u == 0u) {
                    *(u32x4 *)(stage + (uint32_t)i * 1024u + lane * 16u) = p[i];
                }
            }
        } else {
            const uint32_t last = row_end - 1u - r0;
#pragma unroll
            for (int i = 0; i < NL; ++i) {
                if (i < NL - 1 || lane < PIECES % 64u || PIECES % 64u == 0u) {
                    if constexpr (WHOLE) {
                        *(u32x4_a8 *)(stage + stage_at(i, last)) = p[i];
                    } else {
                        *(u32x4 *)(stage + stage_at(i, last)) = p[i];
                    }
                }
            }
        }
        int32_t segn = seg + 1;
        uint32_t rn = r0;
        if (segn == (int32_t)full) {
            segn = SEG0;
            rn = r0 + (uint32_t)R;
        }
        if (step + 1u < nsteps) {
            fetch(rn, segn, p);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (TSEG && seg < 0) {
            // the pass starts with its tail pieces, widest first
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint8_t *row = stage + (uint32_t)r * TAILB;
                const uint32_t *w8 = (const uint32_t *)(row + (q8_at & ~3u));
                const uint32_t *w4 = (const uint32_t *)(row + (q4_at & ~3u));
                const uint32_t e0 = w8[0], e1 = w8[1], e2 = w8[2], f0 = w4[0], f1 = w4[1];
                const uint32_t q8[2] = {__builtin_amdgcn_perm(e1, e0, raw_sel(q8_at)),
                                        __builtin_amdgcn_perm(e2, e1, raw_sel(q8_at))};
                const uint32_t q4[1] = {__builtin_amdgcn_perm(f1, f0, raw_sel(q4_at))};
                const uint32_t s8 = *(const uint16_t *)(row + s8_at);
                const uint32_t s4 = *(const uint16_t *)(row + s4_at);
                float a = __builtin_fmaf(f16_bits_to_f32(s8), piece_dot<8>(q8, x8), 0.0f);
                a = __builtin_fmaf(f16_bits_to_f32(s4), piece_dot<4>(q4, x4), a);
                acc[r] = a;
            }
        } else {
            if (full > 1u) {
                load_x<16, XA>(x + ((uint32_t)seg << 10) + lane * 16u, xv);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                float a = acc[r];
                if (!TSEG && seg == 0) {
                    a = 0.0f;
                    if constexpr (WHOLE) {
                        const uint8_t *row = stage + (uint32_t)r * ROWB;
                        const uint32_t q2[1] = {*(const uint16_t *)(row + q2_at)};
                        const uint32_t s2 = *(const uint16_t *)(row + s2_at);
                        a = __builtin_fmaf(f16_bits_to_f32(s2), piece_dot<2>(q2, x2), a);
                    }
                }
                const uint32_t *w = (const uint32_t *)(window + (uint32_t)r * ROWB);
                const uint32_t d0 = w[0], d1 = w[1], d2 = w[2], d3 = w[3], d4 = w[4];
                uint32_t q[4];
                q[0] = __builtin_amdgcn_perm(d1, d0, sel);
                q[1] = __builtin_amdgcn_perm(d2, d1, sel);
                q[2] = __builtin_amdgcn_perm(d3, d2, sel);
                q[3] = __builtin_amdgcn_perm(d4, d3, sel);
                const uint32_t own = high ? d0 >> 16 : d0;
                // quad_perm [0, 0, 2, 2]: odd lanes take their even neighbour's scale
                const uint32_t sb =
                    (uint32_t)__builtin_amdgcn_update_dpp(0, (int)own, 0xA0, 0xf, 0xf, false) &
                    0xffffu;
                acc[r] = __builtin_fmaf(f16_bits_to_f32(sb), piece_dot<16>(q, xv), a);
            }
        }
        if (segn == SEG0) {
            reduce_store<R>(acc, y, r0, row_end, lane, true, res, alpha);
        }
        seg = segn;
        r0 = rn;
    }
}

// Gate and up projection of the same activations with the gated activation on
// top: out[r] = act(gate[r]) * up[r], act = silu (kind 0) or ggml's tanh GELU
// (kind 1), the expressions of silu_mul_kernel / gelu_tanh_mul_kernel. After
// the butterfly of reduce_store<8>, lanes 0, 8, 16, 24 hold the gate rows
// r0..r0+3 and lanes 32, 40, 48, 56 the up rows; one exchange pairs them. The
// raw projections are stored as well (the gate's only when `out` is another
// buffer: in place, the activation replaces it as the separate operator would).
// The same with passes of 2 gate rows and 2 up rows (a pair of few rows cut
// into short tiles, so that more waves share it): acc = [g0, g1, u0, u1]; the
// butterfly halves the values per lane at the shuffles over 32 and 16 lanes,
// every addition with the two operands q8::wave_sum gives it.
template <bool XA, int TAILMASK, class XS>
__device__ __forceinline__ void stream_rows_glu_short(const WView<PACKED> &wg,
                                                      const WView<PACKED> &wu, const XS xs,
                                                      float *gate_out, float *up_out, float *out,
                                                      uint32_t kind, uint32_t cols,
                                                      uint32_t row_first, uint32_t row_end,
                                                      uint32_t lane) {
    constexpr int R = 4;
    stream_rows_to<R, XA, TAILMASK>(
        PairRows{wg, wu}, xs, cols, row_first, row_end, lane,
        [&](const float (&acc)[R], uint32_t r0) {
            float a2[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const float keep = (lane & 32u) ? acc[i + 2] : acc[i];
                const float send = (lane & 32u) ? acc[i] : acc[i + 2];
                a2[i] = keep + __shfl_xor(send, 32, WAVE);
            }
            const float keep = (lane & 16u) ? a2[1] : a2[0];
            const float send = (lane & 16u) ? a2[0] : a2[1];
            float a1 = keep + __shfl_xor(send, 16, WAVE);
            a1 += __shfl_xor(a1, 8, WAVE);
            a1 += __shfl_xor(a1, 4, WAVE);
            a1 += __shfl_xor(a1, 2, WAVE);
            a1 += __shfl_xor(a1, 1, WAVE);
            const float other = __shfl_xor(a1, 32, WAVE);
            const uint32_t row = r0 + ((lane >> 4) & 1u);
            if ((lane & 15u) == 0u && row < row_end) {
                if (lane & 32u) {
                    up_out[row] = a1;
                } else {
                    const float act = glu_act(a1, other, kind);
                    if (out != gate_out) {
                        gate_out[row] = a1;
                    }
                    out[row] = act;
                }
            }
        });
}

template <bool XA, int TAILMASK, class XS>
__device__ __forceinline__ void stream_rows_glu(const WView<PACKED> &wg, const WView<PACKED> &wu,
                                                const XS xs, float *gate_out, float *up_out,
                                                float *out, uint32_t kind, uint32_t cols,
                                                uint32_t row_first, uint32_t row_end,
                                                uint32_t lane) {
    constexpr int R = 8;
    stream_rows_to<R, XA, TAILMASK>(
        PairRows{wg, wu}, xs, cols, row_first, row_end, lane,
        [&](const float (&acc)[R], uint32_t r0) {
            // the butterfly of reduce_store<8>: same operands per addition
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
            const float other = __shfl_xor(a1, 32, WAVE);
            const uint32_t row = r0 + ((lane >> 4) & 1u) * 2u + ((lane >> 3) & 1u);
            if ((lane & 7u) == 0u && row < row_end) {
                if (lane & 32u) {
                    up_out[row] = a1;
                } else {
                    const float act = glu_act(a1, other, kind);
                    if (out != gate_out) {
                        gate_out[row] = a1;
                    }
                    out[row] = act;
                }
            }
        });
}

// TAILS selects which column tails get the streaming decode path: 0 = none
// (cols a multiple of 1024 only; fewest registers, the Qwen3 shapes), 1 = also
// cols % 1024 == 128 and == 768 (the Gemma-3-1B shapes), 2 = also == 768 but
// not 128 (a launch of Gemma's down projections only), 3 = as 1. In the plain
// kernel (neither NORM nor WIDE) 1 stands for "every row with a 128-column tail
// is 1152 columns long": its tiles are single steps (stream_rows_once), and
// without the pipelined form for that tail, which is what costs the registers,
// four waves fit a SIMD (120 registers against 164; Gemma-3-1B's 79-GEMV step
// 152.2 -> 143.2 us, its vocabulary alone 47.2 -> 44.5); 3 is the pipelined
// form for any number of whole chunks in front of the tail. The host picks the
// cheapest set that covers the products of a launch.
// NORM: the launch carries fused forms, an RMSNorm in front of its products
// and/or gate-up pairs with their activation (a separate instantiation, so that
// the plain decode kernel keeps its register budget).
// WIDE: short tiles under a long K take steps of several chunks
// (stream_rows_wide; a separate instantiation for the same reason).
template <int L, int R, int TB, bool XA, int TAILS = 0, int ND = GEMV_MAX_DESCS, bool NORM = false,
          bool WIDE = false>
__global__ __launch_bounds__(256) void gemv_list_kernel(const GemvArgsT<ND> args) {
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

    if constexpr (NORM && TB == 1 && L == PACKED) {
        if (d.pad & (GEMV_X_NORMED | GEMV_PAIR)) {
            // Every wave recomputes the row's scale (a few hundred operations)
            // instead of waiting for a separate kernel to publish it.
            // (d.pad2: which row of the norm this descriptor's token is, when a
            // few tokens go through the launch as one descriptor each)
            const float *norm_h = args.norm_h + (size_t)d.pad2 * cols;
            float *norm_out = args.norm_out + (size_t)d.pad2 * cols;
            float inv = 0.0f;
            if (d.pad & GEMV_X_NORMED) {
                const float sumsq = row_sumsq<true>(norm_h, cols, lane);
                inv = 1.0f / sqrtf(sumsq / (float)cols + args.norm_eps);
            }
            const NormedX xn{norm_h, args.norm_w, inv};
            const uint32_t tail = cols & 1023u; // 0, or (TAILS == 1) 128: the host fuses nothing else
            if ((d.pad & GEMV_WRITES_NORM) && tile == d.tile_begin) {
                for (uint32_t c = 0; c < full; ++c) {
                    float o[16];
                    xn.template load16<true>((c << 10) + lane * 16u, o);
                    float4 *dst = (float4 *)(norm_out + (c << 10) + lane * 16u);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        dst[i] = make_float4(o[4 * i], o[4 * i + 1], o[4 * i + 2], o[4 * i + 3]);
                    }
                }
                if constexpr (TAILS == 1) {
                    if (tail == 128u) {
                        float o[2];
                        xn.template loadn<2, true>(tail0 + lane * 2u, o);
                        *(float2 *)(norm_out + tail0 + lane * 2u) = make_float2(o[0], o[1]);
                    }
                }
            }
            // (a small product may be cut into shorter tiles, as below)
#define Q8_NORMED_STREAM(TAILMASK)                                                               \
    if (d.pad & GEMV_PAIR) {                                                                     \
        /* gate (this descriptor) and up (the next one, which owns no tiles; its                 \
           `res` is the activation's output, its `alpha` the kind) */                            \
        const GemvDesc &d2 = args.d[lo + 1];                                                     \
        const WView<PACKED> wu(d2.w, rows, cols);                                                \
        const uint32_t kind = (uint32_t)d2.alpha;                                                \
        /* (tiles of 2 rows of each: the short form, for whole chunks only) */                   \
        const bool short_pair = (TAILMASK) == 0 && d.rows_per_tile % 4u != 0u;                   \
        if (d.pad & GEMV_X_NORMED) {                                                             \
            if (short_pair) {                                                                    \
                stream_rows_glu_short<true, TAILMASK>(wv, wu, xn, y, d2.y, d2.res, kind, cols,   \
                                                      row_first, row_end, lane);                 \
            } else {                                                                             \
                stream_rows_glu<true, TAILMASK>(wv, wu, xn, y, d2.y, d2.res, kind, cols,         \
                                                row_first, row_end, lane);                       \
            }                                                                                    \
        } else if (short_pair) {                                                                 \
            stream_rows_glu_short<true, TAILMASK>(wv, wu, PlainX{x}, y, d2.y, d2.res, kind,      \
                                                  cols, row_first, row_end, lane);               \
        } else {                                                                                 \
            stream_rows_glu<true, TAILMASK>(wv, wu, PlainX{x}, y, d2.y, d2.res, kind, cols,      \
                                            row_first, row_end, lane);                           \
        }                                                                                        \
    } else if (d.rows_per_tile % (R / 2) != 0u) {                                                \
        stream_rows<R / 4, true, TAILMASK, NormedX>(wv, xn, y, cols, row_first, row_end, lane,   \
                                                    d.res, d.alpha);                             \
    } else if (d.rows_per_tile % R != 0u) {                                                      \
        stream_rows<R / 2, true, TAILMASK, NormedX>(wv, xn, y, cols, row_first, row_end, lane,   \
                                                    d.res, d.alpha);                             \
    } else {                                                                                     \
        stream_rows<R, true, TAILMASK, NormedX>(wv, xn, y, cols, row_first, row_end, lane,       \
                                                d.res, d.alpha);                                 \
    }
            if constexpr (TAILS == 1) {
                if (tail == 128u) {
                    Q8_NORMED_STREAM(128)
                    return;
                }
            }
            Q8_NORMED_STREAM(0)
#undef Q8_NORMED_STREAM
            return;
        }
    }
    if constexpr (TB == 1 && L == PACKED) {
        // One token, sealed weights: the decode path, software-pipelined (see
        // stream_rows). Column tails seen in practice are instantiated; other
        // shapes take the general path below. Same arithmetic either way.
        if (full >= 1u) {
            const uint32_t tail = cols & 1023u;
            if (tail == 0u) {
                // a small product may be cut into shorter tiles
                const bool quarter = d.rows_per_tile % (R / 2) != 0u;
                const bool half = !quarter && d.rows_per_tile % R != 0u;
                if constexpr (WIDE) {
                    if (full >= 2u && quarter) {
                        stream_rows_wide<R / 4, 4, XA, 0>(wv, PlainX{x}, y, cols, row_first, row_end,
                                                          lane, d.res, d.alpha);
                        return;
                    }
                    if (full >= 2u && half) {
                        stream_rows_wide<R / 2, 2, XA, 0>(wv, PlainX{x}, y, cols, row_first, row_end,
                                                          lane, d.res, d.alpha);
                        return;
                    }
                }
                if (quarter) {
                    stream_rows<R / 4, XA, 0>(wv, PlainX{x}, y, cols, row_first, row_end, lane,
                                              d.res, d.alpha);
                } else if (half) {
                    stream_rows<R / 2, XA, 0>(wv, PlainX{x}, y, cols, row_first, row_end, lane,
                                              d.res, d.alpha);
                } else {
                    stream_rows<R, XA, 0>(wv, PlainX{x}, y, cols, row_first, row_end, lane, d.res,
                                          d.alpha);
                }
                return;
            }
            // (as above, a small product may be cut into shorter tiles)
            if constexpr (TAILS == 1 && !NORM && !WIDE) {
                // every product with this tail has one whole chunk per row (the host
                // chose the instantiation by that): a tile is a single step
                if (tail == 128u && full == 1u && d.rows_per_tile <= (uint32_t)R) {
                    if (d.rows_per_tile % (R / 2) != 0u) {
                        stream_rows_once<R / 4, XA, 128>(wv, PlainX{x}, y, row_first, row_end, lane, d.res, d.alpha);
                    } else if (d.rows_per_tile % R != 0u) {
                        stream_rows_once<R / 2, XA, 128>(wv, PlainX{x}, y, row_first, row_end, lane, d.res, d.alpha);
                    } else {
                        stream_rows_once<R, XA, 128>(wv, PlainX{x}, y, row_first, row_end, lane, d.res, d.alpha);
                    }
                    return;
                }
            }
            if constexpr ((TAILS == 1 && (NORM || WIDE)) || TAILS == 3) {
                if (tail == 128u) { // any number of whole chunks, pipelined
                    if (d.rows_per_tile % (R / 2) != 0u) {
                        stream_rows<R / 4, XA, 128>(wv, PlainX{x}, y, cols, row_first, row_end, lane,
                                                    d.res, d.alpha);
                    } else if (d.rows_per_tile % R != 0u) {
                        stream_rows<R / 2, XA, 128>(wv, PlainX{x}, y, cols, row_first, row_end, lane,
                                                    d.res, d.alpha);
                    } else {
                        stream_rows<R, XA, 128>(wv, PlainX{x}, y, cols, row_first, row_end, lane,
                                                d.res, d.alpha);
                    }
                    return;
                }
            }
            if constexpr (TAILS >= 1) {
                if (tail == 768u) { // FFN 6912 (Gemma-3-1B); half the rows per pass
                    if (d.rows_per_tile % (R / 2) != 0u) {
                        if constexpr (WIDE) {
                            stream_rows_wide<R / 4, 4, XA, 768>(wv, PlainX{x}, y, cols, row_first,
                                                                row_end, lane, d.res, d.alpha);
                        } else {
                            stream_rows<R / 4, XA, 768>(wv, PlainX{x}, y, cols, row_first, row_end,
                                                        lane, d.res, d.alpha);
                        }
                    } else {
                        stream_rows<R / 2, XA, 768>(wv, PlainX{x}, y, cols, row_first, row_end, lane,
                                                    d.res, d.alpha);
                    }
                    return;
                }
            }
        }
    }

    if constexpr (TB == 1 && L == RAW) {
        // One token over weights as uploaded: rows of whole 1024-column chunks,
        // and the column tails that have a decode path of their own, stream
        // through LDS (stream_rows_raw); other shapes take the general path
        // (rows of 2^27 columns and more too: the staging indexes a pass in 32 bits).
        if (full >= 1u && cols < (1u << 27)) {
            __shared__ __attribute__((aligned(16))) uint8_t raw_stage[4][raw_stage_bytes<R, TAILS>()];
            const uint32_t tail = cols & 1023u;
            // (a small product may be cut into shorter tiles, as in the sealed layout)
#define Q8_RAW_STREAM(TAILMASK)                                                                  \
    if (d.rows_per_tile % (R / 2) != 0u) {                                                       \
        stream_rows_raw<R / 4, XA, TAILMASK>(wv, x, y, cols, row_first, row_end, lane,           \
                                             raw_stage[wave], d.res, d.alpha);                   \
    } else if (d.rows_per_tile % R != 0u) {                                                      \
        stream_rows_raw<R / 2, XA, TAILMASK>(wv, x, y, cols, row_first, row_end, lane,           \
                                             raw_stage[wave], d.res, d.alpha);                   \
    } else {                                                                                     \
        stream_rows_raw<R, XA, TAILMASK>(wv, x, y, cols, row_first, row_end, lane,               \
                                         raw_stage[wave], d.res, d.alpha);                       \
    }                                                                                            \
    return;
            if (tail == 0u) {
                Q8_RAW_STREAM(0)
            }
            if constexpr (TAILS == 1) {
                if (tail == 128u && full == 1u) { // hidden 1152 (Gemma-3-1B)
                    Q8_RAW_STREAM(128)
                }
            }
            if constexpr (TAILS >= 1) {
                if (tail == 768u) { // FFN 6912 (Gemma-3-1B)
                    Q8_RAW_STREAM(768)
                }
            }
#undef Q8_RAW_STREAM
        }
    }

    // The general form (raw layout, narrow matrices, other column tails).
    // Token groups outermost: with the row passes outermost this path, which
    // the decode shapes never take, doubled the kernel's register count and
    // halved the occupancy of the streaming path above.
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
            // Column order is part of the arithmetic: tail pieces first, then
            // the whole 1024-column chunks in ascending order.
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
            for (uint32_t c = 0; c < full; ++c) {
                chunk<L, R, TB, 16, XA, NT>(wv, x, cols, row, tok, c << 10, lane, true, acc);
            }
#pragma unroll
            for (int t = 0; t < TB; ++t) {
                float col_acc[R];
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    col_acc[r] = acc[r][t];
                }
                reduce_store<R>(col_acc, y + (size_t)(t0 + t) * rows, r0, row_end, lane,
                                t0 + t < batch, d.res, d.alpha); // res is only set for one token
            }
        }
    }
}

} // namespace q8
