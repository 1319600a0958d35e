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

struct MmaDesc {
    const uint8_t *w;
    const float *x;      // x_off already applied
    float *y;            // y_off already applied
    uint32_t rows, cols, batch;
    uint32_t tile_begin; // index of this product's first output tile in the launch
    uint32_t tiles_t;    // token tiles per row tile
    uint32_t pad;
};

// A launch of gemm_mma_kernel<..., GLU>: its one descriptor is the gate projection,
// this the up projection over the same activations and what becomes of the pair.
struct MmaGlu {
    const uint8_t *w2 = nullptr; // the up projection's weights (the descriptor's shape)
    float *y2 = nullptr;         // its output
    float *act = nullptr;        // act(gate) * up, [batch][rows]; may be the gate's output (in place)
    uint16_t *act_split = nullptr; // the split form of `act` as [rows / 32][3][batch][32] bf16, or null
    uint32_t kind = 0;           // 0 silu, 1 tanh GELU
    uint32_t pad = 0;
};

struct MmaArgs {
    uint32_t n;
    uint32_t total_tiles;
    uint32_t chunk_wgs; // workgroups that share one weight row-tile (see the XCD mapping)
    uint32_t z;         // workgroups that share one output tile, each with a part of K (1: none)
    float *partials;    // z > 1: total_tiles x z partial tiles
    uint32_t *arrivals; // z > 1: one counter per output tile, zero between launches
    MmaGlu glu;
    MmaDesc d[MMA_MAX_DESCS];
};

// Operands of one Q8_0 block for a wave's TMW x TNW tiles, as loaded.
template <int TMW, int TNW> struct MmaRaw {
    uint32_t q[TNW][4];
    uint32_t sb[TNW];
    float xv[TMW][16];
};

template <int L, int TMW, int TNW, bool XA>
__device__ __forceinline__ void mma_load_block(const WView<L> &wv, const float *x, uint32_t cols,
                                               const uint32_t (&wrow)[TNW],
                                               const uint32_t (&tok)[TMW], uint32_t kb,
                                               uint32_t half, MmaRaw<TMW, TNW> &raw) {
    const uint32_t col = (kb << 5) + (half << 4);
#pragma unroll
    for (int j = 0; j < TNW; ++j) {
        wv.template load_quants<16>(wrow[j], col, raw.q[j]);
        raw.sb[j] = wv.scale_bits(wrow[j], kb);
    }
#pragma unroll
    for (int i = 0; i < TMW; ++i) {
        load_x16<XA>(x + (size_t)tok[i] * cols + col, raw.xv[i]);
    }
}

// One launch runs a list of products (the q/k/v or gate/up projections of a
// prefill chunk share their input and do not depend on each other).
// Workgroup = 4 waves = P slots x S k-slices. Slot p of workgroup g owns
// output tile g*P + p of the launch; its S waves each take a contiguous share
// of the Q8_0 blocks; the partial tiles are added in wave order, each wave
// finishing and storing 16 / S of a lane's 16 values per tile. The k loop is
// software-pipelined: the operands of block kb+1 are requested before the
// 16*TMW*TNW MFMAs of block kb are issued.
// ZS: args.z workgroups share an output tile (S == 4 only: one tile per
// workgroup). Workgroup g takes part g % z of the K range of tile g / z; what its
// four waves add up goes to args.partials, and the workgroup that arrives last
// at the tile's counter adds the z partial tiles in part order (whoever it is:
// the result does not depend on the order of arrival), stores the sum and puts
// the counter back to zero.
//
// XP: the activations come in split form (d.x points at [cols / 32][3][batch][32]
// bf16, split_index; an operator in front of the launch has written it) and the
// products run on the bf16 matrix cores, exactly (q8_gemm_bf16x3.hpp has the
// argument): the lane's 16 quants of a block are exact in bf16, six
// v_mfma_f32_32x32x16_bf16 (pieces l, m, h times the two halves of the lane's k
// range) leave the block's sum of q*x in f32, and  acc += d * S  rescales it.
// Six matrix instructions of 8 passes stand where sixteen of 16 passes stood.
//
// GLU (with XP): the launch is the gate and the up projection of a gated unit
// (same shape, same activations) and the activation behind them. A wave's two
// accumulator tiles are the same 32 x 32 outputs of both; where the sums are
// finished, the projections, act(gate) * up and, for a product launched right
// behind, its split form are stored: one launch and one pass over the outputs in
// the place of two. Every sum is formed as in the launch without the activation.
template <int L, int TMW, int TNW, int S, bool XA, bool ZS = false, bool XP = false, bool GLU = false>
__global__ __launch_bounds__(256, XP ? 2 : 1) void gemm_mma_kernel(const MmaArgs args) {
    static_assert(!ZS || S == 4, "shared tiles: one tile per workgroup");
    static_assert(!GLU || (XP && TMW == 1 && TNW == 2 && !ZS), "gated pair: two accumulators over one 32 x 32 tile");
    constexpr int TNG = GLU ? 1 : TNW; // row tiles of 32 that a wave's outputs span
    constexpr int P = 4 / S;
    constexpr int TILE_FLOATS = TMW * TNW * 16 * WAVE;
    extern __shared__ float red[]; // S > 1: [P][S][TILE_FLOATS] (+ one word with shared tiles)

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t p = wave / S, s = wave % S;
    const uint32_t idx = lane & 31u, half = lane >> 5;

    // Workgroups are dealt round-robin to the 8 XCDs (workgroup g runs on XCD
    // g % 8), each with its own L2. Tiles are numbered token-tile fastest, so
    // `chunk_wgs` consecutive workgroups share one weight row-tile: hand whole
    // chunks to the XCDs in turn. A weight tile then lives in one L2, and
    // heavy products (large K) are spread over all XCDs instead of landing on
    // the one that owns their index range.
    uint32_t g = blockIdx.x;
    uint32_t zpart = 0;
    if constexpr (ZS) {
        zpart = g % args.z;
        g = g / args.z;
    } else {
        const uint32_t cw = args.chunk_wgs;
        const uint32_t span = 8u * cw;
        const uint32_t g_full = (gridDim.x / span) * span;
        if (g < g_full) {
            const uint32_t xcd = g & 7u, j = g >> 3;
            g = ((j / cw) * 8u + xcd) * cw + (j % cw);
        }
    }
    const uint32_t tile = g * P + p;
    const bool valid = tile < args.total_tiles;
    uint32_t lo = 0, hi = args.n;
    while (hi - lo > 1u) {
        const uint32_t mid = (lo + hi) >> 1;
        if (args.d[mid].tile_begin <= tile) {
            lo = mid;
        } else {
            hi = mid;
        }
    }
    const MmaDesc &d = args.d[lo];
    const uint32_t rows = d.rows, cols = d.cols, batch = d.batch;
    const uint32_t local = valid ? tile - d.tile_begin : 0u;
    const uint32_t tn = local / d.tiles_t, tt = local % d.tiles_t;
    const uint32_t t0 = tt * (32u * TMW), n0 = tn * (32u * TNG);
    const float *x = d.x;
    float *y = d.y;

    const WView<L> wv(d.w, rows, cols);
    const WView<L> wv2(GLU ? args.glu.w2 : d.w, rows, cols); // GLU: the up projection
    const uint32_t blocks = cols >> 5;
    // this wave's part of K: one of S, or with shared tiles one of z x S
    const uint32_t kparts = ZS ? args.z * (uint32_t)S : (uint32_t)S;
    const uint32_t kpart = ZS ? zpart * (uint32_t)S + s : s;
    const uint32_t kb_begin = (uint32_t)(((uint64_t)blocks * kpart) / kparts);
    const uint32_t kb_end = (uint32_t)(((uint64_t)blocks * (kpart + 1u)) / kparts);

    uint32_t wrow[TNW], tok[TMW];
#pragma unroll
    for (int j = 0; j < TNW; ++j) {
        const uint32_t r = n0 + (GLU ? 0u : 32u * j) + idx;
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

    if constexpr (XP) {
        // Activations in split form, sealed weights. What limits this path is what
        // the waves pull through the L2, so nothing is fetched twice: the wave's
        // K range is made of groups of four Q8_0 blocks, a group's weights are one
        // whole 128-byte line per row (four 16-byte loads per lane, issued
        // together) and its four scales one 8-byte load; the activations' pieces
        // are whole lines as they are. The next block's activations (and behind a
        // group's last block the next group's weights) are asked for as soon as
        // the block's operands are converted; more in flight than that costs the
        // registers that let two workgroups share a CU (measured with two blocks
        // of activations and two weight groups held: the gated pair at 128 tokens
        // 17.7 us against 15.3, 4096 x 1024 with two row tiles 11.1 against 9.0).
        static_assert(L == PACKED, "split-form activations: sealed weights");
        const uint32_t groups = (blocks + 3u) >> 2;
        const uint32_t g_begin = (uint32_t)(((uint64_t)groups * kpart) / kparts);
        const uint32_t g_end = (uint32_t)(((uint64_t)groups * (kpart + 1u)) / kparts);
        const uint32_t xkb_begin = g_begin * 4u;
        const uint32_t xkb_end = g_end * 4u < blocks ? g_end * 4u : blocks;
        if (valid && g_begin < g_end) {
            const uint16_t *xs = (const uint16_t *)x;
            const bool scales8 = (blocks & 3u) == 0u; // a group's scales: one aligned 8-byte load
            struct WGroup {
                u32x4 q[TNW][4];
                u32x2 sc[TNW];
            };
            struct XBlock {
                u32x4 p[TMW][3][2];
            };
            auto load_w = [&](uint32_t grp, WGroup &into) {
#pragma unroll
                for (int j = 0; j < TNW; ++j) {
                    const WView<L> &view = GLU && j == 1 ? wv2 : wv;
                    const uint8_t *row = view.q + (size_t)wrow[j] * cols + (half << 4);
#pragma unroll
                    for (int b = 0; b < 4; ++b) {
                        uint32_t kb = grp * 4u + (uint32_t)b;
                        kb = kb < blocks ? kb : blocks - 1u;
                        into.q[j][b] = *(const u32x4 *)(row + (kb << 5));
                    }
                    const uint16_t *sp = view.s + (size_t)wrow[j] * blocks + grp * 4u;
                    if (scales8) {
                        into.sc[j] = *(const u32x2 *)sp;
                    } else {
                        uint32_t h4[4];
#pragma unroll
                        for (int b = 0; b < 4; ++b) {
                            h4[b] = grp * 4u + (uint32_t)b < blocks ? (uint32_t)sp[b] : 0u;
                        }
                        into.sc[j] = u32x2{h4[0] | (h4[1] << 16), h4[2] | (h4[3] << 16)};
                    }
                }
            };
            auto load_x = [&](uint32_t kb, XBlock &into) {
#pragma unroll
                for (int i = 0; i < TMW; ++i) {
                    const uint16_t *base = xs + ((size_t)kb * 3u * batch + tok[i]) * 32u + (half << 4);
#pragma unroll
                    for (int pc = 0; pc < 3; ++pc) {
#pragma unroll
                        for (int k2 = 0; k2 < 2; ++k2) {
                            into.p[i][pc][k2] = *(const u32x4 *)(base + (size_t)pc * batch * 32u + 8u * k2);
                        }
                    }
                }
            };
            WGroup wg;
            XBlock xb;
            load_w(g_begin, wg);
            load_x(xkb_begin, xb);
            for (uint32_t grp = g_begin; grp < g_end; ++grp) {
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const uint32_t kb = grp * 4u + (uint32_t)b;
                    if (kb >= xkb_end) { // (uniform over the wave)
                        break;
                    }
                    bf16x8_t wb[TNW][2], xp[TMW][3][2];
                    float dsc[TNW];
#pragma unroll
                    for (int j = 0; j < TNW; ++j) {
                        const uint32_t pair = b < 2 ? wg.sc[j].x : wg.sc[j].y;
                        dsc[j] = f16_bits_to_f32(b % 2 ? pair >> 16 : pair & 0xffffu);
                        wb[j][0] = sbytes_to_bf16x8(wg.q[j][b].x, wg.q[j][b].y);
                        wb[j][1] = sbytes_to_bf16x8(wg.q[j][b].z, wg.q[j][b].w);
                    }
#pragma unroll
                    for (int i = 0; i < TMW; ++i) {
#pragma unroll
                        for (int pc = 0; pc < 3; ++pc) {
#pragma unroll
                            for (int k2 = 0; k2 < 2; ++k2) {
                                xp[i][pc][k2] = __builtin_bit_cast(bf16x8_t, xb.p[i][pc][k2]);
                            }
                        }
                    }
                    // the block's operands are converted: ask for the next ones
                    if (b == 3 && grp + 1u < g_end) {
                        load_w(grp + 1u, wg);
                    }
                    if (kb + 1u < xkb_end) {
                        load_x(kb + 1u, xb);
                    }
#pragma unroll
                    for (int i = 0; i < TMW; ++i) {
#pragma unroll
                        for (int j = 0; j < TNW; ++j) {
                            floatx16 sum = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f,
                                            0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                            for (int piece = 2; piece >= 0; --piece) { // smallest pieces first
#pragma unroll
                                for (int k2 = 0; k2 < 2; ++k2) {
                                    sum = __builtin_amdgcn_mfma_f32_32x32x16_bf16(xp[i][piece][k2], wb[j][k2],
                                                                                  sum, 0, 0, 0);
                                }
                            }
#pragma unroll
                            for (int v = 0; v < 16; ++v) {
                                acc[i][j][v] = __builtin_fmaf(dsc[j], sum[v], acc[i][j][v]);
                            }
                        }
                    }
                }
            }
        }
    } else if (valid && kb_begin < kb_end) {
        MmaRaw<TMW, TNW> raw;
        mma_load_block<L, TMW, TNW, XA>(wv, x, cols, wrow, tok, kb_begin, half, raw);
        for (uint32_t kb = kb_begin; kb < kb_end; ++kb) {
            float wf[TNW][16];
            float xa[TMW][16];
#pragma unroll
            for (int j = 0; j < TNW; ++j) {
                const float dsc = f16_bits_to_f32(raw.sb[j]);
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    wf[j][e] = dsc * sbyte_to_float(raw.q[j][e / 4], e % 4);
                }
            }
#pragma unroll
            for (int i = 0; i < TMW; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    xa[i][e] = raw.xv[i][e];
                }
            }
            if (kb + 1u < kb_end) {
                mma_load_block<L, TMW, TNW, XA>(wv, x, cols, wrow, tok, kb + 1u, half, raw);
            }
#pragma unroll
            for (int e = 0; e < 16; ++e) {
#pragma unroll
                for (int i = 0; i < TMW; ++i) {
#pragma unroll
                    for (int j = 0; j < TNW; ++j) {
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(xa[i][e], wf[j][e],
                                                                         acc[i][j], 0, 0, 0);
                    }
                }
            }
        }
    }

    if constexpr (S > 1) {
        // What follows the matrix instructions counts in these launches (short K
        // ranges, workgroups that share a tile): every wave leaves its partial tile
        // in LDS, and wave s adds up (in wave order) and finishes the 16 / S values
        // per lane and tile that start at value (16 / S) * s.
        constexpr int VQ = 16 / S;
        float *slot = red + (size_t)p * S * TILE_FLOATS; // [S][TILE_FLOATS]
#pragma unroll
        for (int i = 0; i < TMW; ++i) {
#pragma unroll
            for (int j = 0; j < TNW; ++j) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    slot[(size_t)s * TILE_FLOATS + ((i * TNW + j) * 16 + v) * WAVE + lane] = acc[i][j][v];
                }
            }
        }
        __syncthreads();
        if (!valid) {
            return; // (with shared tiles a workgroup is one tile: all of its waves leave here)
        }
        float fin[TMW][TNW][VQ];
#pragma unroll
        for (int i = 0; i < TMW; ++i) {
#pragma unroll
            for (int j = 0; j < TNW; ++j) {
#pragma unroll
                for (int vv = 0; vv < VQ; ++vv) {
                    const uint32_t at = ((i * TNW + j) * 16 + (uint32_t)VQ * s + vv) * WAVE + lane;
                    float sum = slot[at];
#pragma unroll
                    for (int o = 1; o < S; ++o) {
                        sum += slot[(size_t)o * TILE_FLOATS + at];
                    }
                    fin[i][j][vv] = sum;
                }
            }
        }
        if constexpr (ZS) {
            // The tile's z workgroups exchange their sums through memory with
            // device-scope accesses (sc1: past this XCD's L2, so no cache has to be
            // written back or invalidated to publish them; what is needed is
            // order). Producer: every wave waits until its stores are acknowledged
            // (vmcnt(0)), the workgroup's barrier follows, and only then does one
            // lane count the arrival. Consumer: the count comes back to every wave
            // through LDS behind a second barrier, and the loads of the last
            // workgroup to arrive are issued after it. The empty asm statements
            // keep the compiler from moving the relaxed atomics across either
            // point. Device-scope release and acquire fences in their place write
            // back and invalidate the whole L2 under the other workgroups: measured
            // 1.7 us per launch of 12-15 us, and far more on launches with hundreds
            // of workgroups.
            const uint32_t z = args.z;
            uint32_t *flag = (uint32_t *)(red + (size_t)S * TILE_FLOATS); // (one tile per workgroup)
            float *mine = args.partials + ((size_t)tile * z + zpart) * TILE_FLOATS + lane;
#pragma unroll
            for (int i = 0; i < TMW; ++i) {
#pragma unroll
                for (int j = 0; j < TNW; ++j) {
#pragma unroll
                    for (int vv = 0; vv < VQ; ++vv) {
                        __hip_atomic_store(mine + ((i * TNW + j) * 16 + (uint32_t)VQ * s + vv) * WAVE,
                                           fin[i][j][vv], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                }
            }
            __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8)); // vmcnt(0)
            asm volatile("" ::: "memory");
            __syncthreads();
            if (threadIdx.x == 0u) {
                *flag = __hip_atomic_fetch_add(&args.arrivals[tile], 1u, __ATOMIC_RELAXED,
                                               __HIP_MEMORY_SCOPE_AGENT);
            }
            __syncthreads();
            const uint32_t arrived = __builtin_amdgcn_readfirstlane(*flag);
            if (arrived != z - 1u) {
                return;
            }
            asm volatile("" ::: "memory");
            if (threadIdx.x == 0u) { // (every workgroup of the tile has counted itself)
                __hip_atomic_store(&args.arrivals[tile], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            const float *first = args.partials + (size_t)tile * z * TILE_FLOATS + lane;
            for (uint32_t c = 0; c < z; ++c) { // in part order, whoever arrived last
                const float *part = first + (size_t)c * TILE_FLOATS;
#pragma unroll
                for (int i = 0; i < TMW; ++i) {
#pragma unroll
                    for (int j = 0; j < TNW; ++j) {
#pragma unroll
                        for (int vv = 0; vv < VQ; ++vv) {
                            const float pv = __hip_atomic_load(
                                part + ((i * TNW + j) * 16 + (uint32_t)VQ * s + vv) * WAVE, __ATOMIC_RELAXED,
                                __HIP_MEMORY_SCOPE_AGENT);
                            fin[i][j][vv] = c == 0u ? pv : fin[i][j][vv] + pv;
                        }
                    }
                }
            }
        }
        // value v of a 32x32 tile is (token 8*(v/4) + 4*half + v%4, row idx)
        if constexpr (GLU) {
            const uint32_t n = n0 + idx;
            float *y2 = args.glu.y2, *act = args.glu.act;
            uint16_t *act_split = args.glu.act_split;
            const uint32_t kind = args.glu.kind;
#pragma unroll
            for (int vv = 0; vv < VQ; ++vv) {
                const uint32_t v = (uint32_t)VQ * s + vv;
                const uint32_t t = t0 + 8u * (v / 4u) + 4u * half + (v % 4u);
                if (t < batch && n < rows) {
                    const float gv = fin[0][0][vv], uv = fin[0][1][vv];
                    const float a = glu_act(gv, uv, kind);
                    const size_t at = (size_t)t * rows + n;
                    if (act != y) {
                        y[at] = gv;
                    }
                    y2[at] = uv;
                    act[at] = a;
                    if (act_split != nullptr) {
                        split_store(act_split, batch, t, n, a);
                    }
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < TMW; ++i) {
#pragma unroll
                for (int j = 0; j < TNW; ++j) {
                    const uint32_t n = n0 + 32u * j + idx;
#pragma unroll
                    for (int vv = 0; vv < VQ; ++vv) {
                        const uint32_t v = (uint32_t)VQ * s + vv;
                        const uint32_t t = t0 + 32u * i + 8u * (v / 4u) + 4u * half + (v % 4u);
                        if (t < batch && n < rows) {
                            y[(size_t)t * rows + n] = fin[i][j][vv];
                        }
                    }
                }
            }
        }
        return;
    }
    if (!valid) {
        return;
    }
    // acc[v] of a 32x32 tile is (token 8*(v/4) + 4*half + v%4, row idx).
    if constexpr (GLU) {
        const uint32_t n = n0 + idx;
        float *y2 = args.glu.y2, *act = args.glu.act;
        uint16_t *act_split = args.glu.act_split;
        const uint32_t kind = args.glu.kind;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const uint32_t t = t0 + 8u * (v / 4) + 4u * half + (v % 4);
            if (t < batch && n < rows) {
                const float gv = acc[0][0][v], uv = acc[0][1][v];
                const float a = glu_act(gv, uv, kind);
                const size_t at = (size_t)t * rows + n;
                if (act != y) {
                    y[at] = gv;
                }
                y2[at] = uv;
                act[at] = a;
                if (act_split != nullptr) {
                    split_store(act_split, batch, t, n, a);
                }
            }
        }
        return;
    }
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

// ---------------------------------------------------------------------------
// Persistent form of the kernel above for the common configuration (one slot
// per workgroup, K split over its 4 waves, TNW = 1, sealed or raw weights).
//
// Measured on the M = 512 projection set: a wave of the one-tile-per-workgroup
// kernel spends about as long before its first MFMA (first operands: 11 k
// cycles median) and after its last (barrier, reduction by one wave, stores:
// 7 k median) as it needs to issue its MFMAs (16 k), and vector instructions
// do not overlap with f32 MFMAs on this part (each costs the matrix pipe about
// five cycles). So here
//   * a workgroup walks a strided list of tiles and requests the first block
//     of the next tile before it finishes the current one;
//   * the two operand sets are used in turn with no register copies: per
//     block only the dequantisation d*q remains beside the MFMAs;
//   * every wave writes its partial tile to LDS and reduces and stores one
//     quarter of it (sum order wave 0, 1, 2, 3 as before).
struct MmaTileCtx {
    const uint8_t *w;
    const float *x;
    float *y;
    uint32_t rows, cols, batch, t0, n0, kb_begin, kb_end;
};

template <int L, int TMW, bool XA>
__global__ __launch_bounds__(256) void gemm_mma_persistent_kernel(const MmaArgs args) {
    constexpr int S = 4;
    constexpr int NV = TMW * 16;          // accumulator values per lane
    constexpr int QV = NV / S;            // values a wave reduces and stores
    __shared__ float red[S][NV][WAVE];

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t s = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t idx = lane & 31u, half = lane >> 5;
    const uint32_t nwg = gridDim.x;

    // Same workgroup -> XCD dealing as gemm_mma_kernel (gridDim.x is a multiple
    // of 8, so workgroup b keeps its XCD for every tile of its list).
    auto tile_of = [&](uint32_t g) -> uint32_t {
        const uint32_t cw = args.chunk_wgs;
        const uint32_t span = 8u * cw;
        const uint32_t g_full = (args.total_tiles / span) * span;
        if (g < g_full) {
            const uint32_t xcd = g & 7u, j = g >> 3;
            g = ((j / cw) * 8u + xcd) * cw + (j % cw);
        }
        return g;
    };
    auto decode = [&](uint32_t g, MmaTileCtx &c) {
        const uint32_t tile = tile_of(g);
        uint32_t lo = 0, hi = args.n;
        while (hi - lo > 1u) {
            const uint32_t mid = (lo + hi) >> 1;
            if (args.d[mid].tile_begin <= tile) {
                lo = mid;
            } else {
                hi = mid;
            }
        }
        const MmaDesc &d = args.d[lo];
        c.w = d.w; c.x = d.x; c.y = d.y;
        c.rows = d.rows; c.cols = d.cols; c.batch = d.batch;
        const uint32_t local = tile - d.tile_begin;
        c.t0 = (local % d.tiles_t) * (32u * TMW);
        c.n0 = (local / d.tiles_t) * 32u;
        const uint32_t blocks = d.cols >> 5;
        c.kb_begin = (uint32_t)(((uint64_t)blocks * s) / S);
        c.kb_end = (uint32_t)(((uint64_t)blocks * (s + 1u)) / S);
    };
    auto load = [&](const MmaTileCtx &c, uint32_t kb, MmaRaw<TMW, 1> &raw) {
        const WView<L> wv(c.w, c.rows, c.cols);
        const uint32_t r = c.n0 + idx;
        const uint32_t wrow[1] = {r < c.rows ? r : c.rows - 1u};
        uint32_t tok[TMW];
#pragma unroll
        for (int i = 0; i < TMW; ++i) {
            const uint32_t t = c.t0 + 32u * i + idx;
            tok[i] = t < c.batch ? t : c.batch - 1u;
        }
        mma_load_block<L, TMW, 1, XA>(wv, c.x, c.cols, wrow, tok, kb, half, raw);
    };

    floatx16 acc[TMW];
    auto block = [&](const MmaRaw<TMW, 1> &cur) {
        float wf[16];
        const float dsc = f16_bits_to_f32(cur.sb[0]);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            wf[e] = dsc * sbyte_to_float(cur.q[0][e / 4], e % 4);
        }
#pragma unroll
        for (int e = 0; e < 16; ++e) {
#pragma unroll
            for (int i = 0; i < TMW; ++i) {
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(cur.xv[i][e], wf[e], acc[i], 0, 0, 0);
            }
        }
    };

    uint32_t g = blockIdx.x;
    if (g >= args.total_tiles) {
        return;
    }
    MmaTileCtx cur;
    decode(g, cur);
    MmaRaw<TMW, 1> ra, rb;
    load(cur, cur.kb_begin, ra); // invariant: `ra` holds the first block of the tile about to run
    while (true) {
        const uint32_t gn = g + nwg;
        const bool more = gn < args.total_tiles; // uniform over the workgroup
        MmaTileCtx nxt = cur;
        if (more) {
            decode(gn, nxt);
        }
#pragma unroll
        for (int i = 0; i < TMW; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                acc[i][v] = 0.0f;
            }
        }
        // The wave's blocks, two per trip; every step requests the operands
        // of the following step first (the next tile's first block at the
        // end: without a next tile the last block is requested once more).
        uint32_t kb = cur.kb_begin;
        const uint32_t ke = cur.kb_end;
        for (; kb + 2u < ke; kb += 2u) {
            load(cur, kb + 1u, rb);
            __builtin_amdgcn_sched_barrier(0);
            block(ra);
            load(cur, kb + 2u, ra);
            __builtin_amdgcn_sched_barrier(0);
            block(rb);
        }
        if (kb + 2u == ke) { // two blocks left
            load(cur, kb + 1u, rb);
            __builtin_amdgcn_sched_barrier(0);
            block(ra);
            load(nxt, more ? nxt.kb_begin : kb + 1u, ra);
            __builtin_amdgcn_sched_barrier(0);
            block(rb);
        } else if (kb + 1u == ke) { // one block left
            load(nxt, more ? nxt.kb_begin : kb, rb);
            __builtin_amdgcn_sched_barrier(0);
            block(ra);
            ra = rb;
        } else if (more) { // a wave without blocks (fewer blocks than waves)
            load(nxt, nxt.kb_begin, ra);
        }

        // Reduction over the 4 k-slices: everybody parks its partial tile,
        // then wave s adds values s*QV .. s*QV+QV-1 in slice order and stores.
        __syncthreads(); // the previous tile's partials have been read
#pragma unroll
        for (int i = 0; i < TMW; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                red[s][i * 16 + v][lane] = acc[i][v];
            }
        }
        __syncthreads();
        const uint32_t n = cur.n0 + idx;
#pragma unroll
        for (int k = 0; k < QV; ++k) {
            const uint32_t q = s * QV + k;
            float sum = red[0][q][lane];
#pragma unroll
            for (int o = 1; o < S; ++o) {
                sum += red[o][q][lane];
            }
            const uint32_t i = q >> 4, v = q & 15u;
            const uint32_t t = cur.t0 + 32u * i + 8u * (v >> 2) + 4u * half + (v & 3u);
            if (t < cur.batch && n < cur.rows) {
                cur.y[(size_t)t * cur.rows + n] = sum;
            }
        }
        if (!more) {
            break;
        }
        g = gn;
        cur = nxt;
    }
}

// ---------------------------------------------------------------------------
// Work-queue form for launches with more wave tiles than the chip holds waves.
//
// A wave owns a 32*TMW-token x 32-row tile over the WHOLE of K and takes its
// next tile from a counter in device memory, so nothing synchronises: no
// workgroup barrier, no partial tiles through LDS, and tiles of different
// length (products with different K share a launch, longest first) balance
// themselves. The result has the bits of the K-split kernels above: the wave
// runs the four K quarters one after the other, each as its own MFMA chain
// from zero, and adds the four partial tiles in slice order.
//
// queue[0] hands out tiles beyond the first one per wave, queue[1] counts
// finished waves; the last wave to finish sets both back to zero, so a launch
// needs them zero on entry and leaves them zero (launches that share the
// counters must not overlap: one stream per context). Every wave ends after
// exactly one grab past the end of the list.
template <int L, int TMW, bool XA>
__global__ __launch_bounds__(256, 2) void gemm_mma_queue_kernel(const MmaArgs args, uint32_t *queue) {
    constexpr int S = 4;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t idx = lane & 31u, half = lane >> 5;
    const uint32_t nwaves = gridDim.x * 4u; // <= total_tiles (the launcher sees to it)
    const uint32_t total = args.total_tiles;

    auto decode = [&](uint32_t tile, MmaTileCtx &c) {
        uint32_t lo = 0, hi = args.n;
        while (hi - lo > 1u) {
            const uint32_t mid = (lo + hi) >> 1;
            if (args.d[mid].tile_begin <= tile) {
                lo = mid;
            } else {
                hi = mid;
            }
        }
        const MmaDesc &d = args.d[lo];
        c.w = d.w; c.x = d.x; c.y = d.y;
        c.rows = d.rows; c.cols = d.cols; c.batch = d.batch;
        const uint32_t local = tile - d.tile_begin;
        c.t0 = (local % d.tiles_t) * (32u * TMW);
        c.n0 = (local / d.tiles_t) * 32u;
        c.kb_begin = 0;
        c.kb_end = d.cols >> 5;
    };
    auto load = [&](const MmaTileCtx &c, uint32_t kb, MmaRaw<TMW, 1> &raw) {
        const WView<L> wv(c.w, c.rows, c.cols);
        const uint32_t r = c.n0 + idx;
        const uint32_t wrow[1] = {r < c.rows ? r : c.rows - 1u};
        uint32_t tok[TMW];
#pragma unroll
        for (int i = 0; i < TMW; ++i) {
            const uint32_t t = c.t0 + 32u * i + idx;
            tok[i] = t < c.batch ? t : c.batch - 1u;
        }
        mma_load_block<L, TMW, 1, XA>(wv, c.x, c.cols, wrow, tok, kb, half, raw);
    };

    floatx16 acc[TMW];
    auto block = [&](const MmaRaw<TMW, 1> &cur) {
        float wf[16];
        const float dsc = f16_bits_to_f32(cur.sb[0]);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            wf[e] = dsc * sbyte_to_float(cur.q[0][e / 4], e % 4);
        }
#pragma unroll
        for (int e = 0; e < 16; ++e) {
#pragma unroll
            for (int i = 0; i < TMW; ++i) {
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(cur.xv[i][e], wf[e], acc[i], 0, 0, 0);
            }
        }
    };

    MmaRaw<TMW, 1> ra, rb;
    // Blocks [kb0, kb1) of `c` (at least one), `ra` holding block kb0 on entry
    // and block `nkb` of `nc` on exit: every step requests the operands of the
    // following step before it issues its own MFMAs.
    auto quarter = [&](const MmaTileCtx &c, uint32_t kb0, uint32_t kb1, const MmaTileCtx &nc,
                       uint32_t nkb) {
        uint32_t kb = kb0;
        for (; kb + 2u < kb1; kb += 2u) {
            load(c, kb + 1u, rb);
            __builtin_amdgcn_sched_barrier(0);
            block(ra);
            load(c, kb + 2u, ra);
            __builtin_amdgcn_sched_barrier(0);
            block(rb);
        }
        if (kb + 2u == kb1) {
            load(c, kb + 1u, rb);
            __builtin_amdgcn_sched_barrier(0);
            block(ra);
            load(nc, nkb, ra);
            __builtin_amdgcn_sched_barrier(0);
            block(rb);
        } else {
            load(nc, nkb, rb);
            __builtin_amdgcn_sched_barrier(0);
            block(ra);
            ra = rb;
        }
    };

    uint32_t tile = blockIdx.x * 4u + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    MmaTileCtx cur;
    decode(tile, cur);
    load(cur, 0, ra);
    while (true) {
        // Ask for the next tile now; the answer is looked at before the last quarter.
        uint32_t ticket = 0;
        if (lane == 0u) {
            ticket = atomicAdd(&queue[0], 1u);
        }
        const uint32_t blocks = cur.kb_end;
        floatx16 sum[TMW];
#pragma unroll
        for (int i = 0; i < TMW; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                sum[i][v] = 0.0f;
            }
        }
        auto fold = [&]() {
#pragma unroll
            for (int i = 0; i < TMW; ++i) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    sum[i][v] += acc[i][v];
                    acc[i][v] = 0.0f;
                }
            }
        };
#pragma unroll
        for (int i = 0; i < TMW; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                acc[i][v] = 0.0f;
            }
        }
        for (uint32_t s = 0; s + 1u < (uint32_t)S; ++s) {
            const uint32_t kb0 = (uint32_t)(((uint64_t)blocks * s) / S);
            const uint32_t kb1 = (uint32_t)(((uint64_t)blocks * (s + 1u)) / S);
            quarter(cur, kb0, kb1, cur, kb1);
            fold();
        }
        const uint32_t next = nwaves + __builtin_amdgcn_readfirstlane(ticket);
        const bool more = next < total;
        MmaTileCtx nxt = cur;
        if (more) {
            decode(next, nxt);
        }
        const uint32_t kb3 = (uint32_t)(((uint64_t)blocks * 3u) / S);
        quarter(cur, kb3, blocks, nxt, more ? 0u : blocks - 1u);
        fold();

        // sum[i][v] is (token 8*(v/4) + 4*half + v%4, row idx) of token tile i
        const uint32_t n = cur.n0 + idx;
#pragma unroll
        for (int i = 0; i < TMW; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const uint32_t t = cur.t0 + 32u * i + 8u * (v / 4) + 4u * half + (v % 4);
                if (t < cur.batch && n < cur.rows) {
                    cur.y[(size_t)t * cur.rows + n] = sum[i][v];
                }
            }
        }
        if (!more) {
            break;
        }
        tile = next;
        cur = nxt;
    }
    if (lane == 0u) {
        const uint32_t done = atomicAdd(&queue[1], 1u);
        if (done == nwaves - 1u) { // every other wave has made its last grab
            atomicExch(&queue[0], 0u);
            atomicExch(&queue[1], 0u);
        }
    }
}

// Resident workgroups of a 256-thread kernel on the current device (a multiple of 8).
template <class K> inline uint32_t mma_resident_wgs(K kernel) {
    int per_cu = 0, dev = 0, cus = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void *)kernel, 256, 0) !=
            hipSuccess ||
        hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        per_cu <= 0 || cus <= 0) {
        (void)hipGetLastError();
        return 512u;
    }
    return ((uint32_t)per_cu * (uint32_t)cus) & ~7u;
}

// Launches with at least this many wave tiles per resident wave use the work-queue kernel.
constexpr uint32_t MMA_QUEUE_MIN_TILES_PER_WAVE = 8;

// What a launch whose output tiles are shared between workgroups needs beside
// the products: MMA_SHARED_PARTIAL_FLOATS floats for the partial tiles and
// MMA_SHARED_MAX_TILES zeroed counters (null: no such launches).
struct MmaShared {
    float *partials = nullptr;
    uint32_t *arrivals = nullptr;
};

// Floats of one partial tile.
constexpr uint32_t mma_tile_floats(int tmw) { return (uint32_t)tmw * 16u * WAVE; }

template <int L, int TMW, int TNW, int S, bool XA>
inline hipError_t launch_mma_cfg(hipStream_t stream, hipEvent_t stop, const MmaProduct *prods_in,
                                 int n, uint32_t *queue, const MmaShared &shared) {
    constexpr int P = 4 / S;
    MmaArgs args;
    args.n = (uint32_t)n;
    args.z = 1;
    args.partials = nullptr;
    args.arrivals = nullptr;
    const MmaConfig c{TMW, TNW, S};
    uint64_t tiles = 0;
    uint32_t min_batch = 0xffffffffu;
    for (int i = 0; i < n; ++i) {
        tiles += mma_tiles(prods_in[i], c);
        min_batch = prods_in[i].batch < min_batch ? prods_in[i].batch : min_batch;
    }
    // Which form runs (see the kernels): the work queue from 8 wave tiles per
    // resident wave, else persistent workgroups from 256 tokens (measured on the
    // 2B-class shapes: below that their static tile lists balance worse than the
    // hardware's workgroup dispatch, M = 64 was 1.8x slower), else one tile per
    // workgroup.
    bool use_queue = false, use_persistent = false;
    uint32_t launch_wgs = 0;
    const uint32_t groups = (uint32_t)((tiles + P - 1) / P);
    uint32_t z = 1;
    if constexpr (S == 4 && TNW == 1) if (shared.partials != nullptr && shared.arrivals != nullptr) {
        uint32_t min_blocks = 0xffffffffu;
        for (int i = 0; i < n; ++i) {
            const uint32_t blocks = prods_in[i].cols / 32u;
            min_blocks = blocks < min_blocks ? blocks : min_blocks;
        }
        z = mma_shared_parts(tiles, min_blocks);
    }
    const bool shared_tiles = z > 1u;
    if constexpr (S == 4 && TNW == 1 && TMW == 2) if (queue != nullptr && !shared_tiles) {
        static const uint32_t resident = mma_resident_wgs(gemm_mma_queue_kernel<L, TMW, XA>);
        if (tiles >= (uint64_t)resident * 4u * MMA_QUEUE_MIN_TILES_PER_WAVE) {
            use_queue = true;
            launch_wgs = resident;
        }
    }
    if constexpr (S == 4 && TNW == 1) if (!use_queue && !shared_tiles && min_batch >= 256u) {
        static const uint32_t resident = mma_resident_wgs(gemm_mma_persistent_kernel<L, TMW, XA>);
        const uint32_t wgs = groups < resident ? groups : resident;
        if (wgs == groups || wgs % 8u == 0u) {
            use_persistent = true;
            launch_wgs = wgs;
        }
    }
    // Longest K first where tiles are handed out in list order (the work queue,
    // the hardware's workgroup dispatch): the long ones must not be the last to
    // start (M = 64 on the 2B shapes: 87 -> 98 TFLOP/s). The persistent form's
    // strided lists did better in the caller's order. The order of the list
    // does not change any product's result.
    MmaProduct prods[MMA_MAX_DESCS];
    for (int i = 0; i < n; ++i) {
        int at = i;
        while (!use_persistent && at > 0 && prods[at - 1].cols < prods_in[i].cols) {
            prods[at] = prods[at - 1];
            --at;
        }
        prods[at] = prods_in[i];
    }
    tiles = 0;
    for (int i = 0; i < n; ++i) {
        MmaDesc &d = args.d[i];
        d.w = prods[i].w;
        d.x = prods[i].x;
        d.y = prods[i].y;
        d.rows = prods[i].rows;
        d.cols = prods[i].cols;
        d.batch = prods[i].batch;
        d.tile_begin = (uint32_t)tiles;
        d.tiles_t = (prods[i].batch + 32u * TMW - 1) / (32u * TMW);
        d.pad = 0;
        tiles += mma_tiles(prods[i], c);
    }
    args.total_tiles = (uint32_t)tiles;
    args.chunk_wgs = args.d[0].tiles_t >= (uint32_t)P ? args.d[0].tiles_t / P : 1u;
    if constexpr (S == 4 && TNW == 1) if (shared_tiles) {
        static_assert(256u * mma_tile_floats(2) <= MMA_SHARED_PARTIAL_FLOATS, "partial tiles");
        args.z = z;
        args.partials = shared.partials;
        args.arrivals = shared.arrivals;
        // (every wave's partial tile, and the word through which the arrival count reaches them)
        const size_t lds = (size_t)S * TMW * TNW * 16 * WAVE * sizeof(float) + 16u;
        Q8_LAUNCH((gemm_mma_kernel<L, TMW, TNW, S, XA, true>), dim3(groups * z), dim3(256), lds,
                  stream, stop, args);
        return hipGetLastError();
    }
    if constexpr (S == 4 && TNW == 1 && TMW == 2) if (use_queue) {
        Q8_LAUNCH((gemm_mma_queue_kernel<L, TMW, XA>), dim3(launch_wgs), dim3(256), 0, stream, stop,
                  args, queue);
        return hipGetLastError();
    }
    if constexpr (S == 4 && TNW == 1) if (use_persistent) {
        Q8_LAUNCH((gemm_mma_persistent_kernel<L, TMW, XA>), dim3(launch_wgs), dim3(256), 0, stream,
                  stop, args);
        return hipGetLastError();
    }
    const size_t lds = S > 1 ? (size_t)P * S * TMW * TNW * 16 * WAVE * sizeof(float) : 0; // every wave's partial tile
    Q8_LAUNCH((gemm_mma_kernel<L, TMW, TNW, S, XA>), dim3(groups), dim3(256), lds, stream, stop,
              args);
    return hipGetLastError();
}

// Products over sealed weights whose activations are in split form: prods[i].x
// points at the split form ([cols / 32][3][batch][32] bf16) of the product's
// activations, not at the activations.
template <int TNW, int S>
inline hipError_t launch_mma_split_cfg(hipStream_t stream, hipEvent_t stop, const MmaProduct *prods_in,
                                       int n, const MmaShared &shared, const MmaGlu *glu = nullptr) {
    constexpr int P = 4 / S;
    MmaArgs args;
    args.n = (uint32_t)n;
    args.z = 1;
    args.partials = nullptr;
    args.arrivals = nullptr;
    const MmaConfig c{1, TNW, S};
    // longest K first: the hardware hands the tiles out in list order
    MmaProduct prods[MMA_MAX_DESCS];
    for (int i = 0; i < n; ++i) {
        int at = i;
        while (at > 0 && prods[at - 1].cols < prods_in[i].cols) {
            prods[at] = prods[at - 1];
            --at;
        }
        prods[at] = prods_in[i];
    }
    uint64_t tiles = 0;
    uint32_t min_blocks = 0xffffffffu;
    for (int i = 0; i < n; ++i) {
        MmaDesc &d = args.d[i];
        d.w = prods[i].w;
        d.x = prods[i].x;
        d.y = prods[i].y;
        d.rows = prods[i].rows;
        d.cols = prods[i].cols;
        d.batch = prods[i].batch;
        d.tile_begin = (uint32_t)tiles;
        d.tiles_t = (prods[i].batch + 31u) / 32u;
        d.pad = 0;
        tiles += mma_tiles(prods[i], c);
        const uint32_t blocks = prods[i].cols / 32u;
        min_blocks = blocks < min_blocks ? blocks : min_blocks;
    }
    if (tiles >= (1ull << 31)) {
        return hipErrorInvalidValue;
    }
    args.total_tiles = (uint32_t)tiles;
    args.chunk_wgs = args.d[0].tiles_t >= (uint32_t)P ? args.d[0].tiles_t / P : 1u;
    const uint32_t groups = (uint32_t)((tiles + P - 1) / P);
    if constexpr (TNW == 1) if (glu != nullptr) { // (n == 1: the gate projection's descriptor)
        args.glu = *glu;
        const size_t lds = S > 1 ? (size_t)P * S * 2 * 16 * WAVE * sizeof(float) : 0;
        Q8_LAUNCH((gemm_mma_kernel<PACKED, 1, 2, S, true, false, true, true>), dim3(groups), dim3(256), lds,
                  stream, stop, args);
        return hipGetLastError();
    }
    if constexpr (S == 4) if (glu == nullptr && shared.partials != nullptr && shared.arrivals != nullptr) {
        static_assert(256u * (uint32_t)TNW * 16u * WAVE <= MMA_SHARED_PARTIAL_FLOATS, "partial tiles");
        const uint32_t z = mma_shared_parts(tiles, min_blocks);
        if (z > 1u) {
            args.z = z;
            args.partials = shared.partials;
            args.arrivals = shared.arrivals;
            const size_t lds = (size_t)S * TNW * 16 * WAVE * sizeof(float) + 16u;
            Q8_LAUNCH((gemm_mma_kernel<PACKED, 1, TNW, S, true, true, true>), dim3(groups * z), dim3(256),
                      lds, stream, stop, args);
            return hipGetLastError();
        }
    }
    const size_t lds = S > 1 ? (size_t)P * S * TNW * 16 * WAVE * sizeof(float) : 0; // every wave's partial tile
    Q8_LAUNCH((gemm_mma_kernel<PACKED, 1, TNW, S, true, false, true>), dim3(groups), dim3(256), lds,
              stream, stop, args);
    return hipGetLastError();
}

// `glu`: the list is the gate projection alone; glu names the up projection, the
// activation's kind and where its result goes (gemm_mma_kernel<..., GLU>).
inline hipError_t launch_gemm_mma_split_list(hipStream_t stream, hipEvent_t stop, const MmaProduct *prods,
                                             int n, const MmaShared &shared, const MmaGlu *glu = nullptr) {
    if (n <= 0 || n > MMA_MAX_DESCS) {
        return hipErrorInvalidValue;
    }
    if (glu != nullptr) {
        if (n != 1 || glu->w2 == nullptr || glu->y2 == nullptr || glu->act == nullptr || glu->kind > 1u ||
            (uint64_t)prods[0].batch * prods[0].cols * 3u >= (1ull << 32) || prods[0].cols % 32u != 0u ||
            (glu->act_split != nullptr &&
             ((uint64_t)prods[0].batch * prods[0].rows * 3u >= (1ull << 32) || prods[0].rows % 32u != 0u))) {
            return hipErrorInvalidValue;
        }
        const uint32_t blocks = prods[0].cols / 32u;
        if (blocks >= 16u) {
            return launch_mma_split_cfg<1, 4>(stream, stop, prods, 1, shared, glu);
        }
        if (blocks >= 8u) {
            return launch_mma_split_cfg<1, 2>(stream, stop, prods, 1, shared, glu);
        }
        return launch_mma_split_cfg<1, 1>(stream, stop, prods, 1, shared, glu);
    }
    for (int i = 0; i < n; ++i) {
        // (the kernel indexes a product's split form in 32 bits of bf16 units)
        if ((uint64_t)prods[i].batch * prods[i].cols * 3u >= (1ull << 32) || prods[i].cols % 32u != 0u) {
            return hipErrorInvalidValue;
        }
    }
    const MmaConfig c = pick_mma_split_config(prods, n);
    if (c.tnw == 2) {
        return launch_mma_split_cfg<2, 4>(stream, stop, prods, n, shared);
    }
    if (c.s == 4) {
        return launch_mma_split_cfg<1, 4>(stream, stop, prods, n, shared);
    }
    if (c.s == 2) {
        return launch_mma_split_cfg<1, 2>(stream, stop, prods, n, shared);
    }
    return launch_mma_split_cfg<1, 1>(stream, stop, prods, n, shared);
}

template <int L, bool XA>
inline hipError_t launch_mma_layout(hipStream_t stream, hipEvent_t stop, const MmaProduct *prods,
                                    int n, const MmaConfig *forced, uint32_t *queue,
                                    const MmaShared &shared) {
    const MmaConfig c = forced != nullptr ? *forced : pick_mma_config(prods, n);
#define TM_MMA_CASE(A, B, C)                                                          \
    if (c.tmw == A && c.tnw == B && c.s == C) {                                       \
        return launch_mma_cfg<L, A, B, C, XA>(stream, stop, prods, n, queue, shared); \
    }
    TM_MMA_CASE(2, 1, 1)
    TM_MMA_CASE(1, 1, 1)
    TM_MMA_CASE(2, 1, 2)
    TM_MMA_CASE(1, 1, 2)
    TM_MMA_CASE(2, 1, 4)
    TM_MMA_CASE(1, 1, 4)
#undef TM_MMA_CASE
    return hipErrorInvalidValue;
}

// All products of one call share the weight layout and the 16-byte alignment
// class of their activations (the caller groups them so). `queue`: two zeroed
// uint32 counters in device memory owned by the stream's context (see
// gemm_mma_queue_kernel), or null to do without that kernel.
inline hipError_t launch_gemm_mma_list(hipStream_t stream, hipEvent_t stop, bool packed,
                                       bool xaligned, const MmaProduct *prods, int n,
                                       const MmaConfig *forced = nullptr,
                                       uint32_t *queue = nullptr,
                                       const MmaShared &shared = MmaShared()) {
    if (n <= 0 || n > MMA_MAX_DESCS) {
        return hipErrorInvalidValue;
    }
    if (packed) {
        return xaligned
                   ? launch_mma_layout<PACKED, true>(stream, stop, prods, n, forced, queue, shared)
                   : launch_mma_layout<PACKED, false>(stream, stop, prods, n, forced, queue, shared);
    }
    return xaligned ? launch_mma_layout<RAW, true>(stream, stop, prods, n, forced, queue, shared)
                    : launch_mma_layout<RAW, false>(stream, stop, prods, n, forced, queue, shared);
}

} // namespace q8
