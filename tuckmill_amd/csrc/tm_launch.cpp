// tm_launch.cpp — the HIP side of libtm_hip's launch interface (tm_launch.hpp):
// the kernels, the static device workspace of the entry point that allocates
// nothing, and the launchers that turn a planned launch (tm_plan.hpp) into
// kernel arguments, a kernel instantiation and a grid sized for its shapes.
// Everything the host logic in tm_hip.cpp knows about the device goes through
// here or through the HIP runtime API.
#include "tm_launch.hpp"

#include <mutex>
#include <vector>

#include "q8_gemm_i8.hpp"
#include "q8_gemv_i8.hpp"
#include "q8_gemm_bf16x3.hpp"
#include "q8_gemm_i8_lds.hpp"
#include "q8_gemm_mma.hpp"
#include "q8_gemv.hpp"
#include "q8_gemm_small.hpp"
#include "q8_misc.hpp"
#include "q8_neighbors.hpp"
#include "f16_gemv.hpp"

using namespace tmh;

static __device__ __align__(256) uint8_t scratch[kScratchBytes];

namespace {

// In host code `scratch` is only a stand-in for the device array: its address on
// a GPU comes from hipGetSymbolAddress, asked once per device with that device
// current (every GPU holds its own copy at its own address).
constexpr int kMaxDevices = 64;
uint8_t *g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mu;

} // namespace

hipError_t tmdev::scratch_on_current_device(int device, uint8_t **out) {
    if (device < 0 || device >= kMaxDevices) {
        return hipErrorInvalidDevice;
    }
    std::lock_guard<std::mutex> g(g_scratch_mu);
    if (g_scratch_ptr[device] == nullptr) {
        void *ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) {
            return e;
        }
        if (ptr == nullptr) {
            return hipErrorInvalidSymbol;
        }
        g_scratch_ptr[device] = (uint8_t *)ptr;
    }
    *out = g_scratch_ptr[device];
    return hipSuccess;
}

namespace {

uint32_t pick_rows_per_tile(uint32_t rows, uint32_t cols, uint32_t tile_bytes, int R) {
    // About 8 KiB of weights per wave (measured best for streaming; 32 KiB
    // and more lose bandwidth), at least one pass of R rows; a matrix that
    // would give fewer than 256 tiles gets smaller ones so that a lone
    // product still spreads over the CUs.
    uint32_t rpt = (tile_bytes / cols);
    if (rpt < (uint32_t)R) {
        rpt = (uint32_t)R;
    }
    rpt = (rpt / (uint32_t)R) * (uint32_t)R;
    while (rpt > (uint32_t)R && (rows + rpt - 1) / rpt < 256u) {
        rpt -= (uint32_t)R;
    }
    return rpt;
}

// Workgroups of `per` elements that cover n (n + per - 1 may not fit 32 bits).
inline unsigned blocks_of(uint32_t n, uint32_t per) {
    return (unsigned)(((uint64_t)n + per - 1u) / per);
}

// The same for the element-wise kernels that stride over what one pass of the
// grid leaves: at most 2^22 workgroups (a launch holds fewer than 2^32 threads).
inline unsigned strided_blocks_of(uint32_t n, uint32_t per) {
    const unsigned blocks = blocks_of(n, per);
    return blocks < (1u << 22) ? blocks : (1u << 22);
}

template <int L, int R, int TB, bool XA>
hipError_t launch_gemv(hipStream_t stream, hipEvent_t stop, const q8::GemvArgs &args, int tails,
                       bool fused, bool wide, bool tail128_long = false) {
    const uint32_t groups = (args.total_tiles + 3u) / 4u;
    if constexpr (L == q8::PACKED && TB == 1) {
        const bool norm = fused; // the planner only fuses into aligned launches of the decode kernel
        if (args.n <= (uint32_t)q8::GEMV_FEW_DESCS) { // short argument block
            q8::GemvArgsT<q8::GEMV_FEW_DESCS> few;
            few.n = args.n;
            few.total_tiles = args.total_tiles;
            few.norm_eps = args.norm_eps;
            few.pad = 0;
            few.norm_h = args.norm_h;
            few.norm_w = args.norm_w;
            few.norm_out = args.norm_out;
            for (uint32_t i = 0; i < args.n; ++i) {
                few.d[i] = args.d[i];
            }
            if (norm) {
                if constexpr (XA) {
                    if (tails == 1) {
                        Q8_LAUNCH((q8::gemv_list_kernel<L, R, TB, true, 1, q8::GEMV_FEW_DESCS, true>),
                                  dim3(groups), dim3(256), 0, stream, stop, few);
                    } else {
                        Q8_LAUNCH((q8::gemv_list_kernel<L, R, TB, true, 0, q8::GEMV_FEW_DESCS, true>),
                                  dim3(groups), dim3(256), 0, stream, stop, few);
                    }
                    return hipGetLastError();
                }
                return hipErrorInvalidValue;
            }
            if (wide) { // short tiles under a long K: the instantiation with steps of several chunks
                if (tails == 1) {
                    Q8_LAUNCH((q8::gemv_list_kernel<L, R, TB, XA, 1, q8::GEMV_FEW_DESCS, false, true>),
                              dim3(groups), dim3(256), 0, stream, stop, few);
                } else if (tails == 2) {
                    Q8_LAUNCH((q8::gemv_list_kernel<L, R, TB, XA, 2, q8::GEMV_FEW_DESCS, false, true>),
                              dim3(groups), dim3(256), 0, stream, stop, few);
                } else {
                    Q8_LAUNCH((q8::gemv_list_kernel<L, R, TB, XA, 0, q8::GEMV_FEW_DESCS, false, true>),
                              dim3(groups), dim3(256), 0, stream, stop, few);
                }
            } else if (tails == 1 && tail128_long) { // some row has whole chunks in front of its 128-column tail
                Q8_LAUNCH((q8::gemv_list_kernel<L, R, TB, XA, 3, q8::GEMV_FEW_DESCS>), dim3(groups),
                          dim3(256), 0, stream, stop, few);
            } else if (tails == 1) {
                Q8_LAUNCH((q8::gemv_list_kernel<L, R, TB, XA, 1, q8::GEMV_FEW_DESCS>), dim3(groups),
                          dim3(256), 0, stream, stop, few);
            } else if (tails == 2) {
                Q8_LAUNCH((q8::gemv_list_kernel<L, R, TB, XA, 2, q8::GEMV_FEW_DESCS>), dim3(groups),
                          dim3(256), 0, stream, stop, few);
            } else {
                Q8_LAUNCH((q8::gemv_list_kernel<L, R, TB, XA, 0, q8::GEMV_FEW_DESCS>), dim3(groups),
                          dim3(256), 0, stream, stop, few);
            }
            return hipGetLastError();
        }
        if (norm) {
            if constexpr (XA) {
                if (tails == 1) {
                    Q8_LAUNCH((q8::gemv_list_kernel<L, R, TB, true, 1, q8::GEMV_MAX_DESCS, true>),
                              dim3(groups), dim3(256), 0, stream, stop, args);
                } else {
                    Q8_LAUNCH((q8::gemv_list_kernel<L, R, TB, true, 0, q8::GEMV_MAX_DESCS, true>),
                              dim3(groups), dim3(256), 0, stream, stop, args);
                }
                return hipGetLastError();
            }
            return hipErrorInvalidValue;
        }
    }
    if constexpr (TB == 1) { // (either layout: the column tails that stream)
        if constexpr (L == q8::PACKED) {
            if (tails == 1 && tail128_long) {
                Q8_LAUNCH((q8::gemv_list_kernel<L, R, TB, XA, 3>), dim3(groups), dim3(256), 0,
                          stream, stop, args);
                return hipGetLastError();
            }
        }
        if (tails == 1) {
            Q8_LAUNCH((q8::gemv_list_kernel<L, R, TB, XA, 1>), dim3(groups), dim3(256), 0,
                      stream, stop, args);
            return hipGetLastError();
        }
        if (tails == 2) {
            Q8_LAUNCH((q8::gemv_list_kernel<L, R, TB, XA, 2>), dim3(groups), dim3(256), 0,
                      stream, stop, args);
            return hipGetLastError();
        }
    }
    Q8_LAUNCH((q8::gemv_list_kernel<L, R, TB, XA, 0>), dim3(groups), dim3(256), 0, stream,
              stop, args);
    return hipGetLastError();
}

constexpr int kGemvR1 = 8; // rows per pass at one token per pass
constexpr int kGemvR4 = 2; // rows per pass at four tokens per pass

hipError_t launch_mma_list(hipStream_t stream, hipEvent_t stop, const OpList &ops,
                           GemvKey key, const Workspace &ws) {
    q8::MmaProduct prods[q8::MMA_MAX_DESCS];
    int n = 0;
    for (const Op *op : ops) {
        prods[n++] = q8::MmaProduct{(const uint8_t *)op->a[0]->ptr,
                                    (const float *)op->a[1]->ptr + op->x_off,
                                    (float *)op->a[2]->ptr + op->y_off, op->rows, op->cols,
                                    op->batch};
    }
    const q8::MmaConfig c{key.p0, key.p1, key.p2};
    const q8::MmaShared shared{ws.mma_partials, ws.arrivals};
    return q8::launch_gemm_mma_list(stream, stop, key.packed, key.flag, prods, n, &c,
                                    ws.mma_queue, shared);
}

// The f32 kernel's tiles on the bf16 matrix cores: every product reads the one
// split form that the launch before this one has left in the workspace
// (at Launch::xs_in_off).
hipError_t launch_mma_split_list(hipStream_t stream, hipEvent_t stop, const Launch &launch,
                                 const Workspace &ws) {
    const OpList &ops = launch.list;
    if (ops.empty() || launch.bx3_inputs != 1 || launch.bx3_presplit != 1u ||
        launch.bx3_xs_bytes > ws.xs_bytes || launch.xs_in_off + bx3_xs_bytes_of(*ops[0]) > launch.bx3_xs_bytes) {
        return hipErrorInvalidValue;
    }
    q8::MmaProduct prods[q8::MMA_MAX_DESCS];
    int n = 0;
    for (const Op *op : ops) {
        if (n == q8::MMA_MAX_DESCS || !same_input(*ops[0], *op)) {
            return hipErrorInvalidValue;
        }
        prods[n++] = q8::MmaProduct{(const uint8_t *)op->a[0]->ptr,
                                    (const float *)(ws.xs + launch.xs_in_off),
                                    (float *)op->a[2]->ptr + op->y_off, op->rows, op->cols,
                                    op->batch};
    }
    const q8::MmaShared shared{ws.mma_partials, ws.arrivals};
    if (launch.glu.size() == ops.size() && launch.glu[0] != nullptr) {
        // gate, up and the gated activation behind them as one launch
        const Op &act = *launch.glu[0];
        if (n != 2 || ops[0]->rows != ops[1]->rows || ops[0]->cols != ops[1]->cols ||
            ops[0]->y_off != 0 || ops[1]->y_off != 0 || act.a[0] != ops[0]->a[2] || act.a[1] != ops[1]->a[2] ||
            (act.kind != OP_SILU_MUL && act.kind != OP_GELU_MUL) ||
            act.extra != (uint64_t)ops[0]->rows * ops[0]->batch ||
            (launch.split_xs_off >= 0 &&
             (uint64_t)launch.split_xs_off + (uint64_t)ops[0]->batch * ops[0]->rows * 6u > ws.xs_bytes)) {
            return hipErrorInvalidValue;
        }
        q8::MmaGlu glu;
        glu.w2 = prods[1].w;
        glu.y2 = prods[1].y;
        glu.act = (float *)act.a[2]->ptr;
        glu.act_split = launch.split_xs_off >= 0 ? (uint16_t *)(ws.xs + launch.split_xs_off) : nullptr;
        glu.kind = act.kind == OP_SILU_MUL ? 0u : 1u;
        return q8::launch_gemm_mma_split_list(stream, stop, prods, 1, shared, &glu);
    }
    return q8::launch_gemm_mma_split_list(stream, stop, prods, n, shared);
}

// The split-float GEMM: one launch that splits every distinct input of the list
// into its three bf16 planes, then the product list. The workspace was sized by
// ensure_bx3_workspace() when the launches were planned.
hipError_t launch_bx3_list(hipStream_t stream, hipEvent_t stop, const Launch &launch,
                           const Workspace &ws) {
    const OpList &ops = launch.list;
    if (launch.bx3_chunks.size() != ops.size() || launch.bx3_xs_bytes > ws.xs_bytes ||
        launch.bx3_partial_floats * 4u > ws.partial_bytes) {
        return hipErrorInvalidValue;
    }
    q8::SplitInput inputs[q8::SPLIT_MAX_DESCS];
    const Op *input_of[q8::SPLIT_MAX_DESCS];
    q8::Bx3Product prods[q8::BX3_MAX_DESCS];
    int n_in = 0, n = 0;
    uint32_t op_at = 0;
    size_t xs_used = 0;
    for (const Op *op : ops) {
        int at = 0;
        while (at < n_in && !same_input(*input_of[at], *op)) {
            ++at;
        }
        if (at == n_in) {
            if (n_in == q8::SPLIT_MAX_DESCS) {
                return hipErrorInvalidValue;
            }
            input_of[n_in] = op;
            inputs[n_in] = q8::SplitInput{(const float *)op->a[1]->ptr + op->x_off,
                                          (uint16_t *)(ws.xs + xs_used), op->batch, op->cols};
            xs_used += bx3_xs_bytes_of(*op);
            ++n_in;
        }
        const uint32_t chunks = launch.bx3_chunks[(size_t)(op_at)];
        const bool tailed = launch.bx3_tail.row_tiles != 0u && launch.bx3_tail.product == op_at;
        const uint32_t head = tailed ? q8::bx3_head_rows(op->rows, launch.bx3_tail.row_tiles) : op->rows;
        if (n + (tailed ? 2 : 1) > q8::BX3_MAX_DESCS || head == 0u) {
            return hipErrorInvalidValue;
        }
        prods[n++] = q8::Bx3Product{(const uint8_t *)op->a[0]->ptr, inputs[at].xs,
                                    (float *)op->a[2]->ptr + op->y_off, op->rows, op->cols,
                                    op->batch, chunks, 0u, head};
        if (tailed) { // the product's last rows, K in chunks of their own
            prods[n] = prods[n - 1];
            prods[n].chunks = launch.bx3_tail.chunks;
            prods[n].row_begin = head;
            prods[n].row_end = op->rows;
            ++n;
        }
        ++op_at;
    }
    // Inputs that the launch before this one has split already stay out of the
    // split pass (none left: no split pass).
    q8::SplitInput to_split[q8::SPLIT_MAX_DESCS];
    int n_split = 0;
    for (int i = 0; i < n_in; ++i) {
        if (((launch.bx3_presplit >> i) & 1u) == 0u) {
            to_split[n_split++] = inputs[i];
        }
    }
    if (n_split > 0) {
        hipError_t e = q8::launch_split_act_list(stream, to_split, n_split);
        if (e != hipSuccess) {
            return e;
        }
    }
    bool small_batch = n <= q8::MMA_MAX_DESCS;
    for (const Op *op : ops) {
        small_batch = small_batch && q8::bx3_small_batch_tiles(op->batch);
    }
    if (small_batch) { // (no tail segments on the 64-token tile: one entry per product)
        q8::MmaProduct small[q8::MMA_MAX_DESCS];
        for (int i = 0; i < n; ++i) {
            small[i] = q8::MmaProduct{prods[i].w, (const float *)prods[i].xs, prods[i].y, prods[i].rows,
                                      prods[i].cols, prods[i].batch};
        }
        const q8::MmaShared shared{ws.mma_partials, ws.arrivals};
        return q8::launch_gemm_mma_split_list(stream, stop, small, n, shared);
    }
    return q8::launch_gemm_bf16x3_list(stream, stop, launch.key.p0 * 64u, prods, n,
                                       ws.partials, ws.arrivals);
}

hipError_t launch_i8_list(hipStream_t stream, hipEvent_t stop, const OpList &ops,
                          GemvKey key) {
    q8::I8Product prods[q8::I8_MAX_DESCS];
    int n = 0;
    for (const Op *op : ops) {
        prods[n++] = q8::I8Product{(const uint8_t *)op->a[0]->ptr, (const uint8_t *)op->a[1]->ptr,
                                   (float *)op->a[2]->ptr + op->y_off,
                                   op->a[3] != nullptr ? (int32_t *)op->a[3]->ptr : nullptr,
                                   op->rows, op->cols, op->batch};
    }
    if (key.variant == V_I8_LDS) {
        return q8::launch_gemm_i8_lds_list(stream, stop, key.p0, prods, n, key.p1 != 0);
    }
    if (key.variant == V_I8_STREAM) {
        return q8::launch_gemv_i8_list(stream, stop, key.flag, key.p0, prods, n);
    }
    return q8::launch_gemm_i8_list(stream, stop, key.packed, key.flag, key.p0, prods, n);
}

} // namespace

hipError_t tmdev::launch_list(hipStream_t stream, hipEvent_t stop, const Launch &launch,
                              const Workspace &ws) {
    const OpList &ops = launch.list;
    const OpList &residual = launch.residual;
    GemvKey key = launch.key;
    if (key.variant == V_BF16X3) {
        return launch_bx3_list(stream, stop, launch, ws);
    }
    if (key.variant == V_MMA_SPLIT) {
        return launch_mma_split_list(stream, stop, launch, ws);
    }
    if (key.kind == OP_MMA) {
        return launch_mma_list(stream, stop, ops, key, ws);
    }
    if (key.kind == OP_I8) {
        return launch_i8_list(stream, stop, ops, key);
    }
    if (key.kind == OP_F16_GEMM) {
        std::vector<q8::F16Product> prods;
        prods.reserve(ops.size());
        for (const Op *op : ops) {
            prods.push_back(q8::F16Product{(const uint16_t *)op->a[0]->ptr,
                                           (const float *)op->a[1]->ptr + op->x_off,
                                           (float *)op->a[2]->ptr + op->y_off, op->rows, op->cols,
                                           op->batch});
        }
        return q8::launch_f16_list(stream, stop, key.p0, key.flag, prods.data(),
                                   (int)prods.size());
    }
    q8::GemvArgs args; // only the used descriptors are written (the struct is 14 KB)
    args.n = 0;
    args.pad = 0;
    args.norm_eps = launch.norm != nullptr ? launch.norm->scalar : 0.0f;
    args.norm_h = launch.norm != nullptr ? (const float *)launch.norm->a[0]->ptr : nullptr;
    args.norm_w = launch.norm != nullptr ? (const float *)launch.norm->a[1]->ptr : nullptr;
    args.norm_out = launch.norm != nullptr ? (float *)launch.norm->a[2]->ptr : nullptr;
    uint32_t norm_written = 0; // bit t: a descriptor stores row t of the fused norm
    bool fused = launch.norm != nullptr; // the launch needs the kernel variant with fused forms
    const int R = key.variant == V_GENERAL ? kGemvR4 : kGemvR1;
    uint32_t tiles = 0;
    uint64_t launch_bytes = 0;
    for (const Op *op : ops) {
        launch_bytes += (uint64_t)op->rows * (op->cols / 32u) * 34u;
    }
    // The token-split kernel in a launch that is all latency (the projections
    // of one layer between two dependent operators, a few tokens of a
    // speculative step): one pass of rows per workgroup, and the same tokens
    // over twice the waves. A token's result does not depend on either.
    // (the same for a larger launch that has few workgroups anyway, few rows
    // under a long K: 4096 x 14336 at 8 tokens 42.5 -> 32.3 us)
    uint64_t split_wgs = 0;
    for (const Op *op : ops) {
        const uint32_t rpt = pick_rows_per_tile(op->rows, op->cols, 32768u, R);
        split_wgs += (uint64_t)split_token_groups(key, op->batch) * ((op->rows + rpt - 1) / rpt);
    }
    const bool small_split = key.variant == V_SPLIT &&
                             (launch_bytes < (32u << 20) || split_wgs < 1024u);
    if (small_split && key.p1 == 4 && key.p0 <= 2) {
        key.p0 = (uint8_t)(key.p0 * 2);
        key.p1 = 2;
    }
    // Such a launch with few rows (fewer than 160 of the token-split kernel's
    // workgroups of 8 rows: the o and down projections) and up to 4 tokens goes
    // to the one-token kernel instead, one descriptor per token: every token is
    // its own GEMV anyway, and that kernel cuts a small product into tiles of 2
    // rows (lone 1024 x 3072: 2 tokens 6.0 -> 4.2 us, 4 tokens 5.9 -> 5.0; 1152 x 6912:
    // 10.3 -> 6.6 and 10.2 -> 9.0). With more rows the weights read once per
    // token cost more than the waves bring (q,k,v at 4 tokens 4.8 -> 6.1 us; Gemma's,
    // 192 such workgroups, at 3 tokens 4.4 -> 7.4).
    // (A launch with a fused norm or gated activation in it goes there whatever
    // its row count: those forms exist in that kernel only, and the dependent
    // launch a fusion saves, about 4 us, is more than the difference; the planner
    // keeps products of more than 16 M weights out of such launches.)
    bool per_token = launch.per_token;
    if (per_token) {
        key.variant = V_DECODE;
    } else if (small_split) {
        uint32_t max_batch = 0, descs = 0;
        uint64_t row_groups = 0;
        for (const Op *op : ops) {
            max_batch = op->batch > max_batch ? op->batch : max_batch;
            descs += op->batch;
            row_groups += (op->rows + 7u) / 8u;
        }
        if (max_batch <= 4u && row_groups < 160u && descs <= (uint32_t)q8::GEMV_MAX_DESCS) {
            per_token = true;
            key.variant = V_DECODE;
        }
    }
    // The token-split kernel's step: 8 rows, or 4 where a launch of up to 4
    // tokens over sealed weights has at most 512 workgroups of 8 rows and
    // every row is long (3072 columns and more: the plain reduction of the
    // 4-row form is paid once per row pass; 2048 x 2048 at 3 tokens 4.8 -> 5.6
    // us with it). Few rows under a long K then get twice the workgroups, each
    // with a step on its way: lone 4096 x 14336 at 2 / 4 tokens 20.2 / 29.1
    // -> 16.4 / 19.7 us, 2048 x 8192 at 2 tokens 11.5 -> 8.6. (With more
    // workgroups or tokens the 8-row step is ahead: 6144 x 4096 at 4 tokens 10.5
    // against 12.4 us, 4096 x 4096 at 8 tokens 10.7 against 13.7.)
    int split_rows = 8;
    if (key.variant == V_SPLIT && small_split && key.packed && key.p1 == 2 && key.p0 <= 2) {
        uint64_t wgs = 0;
        uint32_t min_cols = 0xffffffffu;
        for (const Op *op : ops) {
            wgs += (uint64_t)split_token_groups(key, op->batch) * ((op->rows + 7u) / 8u);
            min_cols = op->cols < min_cols ? op->cols : min_cols;
        }
        if (wgs <= 512u && min_cols >= 3072u) {
            split_rows = 4;
        }
    }
    // a workgroup's tile in the token-split kernel, a wave's tile otherwise (one
    // token over raw weights: two passes per wave, so that the second pass's
    // loads fly while the first goes through LDS)
    const uint32_t tile_bytes = key.variant == V_SPLIT ? (small_split ? 8192u : 32768u)
                                : (!key.packed && key.variant == V_DECODE) ? 16384u
                                                                           : 8192u;
    // tiles the launch has at one pass of R rows per tile (a product of a few
    // tokens that goes a token a descriptor counts once per token)
    uint64_t full_tiles = 0;
    for (const Op *op : ops) {
        full_tiles += (uint64_t)(per_token ? op->batch : 1u) * ((op->rows + R - 1) / R);
    }
    // which column tails with a streaming path of their own the products have:
    // 0 none, 1 128 columns (and maybe 768), 2 768 columns only
    int tails = 0;
    bool tail128_long = false; // some row with a 128-column tail has more than one whole chunk
    bool wide = false; // some sealed product in short tiles has two chunks and more per row
    // One descriptor: token group `grp` of the product at place `at` of the
    // launch's list (the fusions are recorded per product).
    auto emit = [&](size_t at, uint32_t grp, uint32_t groups, uint32_t group_tokens) {
        const Op *op = ops[at];
        const uint32_t tail = op->cols & 1023u;
        q8::GemvDesc &d = args.d[args.n++];
        d.w = (const uint8_t *)op->a[0]->ptr;
        d.x = (const float *)op->a[1]->ptr + op->x_off + (size_t)grp * group_tokens * op->cols;
        d.y = (float *)op->a[2]->ptr + op->y_off + (size_t)grp * group_tokens * op->rows;
        d.rows = op->rows;
        d.cols = op->cols;
        d.batch = groups == 1u ? op->batch
                               : (op->batch - grp * group_tokens < group_tokens
                                      ? op->batch - grp * group_tokens
                                      : group_tokens);
        d.tile_begin = tiles;
        d.rows_per_tile = pick_rows_per_tile(op->rows, op->cols, tile_bytes,
                                             key.variant == V_SPLIT ? split_rows : R);
        const bool streams = tail == 0u || (op->cols >= 1024u && (tail == 128u || tail == 768u));
        const bool one_token = key.kind == OP_GEMV_LIST && key.variant == V_DECODE;
        if (one_token && d.rows_per_tile == (uint32_t)R && streams && full_tiles < 1024u) {
            // Fewer than 1024 tiles in the whole launch even at one pass per
            // wave (a projection or two between two dependent operators, up to
            // the 4096 x 14336 of an 8 B model): a wave a tile, that leaves
            // three quarters of the chip's wave slots empty, and a tile is one
            // long row pass with 8 KB in flight. Half- and quarter-height
            // tiles put two and four times as many waves on it (quarter-height
            // ones under a very long K only if the launch would otherwise stay
            // under 1024 tiles: 4096 x 14336 runs better on 1024 tiles of 4
            // rows). Lone 4096 x 4096: 8.2 -> 5.6 us, 4096 x 14336: 23.0 ->
            // 13.9, 2048 x 8192: 11.6 -> 6.3. Inside a large launch full-height
            // tiles stream better.
            d.rows_per_tile = (uint32_t)R / 2u;
            if (2u * full_tiles < (op->cols >= 8192u ? 1024u : 2048u)) {
                d.rows_per_tile = (uint32_t)R / 4u;
            }
            wide = wide || (key.packed && op->cols >= 2048u);
        }
        d.pad = 0;
        const bool pair_first = launch.glu[at] != nullptr;
        const bool pair_second = at > 0 && launch.glu[at - 1] != nullptr;
        if (pair_first) { // a tile covers the same rows of both matrices: half the rows each
            d.rows_per_tile = pick_rows_per_tile(op->rows, op->cols, tile_bytes / 2u, 4);
            if (d.rows_per_tile == 4u && tail == 0u &&
                (full_tiles < 1024u || (full_tiles < 2048u && op->cols >= 2048u))) {
                // Few tiles in the launch: tiles of 2 rows of each matrix, as for
                // single products (3072 x 1024 twice, 768 tiles: 6.0 -> 5.6 us;
                // 6144 x 2048 twice, 1536 tiles: 11.6 -> 11.0). Short rows in
                // more tiles lose instead: every wave pays the norm's sum and
                // its share of the activations again (6912 x 1152 twice, 1728
                // tiles: 8.9 -> 11.2 us). Whole chunks only: the instantiation with
                // the 128-column tail is short of registers as it is.
                d.rows_per_tile = 2u;
            }
            d.pad |= q8::GEMV_PAIR;
            fused = true;
        }
        // (with a fusion in the launch a descriptor is one token: grp is the
        // token, the row of the norm, of the residual and of the activation)
        d.pad2 = 0;
        if (launch.norm != nullptr && launch.normed[at]) {
            d.x = args.norm_h; // not read through: the kernel normalises its row of norm_h itself
            d.pad2 = grp;
            d.pad |= q8::GEMV_X_NORMED |
                     ((norm_written >> grp) & 1u ? 0u : q8::GEMV_WRITES_NORM);
            norm_written |= 1u << grp;
        }
        const Op *update = residual[at];
        d.res = update != nullptr
                    ? (float *)update->a[1]->ptr + (size_t)grp * group_tokens * op->rows
                    : nullptr;
        d.alpha = update != nullptr ? update->scalar : 0.0f;
        if (pair_second) { // owns no tiles; carries the activation's output and kind
            const Op *act = launch.glu[at - 1];
            d.res = (float *)act->a[2]->ptr + (size_t)grp * op->rows;
            d.alpha = act->kind == OP_GELU_MUL ? 1.0f : 0.0f;
        } else {
            tiles += (op->rows + d.rows_per_tile - 1) / d.rows_per_tile;
        }
    };
    for (size_t at = 0; at < ops.size(); ++at) {
        const Op *op = ops[at];
        const uint32_t tail = op->cols & 1023u;
        if (op->cols >= 1024u && tail == 128u) {
            tails = 1;
            tail128_long = tail128_long || op->cols != 1152u;
        } else if (op->cols >= 1024u && tail == 768u && tails == 0) {
            tails = 2;
        }
        // The token-split kernel covers waves x tokens-per-wave tokens per
        // descriptor: a larger batch goes as several descriptors over the same
        // weights, each with its own rows of X and Y.
        const uint32_t group_tokens = per_token                  ? 1u
                                      : key.variant == V_SPLIT ? (uint32_t)key.p0 * key.p1
                                                               : op->batch;
        const uint32_t groups = per_token ? op->batch : split_token_groups(key, op->batch);
        if (args.n + groups > (uint32_t)q8::GEMV_MAX_DESCS) {
            return hipErrorInvalidValue;
        }
        if (at > 0 && launch.glu[at - 1] != nullptr) {
            continue; // the up projection of a fused pair: listed right behind its gate, below
        }
        const bool pair_first = launch.glu[at] != nullptr;
        if (pair_first && args.n + 2u * groups > (uint32_t)q8::GEMV_MAX_DESCS) {
            return hipErrorInvalidValue;
        }
        for (uint32_t grp = 0; grp < groups; ++grp) {
            emit(at, grp, groups, group_tokens);
            if (pair_first) {
                emit(at + 1, grp, groups, group_tokens);
            }
        }
    }
    args.total_tiles = tiles;
#define TM_SPLIT_CASE(P, W, T, A, TL)                                                        \
    if (key.variant == V_SPLIT && key.packed == (P) && key.p0 == (W) && key.p1 == (T) &&     \
        key.p2 == ((TL) ? 1 : 0) && key.flag == (A) && split_rows == 8) {                    \
        Q8_LAUNCH((q8::gemm_split_list_kernel<(P) ? q8::PACKED : q8::RAW, W, T, A, TL>),     \
                  dim3(tiles), dim3((W) * 64), 0, stream, stop, args);                  \
        return hipGetLastError();                                                            \
    }
#define TM_SPLIT_ALL(W, T)                                                                   \
    TM_SPLIT_CASE(true, W, T, true, false)                                                   \
    TM_SPLIT_CASE(true, W, T, false, false)                                                  \
    TM_SPLIT_CASE(true, W, T, true, true)                                                    \
    TM_SPLIT_CASE(true, W, T, false, true)                                                   \
    TM_SPLIT_CASE(false, W, T, true, false)                                                  \
    TM_SPLIT_CASE(false, W, T, false, false)                                                 \
    TM_SPLIT_CASE(false, W, T, true, true)                                                   \
    TM_SPLIT_CASE(false, W, T, false, true)
    TM_SPLIT_ALL(1, 2)
    TM_SPLIT_ALL(2, 2)
    TM_SPLIT_ALL(4, 2)
    TM_SPLIT_ALL(1, 4)
    TM_SPLIT_ALL(2, 4)
    TM_SPLIT_ALL(4, 4)
    // (eight tokens per wave: no column-tail form, see gemv_key)
    TM_SPLIT_CASE(true, 4, 8, true, false)
    TM_SPLIT_CASE(true, 4, 8, false, false)
    TM_SPLIT_CASE(false, 4, 8, true, false)
    TM_SPLIT_CASE(false, 4, 8, false, false)
#undef TM_SPLIT_ALL
#undef TM_SPLIT_CASE
#define TM_SPLIT_ROWS4(W, A, TL)                                                             \
    if (key.variant == V_SPLIT && key.packed && key.p0 == (W) && key.p1 == 2 &&              \
        key.p2 == ((TL) ? 1 : 0) && key.flag == (A) && split_rows == 4) {                    \
        Q8_LAUNCH((q8::gemm_split_list_kernel<q8::PACKED, W, 2, A, TL, 4>), dim3(tiles),     \
                  dim3((W) * 64), 0, stream, stop, args);                               \
        return hipGetLastError();                                                            \
    }
#define TM_SPLIT_ROWS4_ALL(W)                                                                \
    TM_SPLIT_ROWS4(W, true, false)                                                           \
    TM_SPLIT_ROWS4(W, false, false)                                                          \
    TM_SPLIT_ROWS4(W, true, true)                                                            \
    TM_SPLIT_ROWS4(W, false, true)
    TM_SPLIT_ROWS4_ALL(1)
    TM_SPLIT_ROWS4_ALL(2)
#undef TM_SPLIT_ROWS4_ALL
#undef TM_SPLIT_ROWS4
#define TM_GEMV_CASE(P, T, A)                                                                \
    if (key.packed == (P) && key.variant == ((T) == 1 ? V_DECODE : V_GENERAL) &&             \
        key.flag == (A)) {                                                                   \
        return launch_gemv<(P) ? q8::PACKED : q8::RAW, (T) == 1 ? kGemvR1 : kGemvR4, T, A>(  \
            stream, stop, args, tails, fused, wide, tail128_long);                                    \
    }
    TM_GEMV_CASE(true, 1, true)
    TM_GEMV_CASE(true, 1, false)
    TM_GEMV_CASE(true, 4, true)
    TM_GEMV_CASE(true, 4, false)
    TM_GEMV_CASE(false, 1, true)
    TM_GEMV_CASE(false, 1, false)
    TM_GEMV_CASE(false, 4, true)
    TM_GEMV_CASE(false, 4, false)
#undef TM_GEMV_CASE
    return hipErrorInvalidValue;
}

// `split_to`: where an RMSNorm or gated activation writes the split form of its
// result as well (the planner's fuse_split_passes), or null.
// `update`: a residual update h += alpha * t that an RMSNorm of h takes in
// front of itself (plan_launches), or null.
hipError_t tmdev::launch_single(hipStream_t stream, hipEvent_t stop, const Op &op,
                                uint16_t *split_to, uint32_t split_cols, const Op *update) {
    const uint8_t *w = op.a[0] ? (const uint8_t *)op.a[0]->ptr : nullptr;
    hipStream_t st = stream;
    switch (op.kind) {
    case OP_ROW: {
        float *out = (float *)op.a[1]->ptr;
        dim3 grid(blocks_of(op.cols, 256u));
        if (op.packed) {
            Q8_LAUNCH(q8::row_kernel<q8::PACKED>, grid, dim3(256), 0, st, stop, w, out, op.rows,
                      op.cols, op.extra, op.y_off);
        } else {
            Q8_LAUNCH(q8::row_kernel<q8::RAW>, grid, dim3(256), 0, st, stop, w, out, op.rows, op.cols,
                      op.extra, op.y_off);
        }
        break;
    }
    case OP_ROW_INDIRECT: {
        float *out = (float *)op.a[1]->ptr;
        const uint32_t *ids = (const uint32_t *)op.a[2]->ptr;
        dim3 grid(blocks_of(op.cols, 256u));
        if (op.packed) {
            Q8_LAUNCH(q8::row_indirect_kernel<q8::PACKED>, grid, dim3(256), 0, st, stop, w, out, ids,
                      op.extra, op.rows, op.cols);
        } else {
            Q8_LAUNCH(q8::row_indirect_kernel<q8::RAW>, grid, dim3(256), 0, st, stop, w, out, ids,
                      op.extra, op.rows, op.cols);
        }
        break;
    }
    case OP_COPY: {
        const float *src = (const float *)op.a[0]->ptr + op.x_off;
        float *dst = (float *)op.a[1]->ptr + op.y_off;
        Q8_LAUNCH(q8::copy_f32_kernel, dim3(strided_blocks_of(op.extra, 256u)), dim3(256), 0, st,
                  stop, src, dst, op.extra);
        break;
    }
    case OP_CHECKSUM:
        Q8_LAUNCH(q8::xor_checksum_kernel, dim3(q8::CHECKSUM_GROUPS), dim3(256), 0, st, stop,
                  (const uint32_t *)op.a[0]->ptr + op.x_off, (uint32_t *)op.a[1]->ptr, op.extra);
        break;
    case OP_SCALE:
        Q8_LAUNCH(q8::scale_kernel, dim3(strided_blocks_of(op.extra, 256u)), dim3(256), 0, st,
                  stop, (const float *)op.a[0]->ptr, (float *)op.a[1]->ptr, op.scalar, op.extra);
        break;
    case OP_CAST_F16_F32:
        Q8_LAUNCH(q8::cast_f16_f32_kernel, dim3(blocks_of(op.extra, 2048u)), dim3(256), 0, st, stop,
                  (const uint16_t *)op.a[0]->ptr, (float *)op.a[1]->ptr, op.extra);
        break;
    case OP_CAST_F32_F16:
        Q8_LAUNCH(q8::cast_f32_f16_kernel, dim3(blocks_of(op.extra, 2048u)), dim3(256), 0, st, stop,
                  (const float *)op.a[0]->ptr, (uint16_t *)op.a[1]->ptr, op.extra);
        break;
    case OP_AXPY:
        Q8_LAUNCH(q8::axpy_kernel, dim3(strided_blocks_of(op.extra, 256u)), dim3(256), 0, st,
                  stop, (const float *)op.a[0]->ptr, (float *)op.a[1]->ptr, op.scalar, op.extra);
        break;
    case OP_SILU_MUL:
        Q8_LAUNCH(q8::silu_mul_kernel, dim3(strided_blocks_of(op.extra, 256u)), dim3(256), 0, st,
                  stop, (const float *)op.a[0]->ptr, (const float *)op.a[1]->ptr, (float *)op.a[2]->ptr,
                  op.extra, split_to, split_cols);
        break;
    case OP_GELU_MUL:
        Q8_LAUNCH(q8::gelu_tanh_mul_kernel, dim3(strided_blocks_of(op.extra, 256u)), dim3(256), 0,
                  st, stop, (const float *)op.a[0]->ptr, (const float *)op.a[1]->ptr, (float *)op.a[2]->ptr,
                  op.extra, split_to, split_cols);
        break;
    case OP_RMSNORM:
        Q8_LAUNCH(q8::rmsnorm_kernel, dim3((op.rows + q8::RMSNORM_ROWS - 1u) / q8::RMSNORM_ROWS),
                  dim3(64u * q8::RMSNORM_ROWS), 0, st, stop,
                  (float *)op.a[0]->ptr, (const float *)op.a[1]->ptr, (float *)op.a[2]->ptr,
                  op.rows, op.cols, op.scalar, split_to,
                  update != nullptr ? (const float *)update->a[0]->ptr : (const float *)nullptr,
                  update != nullptr ? update->scalar : 0.0f);
        break;
    case OP_ARGMAX: {
        float *part_v = (float *)op.a[1]->ptr;
        uint32_t *part_i = (uint32_t *)((uint8_t *)op.a[1]->ptr + q8::ARGMAX_GROUPS * 4u);
        hipLaunchKernelGGL(q8::argmax_partial_kernel, dim3(q8::ARGMAX_GROUPS), dim3(256), 0, st,
                           (const float *)op.a[0]->ptr, part_v, part_i, op.extra);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) {
            return e;
        }
        Q8_LAUNCH(q8::argmax_final_kernel, dim3(1), dim3(256), 0, st, stop, (const float *)part_v,
                  (const uint32_t *)part_i, (uint32_t *)op.a[2]->ptr, op.y_off);
        break;
    }
    case OP_F16_ROW:
        Q8_LAUNCH(q8::f16_row_kernel, dim3(blocks_of(op.cols, 256u)), dim3(256), 0, st, stop,
                  (const uint16_t *)op.a[0]->ptr, (float *)op.a[1]->ptr, op.cols, op.extra,
                  op.y_off);
        break;
    case OP_F16_ROW_INDIRECT:
        Q8_LAUNCH(q8::f16_row_indirect_kernel, dim3(blocks_of(op.cols, 256u)), dim3(256), 0, st, stop,
                  (const uint16_t *)op.a[0]->ptr, (float *)op.a[1]->ptr,
                  (const uint32_t *)op.a[2]->ptr, op.extra, op.rows, op.cols);
        break;
    case OP_PACK: {
        const size_t nblocks = (size_t)op.rows * (op.cols / 32u);
        Q8_LAUNCH(q8::pack_kernel, dim3((unsigned)((nblocks + 255u) / 256u)), dim3(256), 0, st, stop,
                  w, (uint8_t *)op.a[1]->ptr, op.rows, op.cols);
        break;
    }
    case OP_QUANT:
        return q8::launch_quantize_act(st, stop, (const float *)op.a[0]->ptr + op.x_off,
                                       (uint8_t *)op.a[1]->ptr, op.cols, op.batch);
    default:
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t tmdev::kernels_present() {
    hipFuncAttributes attr;
    return hipFuncGetAttributes(&attr,
                                (const void *)q8::gemv_list_kernel<q8::PACKED, kGemvR1, 1, true, 0>);
}

hipError_t tmdev::zero_words(hipStream_t stream, uint32_t *dst, uint32_t n) {
    hipLaunchKernelGGL(q8::zero_u32_kernel, dim3((n + 255u) / 256u), dim3(256), 0, stream, dst, n);
    return hipGetLastError();
}
