// A recording stand-in for libtm_hip's launch interface (tm_launch.hpp): where
// tm_launch.cpp turns a planned launch into kernels, this writes it down and
// checks what the real launchers rely on: every buffer a launch names is alive
// and large enough, lists fit their kernels' capacities, a launch on the bf16
// matrix cores has its K chunks and its share of the workspace, fusions are
// wired to the products they ride with. Nothing computes.
#include "tm_launch.hpp"

#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include <mutex>

#include "recorder.hpp"

using namespace tmh;

namespace rec {
std::vector<std::string> log;
std::string (*name_of)(const void *) = nullptr;
} // namespace rec

namespace {
// Contexts may launch from several threads at once (each on its own stream).
std::mutex rec_mu;
void record(std::string line) {
    std::lock_guard<std::mutex> g(rec_mu);
    rec::log.push_back(std::move(line));
}
} // namespace

namespace {

[[noreturn]] void die(const char *what) {
    fprintf(stderr, "stub launcher: %s\n", what);
    abort();
}

std::string nm(const Alloc *a) {
    if (a == nullptr) {
        return "null";
    }
    return "\"" + (rec::name_of != nullptr ? rec::name_of(a->ptr) : std::string("?")) + "\"";
}

void need(const Alloc *a, size_t bytes, const char *what) {
    if (a == nullptr || a->ptr == nullptr) {
        die(what);
    }
    if (a->refs.load() <= 0) {
        die("allocation with no reference left");
    }
    if (bytes > a->len || !fake::device_range_live(a->ptr, bytes)) {
        die(what);
    }
}

const char *variant_name(Variant v) {
    switch (v) {
    case V_DECODE: return "decode";
    case V_GENERAL: return "general";
    case V_SPLIT: return "split";
    case V_MMA: return "mma_f32";
    case V_BF16X3: return "bf16x3";
    case V_MMA_SPLIT: return "mma_split";
    case V_I8_TILE: return "i8_tile";
    case V_I8_STREAM: return "i8_stream";
    case V_I8_LDS: return "i8_lds";
    case V_F16: return "f16";
    }
    return "?";
}

void check_product(const Op &op, const GemvKey &key) {
    const size_t blocks = op.cols / 32u;
    if (op.rows == 0 || op.cols == 0 || op.batch == 0) {
        die("product with a zero dimension");
    }
    if (op.kind == OP_F16_GEMM) {
        need(op.a[0], (size_t)op.rows * op.cols * 2u, "f16 weights");
    } else {
        if ((op.cols & 31u) != 0u) {
            die("Q8_0 product whose cols is not a multiple of 32");
        }
        need(op.a[0], (size_t)op.rows * blocks * 34u, "Q8_0 weights");
        if (op.a[0]->packed != op.packed || key.packed != op.packed) {
            die("weight layout of the product, its allocation and its launch disagree");
        }
    }
    if (op.kind == OP_I8) {
        need(op.a[1], q8::xq_bytes(op.cols, op.batch), "quantized activations");
    } else {
        need(op.a[1], ((size_t)op.x_off + (size_t)op.batch * op.cols) * 4u, "activations");
    }
    need(op.a[2], ((size_t)op.y_off + (size_t)op.batch * op.rows) * 4u, "outputs");
    if (op.a[3] != nullptr) {
        need(op.a[3], (size_t)op.batch * op.rows * blocks * 4u, "block dots");
    }
}

} // namespace

hipError_t tmdev::kernels_present() { return hipSuccess; }

hipError_t tmdev::scratch_on_current_device(int device, uint8_t **out) {
    static uint8_t *scratch = nullptr; // (lives as long as the process, like the real one)
    static std::mutex mu;
    if (device != 0) {
        return hipErrorInvalidDevice;
    }
    std::lock_guard<std::mutex> g(mu);
    if (scratch == nullptr) {
        scratch = (uint8_t *)malloc(kScratchBytes);
    }
    *out = scratch;
    return scratch != nullptr ? hipSuccess : hipErrorOutOfMemory;
}

hipError_t tmdev::zero_words(hipStream_t stream, uint32_t *dst, uint32_t n) {
    if (dst == nullptr || n == 0) {
        die("zero_words: nothing to clear");
    }
    if (!fake::enqueue(stream, "zero_words")) {
        return hipErrorInvalidValue;
    }
    record("{\"k\":\"zero_words\",\"n\":" + std::to_string(n) + "}");
    return hipSuccess;
}

hipError_t tmdev::launch_list(hipStream_t stream, hipEvent_t stop, const Launch &l,
                              const Workspace &ws) {
    const size_t n = l.list.size();
    if (l.single != nullptr || n == 0) {
        die("launch_list: not a product list");
    }
    if (l.residual.size() != n || l.glu.size() != n || l.normed.size() != n) {
        die("launch_list: per-product lists of different lengths");
    }
    const GemvKey &key = l.key;
    const size_t cap = key.kind == OP_MMA  ? (key.variant == V_BF16X3 ? q8::BX3_MAX_DESCS : q8::MMA_MAX_DESCS)
                       : key.kind == OP_I8 ? (size_t)q8::I8_MAX_DESCS
                                           : (size_t)q8::GEMV_MAX_DESCS;
    if (n > cap) {
        die("launch_list: more products than the kernel's list holds");
    }
    if (key.kind == OP_GEMV_LIST) {
        uint64_t descs = 0;
        for (const Op *op : l.list) {
            descs += l.per_token ? op->batch : split_token_groups(key, op->batch);
        }
        if (descs > (uint64_t)q8::GEMV_MAX_DESCS) {
            die("launch_list: more descriptors than the kernel's list holds");
        }
    }
    std::string out = "{\"k\":\"list\",\"variant\":\"" + std::string(variant_name(key.variant)) +
                      "\",\"p\":[" + std::to_string(key.p0) + "," + std::to_string(key.p1) + "," +
                      std::to_string(key.p2) + "],\"packed\":" + (key.packed ? "true" : "false") +
                      ",\"flag\":" + (key.flag ? "true" : "false") +
                      ",\"per_token\":" + (l.per_token ? "true" : "false") +
                      ",\"recording\":" + (fake::capturing(stream) ? "true" : "false");
    if (key.variant == V_BF16X3) {
        if (l.bx3_chunks.size() != n) {
            die("bf16 launch without its K chunks");
        }
        if (ws.xs == nullptr || l.bx3_xs_bytes > ws.xs_bytes) {
            die("bf16 launch: split activations do not fit the workspace");
        }
        uint64_t split_tiles = 0, partial_floats = 0;
        size_t xs_bytes = 0;
        int inputs = 0;
        const Op *seen[q8::SPLIT_MAX_DESCS];
        for (size_t i = 0; i < n; ++i) {
            const Op &op = *l.list[i];
            const q8::Bx3Plan p = q8::bx3_plan_chunked(op.rows, op.cols, op.batch, key.p0 * 64u,
                                                      l.bx3_chunks[i]);
            if (p.chunks != l.bx3_chunks[i] || p.chunk_blocks == 0) {
                die("bf16 launch: chunk count that its product cannot have");
            }
            split_tiles += p.split_tiles;
            partial_floats += p.partial_floats;
            int at = 0;
            while (at < inputs && !same_input(*seen[at], op)) {
                ++at;
            }
            if (at == inputs) {
                if (inputs == q8::SPLIT_MAX_DESCS) {
                    die("bf16 launch: more distinct inputs than the split pass holds");
                }
                seen[inputs++] = &op;
                xs_bytes += bx3_xs_bytes_of(op);
            }
        }
        if (l.bx3_tail.row_tiles != 0u) { // one product's last rows as a segment with chunks of its own
            const q8::Bx3Tail &t = l.bx3_tail;
            if (t.product >= n || l.bx3_chunks[t.product] != 1u || n + 1 > (size_t)q8::BX3_MAX_DESCS) {
                die("bf16 launch: tail segment on a product that cannot have one");
            }
            const Op &op = *l.list[t.product];
            const uint32_t row_tiles = (op.rows + q8::BX3_TILE_ROWS - 1u) / q8::BX3_TILE_ROWS;
            if (t.row_tiles >= row_tiles) {
                die("bf16 launch: tail segment leaves its product no head");
            }
            const uint32_t head = q8::bx3_head_rows(op.rows, t.row_tiles);
            const q8::Bx3Plan p = q8::bx3_plan_chunked(op.rows - head, op.cols, op.batch, key.p0 * 64u, t.chunks);
            if (p.chunks != t.chunks || t.chunks < 2u || t.chunks > q8::BX3_TAIL_MAX_CHUNKS || key.p0 != 2 ||
                p.chunk_blocks < q8::BX3_TAIL_CHUNK_BLOCKS) {
                die("bf16 launch: tail segment with chunks it cannot have");
            }
            split_tiles += p.split_tiles;
            partial_floats += p.partial_floats;
            out += ",\"tail\":{\"product\":" + std::to_string(t.product) + ",\"row_tiles\":" +
                   std::to_string(t.row_tiles) + ",\"chunks\":" + std::to_string(t.chunks) + "}";
        }
        if (split_tiles != l.bx3_split_tiles || partial_floats != l.bx3_partial_floats ||
            xs_bytes != l.bx3_xs_bytes || inputs != l.bx3_inputs) {
            die("bf16 launch: workspace figures do not match its products");
        }
        if (split_tiles > q8::BX3_MAX_SPLIT_TILES ||
            (split_tiles > 0 && (ws.arrivals == nullptr || ws.partials == nullptr)) ||
            partial_floats * 4u > ws.partial_bytes) {
            die("bf16 launch: partial tiles do not fit the workspace");
        }
        out += ",\"presplit\":" + std::to_string(l.bx3_presplit);
        bool small_batch = true; // up to 32 tokens: the f32 kernel's tiles fed from the split form
        for (size_t i = 0; i < n; ++i) {
            small_batch = small_batch && q8::bx3_small_batch_tiles(l.list[i]->batch);
        }
        out += std::string(",\"small_tiles\":") + (small_batch ? "true" : "false");
    }
    if (key.variant == V_MMA_SPLIT) { // every product reads the one split form the launch before has written
        if (!key.packed || l.bx3_inputs != 1 || l.bx3_presplit != 1u) {
            die("split-form f32-tile launch: not one input split by the launch before");
        }
        const uint64_t in_end = l.xs_in_off + bx3_xs_bytes_of(*l.list[0]);
        if (ws.xs == nullptr || l.bx3_xs_bytes > ws.xs_bytes || in_end > l.bx3_xs_bytes || l.xs_in_off % 256u != 0u) {
            die("split-form f32-tile launch: split activations do not fit the workspace");
        }
        if (l.glu[0] != nullptr) { // gate, up and the gated activation; its split form goes behind the input's
            const Op &act = *l.glu[0];
            if (n != 2 || l.list[0]->rows != l.list[1]->rows || l.list[0]->cols != l.list[1]->cols ||
                act.extra != (uint64_t)l.list[0]->rows * l.list[0]->batch) {
                die("split-form f32-tile launch: gated pair of unlike projections");
            }
            if (l.split_xs_off >= 0 &&
                ((uint64_t)l.split_xs_off < in_end ||
                 (uint64_t)l.split_xs_off + (uint64_t)act.extra * 6u > l.bx3_xs_bytes || l.split_cols != l.list[0]->rows)) {
                die("split-form f32-tile launch: the activation's split form overlaps the input's or the end");
            }
            out += std::string(",\"split_out\":") + (l.split_xs_off >= 0 ? "true" : "false");
        } else if (l.split_xs_off >= 0 || in_end != l.bx3_xs_bytes) {
            die("split-form f32-tile launch: workspace figures do not match its products");
        }
        out += ",\"xs_in_off\":" + std::to_string(l.xs_in_off);
        for (size_t i = 0; i < n; ++i) {
            if (!same_input(*l.list[0], *l.list[i])) {
                die("split-form f32-tile launch: products over different inputs");
            }
        }
        out += ",\"presplit\":1";
    }
    if (l.norm != nullptr) {
        const Op &nrm = *l.norm;
        if (nrm.kind != OP_RMSNORM || !key.fusable()) {
            die("fused norm in a launch that has no such form");
        }
        need(nrm.a[0], (size_t)nrm.rows * nrm.cols * 4u, "fused norm input");
        need(nrm.a[1], (size_t)nrm.cols * 4u, "fused norm weight");
        need(nrm.a[2], (size_t)nrm.rows * nrm.cols * 4u, "fused norm output");
        out += ",\"norm\":{\"x\":" + nm(nrm.a[0]) + ",\"y\":" + nm(nrm.a[2]) + "}";
    }
    out += ",\"ops\":[";
    for (size_t i = 0; i < n; ++i) {
        const Op &op = *l.list[i];
        check_product(op, key);
        out += std::string(i ? "," : "") + "{\"what\":\"" + op.what + "\",\"w\":" + nm(op.a[0]) +
               ",\"x\":" + nm(op.a[1]) + ",\"y\":" + nm(op.a[2]) + ",\"rows\":" + std::to_string(op.rows) +
               ",\"cols\":" + std::to_string(op.cols) + ",\"batch\":" + std::to_string(op.batch);
        if (l.normed[i]) {
            if (l.norm == nullptr || op.a[1] != l.norm->a[2]) {
                die("product reads a fused norm that is not its input");
            }
            out += ",\"normed\":true";
        }
        if (l.residual[i] != nullptr) {
            const Op &up = *l.residual[i];
            if (up.kind != OP_AXPY || up.a[0] != op.a[2] || up.extra != (uint64_t)op.rows * op.batch) {
                die("fused residual update is not over the product's output");
            }
            need(up.a[1], (size_t)up.extra * 4u, "fused residual");
            out += ",\"residual\":" + nm(up.a[1]);
        }
        if (l.glu[i] != nullptr) {
            const Op &act = *l.glu[i];
            if (i + 1 >= n || (act.kind != OP_SILU_MUL && act.kind != OP_GELU_MUL) ||
                act.a[0] != op.a[2] || act.a[1] != l.list[i + 1]->a[2]) {
                die("fused gated activation is not over this product and the next");
            }
            need(act.a[2], (size_t)act.extra * 4u, "fused activation output");
            out += ",\"glu\":" + nm(act.a[2]);
        }
        if (key.variant == V_BF16X3) {
            out += ",\"chunks\":" + std::to_string(l.bx3_chunks[i]);
        }
        out += "}";
    }
    out += "]}";
    if (!fake::enqueue(stream, "launch_list")) {
        return hipErrorInvalidValue;
    }
    if (stop != nullptr) {
        if (fake::capturing(stream)) {
            die("stop event on a recorded launch");
        }
        fake::attach_event(stop, stream);
    }
    record(out);
    return hipSuccess;
}

hipError_t tmdev::launch_single(hipStream_t stream, hipEvent_t stop, const Op &op, uint16_t *split_to,
                                uint32_t split_cols, const Op *update) {
    for (int i = 0; i < op.n_alloc; ++i) {
        if (op.a[i] != nullptr) {
            need(op.a[i], 1, "operand of a single operation");
        }
    }
    switch (op.kind) {
    case OP_RMSNORM:
        need(op.a[0], (size_t)op.rows * op.cols * 4u, "norm input");
        need(op.a[1], (size_t)op.cols * 4u, "norm weight");
        need(op.a[2], (size_t)op.rows * op.cols * 4u, "norm output");
        break;
    case OP_SILU_MUL:
    case OP_GELU_MUL:
        for (int i = 0; i < 3; ++i) {
            need(op.a[i], (size_t)op.extra * 4u, "gated activation operand");
        }
        break;
    case OP_AXPY:
    case OP_SCALE:
        need(op.a[0], (size_t)op.extra * 4u, "element-wise input");
        need(op.a[1], (size_t)op.extra * 4u, "element-wise output");
        break;
    case OP_COPY:
        need(op.a[0], ((size_t)op.x_off + op.extra) * 4u, "copy source");
        need(op.a[1], ((size_t)op.y_off + op.extra) * 4u, "copy destination");
        break;
    case OP_PACK:
        need(op.a[0], (size_t)op.rows * (op.cols / 32u) * 34u, "raw weights");
        need(op.a[1], (size_t)op.rows * (op.cols / 32u) * 34u, "sealed weights");
        break;
    case OP_QUANT:
        need(op.a[0], ((size_t)op.x_off + (size_t)op.batch * op.cols) * 4u, "activations");
        need(op.a[1], q8::xq_bytes(op.cols, op.batch), "quantized activations");
        break;
    case OP_ARGMAX:
        need(op.a[0], (size_t)op.extra * 4u, "argmax input");
        need(op.a[1], q8::ARGMAX_PARTIAL_BYTES, "argmax partials");
        need(op.a[2], ((size_t)op.y_off + 1u) * 4u, "argmax output");
        break;
    case OP_CHECKSUM:
        need(op.a[0], ((size_t)op.x_off + op.extra) * 4u, "checksum input");
        need(op.a[1], q8::CHECKSUM_GROUPS * 4u, "checksum partials");
        break;
    default:
        break;
    }
    if (update != nullptr) {
        if (op.kind != OP_RMSNORM || update->kind != OP_AXPY || update->a[1] != op.a[0]) {
            die("residual update in front of something that is not the norm of its result");
        }
        need(update->a[0], (size_t)update->extra * 4u, "residual update input");
    }
    if (split_to != nullptr &&
        (op.kind != OP_RMSNORM && op.kind != OP_SILU_MUL && op.kind != OP_GELU_MUL)) {
        die("split form asked of an operation that cannot write it");
    }
    (void)split_cols;
    std::string out = std::string("{\"k\":\"single\",\"what\":\"") + op.what + "\",\"bufs\":[";
    for (int i = 0; i < op.n_alloc; ++i) {
        out += std::string(i ? "," : "") + nm(op.a[i]);
    }
    out += std::string("],\"update\":") + (update != nullptr ? nm(update->a[0]) : "null") +
           ",\"split\":" + (split_to != nullptr ? "true" : "false") +
           ",\"recording\":" + (fake::capturing(stream) ? "true" : "false") + "}";
    // (argmax is two kernels, one enqueue each would change nothing here)
    if (!fake::enqueue(stream, "launch_single")) {
        return hipErrorInvalidValue;
    }
    if (stop != nullptr) {
        if (fake::capturing(stream)) {
            die("stop event on a recorded launch");
        }
        fake::attach_event(stop, stream);
    }
    record(out);
    return hipSuccess;
}
