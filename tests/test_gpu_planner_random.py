"""GPU: random operator sequences through the dispatch-group planner.

The planner shares launches between independent products, lets operators ride
in a neighbouring launch (a residual update behind a one-token product or in
front of a norm, a norm or gated activation in front of or behind its
products, the split form of a bf16 product's input written by the operator
before it) and picks kernels per launch. None of that may change what a
sequence computes: every random program here is run three ways - one commit
per operator, as one dispatch group, and as a recorded group replayed - and the
contents of every buffer are compared afterwards. Programs made of the exact
kernels only (GEMV, exact GEMM, operators) must agree bit for bit; programs
with matrix-core products, whose tile (and so the order of their f32 sums) may
depend on what shares the launch, within the path's tolerance.
(The reference's own grouping tests: crates/metal/src/tests.rs:922-1056.)
"""
import numpy as np
import pytest

from tuckmill_amd import synth as S

from q8util import bits, require_gpu, upload_new, weights_buffer

pytestmark = pytest.mark.gpu

# Qwen3-0.6B's widths, Gemma-3-1B's (column tails of 128 and 768 behind the 1024-column steps)
# and Qwen3-1.7B's (rows of 2048 and 6144 columns: short tiles in steps of several chunks,
# the token-split kernel's 4-row steps, short gated pairs)
DIMS = [(1024, 3072), (1152, 6912), (2048, 6144)]


@pytest.fixture(scope="module")
def ctx():
    c = require_gpu()
    yield c
    c.close()


@pytest.fixture(scope="module", params=DIMS, ids=lambda d: f"{d[0]}x{d[1]}")
def weights(ctx, request):
    """Sealed matrices hidden -> hidden, hidden -> ffn, ffn -> hidden (two each)."""
    hidden, ffn = request.param
    out = {}
    for kind, rows, cols in (("hh", hidden, hidden), ("hf", ffn, hidden), ("fh", hidden, ffn)):
        out[kind] = [(weights_buffer(ctx, S.make_weights(rows, cols, 40 + 7 * i + rows % 13), rows,
                                     cols, True), rows, cols) for i in range(2)]
    norm_w = upload_new(ctx, (1.0 + 0.2 * S.make_activations(hidden, 3)).astype(np.float32))
    yield out, norm_w, hidden, ffn
    for mats in out.values():
        for wb, _, _ in mats:
            wb.free()
    norm_w.free()


def make_program(rng, batch, with_mma):
    """A list of operators over 4 hidden-width and 3 ffn-width buffers of
    `batch` rows each. Reads come before writes in the tuple; an operator never
    writes a buffer it reads unless the ABI allows it (axpy, in-place norm)."""
    ops = []
    call = "mma" if with_mma else "exact"
    for _ in range(int(rng.integers(6, 14))):
        kind = rng.choice(["product", "product", "product", "rmsnorm", "silu", "gelu", "axpy",
                           "block", "block", "ffn", "ffn"])
        if kind == "block":
            # the shapes the planner fuses: residual update, norm, products that read the norm
            t, hid, xn = (int(v) for v in rng.permutation(4)[:3])
            ops.append(("axpy", "h", t, hid, 1.0))
            ops.append(("rmsnorm", hid, xn))
            outs = rng.permutation(3)
            for k in range(int(rng.integers(1, 4))):
                ops.append(("product", "hf", int(rng.integers(2)), xn, int(outs[k]), call))
            continue
        if kind == "ffn":
            # gate and up from one input, the gated activation, down, the residual update
            x, t, hid = (int(v) for v in rng.permutation(4)[:3])
            g, u, act = (int(v) for v in rng.permutation(3))
            ops.append(("product", "hf", 0, x, g, call))
            ops.append(("product", "hf", 1, x, u, call))
            ops.append((str(rng.choice(["silu", "gelu"])), g, u, g if rng.random() < 0.5 else act))
            ops.append(("product", "fh", int(rng.integers(2)), ops[-1][3], t, call))
            ops.append(("axpy", "h", t, hid, 1.0))
            continue
        if kind == "product":
            shape = rng.choice(["hh", "hf", "fh"])
            src_pool, dst_pool = (4 if shape[0] == "h" else 3), (4 if shape[1] == "h" else 3)
            src = int(rng.integers(src_pool))
            dst = int(rng.integers(dst_pool))
            if shape == "hh":
                while dst == src:
                    dst = int(rng.integers(dst_pool))
            ops.append(("product", shape, int(rng.integers(2)), src, dst, call))
        elif kind == "rmsnorm":
            src = int(rng.integers(4))
            dst = src if rng.random() < 0.25 else int(rng.integers(4))
            ops.append(("rmsnorm", src, dst))
        elif kind in ("silu", "gelu"):
            g, u = int(rng.integers(3)), int(rng.integers(3))
            out = g if rng.random() < 0.3 else int(rng.integers(3))
            if out == u and out != g:
                out = g
            ops.append((kind, g, u, out))
        else:
            width = rng.choice(["h", "f"])
            pool = 4 if width == "h" else 3
            a, y = int(rng.integers(pool)), int(rng.integers(pool))
            while y == a:
                y = int(rng.integers(pool))
            ops.append(("axpy", width, a, y, float(rng.choice([1.0, 0.5, -0.25]))))
    return ops


def encode(ctx, op, bufs, weights, norm_w, batch, dims):
    h, f = bufs
    HIDDEN, FFN = dims
    if op[0] == "product":
        _, shape, which, src, dst, call = op
        wb, rows, cols = weights[shape][which]
        x = (h if shape[0] == "h" else f)[src]
        y = (h if shape[1] == "h" else f)[dst]
        if call == "mma":
            ctx.q8_0_gemm_mma(wb, x, y, rows, cols, batch, 0, 0)
        elif batch == 1:
            ctx.q8_0_gemv(wb, x, y, rows, cols)
        else:
            ctx.q8_0_gemm(wb, x, y, rows, cols, batch, 0, 0)
    elif op[0] == "rmsnorm":
        ctx.rmsnorm(h[op[1]], norm_w, h[op[2]], batch, HIDDEN, 1e-6)
    elif op[0] == "silu":
        ctx.silu_mul(f[op[1]], f[op[2]], f[op[3]], batch * FFN)
    elif op[0] == "gelu":
        ctx.gelu_tanh_mul(f[op[1]], f[op[2]], f[op[3]], batch * FFN)
    else:
        _, width, a, y, alpha = op
        pool, n = (h, batch * HIDDEN) if width == "h" else (f, batch * FFN)
        ctx.f32_axpy(pool[a], pool[y], alpha, n)


# kernel launches and runs over all programs, per way of running them
LAUNCHES = {"apart": 0, "group": 0}
RUNS = {"apart": 0, "group": 0}


def run(ctx, program, weights, norm_w, batch, start, mode, dims):
    HIDDEN, FFN = dims
    h = [upload_new(ctx, v) for v in start[0]]
    f = [upload_new(ctx, v) for v in start[1]]
    before = ctx.kernel_launches()
    if mode == "apart":
        for op in program:
            encode(ctx, op, (h, f), weights, norm_w, batch, dims)
    elif mode == "group":
        ctx.begin_group()
        for op in program:
            encode(ctx, op, (h, f), weights, norm_w, batch, dims)
        ctx.end_group()
    else:
        ctx.begin_group()
        for op in program:
            encode(ctx, op, (h, f), weights, norm_w, batch, dims)
        step = ctx.end_group_recorded()
        step.run()
        ctx.fence()
        step.free()
    ctx.fence()
    if mode in LAUNCHES:
        LAUNCHES[mode] += ctx.kernel_launches() - before
        RUNS[mode] += 1
    out = [b.download_f32(0, batch * HIDDEN).copy() for b in h] + \
          [b.download_f32(0, batch * FFN).copy() for b in f]
    for b in h + f:
        b.free()
    return out


def starting_values(seed, batch, dims):
    HIDDEN, FFN = dims
    # small magnitudes: a dozen products and residual updates in a row must not overflow
    return ([0.5 * S.make_activations(batch * HIDDEN, seed + i) for i in range(4)],
            [0.5 * S.make_activations(batch * FFN, seed + 10 + i) for i in range(3)])


@pytest.mark.parametrize("seed", range(32))
def test_exact_programs_give_the_same_bits_however_they_are_grouped(ctx, weights, seed):
    mats, norm_w, hidden, ffn = weights
    dims = (hidden, ffn)
    rng = np.random.default_rng(1000 + seed)
    batch = int(rng.choice([1, 1, 2, 3, 4, 8, 20, 32]))
    program = make_program(rng, batch, with_mma=False)
    start = starting_values(seed, batch, dims)
    apart = run(ctx, program, mats, norm_w, batch, start, "apart", dims)
    for mode in ("group", "recorded"):
        got = run(ctx, program, mats, norm_w, batch, start, mode, dims)
        for i, (a, b) in enumerate(zip(apart, got)):
            assert np.array_equal(bits(a), bits(b)), f"{mode}: buffer {i}, batch {batch}, program {program}"


@pytest.mark.parametrize("seed", range(24))
def test_matrix_core_programs_agree_within_tolerance_however_they_are_grouped(ctx, weights, seed):
    mats, norm_w, hidden, ffn = weights
    dims = (hidden, ffn)
    rng = np.random.default_rng(2000 + seed)
    batch = int(rng.choice([17, 40, 64, 100, 128, 256, 512]))
    program = make_program(rng, batch, with_mma=True)
    start = starting_values(seed, batch, dims)
    apart = run(ctx, program, mats, norm_w, batch, start, "apart", dims)
    group = run(ctx, program, mats, norm_w, batch, start, "group", dims)
    again = run(ctx, program, mats, norm_w, batch, start, "group", dims)
    recorded = run(ctx, program, mats, norm_w, batch, start, "recorded", dims)
    for i, a in enumerate(apart):
        finite = np.isfinite(a)
        assert np.array_equal(finite, np.isfinite(group[i])), f"buffer {i}, program {program}"
        scale = max(float(np.max(np.abs(a[finite]))) if finite.any() else 0.0, 1.0)
        # errors of 1e-7 per product compound through at most a dozen dependent operators
        assert np.max(np.abs(a[finite] - group[i][finite])) <= 2e-5 * scale, \
            f"buffer {i}, batch {batch}, program {program}"
        # the same group gives the same bits every time, eager or replayed
        assert np.array_equal(bits(group[i]), bits(again[i])), f"buffer {i}, program {program}"
        assert np.array_equal(bits(group[i]), bits(recorded[i])), f"buffer {i}, program {program}"


def test_zz_the_programs_above_exercised_the_planner():
    # (runs after the two tests above: grouped, the same programs took far fewer launches)
    assert RUNS["apart"] > 0 and RUNS["group"] > 0
    apart, group = LAUNCHES["apart"] / RUNS["apart"], LAUNCHES["group"] / RUNS["group"]
    assert group < 0.8 * apart, (LAUNCHES, RUNS)
