"""GPU parity: the prefill GEMM from 17 tokens over sealed weights large enough
to fill the chip with 128-token x 256-row tiles, which runs on the bf16 matrix
cores with every f32 activation split into three exact bf16 pieces (contract: native/metal/tm_metal.h:172-175, tolerance-qualified like
every matrix-core kernel; crates/metal/src/tests.rs:1169-1233 for the shapes).
"""
import numpy as np
import pytest

import oracle as O
from tuckmill_amd import hip as H
from tuckmill_amd import synth as S

from q8util import bits, norm_err, ref_scale, require_gpu, upload_new, weights_buffer

pytestmark = pytest.mark.gpu

M0 = 17  # the least batch at which every sealed product is left to the matrix cores


@pytest.fixture(scope="module")
def ctx():
    c = require_gpu()
    yield c
    c.close()


def product(ctx, wb, x, rows, cols, batch, x_off=0, y_off=0):
    xs = np.zeros(x_off + batch * cols, np.float32)
    xs[x_off:] = x
    xb = upload_new(ctx, xs)
    yb = ctx.buffer((y_off + batch * rows) * 4)
    yb.zero(0, (y_off + batch * rows) * 4)
    ctx.q8_0_gemm_mma(wb, xb, yb, rows, cols, batch, x_off, y_off)
    ctx.fence()
    out = yb.download_f32(0, y_off + batch * rows).copy()
    xb.free()
    yb.free()
    return out


# K of 1, 3, 32 (whole, or two chunks of 16 blocks), 33 (17 + 16), 36, 64 and 96 blocks;
# ragged rows; a ragged last token tile; the smallest batch of the kernel and
# the largest; every product has at least 128 work units of its own.
SHAPES = [(8192, 1024, 512), (33000, 96, 65), (8300, 1056, 500), (4096, 3072, 512),
          (33000, 2048, 66), (33000, 32, 512), (8500, 1152, 450), (11000, 1024, 384),
          (16500, 1024, 129),
          # tiles of 64 tokens (fewer than 192 units of the large tile)
          (4096, 1024, 512), (2048, 2048, 512), (1024, 4096, 512), (6144, 2048, 128),
          (4100, 1056, 200), (33000, 96, 80),
          # one tile of 64 tokens (matrices of 16 M weights and more)
          (33000, 1024, M0), (4096, 4096, 64), (16500, 1056, 40),
          # few tiles under a deep K (3072 columns and more, where the f32 kernel is estimated
          # slower): tiles of 64 tokens, up to 8 K chunks
          (1024, 3072, 384), (1152, 6912, 100), (1536, 8960, 70), (1030, 4096, 256)]


@pytest.mark.parametrize("rows,cols,batch", SHAPES)
def test_gaussian_products_within_1e5(ctx, rows, cols, batch):
    w = S.make_weights(rows, cols, 5 * rows + cols)
    x = S.make_activations(batch * cols, batch + cols)
    wb = weights_buffer(ctx, w, rows, cols, True)
    launches = ctx.kernel_launches()
    got = product(ctx, wb, x, rows, cols, batch, 32, 8)
    assert ctx.kernel_launches() == launches + 2  # the split of x, then the product
    assert not got[:8].any(), "nothing before y_off"
    want = O.gemm_q8_0_f32(w, rows, cols, x, batch, threads=8)
    assert norm_err(got[8:].reshape(batch, rows), want) <= 1e-5
    wb.free()


# Up to 32 tokens a launch large enough for the bf16 matrix cores runs on 32-token tiles
# behind the split pass, and from 9 tokens (34 M weights) or 5 (128 M and more) so does the
# MFMA entry point over a product that is that large on its own. Ragged rows and a K of
# 33 blocks; the smallest batches; a batch of 16 and of 32.
@pytest.mark.parametrize("rows,cols,batch", [(33001, 1024, 9), (33001, 1024, 16), (33000, 1056, 32),
                                             (131100, 1024, 5), (131100, 1024, 8), (66000, 2048, 12)])
def test_large_products_at_few_tokens_within_1e5(ctx, rows, cols, batch):
    assert H.gemm_mma_on_bf16(rows, cols, batch)
    w = S.make_weights(rows, cols, 300 + batch)
    wb = weights_buffer(ctx, w, rows, cols, True)
    x = S.make_activations(batch * cols, 301)
    before = ctx.kernel_launches()
    got = product(ctx, wb, x, rows, cols, batch).reshape(batch, rows)
    assert ctx.kernel_launches() == before + 2  # the split pass and the products
    again = product(ctx, wb, x, rows, cols, batch).reshape(batch, rows)
    assert np.array_equal(bits(got), bits(again))
    tokens = sorted({0, batch - 1, batch // 2})
    want = O.gemm_q8_0_f32(w, rows, cols, np.ascontiguousarray(x.reshape(batch, cols)[tokens]).ravel(),
                           len(tokens), threads=8)
    assert norm_err(got[tokens], want) <= 1e-5
    # one token fewer than the rule asks for: the vector kernel, the GEMV's bits
    if batch in (5, 9):
        assert not H.gemm_mma_on_bf16(rows, cols, batch - 1)
        small = product(ctx, wb, x[:(batch - 1) * cols], rows, cols, batch - 1).reshape(batch - 1, rows)
        yb = ctx.buffer(rows * 4)
        xb = upload_new(ctx, x[:cols])
        ctx.q8_0_gemv(wb, xb, yb, rows, cols)
        ctx.fence()
        assert np.array_equal(bits(small[0]), bits(yb.download_f32(0, rows)))
        xb.free()
        yb.free()
    wb.free()


def test_few_token_products_that_are_large_together_share_the_small_tiles(ctx):
    # Six products of 8 to 13 M weights each over two inputs at 12 tokens through the MFMA
    # entry point: alone each runs the vector kernel (the GEMV's bits), in one group they are
    # one split pass and one launch on the bf16 matrix cores.
    batch = 12
    shapes = [(6144, 2048), (6144, 2048), (4096, 2048), (2048, 6144), (2048, 6144), (2048, 6144)]
    xs = {2048: S.make_activations(batch * 2048, 501), 6144: S.make_activations(batch * 6144, 502)}
    xbs = {c: upload_new(ctx, x) for c, x in xs.items()}
    mats = []
    for i, (rows, cols) in enumerate(shapes):
        w = S.make_weights(rows, cols, 510 + i)
        mats.append((w, rows, cols, weights_buffer(ctx, w, rows, cols, True), ctx.buffer(batch * rows * 4)))
    before = ctx.kernel_launches()
    w, rows, cols, wb, yb = mats[0]
    ctx.q8_0_gemm_mma(wb, xbs[cols], yb, rows, cols, batch, 0, 0)
    ctx.fence()
    assert ctx.kernel_launches() == before + 1
    alone = yb.download_f32(0, batch * rows).copy()
    runs = []
    for attempt in range(2):
        for m in mats:
            m[4].zero(0, batch * m[1] * 4)
        before = ctx.kernel_launches()
        ctx.begin_group()
        for w, rows, cols, wb, yb in mats:
            ctx.q8_0_gemm_mma(wb, xbs[cols], yb, rows, cols, batch, 0, 0)
        ctx.end_group()
        ctx.fence()
        assert ctx.kernel_launches() == before + 2
        runs.append([m[4].download_f32(0, batch * m[1]).copy() for m in mats])
    for i, (w, rows, cols, wb, yb) in enumerate(mats):
        assert np.array_equal(bits(runs[0][i]), bits(runs[1][i])), f"product {i}"
        want = O.gemm_q8_0_f32(w, rows, cols, xs[cols], batch, threads=8)
        assert norm_err(runs[0][i].reshape(batch, rows), want) <= 1e-5, f"product {i}"
    assert norm_err(alone.reshape(batch, shapes[0][0]), runs[0][0].reshape(batch, shapes[0][0])) <= 1e-5
    for b in list(xbs.values()) + [m[3] for m in mats] + [m[4] for m in mats]:
        b.free()


def test_boundary_values_and_wide_ranges(ctx):
    # crates/metal/src/tests.rs:1169-1233 (boundary weights and inputs), and
    # activations that span 60 binades: every piece of the split is exact, so the
    # large terms do not swamp the small ones any more than in the CPU's sum.
    rows, cols, batch = 33000, 1024, 65
    w = O.boundary_weights(rows, cols, 11)
    x = O.boundary_input(cols * batch, 13)
    wb = weights_buffer(ctx, w, rows, cols, True)
    launches = ctx.kernel_launches()
    got = product(ctx, wb, x, rows, cols, batch).reshape(batch, rows)
    assert ctx.kernel_launches() == launches + 2
    cpu = O.gemm_q8_0_f32(w, rows, cols, x, batch, threads=8)
    for b in range(batch):
        assert np.max(np.abs(got[b] - cpu[b])) <= 1e-4 * ref_scale(cpu[b]), f"token {b}"
    rng = np.random.default_rng(3)
    x = (S.make_activations(batch * cols, 9) *
         np.exp2(rng.integers(-30, 30, batch * cols)).astype(np.float32)).astype(np.float32)
    x[::97] = 0.0
    x[5::101] = np.float32(1e-41)  # subnormal
    got = product(ctx, wb, x, rows, cols, batch).reshape(batch, rows)
    cpu = O.gemm_q8_0_f32(w, rows, cols, x, batch, threads=8)
    assert norm_err(got, cpu) <= 1e-5
    # An infinite or NaN activation reaches the outputs as through f32 products:
    # +-inf where the weight is not zero, NaN where it is (0 * inf) and for NaN.
    x = S.make_activations(batch * cols, 10)
    x[3 * cols + 17] = np.inf
    x[5 * cols + 200] = np.nan
    x[7 * cols + 999] = -np.inf
    x[9 * cols + 40] = np.float32(np.uint32(0x7F800001).view(np.float32))  # a NaN in the low bits only
    got = product(ctx, wb, x, rows, cols, batch).reshape(batch, rows)
    with np.errstate(invalid="ignore", over="ignore"):
        cpu = O.gemm_q8_0_f32(w, rows, cols, x, batch, threads=8)
    assert np.array_equal(np.isnan(got), np.isnan(cpu))
    assert np.array_equal(np.isposinf(got), np.isposinf(cpu))
    assert np.array_equal(np.isneginf(got), np.isneginf(cpu))
    assert np.isnan(got[5]).all() and np.isnan(got[9]).all() and np.isinf(got[3]).any()
    ok = np.isfinite(cpu)
    assert np.max(np.abs(got[ok] - cpu[ok])) <= 1e-5 * np.max(np.abs(cpu[ok]))
    wb.free()


def test_activations_off_a_16_byte_boundary_take_the_f32_kernels(ctx):
    rows, cols, batch = 8192, 1024, 512
    w = S.make_weights(rows, cols, 77)
    x = S.make_activations(batch * cols, 78)
    wb = weights_buffer(ctx, w, rows, cols, True)
    launches = ctx.kernel_launches()
    got = product(ctx, wb, x, rows, cols, batch, 3, 0)
    assert ctx.kernel_launches() == launches + 1
    want = O.gemm_q8_0_f32(w, rows, cols, x, batch, threads=8)
    assert norm_err(got.reshape(batch, rows), want) <= 1e-5
    wb.free()


def test_a_group_splits_each_input_once_and_is_deterministic(ctx):
    # q/k/v share their activations, o and down have their own (K of 2 and 3
    # chunks: partial tiles added by whichever chunk arrives last, in chunk
    # order). The second product would be too small on its own; the launch
    # decides for all of them together, so all six share one launch (plus the one
    # that splits the three distinct inputs). Three times: every launch finds the
    # arrival counters as the last left them and gives the same bits; a replayed
    # recording of the group gives them again.
    batch = 512
    xs = {c: S.make_activations(batch * c, c) for c in (1024, 2048, 3072)}
    xbs = {c: upload_new(ctx, x) for c, x in xs.items()}
    mats = []
    shapes = [(8192, 1024), (1024, 1024), (9000, 1024), (8192, 1024), (4096, 2048), (4100, 3072)]
    assert not H.gemm_mma_on_bf16(1024, 1024, batch)
    assert H.gemm_mma_launch_tile([(r, c, batch) for r, c in shapes]) == 128
    for i, (rows, cols) in enumerate(shapes):
        w = S.make_weights(rows, cols, 600 + i)
        mats.append((w, rows, cols, weights_buffer(ctx, w, rows, cols, True),
                     ctx.buffer(batch * rows * 4)))

    def encode():
        for w, rows, cols, wb, yb in mats:
            ctx.q8_0_gemm_mma(wb, xbs[cols], yb, rows, cols, batch, 0, 0)

    launches = ctx.kernel_launches()
    runs = []
    for _ in range(3):
        for m in mats:
            m[4].zero(0, batch * m[1] * 4)
        ctx.begin_group()
        encode()
        ctx.end_group()
        ctx.fence()
        runs.append([m[4].download_f32(0, batch * m[1]).copy() for m in mats])
    assert ctx.kernel_launches() == launches + 3 * 2
    grouped = runs[0]
    picked = [0, 1, 77, 255, 256, 510, 511]
    for i, (w, rows, cols, wb, yb) in enumerate(mats):
        assert np.array_equal(bits(grouped[i]), bits(runs[1][i])), f"product {i}"
        assert np.array_equal(bits(grouped[i]), bits(runs[2][i])), f"product {i}"
        if i in (2, 5):
            want = O.gemm_q8_0_f32(w, rows, cols, xs[cols], batch, threads=8)
            assert norm_err(grouped[i].reshape(batch, rows), want) <= 1e-5
        else:
            x = np.ascontiguousarray(xs[cols].reshape(batch, cols)[picked]).reshape(-1)
            want = O.gemm_q8_0_f32(w, rows, cols, x, len(picked), threads=8)
            assert norm_err(grouped[i].reshape(batch, rows)[picked], want) <= 1e-5

    ctx.begin_group()
    encode()
    step = ctx.end_group_recorded()
    assert step.launches == 2
    for replay in range(3):
        for m in mats:
            m[4].zero(0, batch * m[1] * 4)
        step.run()
        ctx.fence()
        for i, m in enumerate(mats):
            assert np.array_equal(bits(m[4].download_f32(0, batch * m[1])), bits(grouped[i])), \
                f"replay {replay}, product {i}"
    step.free()
    for m in mats:
        m[3].free()
        m[4].free()


@pytest.mark.parametrize("kind", ["rmsnorm", "silu_mul", "gelu_tanh_mul"])
@pytest.mark.parametrize("batch", [500, 64])
def test_the_operator_in_front_writes_the_split_form_itself(ctx, kind, batch):
    # A layer as the executor encodes it: the norm before q/k/v (or the gated
    # activation before the down projection), then the products that read its
    # result. Inside one group the operator writes the split form of its result
    # as well and the products' launch does without its split pass: one kernel
    # launch fewer, the same bits as with the operator committed on its own
    # first (where the products' launch splits the input itself). A product
    # that reads the result from an offset, or another buffer, keeps its pass.
    cols = 1024
    shapes = [(8192, cols), (2048, cols), (9000, cols)]
    assert H.gemm_mma_launch_tile([(r, c, batch) for r, c in shapes]) != 0
    src = [upload_new(ctx, S.make_activations(batch * cols, 40 + i)) for i in range(2)]
    wn = upload_new(ctx, (1.0 + 0.1 * S.make_activations(cols, 9)).astype(np.float32))
    xb = ctx.buffer((batch * cols + 32) * 4)
    mats = []
    for i, (rows, c) in enumerate(shapes):
        w = S.make_weights(rows, c, 700 + i)
        mats.append((w, rows, c, weights_buffer(ctx, w, rows, c, True), ctx.buffer(batch * rows * 4)))

    def operator():
        if kind == "rmsnorm":
            ctx.rmsnorm(src[0], wn, xb, batch, cols, 1e-6)
        elif kind == "silu_mul":
            ctx.silu_mul(src[0], src[1], xb, batch * cols)
        else:
            ctx.gelu_tanh_mul(src[0], src[1], xb, batch * cols)

    def products(x_off=0):
        for w, rows, c, wb, yb in mats:
            ctx.q8_0_gemm_mma(wb, xb, yb, rows, c, batch, x_off, 0)

    def outputs():
        ctx.fence()
        return [m[4].download_f32(0, batch * m[1]).copy() for m in mats]

    def clear():
        xb.zero(0, (batch * cols + 32) * 4)
        for m in mats:
            m[4].zero(0, batch * m[1] * 4)

    clear()
    operator()
    ctx.fence()
    x = xb.download_f32(0, batch * cols).copy()
    before = ctx.kernel_launches()
    ctx.begin_group()
    products()
    ctx.end_group()
    apart = outputs()
    assert ctx.kernel_launches() == before + 2  # the split pass and the products

    for attempt in range(2):  # the second run finds the workspace as the first left it
        clear()
        before = ctx.kernel_launches()
        ctx.begin_group()
        operator()
        products()
        ctx.end_group()
        fused = outputs()
        assert ctx.kernel_launches() == before + 2  # the operator and the products
        assert np.array_equal(bits(xb.download_f32(0, batch * cols)), bits(x))
        for i in range(len(mats)):
            assert np.array_equal(bits(fused[i]), bits(apart[i])), f"attempt {attempt}, product {i}"
    w, rows, c, wb, yb = mats[1]
    want = O.gemm_q8_0_f32(w, rows, c, x, batch, threads=8)
    assert norm_err(fused[1].reshape(batch, rows), want) <= 1e-5

    # recorded and replayed
    ctx.begin_group()
    operator()
    products()
    step = ctx.end_group_recorded()
    assert step.launches == 2
    for replay in range(2):
        clear()
        step.run()
        got = outputs()
        for i in range(len(mats)):
            assert np.array_equal(bits(got[i]), bits(apart[i])), f"replay {replay}, product {i}"
    step.free()

    # read from an offset: not the operator's whole result, so the launch splits it itself
    clear()
    operator()
    ctx.fence()
    before = ctx.kernel_launches()
    ctx.begin_group()
    operator()
    products(x_off=32)
    ctx.end_group()
    off = outputs()
    assert ctx.kernel_launches() == before + 3
    full = xb.download_f32(0, batch * cols + 32)
    w, rows, c, wb, yb = mats[1]
    want = O.gemm_q8_0_f32(w, rows, c, np.ascontiguousarray(full[32:]), batch, threads=8)
    assert norm_err(off[1].reshape(batch, rows), want) <= 1e-5

    for b in src + [wn, xb]:
        b.free()
    for m in mats:
        m[3].free()
        m[4].free()


# Launches with too few work units for the staged kernel (they keep the f32 kernel's
# 32 x 32 tiles) right behind the operator that writes their one input: the operator
# leaves the split form and the tiles run on the bf16 matrix cores. q,k,v at 128 tokens
# (K over the four waves of a workgroup); one ragged product whose K is 33 blocks
# (a last group of one block, scales off an 8-byte boundary) over two workgroups per
# tile; K of 8 and of 2 blocks (two waves, one wave per tile); q,k,v at 256 tokens (two
# row tiles per wave); the down projection behind the gated activation (K of 96 blocks,
# two workgroups per tile).
SMALL_BEHIND = [("rmsnorm", 128, 1024, [2048, 1024, 1024]), ("rmsnorm", 100, 1056, [1000]),
                ("rmsnorm", 40, 256, [512, 33]), ("rmsnorm", 17, 64, [300]),
                ("rmsnorm", 256, 1024, [2048, 1024, 1024]), ("silu_mul", 128, 3072, [1024]),
                ("gelu_tanh_mul", 96, 3072, [1024])]


@pytest.mark.parametrize("kind,batch,cols,rows_list", SMALL_BEHIND)
def test_small_launches_behind_an_operator_read_its_split_form(ctx, kind, batch, cols, rows_list):
    assert H.gemm_mma_launch_tile([(r, cols, batch) for r in rows_list]) == 0  # not the staged kernel
    src = [upload_new(ctx, S.make_activations(batch * cols, 60 + i)) for i in range(2)]
    wn = upload_new(ctx, (1.0 + 0.1 * S.make_activations(cols, 9)).astype(np.float32))
    xb = ctx.buffer(batch * cols * 4)
    mats = []
    for i, rows in enumerate(rows_list):
        w = S.make_weights(rows, cols, 900 + i)
        mats.append((w, rows, weights_buffer(ctx, w, rows, cols, True), ctx.buffer(batch * rows * 4)))

    def operator():
        if kind == "rmsnorm":
            ctx.rmsnorm(src[0], wn, xb, batch, cols, 1e-6)
        elif kind == "silu_mul":
            ctx.silu_mul(src[0], src[1], xb, batch * cols)
        else:
            ctx.gelu_tanh_mul(src[0], src[1], xb, batch * cols)

    def products():
        for w, rows, wb, yb in mats:
            ctx.q8_0_gemm_mma(wb, xb, yb, rows, cols, batch, 0, 0)

    def outputs():
        ctx.fence()
        return [m[3].download_f32(0, batch * m[1]).copy() for m in mats]

    def clear():
        xb.zero(0, batch * cols * 4)
        for m in mats:
            m[3].zero(0, batch * m[1] * 4)

    operator()
    ctx.fence()
    x = xb.download_f32(0, batch * cols).copy()
    wants = [O.gemm_q8_0_f32(w, rows, cols, x, batch, threads=8) for w, rows, _, _ in mats]
    runs = []
    for attempt in range(2):  # the second run finds the workspace as the first left it
        clear()
        before = ctx.kernel_launches()
        ctx.begin_group()
        operator()
        products()
        ctx.end_group()
        runs.append(outputs())
        assert ctx.kernel_launches() == before + 2  # the operator and the products: no split pass
        assert np.array_equal(bits(xb.download_f32(0, batch * cols)), bits(x))
    for i, want in enumerate(wants):
        assert np.array_equal(bits(runs[0][i]), bits(runs[1][i])), f"product {i}"
        assert norm_err(runs[0][i].reshape(batch, mats[i][1]), want) <= 1e-5, f"product {i}"

    # recorded and replayed, with other work on the context in between
    ctx.begin_group()
    operator()
    products()
    step = ctx.end_group_recorded()
    assert step.launches == 2
    for replay in range(2):
        clear()
        step.run()
        got = outputs()
        for i in range(len(mats)):
            assert np.array_equal(bits(got[i]), bits(runs[0][i])), f"replay {replay}, product {i}"
    step.free()
    for b in src + [wn, xb] + [m[2] for m in mats] + [m[3] for m in mats]:
        b.free()


@pytest.mark.parametrize("kind,batch,hid,ffn,in_place",
                         [("silu_mul", 128, 1024, 3072, False), ("gelu_tanh_mul", 100, 1056, 1120, False),
                          ("silu_mul", 64, 1024, 3072, True), ("silu_mul", 40, 256, 512, False),
                          ("silu_mul", 256, 1024, 3072, False)])
def test_the_gated_activation_rides_in_the_launch_of_gate_and_up(ctx, kind, batch, hid, ffn, in_place):
    # The feed-forward half of a layer at a small prefill size: norm, gate and up, the
    # gated activation, down. In one group that is three launches: gate and up with the
    # activation in their launch, which also leaves the activation's split form for the
    # down projection. Every buffer comes out bit for bit as from the same operations in
    # two groups (norm, gate, up | activation, down), where the activation launches on
    # its own. In place (the activation over the gate's buffer) the raw gate is not kept,
    # as with the operator on its own. At 256 tokens gate and up alone have enough work for
    # the staged kernel's 64-token tile; with the activation and the down projection behind
    # them they take the small tiles with the activation fused in, and the results then
    # agree with the two-group run to the products' tolerance, not bit for bit.
    staged_apart = H.gemm_mma_launch_tile([(ffn, hid, batch)] * 2) != 0
    h = upload_new(ctx, S.make_activations(batch * hid, 31))
    wn = upload_new(ctx, (1.0 + 0.1 * S.make_activations(hid, 9)).astype(np.float32))
    xn = ctx.buffer(batch * hid * 4)
    wg, wu, wd = (S.make_weights(ffn, hid, 960), S.make_weights(ffn, hid, 961), S.make_weights(hid, ffn, 962))
    bg, bu, bd = (weights_buffer(ctx, wg, ffn, hid, True), weights_buffer(ctx, wu, ffn, hid, True),
                  weights_buffer(ctx, wd, hid, ffn, True))
    yg, yu, yd = ctx.buffer(batch * ffn * 4), ctx.buffer(batch * ffn * 4), ctx.buffer(batch * hid * 4)
    act = yg if in_place else ctx.buffer(batch * ffn * 4)
    bufs = [(xn, batch * hid), (yg, batch * ffn), (yu, batch * ffn), (act, batch * ffn), (yd, batch * hid)]

    def front():
        ctx.rmsnorm(h, wn, xn, batch, hid, 1e-6)
        ctx.q8_0_gemm_mma(bg, xn, yg, ffn, hid, batch, 0, 0)
        ctx.q8_0_gemm_mma(bu, xn, yu, ffn, hid, batch, 0, 0)

    def back():
        (ctx.silu_mul if kind == "silu_mul" else ctx.gelu_tanh_mul)(yg, yu, act, batch * ffn)
        ctx.q8_0_gemm_mma(bd, act, yd, hid, ffn, batch, 0, 0)

    def state():
        ctx.fence()
        return [b.download_f32(0, n).copy() for b, n in bufs]

    def clear():
        for b, n in bufs:
            b.zero(0, n * 4)

    clear()
    before = ctx.kernel_launches()
    ctx.begin_group()
    front()
    ctx.end_group()
    raw_gate = yg.download_f32(0, batch * ffn).copy()
    ctx.begin_group()
    back()
    ctx.end_group()
    apart = state()
    assert ctx.kernel_launches() == before + 4

    for attempt in range(2):
        clear()
        before = ctx.kernel_launches()
        ctx.begin_group()
        front()
        back()
        ctx.end_group()
        fused = state()
        assert ctx.kernel_launches() == before + 3
        for i, (a, b) in enumerate(zip(apart, fused)):
            if staged_apart and i > 0:
                scale = max(1.0, float(np.abs(a).max()))
                assert np.abs(a - b).max() <= 2e-5 * scale, f"attempt {attempt}, buffer {i}"
            else:
                assert np.array_equal(bits(a), bits(b)), f"attempt {attempt}, buffer {i}"
        if attempt == 0:
            first = fused
        else:
            for i, (a, b) in enumerate(zip(first, fused)):
                assert np.array_equal(bits(a), bits(b)), f"buffer {i} differs between two runs"
    if staged_apart:
        apart = first
        raw_gate = first[1]

    x = apart[0]
    g_want = O.gemm_q8_0_f32(wg, ffn, hid, x, batch, threads=8)
    assert norm_err(raw_gate.reshape(batch, ffn), g_want) <= 1e-5
    u = apart[2].astype(np.float64)
    g = raw_gate.astype(np.float64)
    if kind == "silu_mul":
        a_want = g / (1.0 + np.exp(-g)) * u
    else:
        a_want = 0.5 * g * (1.0 + np.tanh(0.7978845608028654 * g * (1.0 + 0.044715 * g * g))) * u
    assert np.abs(apart[3] - a_want).max() <= 1e-5 * max(1.0, np.abs(a_want).max())
    d_want = O.gemm_q8_0_f32(wd, hid, ffn, apart[3], batch, threads=8)
    assert norm_err(apart[4].reshape(batch, hid), d_want) <= 1e-5

    ctx.begin_group()
    front()
    back()
    step = ctx.end_group_recorded()
    assert step.launches == 3
    for replay in range(2):
        clear()
        step.run()
        got = state()
        for i, (a, b) in enumerate(zip(apart, got)):
            assert np.array_equal(bits(a), bits(b)), f"replay {replay}, buffer {i}"
    step.free()
    for b in {h, wn, xn, bg, bu, bd, yg, yu, yd, act}:
        b.free()


def test_an_infinite_or_nan_activation_reaches_the_outputs_through_the_operators_split_form(ctx):
    # silu_mul passes its second operand's non-finite values on; the products behind it
    # then see them in the split form (whole in the first piece).
    batch, cols, rows = 64, 1024, 512
    g = S.make_activations(batch * cols, 71)
    u = S.make_activations(batch * cols, 72)
    u[5 * cols + 100] = np.inf
    u[9 * cols + 7] = np.nan
    gb, ub = upload_new(ctx, g), upload_new(ctx, u)
    xb = ctx.buffer(batch * cols * 4)
    w = S.make_weights(rows, cols, 950)
    wb = weights_buffer(ctx, w, rows, cols, True)
    yb = ctx.buffer(batch * rows * 4)
    ctx.begin_group()
    ctx.silu_mul(gb, ub, xb, batch * cols)
    ctx.q8_0_gemm_mma(wb, xb, yb, rows, cols, batch, 0, 0)
    ctx.end_group()
    ctx.fence()
    y = yb.download_f32(0, batch * rows).reshape(batch, rows)
    x = xb.download_f32(0, batch * cols).reshape(batch, cols)
    assert np.isinf(x[5, 100]) and np.isnan(x[9, 7])
    assert not np.isfinite(y[5]).any() and np.isnan(y[9]).all()
    ok = np.ones(batch, bool)
    ok[[5, 9]] = False
    assert np.isfinite(y[ok]).all()
    want = O.gemm_q8_0_f32(w, rows, cols, np.ascontiguousarray(x[ok]).ravel(), int(ok.sum()), threads=8)
    assert norm_err(y[ok], want) <= 1e-5
    for b in [gb, ub, xb, wb, yb]:
        b.free()


@pytest.mark.parametrize("batch", [512, 128, 40])
def test_update_norm_and_products_in_one_group(ctx, batch):
    # The seam between two blocks of a layer: h += t, xn = rmsnorm(h), then the
    # products that read xn. In one group that is two launches (the norm does the
    # update in front of itself and writes xn's split form for the products
    # behind it); h, xn and the products come out bit for bit as with the
    # update, the norm and the products' group issued one after the other.
    cols = 1024
    shapes = [(6144, cols), (6144, cols), (6144, cols)]
    assert H.gemm_mma_launch_tile([(r, c, batch) for r, c in shapes]) != 0
    h0 = S.make_activations(batch * cols, 91)
    t = S.make_activations(batch * cols, 92)
    wn = upload_new(ctx, (1.0 + 0.1 * S.make_activations(cols, 9)).astype(np.float32))
    hb, tb = upload_new(ctx, h0), upload_new(ctx, t)
    xb = ctx.buffer(batch * cols * 4)
    mats = []
    for i, (rows, c) in enumerate(shapes):
        w = S.make_weights(rows, c, 800 + i)
        mats.append((rows, weights_buffer(ctx, w, rows, c, True), ctx.buffer(batch * rows * 4)))

    def products():
        for rows, wb, yb in mats:
            ctx.q8_0_gemm_mma(wb, xb, yb, rows, cols, batch, 0, 0)

    def state():
        ctx.fence()
        return [hb.download_f32(0, batch * cols).copy(), xb.download_f32(0, batch * cols).copy()] + \
               [yb.download_f32(0, batch * rows).copy() for rows, _, yb in mats]

    ctx.f32_axpy(tb, hb, 1.0, batch * cols)
    ctx.rmsnorm(hb, wn, xb, batch, cols, 1e-6)
    ctx.begin_group()
    products()
    ctx.end_group()
    apart = state()
    assert np.array_equal(bits(apart[0]), bits(h0 + t))

    for attempt in range(2):
        hb.upload(0, h0)
        xb.zero(0, batch * cols * 4)
        for _, _, yb in mats:
            yb.zero(0, yb.len())
        before = ctx.kernel_launches()
        ctx.begin_group()
        ctx.f32_axpy(tb, hb, 1.0, batch * cols)
        ctx.rmsnorm(hb, wn, xb, batch, cols, 1e-6)
        products()
        ctx.end_group()
        fused = state()
        assert ctx.kernel_launches() == before + 2
        for i, (a, b) in enumerate(zip(apart, fused)):
            assert np.array_equal(bits(a), bits(b)), f"attempt {attempt}, buffer {i}"
    for b in [wn, hb, tb, xb] + [m[1] for m in mats] + [m[2] for m in mats]:
        b.free()


# Launches whose work units leave the last round of the chip's workgroup slots
# partly empty: the units of that round are cut off one product's last rows as a
# tail segment whose K goes in chunks (q8::bx3_plan_launch). 300 units on the 256
# slots of the 128-token tile; one ragged row in the tail's last tile and a ragged
# token tile; two token tiles per row tile, ragged both ways, K of 48 blocks.
TAIL_SHAPES = [(76800, 1024, 128), (76801, 1024, 100), (38500, 1536, 250)]


@pytest.mark.parametrize("rows,cols,batch", TAIL_SHAPES)
def test_a_ragged_last_round_goes_as_a_tail_segment(ctx, rows, cols, batch):
    w = S.make_weights(rows, cols, 3 * rows + cols)
    x = S.make_activations(batch * cols, batch + rows)
    wb = weights_buffer(ctx, w, rows, cols, True)
    got = product(ctx, wb, x, rows, cols, batch, 0, 8)
    assert not got[:8].any(), "nothing before y_off"
    want = O.gemm_q8_0_f32(w, rows, cols, x, batch, threads=16)
    got = got[8:].reshape(batch, rows)
    assert norm_err(got, want) <= 1e-5
    # the boundary between the two segments and the last rows, row by row
    scale = np.abs(want).max()
    for r in (0, rows // 2, rows - 1, rows - 256, rows - 257):
        assert np.abs(got[:, r] - want[:, r]).max() <= 1e-5 * scale, r
    worst_row = np.abs(got - want).max(axis=0)
    assert worst_row.max() <= 1e-5 * scale, int(worst_row.argmax())
    again = product(ctx, wb, x, rows, cols, batch, 0, 8)[8:].reshape(batch, rows)
    assert np.array_equal(bits(got), bits(again)), "the same launch gives the same bits"
    wb.free()


def test_a_tail_segment_inside_a_group(ctx):
    """Two products share the launch; the larger one gives up its last rows."""
    cols, batch = 1024, 128
    shapes = [(70000, cols), (8192, cols)]
    ws = [S.make_weights(r, c, 11 + r) for r, c in shapes]
    wbs = [weights_buffer(ctx, w, r, c, True) for w, (r, c) in zip(ws, shapes)]
    x = S.make_activations(batch * cols, 99)
    xb = upload_new(ctx, x)
    ybs = [ctx.buffer(batch * r * 4) for r, _ in shapes]
    launches = ctx.kernel_launches()
    ctx.begin_group()
    for wb, yb, (r, c) in zip(wbs, ybs, shapes):
        ctx.q8_0_gemm_mma(wb, xb, yb, r, c, batch, 0, 0)
    ctx.end_group()
    ctx.fence()
    assert ctx.kernel_launches() == launches + 2
    for w, yb, (r, c) in zip(ws, ybs, shapes):
        want = O.gemm_q8_0_f32(w, r, c, x, batch, threads=16)
        assert norm_err(yb.download_f32(0, batch * r).reshape(batch, r), want) <= 1e-5
    for b in wbs + ybs + [xb]:
        b.free()


@pytest.mark.parametrize("rows,cols,batch", [(8192, 1024, 512), (8191, 1024, 512), (7936, 1024, 512),
                                             (32768, 1024, 65), (32768, 1024, 64), (32513, 1024, 65),
                                             (4096, 4096, 128), (4096, 4096, 129), (6144, 2048, 512),
                                             (6144, 2048, 256), (1024, 1024, 512), (2048, 6144, 384),
                                             (2048, 1024, 512), (3072, 1024, 512), (1024, 3072, 512),
                                             (1024, 2048, 512), (6144, 2048, 128), (2048, 4096, 128),
                                             (16384, 1024, 64), (16383, 1024, 64), (16384, 1024, 33),
                                             (16384, 1024, 32), (8192, 4096, 48), (6144, 2048, 64)])
def test_the_choice_of_kernel_follows_the_documented_rule(ctx, rows, cols, batch):
    # two launches (split, multiply) on the bf16 matrix cores, one on the f32 ones
    wb = weights_buffer(ctx, S.make_weights(rows, cols, 1), rows, cols, True)
    xb, yb = ctx.buffer(batch * cols * 4), ctx.buffer(batch * rows * 4)
    launches = ctx.kernel_launches()
    ctx.q8_0_gemm_mma(wb, xb, yb, rows, cols, batch, 0, 0)
    ctx.fence()
    assert ctx.kernel_launches() - launches == (2 if H.gemm_mma_on_bf16(rows, cols, batch) else 1)
    for b in (wb, xb, yb):
        b.free()
