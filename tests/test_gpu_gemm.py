"""GPU parity: small-batch GEMM (GEMV arithmetic) and the MFMA prefill GEMM.

Follows crates/metal/src/tests.rs:835-921 (batched GEMM, batch = 1 bit
identity) and :1169-1247 (MMA GEMM: row tails, partial token tiles, offsets,
batch 512, batch 513 refused).
"""
import numpy as np
import pytest

import oracle as O
from tuckmill_amd import hip as H
from tuckmill_amd import synth as S

from q8util import bits, gemv, norm_err, ref_scale, require_gpu, upload_new, weights_buffer

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = require_gpu()
    yield c
    c.close()


def run_gemm(ctx, fn, wb, x, rows, cols, batch, x_off=0, y_off=0):
    xs = np.zeros(x_off + batch * cols, np.float32)
    xs[x_off:] = x
    xb = upload_new(ctx, xs)
    yb = ctx.buffer((y_off + batch * rows) * 4)
    fn(wb, xb, yb, rows, cols, batch, x_off, y_off)
    ctx.fence()
    out = yb.download_f32(0, y_off + batch * rows).copy()
    xb.free()
    yb.free()
    return out


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("rows,cols,all_rows", [(32, 32, True), (64, 1024, True),
                                                (2048, 1024, True), (3072, 1024, True),
                                                (151_936, 1024, False)])
def test_batched_gemm_matches_the_scalar_reference(ctx, rows, cols, all_rows, packed):
    # crates/metal/src/tests.rs:835-892
    w = O.boundary_weights(rows, cols, 101 + rows)
    wb = weights_buffer(ctx, w, rows, cols, packed)
    for batch in (1, 4, 8, 16):
        xs = [O.boundary_input(cols, 200 + b) for b in range(batch)]
        got = run_gemm(ctx, ctx.q8_0_gemm, wb, np.concatenate(xs), rows, cols, batch)
        got = got.reshape(batch, rows)
        check = np.arange(rows) if all_rows else np.array([0, 1, rows // 2, rows - 2, rows - 1])
        for b, x in enumerate(xs):
            if all_rows or b == 0:
                cpu = O.gemv_q8_0_f32(w, rows, cols, x, threads=8)
            scale = ref_scale(cpu)
            if all_rows or b == 0:
                assert np.max(np.abs(got[b][check] - cpu[check])) <= 1e-4 * scale
    wb.free()


def test_batch_one_gemm_is_bit_identical_to_gemv(ctx):
    # crates/metal/src/tests.rs:895-921
    rows, cols = 512, 1024
    w = O.boundary_weights(rows, cols, 7)
    x = O.boundary_input(cols, 9)
    for packed in (False, True):
        wb = weights_buffer(ctx, w, rows, cols, packed)
        single = gemv(ctx, wb, x, rows, cols)
        batch = run_gemm(ctx, ctx.q8_0_gemm, wb, x, rows, cols, 1)
        assert np.array_equal(bits(single), bits(batch))


@pytest.mark.parametrize("x_off", [0, 3])
@pytest.mark.parametrize("rows,cols,batch", [(64, 1024, 32), (100, 1152, 7), (33, 96, 5),
                                             (513, 2048, 13), (40, 6912, 3), (520, 2048, 8),
                                             (100, 3072, 2), (33, 1024, 4), (4099, 6144, 16),
                                             (41, 6912, 9), (64, 1056, 3), (50, 2016, 5),
                                             (8, 1024, 17), (9, 4096, 31),
                                             (70, 1152, 20), (41, 6912, 32), (33, 2016, 25),
                                             # few rows under a long K, up to 4 tokens: steps of 4 rows
                                             (1300, 3072, 2), (1301, 4224, 4), (2050, 6912, 6),
                                             (1290, 3072, 7), (1283, 4096, 3), (4096, 4096, 8),
                                             (1300, 2048, 2), (1290, 6912, 4)])
def test_every_token_of_the_small_gemm_equals_its_own_gemv(ctx, rows, cols, batch, x_off):
    # Stronger than the reference's batch = 1 identity: the exact (speculative
    # verify) path must reproduce decode for every token. Covers every
    # waves x tokens-per-wave split of the small-batch kernel, column tails,
    # row tails and activations that are not 16-byte aligned.
    w = S.make_weights(rows, cols, 31 + rows)
    x = S.make_activations(cols * batch, 77)
    wb = weights_buffer(ctx, w, rows, cols, True)
    got = run_gemm(ctx, ctx.q8_0_gemm, wb, x, rows, cols, batch, x_off, 5)[5:].reshape(batch, rows)
    want = O.gemm_q8_0_f32(w, rows, cols, x, batch)
    assert norm_err(got, want) <= 1e-5
    for b in range(batch):
        single = gemv(ctx, wb, x[b * cols:(b + 1) * cols], rows, cols)
        assert np.array_equal(bits(single), bits(got[b])), f"token {b}"


@pytest.mark.parametrize("x_off", [0, 3])
@pytest.mark.parametrize("rows,cols,batch", [(64, 1024, 32), (513, 2048, 13), (100, 3072, 2),
                                             (33, 1024, 4), (4099, 6144, 16), (8, 1024, 17),
                                             (9, 4096, 31), (520, 2048, 8), (77, 1024, 5),
                                             # column tails (cols a multiple of 64): rows that are
                                             # only 8- or 4-byte aligned, two token groups at 17+
                                             (100, 1152, 7), (40, 6912, 3), (41, 6912, 32),
                                             (70, 1152, 20), (64, 1088, 3), (50, 2112, 5),
                                             # cols not a multiple of 64: the general form
                                             (33, 2016, 6)])
def test_the_small_gemm_over_weights_as_uploaded_gives_the_sealed_bits(ctx, rows, cols, batch, x_off):
    # Weights in the raw layout (never sealed): the token-split kernel reads their
    # whole 1024-column chunks through LDS. Every token equals its own GEMV over
    # the same raw buffer and the sealed kernel's result, bit for bit.
    w = S.make_weights(rows, cols, 57 + rows)
    x = S.make_activations(cols * batch, 91)
    raw_b = weights_buffer(ctx, w, rows, cols, False)
    sealed_b = weights_buffer(ctx, w, rows, cols, True)
    got = run_gemm(ctx, ctx.q8_0_gemm, raw_b, x, rows, cols, batch, x_off, 5)[5:].reshape(batch, rows)
    sealed = run_gemm(ctx, ctx.q8_0_gemm, sealed_b, x, rows, cols, batch, x_off, 5)[5:]
    assert norm_err(got, O.gemm_q8_0_f32(w, rows, cols, x, batch)) <= 1e-5
    assert np.array_equal(bits(got), bits(sealed.reshape(batch, rows)))
    for b in (0, batch // 2, batch - 1):
        single = gemv(ctx, raw_b, x[b * cols:(b + 1) * cols], rows, cols)
        assert np.array_equal(bits(single), bits(got[b])), f"token {b}"
    raw_b.free()
    sealed_b.free()


def test_products_that_go_as_two_token_groups_share_launches_by_descriptor_count(ctx):
    # 17 to 32 tokens over a matrix with a column tail go as two descriptors of up
    # to 16 tokens each (the 8-tokens-per-wave form has no tail variant). A
    # launch holds 224 descriptors: 120 such products in one group take two
    # launches, and every one of them comes out as it does alone.
    rows, cols, batch, n = 40, 1152, 20, 120
    w = S.make_weights(rows, cols, 901)
    wb = weights_buffer(ctx, w, rows, cols, True)
    xs = [S.make_activations(cols * batch, 300 + i) for i in range(3)]
    xbs = [upload_new(ctx, x) for x in xs]
    ybs = [ctx.buffer(batch * rows * 4) for _ in range(n)]
    alone = []
    for x in xs:
        alone.append(run_gemm(ctx, ctx.q8_0_gemm, wb, x, rows, cols, batch).reshape(batch, rows))
        assert norm_err(alone[-1], O.gemm_q8_0_f32(w, rows, cols, x, batch)) <= 1e-5
    before = ctx.kernel_launches()
    ctx.begin_group()
    for i, yb in enumerate(ybs):
        ctx.q8_0_gemm(wb, xbs[i % 3], yb, rows, cols, batch, 0, 0)
    ctx.end_group()
    ctx.fence()
    assert ctx.kernel_launches() == before + 2
    for i, yb in enumerate(ybs):
        got = yb.download_f32(0, batch * rows).reshape(batch, rows)
        assert np.array_equal(bits(got), bits(alone[i % 3])), f"product {i}"
    for b in [wb] + xbs + ybs:
        b.free()


def test_gemm_batch_limits(ctx):
    wb, xb, yb = ctx.buffer(64), ctx.buffer(64), ctx.buffer(64)
    with pytest.raises(H.TuckmillError) as e:
        ctx.q8_0_gemm(wb, xb, yb, 1, 32, H.GEMM_MAX_BATCH + 1, 0, 0)
    assert e.value.abi_code == H.TM_HIP_ERR_UNSUPPORTED
    with pytest.raises(H.TuckmillError):
        ctx.q8_0_gemm(wb, xb, yb, 1, 32, 0, 0, 0)
    with pytest.raises(H.TuckmillError) as e:
        ctx.q8_0_gemm(wb, xb, yb, 1, 32, 1, 16, 0)  # x range past the end
    assert e.value.abi_code == H.TM_HIP_ERR_BOUNDS


MMA_SHAPES = [(16, 1024, 16), (40, 64, 3), (3584, 1024, 16), (3584, 1024, 32), (40, 64, 27),
              (1024, 3584, 64), (100, 96, 77), (40, 64, 512), (1024, 3584, 7), (6144, 1024, 1),
              # few output tiles at a wide batch: 32-token tiles (ragged last token and row tiles)
              (500, 2048, 500), (1000, 1024, 130)]


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("rows,cols,batch", MMA_SHAPES)
def test_gemm_mma_matches_the_cpu_reference_within_tolerance(ctx, rows, cols, batch, packed):
    # crates/metal/src/tests.rs:1169-1233
    w = O.boundary_weights(rows, cols, 11)
    x = O.boundary_input(cols * batch, 13)
    wb = weights_buffer(ctx, w, rows, cols, packed)
    x_off, y_off = 32, 8
    got = run_gemm(ctx, ctx.q8_0_gemm_mma, wb, x, rows, cols, batch, x_off, y_off)
    assert not got[:y_off].any(), "nothing before y_off"
    got = got[y_off:].reshape(batch, rows)
    cpu = O.gemm_q8_0_f32(w, rows, cols, x, batch, threads=8)
    for b in range(batch):
        assert np.max(np.abs(got[b] - cpu[b])) <= 1e-4 * ref_scale(cpu[b]), f"token {b}"
    wb.free()


def test_gemm_mma_refuses_batch_above_the_maximum(ctx):
    # crates/metal/src/tests.rs:1234-1247
    with pytest.raises(H.TuckmillError):
        ctx.q8_0_gemm_mma(ctx.buffer(64), ctx.buffer(64), ctx.buffer(64), 1, 32,
                          H.GEMM_MMA_MAX_BATCH + 1, 0, 0)


@pytest.mark.parametrize("rows,cols", [(1024, 1024), (2048, 1024), (1024, 2048), (3072, 1024),
                                       (1024, 3072)])
def test_config2_prefill_gemm_m512_gaussian_within_1e5(ctx, rows, cols):
    # BASELINE config 2: M = 512 against the Qwen3-0.6B projection shapes.
    batch = 512
    w = S.make_weights(rows, cols, S.tensor_seed(2, 0, f"{rows}x{cols}"))
    x = S.make_activations(batch * cols, rows + cols)
    wb = weights_buffer(ctx, w, rows, cols, True)
    got = run_gemm(ctx, ctx.q8_0_gemm_mma, wb, x, rows, cols, batch).reshape(batch, rows)
    want = O.gemm_q8_0_f32(w, rows, cols, x, batch, threads=8)
    assert norm_err(got, want) <= 1e-5
    wb.free()


@pytest.mark.parametrize("rows,cols,batch", [(6912, 1152, 512), (1152, 6912, 512), (97, 1152, 33),
                                             (6144, 2048, 64), (2048, 6144, 8), (70, 32, 2)])
def test_gemm_mma_gemma_and_sweep_shapes_gaussian(ctx, rows, cols, batch):
    # BASELINE configs 3 and 4 (K not a multiple of 256; 2B-class shapes).
    w = S.make_weights(rows, cols, rows * 7 + cols)
    x = S.make_activations(batch * cols, batch)
    wb = weights_buffer(ctx, w, rows, cols, True)
    got = run_gemm(ctx, ctx.q8_0_gemm_mma, wb, x, rows, cols, batch).reshape(batch, rows)
    want = O.gemm_q8_0_f32(w, rows, cols, x, batch, threads=8)
    assert norm_err(got, want) <= 1e-5
    wb.free()


def test_independent_mma_products_in_a_group_share_one_launch(ctx):
    # q/k/v of a prefill chunk: same X, three weight matrices, one launch. Too
    # little work between them for the bf16 matrix cores: they run on the f32
    # ones. Alone, k and v have few enough output tiles (96) to be shared between
    # two workgroups each, which cuts their K sums differently: within rounding
    # of the grouped result, not the same bits; q alone has the launch's K split.
    assert H.gemm_mma_launch_tile([(2048, 1024, 96), (1024, 1024, 96), (1024, 1024, 96)]) == 0
    cols, batch = 1024, 96
    x = S.make_activations(batch * cols, 5)
    xb = upload_new(ctx, x)
    mats = []
    for i, rows in enumerate((2048, 1024, 1024)):
        w = S.make_weights(rows, cols, 40 + i)
        mats.append((w, rows, weights_buffer(ctx, w, rows, cols, True), ctx.buffer(batch * rows * 4)))
    launches = ctx.kernel_launches()
    ctx.begin_group()
    for w, rows, wb, yb in mats:
        ctx.q8_0_gemm_mma(wb, xb, yb, rows, cols, batch, 0, 0)
    ctx.end_group()
    assert ctx.kernel_launches() == launches + 1
    ctx.fence()
    for w, rows, wb, yb in mats:
        grouped = yb.download_f32(0, batch * rows).copy()
        alone = run_gemm(ctx, ctx.q8_0_gemm_mma, wb, x, rows, cols, batch)
        if rows == 2048:
            assert np.array_equal(bits(grouped), bits(alone))
        want = O.gemm_q8_0_f32(w, rows, cols, x, batch, threads=8)
        assert norm_err(grouped.reshape(batch, rows), want) <= 1e-5
        assert norm_err(alone.reshape(batch, rows), want) <= 1e-5


@pytest.mark.parametrize("packed", [True, False])
@pytest.mark.parametrize("rows,cols,batch", [
    (1024, 2048, 32),    # 32 output tiles, 64 blocks: four workgroups per tile
    (1024, 3072, 128),   # 128 tiles: two
    (500, 4096, 20),     # 16 tiles (ragged rows and tokens), 128 blocks: eight
    (1152, 6912, 70),    # 108 tiles of 32 tokens: two, 216 blocks
    (100, 8192, 200),    # 16 tiles of 64 tokens... few rows under a very deep K
    (1024, 1024, 17),    # 32 tiles, 32 blocks: two workgroups, four blocks per wave
])
def test_f32_launches_with_few_output_tiles_share_them_between_workgroups(ctx, rows, cols, batch,
                                                                          packed):
    # A launch on the f32 matrix cores with few output tiles and a long K hands
    # each tile to 2, 4 or 8 workgroups, each with its own part of K; the last to
    # arrive adds the partial tiles in part order. Within 1e-5 of the oracle,
    # and the same bits every time (the arrival counters go back to zero), also
    # with another launch of the kind in between.
    assert not packed or not H.gemm_mma_on_bf16(rows, cols, batch)
    w = S.make_weights(rows, cols, 300 + rows)
    x = S.make_activations(batch * cols, 301 + cols)
    wb = weights_buffer(ctx, w, rows, cols, packed)
    want = O.gemm_q8_0_f32(w, rows, cols, x, batch, threads=8)
    first = run_gemm(ctx, ctx.q8_0_gemm_mma, wb, x, rows, cols, batch)
    assert norm_err(first.reshape(batch, rows), want) <= 1e-5
    other_w = S.make_weights(64, 4096, 7)
    other = weights_buffer(ctx, other_w, 64, 4096, packed)
    run_gemm(ctx, ctx.q8_0_gemm_mma, other, S.make_activations(40 * 4096, 8), 64, 4096, 40)
    for _ in range(3):
        again = run_gemm(ctx, ctx.q8_0_gemm_mma, wb, x, rows, cols, batch)
        assert np.array_equal(bits(first), bits(again))
    wb.free()
    other.free()


@pytest.mark.parametrize("packed", [True, False])
def test_a_large_mma_group_is_deterministic_and_matches_the_oracle(ctx, packed):
    # Raw weights: enough wave tiles in one launch for the work-queue kernel (a
    # wave owns a tile over the whole of K and takes tiles from a device-side
    # counter); each product alone has too few and runs the K-split kernels, with
    # the same bits. Sealed weights: the products have enough work between them
    # for the bf16 matrix cores and share one launch there (plus the launch that
    # splits their inputs), with K cut as the launch's tile says; the entry point
    # is tolerance-qualified (native/metal/tm_metal.h:172-175), so what is asked
    # is: the same group gives the same bits every time, and every product is
    # within 1e-5 of the oracle. K of 32, 33, 64 and 96 blocks, ragged rows and a
    # ragged last token tile.
    shapes = [(4100, 1024, 500), (2048, 2048, 512), (1024, 3072, 512), (3000, 1056, 450),
              (4096, 1024, 512), (1024, 3072, 200)]
    mats = []
    for i, (rows, cols, batch) in enumerate(shapes):
        w = S.make_weights(rows, cols, 900 + i)
        x = S.make_activations(batch * cols, 950 + i)
        mats.append((w, x, rows, cols, batch, weights_buffer(ctx, w, rows, cols, packed),
                     upload_new(ctx, x), ctx.buffer(batch * rows * 4)))
    launches = ctx.kernel_launches()
    runs = []
    for _ in range(3):   # again and again: each launch finds the counters as the last left them
        for m in mats:
            m[7].zero(0, m[4] * m[2] * 4)
        ctx.begin_group()
        for w, x, rows, cols, batch, wb, xb, yb in mats:
            ctx.q8_0_gemm_mma(wb, xb, yb, rows, cols, batch, 0, 0)
        ctx.end_group()
        ctx.fence()
        runs.append([m[7].download_f32(0, m[4] * m[2]).copy() for m in mats])
    if packed:
        assert H.gemm_mma_launch_tile(shapes) == 128
        assert ctx.kernel_launches() == launches + 3 * 2  # split the inputs, multiply
    for i, (w, x, rows, cols, batch, wb, xb, yb) in enumerate(mats):
        assert np.array_equal(bits(runs[0][i]), bits(runs[1][i])), f"product {i}"
        assert np.array_equal(bits(runs[0][i]), bits(runs[2][i])), f"product {i}"
        want = O.gemm_q8_0_f32(w, rows, cols, x, batch, threads=8)
        assert norm_err(runs[0][i].reshape(batch, rows), want) <= 1e-5, f"product {i}"
        if not packed:  # the f32 kernels: same bits as the product alone (each has too
            # many output tiles alone to share them between workgroups)
            alone = run_gemm(ctx, ctx.q8_0_gemm_mma, wb, x, rows, cols, batch)
            assert np.array_equal(bits(runs[0][i]), bits(alone)), f"product {i}"
    for m in mats:
        for b in m[5:]:
            b.free()
