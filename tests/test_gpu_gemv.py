"""GPU parity: the Q8_0 decode GEMV against the CPU oracle.

Follows the reference's operator tests for this kernel
(crates/metal/src/tests.rs:310-406) and adds the benchmark's Gaussian data
under the 1e-5 normalised-error bar.
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


@pytest.mark.parametrize("packed", [False, True])
def test_gemv_minimal_ones_case(ctx, packed):
    # crates/metal/src/tests.rs:310-330: d = 1, q = 1, x = 2 -> exactly 64
    w = np.frombuffer(O.f32_to_f16_bits(1.0).to_bytes(2, "little") + bytes([1] * 32), np.uint8)
    wb = weights_buffer(ctx, w, 1, 32, packed)
    y = gemv(ctx, wb, np.full(32, 2.0, np.float32), 1, 32)
    assert y[0] == 64.0


REAL_SHAPES = [(1, 32, 1), (3, 32, 2), (17, 64, 3), (1024, 1024, 4), (2048, 1024, 5),
               (3072, 1024, 6), (151_936, 1024, 7)]


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("rows,cols,seed", REAL_SHAPES)
def test_gemv_matches_the_scalar_reference_across_real_shapes(ctx, rows, cols, seed, packed):
    # crates/metal/src/tests.rs:333-383, tolerance 1e-4 * max(|cpu|_inf, 1),
    # checked here on every row and against both CPU summation orders.
    w = O.boundary_weights(rows, cols, seed)
    x = O.boundary_input(cols, seed ^ 0x9E37)
    wb = weights_buffer(ctx, w, rows, cols, packed)
    got = gemv(ctx, wb, x, rows, cols)
    cpu = O.gemv_q8_0_f32(w, rows, cols, x, threads=8)
    scale = ref_scale(cpu)
    assert np.max(np.abs(got - cpu)) <= 1e-4 * scale
    if rows <= 4096:
        cpu2 = O.gemv_q8_0_f32_dequant_first(w, rows, cols, x)
        assert np.max(np.abs(got - cpu2)) <= 1e-4 * ref_scale(cpu2)
    wb.free()


def test_raw_and_packed_layouts_give_identical_bits(ctx):
    # (rows of whole 1024-column chunks stream through LDS in the raw layout: tiles whose
    # last pass is short, one to six chunks per row)
    for rows, cols, seed in [(17, 64, 3), (1024, 1024, 4), (300, 1152, 9), (77, 6912, 10),
                             (64, 2016, 11), (259, 1024, 12), (1021, 2048, 13), (13, 3072, 14),
                             (4100, 1024, 15), (530, 6144, 16),
                             # 1152 and 6912 columns: tails that stream too (rows of 1224 bytes
                             # staged whole, odd and even numbers of rows in the last pass)
                             (1, 1152, 17), (7, 1152, 18), (301, 1152, 19), (1030, 1152, 20),
                             (13, 6912, 21), (260, 6912, 22),
                             # full-height tiles of 1152 columns (a tile is a single step), ragged end
                             (9001, 1152, 25),
                             # whole chunks in front of a 128-column tail (pipelined), other tails
                             (40, 2176, 23), (9000, 3200, 26), (24, 1792, 24)]:
        w = O.boundary_weights(rows, cols, seed)
        x = O.boundary_input(cols, seed + 100)
        a = gemv(ctx, weights_buffer(ctx, w, rows, cols, False), x, rows, cols)
        b = gemv(ctx, weights_buffer(ctx, w, rows, cols, True), x, rows, cols)
        assert np.array_equal(bits(a), bits(b))


def test_rows_of_1152_columns_beside_longer_rows_with_the_same_tail(ctx):
    """Alone, products of 1152 columns run tiles of a single step; in a launch with a
    product whose rows have more whole chunks in front of the 128-column tail (3200
    columns) they take the pipelined form like it. Same bits either way, and the
    oracle's within 1e-5."""
    shapes = [(9000, 1152), (2000, 3200), (300, 1152), (1152, 6912)]
    ws = [S.make_weights(r, c, 40 + i) for i, (r, c) in enumerate(shapes)]
    xs = [S.make_activations(c, 50 + i) for i, (r, c) in enumerate(shapes)]
    wbs = [weights_buffer(ctx, w, r, c, True) for w, (r, c) in zip(ws, shapes)]
    alone = [gemv(ctx, wb, x, r, c) for wb, x, (r, c) in zip(wbs, xs, shapes)]
    for picked in ([0, 1, 2, 3], [0, 2], [0, 2, 3]):
        xbs = [upload_new(ctx, xs[i]) for i in picked]
        ybs = [ctx.buffer(shapes[i][0] * 4) for i in picked]
        launches = ctx.kernel_launches()
        ctx.begin_group()
        for i, xb, yb in zip(picked, xbs, ybs):
            ctx.q8_0_gemv(wbs[i], xb, yb, *shapes[i])
        ctx.end_group()
        ctx.fence()
        assert ctx.kernel_launches() == launches + 1
        for i, yb in zip(picked, ybs):
            assert np.array_equal(bits(yb.download_f32(0, shapes[i][0])), bits(alone[i])), (picked, i)
        for b in xbs + ybs:
            b.free()
    for w, x, got, (r, c) in zip(ws, xs, alone, shapes):
        assert norm_err(got, O.gemv_q8_0_f32(w, r, c, x)) <= 1e-5


@pytest.mark.parametrize("packed", [False, True])
def test_config0_gate_proj_gaussian_within_1e5(ctx, packed):
    # BASELINE config 0: W [3072, 1024] from N(0, 0.02), x ~ N(0, 1), seed 0.
    rows, cols = 3072, 1024
    w = S.make_weights(rows, cols, S.tensor_seed(0, 0, "gate"))
    x = S.make_activations(cols, 0)
    got = gemv(ctx, weights_buffer(ctx, w, rows, cols, packed), x, rows, cols)
    want = O.gemv_q8_0_f32(w, rows, cols, x)
    assert norm_err(got, want) <= 1e-5
    exact = O.gemv_q8_0_f64(w, rows, cols, x)
    # both are roundings of the same exact sum; the GPU must not be further
    # from it than a few times the oracle's own rounding error
    e_gpu = np.max(np.abs(got - exact)) / np.max(np.abs(exact))
    e_cpu = np.max(np.abs(want - exact)) / np.max(np.abs(exact))
    assert e_gpu <= max(4 * e_cpu, 2e-6)


@pytest.mark.parametrize("rows,cols", [(5, 32), (9, 64), (33, 96), (40, 160), (7, 992), (12, 1056),
                                       (31, 1152), (6, 2016), (10, 2048), (3, 3072 + 480),
                                       (2, 6912), (129, 6144)])
def test_every_column_tail_decomposition(ctx, rows, cols):
    # cols = 1024*a + {512,256,128,64,32} tails: each chunk width is exercised,
    # on Gaussian data under the tight bar.
    w = S.make_weights(rows, cols, 1000 + cols)
    x = S.make_activations(cols, 2000 + cols)
    want = O.gemv_q8_0_f32(w, rows, cols, x)
    for packed in (False, True):
        got = gemv(ctx, weights_buffer(ctx, w, rows, cols, packed), x, rows, cols)
        assert norm_err(got, want) <= 1e-5, (rows, cols, packed)


def test_zero_weights_and_zero_x_give_exact_zero(ctx):
    rows, cols = 16, 128
    wz = np.zeros(S.q8_0_bytes(rows, cols), np.uint8)
    x = S.make_activations(cols, 1)
    assert not gemv(ctx, weights_buffer(ctx, wz, rows, cols, True), x, rows, cols).any()
    w = S.make_weights(rows, cols, 2)
    assert not gemv(ctx, weights_buffer(ctx, w, rows, cols, True), np.zeros(cols, np.float32),
                    rows, cols).any()


def test_unaligned_activation_offsets_through_gemm_batch_one(ctx):
    # x_off / y_off are element offsets; odd values break 16-byte alignment.
    rows, cols = 50, 1152
    w = S.make_weights(rows, cols, 5)
    x = S.make_activations(cols, 6)
    want = O.gemv_q8_0_f32(w, rows, cols, x)
    wb = weights_buffer(ctx, w, rows, cols, True)
    ref = gemv(ctx, wb, x, rows, cols)
    for x_off, y_off in [(1, 3), (2, 1), (4, 0), (7, 5)]:
        xs = np.zeros(x_off + cols, np.float32)
        xs[x_off:] = x
        xb = upload_new(ctx, xs)
        yb = ctx.buffer((y_off + rows) * 4)
        ctx.q8_0_gemm(wb, xb, yb, rows, cols, 1, x_off, y_off)
        ctx.fence()
        out = yb.download_f32(0, y_off + rows)
        assert not out[:y_off].any()
        assert np.array_equal(bits(out[y_off:]), bits(ref))
    assert norm_err(ref, want) <= 1e-5


def test_gemv_rejects_malformed_arguments(ctx):
    # crates/metal/src/tests.rs:386-406
    wb = ctx.buffer(2 * 34)
    xb = ctx.buffer(32 * 4)
    yb = ctx.buffer(4)
    with pytest.raises(H.TuckmillError):
        ctx.q8_0_gemv(wb, xb, yb, 2, 30)
    with pytest.raises(H.TuckmillError):
        ctx.q8_0_gemv(wb, xb, yb, 0, 32)
    with pytest.raises(H.TuckmillError) as e:
        ctx.q8_0_gemv(wb, xb, yb, 2, 32)
    assert e.value.code == "InvalidRequest" and e.value.abi_code == H.TM_HIP_ERR_BOUNDS
    big_w = ctx.buffer(34)
    big_y = ctx.buffer(8)
    with pytest.raises(H.TuckmillError):
        ctx.q8_0_gemv(big_w, xb, big_y, 2, 32)
    with pytest.raises(H.TuckmillError):
        ctx.buffer(0)
    # nothing was dispatched by the refused calls
    before = ctx.committed_dispatches()
    with pytest.raises(H.TuckmillError):
        ctx.q8_0_gemv(wb, xb, yb, 1, 0)
    assert ctx.committed_dispatches() == before
