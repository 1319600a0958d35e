"""GPU parity: the int8-activation profile (device activation quantizer and
int8 x int8 -> i32 MFMA block dots) against the CPU oracle's
quantize_row_q8_0 / dot_q8_0_q8_0 (crates/tuckcore/src/tensor.rs:184-206,
crates/tuckcore/src/kernels.rs:206-221).

Bar: quantized activations bit-exact, every i32 block dot bit-exact, and the
f32 result bit-exact as well (the kernel keeps the reference's unfused
multiply, multiply, add in block order).
"""
import numpy as np
import pytest

import oracle as O
from tuckmill_amd import hip as H
from tuckmill_amd import synth as S

from q8util import bits, require_gpu, upload_new, weights_buffer

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = require_gpu()
    yield c
    c.close()


def quantize_on_gpu(ctx, x, cols, batch, x_off=0):
    xs = np.zeros(x_off + batch * cols, np.float32)
    xs[x_off:] = x
    xb = upload_new(ctx, xs)
    xq = ctx.buffer(H.xq_bytes(cols, batch))
    ctx.q8_0_quantize_act(xb, xq, cols, batch, x_off)
    ctx.fence()
    qs, ds = H.xq_split(xq.download(0, H.xq_bytes(cols, batch)), cols, batch)
    return xq, qs, ds


def test_activation_quantizer_known_answer(ctx):
    # crates/tuckcore/src/tensor.rs:373-392
    x = np.zeros(32, np.float32)
    x[0], x[1], x[2] = 127.0, -63.5, 1.0
    _, qs, ds = quantize_on_gpu(ctx, x, 32, 1)
    assert ds[0, 0] == 1.0
    assert qs[0, 0, 0] == 127 and qs[0, 0, 1] == -64 and qs[0, 0, 2] == 1 and qs[0, 0, 3] == 0


@pytest.mark.parametrize("cols,batch,scale", [(32, 1, 1.0), (1024, 7, 1.0), (1152, 33, 0.02),
                                              (2048, 64, 37.5), (96, 5, 1e-6), (64, 3, 6e4)])
def test_activation_quantizer_is_bit_exact(ctx, cols, batch, scale):
    x = (S.make_activations(cols * batch, cols + batch) * np.float32(scale)).astype(np.float32)
    x[:32] = 0.0  # an all-zero block
    if x.size >= 96:
        x[40], x[70] = np.nan, np.inf
    _, qs, ds = quantize_on_gpu(ctx, x, cols, batch, x_off=4)
    want_q, want_d = O.quantize_row_q8_0(x)
    assert np.array_equal(qs.reshape(-1, 32), want_q)
    assert np.array_equal(bits(ds.reshape(-1)), bits(want_d))


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("rows,cols,batch", [(16, 32, 1), (40, 64, 3), (100, 96, 77),
                                             (1024, 1024, 16), (333, 1152, 40), (2048, 2048, 8),
                                             (70, 1024, 17), (48, 160, 33), (65, 2048, 130),
                                             # decode-sized batches: the streaming kernel
                                             (4099, 2048, 1), (33, 6144, 2), (520, 1152, 4),
                                             (41, 6912, 5), (1000, 3072, 8), (9, 2016, 7),
                                             (64, 1056, 6), (17000, 1024, 2)])
def test_gemm_i8_block_dots_and_result_are_bit_exact(ctx, rows, cols, batch, packed):
    blocks = cols // 32
    w = S.make_weights(rows, cols, rows + cols)
    if rows >= 40:  # extremes: q_w = -128 against q_x = +-127
        wv = w.reshape(rows * blocks, 34)
        wv[0, 2:] = 0x80
        wv[blocks, 2:] = 0x80
    x = S.make_activations(cols * batch, batch)
    x[:32] = 5.0
    if batch > 1:
        x[cols:cols + 32] = -5.0
    wb = weights_buffer(ctx, w, rows, cols, packed)
    xq, qs, ds = quantize_on_gpu(ctx, x, cols, batch)
    yb = ctx.buffer((3 + batch * rows) * 4)
    sb = ctx.buffer(batch * rows * blocks * 4)
    ctx.q8_0_gemm_i8(wb, xq, yb, rows, cols, batch, 3, sb)
    ctx.fence()
    out = yb.download_f32(0, 3 + batch * rows)
    assert not out[:3].any()
    got = out[3:].reshape(batch, rows)
    sumi = sb.download(0, batch * rows * blocks * 4).view(np.int32).reshape(batch, rows, blocks)
    want = O.gemm_q8_0_q8_0(w, rows, cols, x, batch, threads=8)
    assert np.array_equal(bits(got), bits(want))
    row_bytes = blocks * 34
    wq = w.reshape(rows, blocks, 34)[:, :, 2:].view(np.int8).astype(np.int64)
    for b in range(batch):
        brute = np.einsum("rkl,kl->rk", wq, qs[b].astype(np.int64))
        assert np.array_equal(sumi[b].astype(np.int64), brute)
        if b == 0:
            for r in (0, rows - 1):
                one = O.block_sumi(w[r * row_bytes:(r + 1) * row_bytes], qs[b])
                assert np.array_equal(sumi[b, r], one)
    if rows >= 40:
        assert sumi[0, 0, 0] == -128 * 127 * 32
    # without the verification output
    ctx.q8_0_gemm_i8(wb, xq, yb, rows, cols, batch, 3)
    ctx.fence()
    assert np.array_equal(bits(yb.download_f32(3, batch * rows)), bits(want.reshape(-1)))


def test_i8_argument_refusals(ctx):
    b = ctx.buffer(4096)
    with pytest.raises(H.TuckmillError):
        ctx.q8_0_quantize_act(b, b, 48, 1, 0)
    with pytest.raises(H.TuckmillError):
        ctx.q8_0_quantize_act(b, b, 32, H.GEMM_I8_MAX_BATCH + 1, 0)
    with pytest.raises(H.TuckmillError) as e:
        ctx.q8_0_quantize_act(b, ctx.buffer(35), 32, 1, 0)
    assert e.value.abi_code == H.TM_HIP_ERR_BOUNDS
    with pytest.raises(H.TuckmillError):
        ctx.q8_0_gemm_i8(b, b, b, 0, 32, 1, 0)
    with pytest.raises(H.TuckmillError) as e:
        ctx.q8_0_gemm_i8(b, b, b, 4, 32, 1, 0, ctx.buffer(8))
    assert e.value.abi_code == H.TM_HIP_ERR_BOUNDS


def test_independent_i8_products_in_a_group_share_one_launch(ctx):
    cols, batch = 1024, 48
    x = S.make_activations(batch * cols, 3)
    xb = upload_new(ctx, x)
    xq = ctx.buffer(H.xq_bytes(cols, batch))
    mats = []
    for i, rows in enumerate((512, 256, 256)):
        w = S.make_weights(rows, cols, 70 + i)
        mats.append((w, rows, weights_buffer(ctx, w, rows, cols, True), ctx.buffer(batch * rows * 4)))
    launches = ctx.kernel_launches()
    ctx.begin_group()
    ctx.q8_0_quantize_act(xb, xq, cols, batch)
    for w, rows, wb, yb in mats:
        ctx.q8_0_gemm_i8(wb, xq, yb, rows, cols, batch)
    ctx.end_group()
    assert ctx.kernel_launches() == launches + 2  # the quantizer, then one list launch
    ctx.fence()
    for w, rows, wb, yb in mats:
        want = O.gemm_q8_0_q8_0(w, rows, cols, x, batch, threads=4)
        assert np.array_equal(bits(yb.download_f32(0, batch * rows)), bits(want.reshape(-1)))


@pytest.mark.parametrize("rows,cols,batch", [(128, 1024, 64), (129, 2048, 65), (300, 1152, 200),
                                             (64, 96, 77), (1000, 64, 512), (257, 6144, 129),
                                             (70, 32, 64), (513, 3072, 300),
                                             # one to three token tiles of 16
                                             (300, 1152, 5), (65, 96, 16), (129, 2080, 9),
                                             (300, 1152, 17), (256, 2048, 32), (65, 96, 20),
                                             (100, 352, 48), (70, 1024, 33), (513, 160, 41),
                                             # several token tiles of equal height, and the
                                             # first batch of the 128-token shape
                                             (200, 1024, 96), (64, 1152, 256), (100, 1024, 257)])
def test_lds_staged_i8_gemm_is_bit_exact(ctx, rows, cols, batch):
    # Batches of five and more over sealed weights without the verification output
    # take the LDS-staged kernel: partial token and row tiles, K stages that end
    # inside the last stage, every workgroup shape.
    w = S.make_weights(rows, cols, 3 * rows + cols)
    x = S.make_activations(cols * batch, batch + 1)
    wb = weights_buffer(ctx, w, rows, cols, True)
    xq, qs, ds = quantize_on_gpu(ctx, x, cols, batch)
    yb = ctx.buffer((5 + batch * rows) * 4)
    ctx.q8_0_gemm_i8(wb, xq, yb, rows, cols, batch, 5)
    ctx.fence()
    out = yb.download_f32(0, 5 + batch * rows)
    assert not out[:5].any()
    want = O.gemm_q8_0_q8_0(w, rows, cols, x, batch, threads=8)
    assert np.array_equal(bits(out[5:]), bits(want.reshape(-1)))


@pytest.mark.parametrize("rows,cols,batch", [(300, 1152, 5), (129, 2080, 17), (100, 352, 48),
                                             (513, 160, 41), (200, 1024, 96), (64, 1152, 256),
                                             (257, 6144, 129), (513, 3072, 300), (1000, 64, 512),
                                             (6144, 2048, 512), (300, 1152, 3), (96, 1024, 1)])
def test_fused_tail_variant_is_within_tolerance_and_never_silent(ctx, rows, cols, batch):
    """tm_hip_q8_0_gemm_i8_fma: the same exact block dots, every term fused into
    the f32 sum. Within 1e-5 (normalised) of the CPU's dot_q8_0_q8_0 and of the
    bit-exact entry point; where the fused multiply-add rounds differently the
    bits differ, which is why it is an entry point of its own. Up to four tokens
    the bit-exact streaming kernel serves it."""
    w = S.make_weights(rows, cols, 7 * rows + cols)
    x = S.make_activations(cols * batch, batch + 3)
    wb = weights_buffer(ctx, w, rows, cols, True)
    xq, qs, ds = quantize_on_gpu(ctx, x, cols, batch)
    y_fma, y_exact = ctx.buffer((5 + batch * rows) * 4), ctx.buffer(batch * rows * 4)
    ctx.begin_group()  # both in one group: they never share a launch
    ctx.q8_0_gemm_i8_fma(wb, xq, y_fma, rows, cols, batch, 5)
    ctx.q8_0_gemm_i8(wb, xq, y_exact, rows, cols, batch, 0)
    ctx.end_group()
    ctx.fence()
    out = y_fma.download_f32(0, 5 + batch * rows)
    assert not out[:5].any()
    want = O.gemm_q8_0_q8_0(w, rows, cols, x, batch, threads=8).reshape(-1)
    exact = y_exact.download_f32(0, batch * rows)
    assert np.array_equal(bits(exact), bits(want))
    scale = float(np.max(np.abs(want)))
    assert float(np.max(np.abs(out[5:] - want))) / scale <= 1e-5
    if batch <= 4:
        assert np.array_equal(bits(out[5:]), bits(want))
    for b in (wb, xq, y_fma, y_exact):
        b.free()


def test_matrix_takes_the_fused_tail_only_when_asked(ctx):
    rows, cols, batch = 512, 2048, 64
    w = S.make_weights(rows, cols, 11)
    x = S.make_activations(cols * batch, 12)
    xb = upload_new(ctx, x)
    want = O.gemm_q8_0_q8_0(w, rows, cols, x, batch, threads=8)
    outs = {}
    for fused in (False, True):
        m = H.Matrix.load(ctx, w, cols, rows, profile=H.NumericalProfile.LLAMA_CPU,
                          fused_i8_tail=fused)
        yb = ctx.buffer(batch * rows * 4)
        m.gemm(ctx, xb, yb, batch, exact=False)
        ctx.fence()
        outs[fused] = yb.download_f32(0, batch * rows).reshape(batch, rows)
        m.buf.free()
        yb.free()
    assert np.array_equal(bits(outs[False]), bits(want)), "the default keeps the CPU's bits"
    assert float(np.max(np.abs(outs[True] - want))) / float(np.max(np.abs(want))) <= 1e-5
    with pytest.raises(H.TuckmillError) as e:
        H.Matrix.load(ctx, w, cols, rows, fused_i8_tail=True)  # oracle-f32 has no int8 tail
    assert e.value.code == "InvalidRequest"
    xb.free()
