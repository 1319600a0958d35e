"""Recorded dispatch groups: a step replays with the bits the committed group
gives, on whatever the buffers hold at the time of the replay.

The reference re-encodes a token's operators for every token
(crates/tuckcore/src/qwen35_gpu.rs:66-85); the recorded step is the same group
kept as a HIP graph. Every replay is checked against the eager group, with
eager work and synchronizations between replays.
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


class Layer:
    """One transformer layer's products around a residual stream `h`, then a
    vocabulary projection and argmax (attention itself left out)."""

    def __init__(self, ctx, hidden=1024, qdim=2048, kvdim=1024, ffn=3072, vocab=4096, seed=300):
        self.ctx, self.hidden, self.qdim, self.kvdim, self.ffn, self.vocab = (
            ctx, hidden, qdim, kvdim, ffn, vocab)

        def mat(rows, cols, s):
            return weights_buffer(ctx, S.make_weights(rows, cols, seed + s), rows, cols, True)

        def vec(n, s):
            return upload_new(ctx, (0.5 + np.abs(S.make_activations(n, seed + s))).astype(np.float32))

        self.wq, self.wk, self.wv = mat(qdim, hidden, 1), mat(kvdim, hidden, 2), mat(kvdim, hidden, 3)
        self.wo, self.wg, self.wu = mat(hidden, qdim, 4), mat(ffn, hidden, 5), mat(ffn, hidden, 6)
        self.wd, self.wl = mat(hidden, ffn, 7), mat(vocab, hidden, 8)
        self.g1, self.g2, self.g3 = vec(hidden, 9), vec(hidden, 10), vec(hidden, 11)
        f32 = lambda n: ctx.buffer(n * 4)  # noqa: E731
        self.h, self.n, self.q, self.k, self.v = f32(hidden), f32(hidden), f32(qdim), f32(kvdim), f32(kvdim)
        self.t, self.gate, self.up, self.logits = f32(hidden), f32(ffn), f32(ffn), f32(vocab)
        self.partial, self.token = ctx.buffer(H.ARGMAX_PARTIAL_BYTES), ctx.buffer(4)

    def encode(self):
        c = self.ctx
        c.rmsnorm(self.h, self.g1, self.n, 1, self.hidden, 1e-6)
        c.q8_0_gemv(self.wq, self.n, self.q, self.qdim, self.hidden)
        c.q8_0_gemv(self.wk, self.n, self.k, self.kvdim, self.hidden)
        c.q8_0_gemv(self.wv, self.n, self.v, self.kvdim, self.hidden)
        c.q8_0_gemv(self.wo, self.q, self.t, self.hidden, self.qdim)
        c.f32_axpy(self.t, self.h, 1.0, self.hidden)
        c.rmsnorm(self.h, self.g2, self.n, 1, self.hidden, 1e-6)
        c.q8_0_gemv(self.wg, self.n, self.gate, self.ffn, self.hidden)
        c.q8_0_gemv(self.wu, self.n, self.up, self.ffn, self.hidden)
        c.silu_mul(self.gate, self.up, self.gate, self.ffn)
        c.q8_0_gemv(self.wd, self.gate, self.t, self.hidden, self.ffn)
        c.f32_axpy(self.t, self.h, 1.0, self.hidden)
        c.rmsnorm(self.h, self.g3, self.n, 1, self.hidden, 1e-6)
        c.q8_0_gemv(self.wl, self.n, self.logits, self.vocab, self.hidden)
        c.argmax_f32(self.logits, self.vocab, self.partial, self.token, 0)

    def outputs(self):
        return (bits(self.h.download_f32(0, self.hidden)).copy(),
                bits(self.k.download_f32(0, self.kvdim)).copy(),
                bits(self.logits.download_f32(0, self.vocab)).copy(),
                int(self.token.download(0, 4).view(np.uint32)[0]))


def same(a, b):
    return all(np.array_equal(x, y) for x, y in zip(a[:3], b[:3])) and a[3] == b[3]


def test_a_recorded_layer_replays_with_the_bits_of_the_committed_group(ctx):
    layer = Layer(ctx)
    other_w = weights_buffer(ctx, S.make_weights(512, 1024, 5), 512, 1024, True)
    other_x, other_y = upload_new(ctx, S.make_activations(1024, 6)), ctx.buffer(512 * 4)

    commits, launches = ctx.committed_dispatches(), ctx.kernel_launches()
    ctx.begin_group()
    layer.encode()
    step = ctx.end_group_recorded()
    # recording runs nothing and commits nothing
    assert ctx.committed_dispatches() == commits and ctx.kernel_launches() == launches
    ctx.fence()
    assert not np.any(layer.logits.download_f32(0, layer.vocab))
    assert 0 < step.launches < 15

    for replay in range(4):
        x = S.make_activations(layer.hidden, 400 + replay)
        layer.h.upload(0, x)
        ctx.begin_group()
        layer.encode()
        ctx.end_group()
        ctx.fence()
        want = layer.outputs()
        # the layer computed something that depends on this replay's input
        logits = want[2].view(np.float32)
        assert np.all(np.isfinite(logits)) and want[3] == O.argmax(logits)

        layer.h.upload(0, x)
        layer.logits.zero(0, layer.vocab * 4)
        commits, launches = ctx.committed_dispatches(), ctx.kernel_launches()
        step.run()
        assert ctx.committed_dispatches() == commits + 1
        assert ctx.kernel_launches() == launches + step.launches
        # unrelated eager work and a synchronization between replays
        ctx.q8_0_gemv(other_w, other_x, other_y, 512, 1024)
        ctx.fence()
        assert same(layer.outputs(), want), f"replay {replay}"

    # two replays back to back without a fence: the residual stream carries over
    x = S.make_activations(layer.hidden, 500)
    layer.h.upload(0, x)
    for _ in range(2):
        ctx.begin_group()
        layer.encode()
        ctx.end_group()
    ctx.fence()
    want = layer.outputs()
    layer.h.upload(0, x)
    step.run()
    step.run()
    ctx.fence()
    assert same(layer.outputs(), want)
    assert ctx.last_gpu_ms() > 0.0
    step.free()


def test_a_recorded_prefill_chunk_replays_every_product_kernel(ctx):
    # MFMA GEMM (persistent and one-tile forms), exact small-batch GEMM, and the
    # int8 profile (quantize + streaming kernel + LDS GEMM) under one recording.
    rows, cols = 1024, 2048
    w = weights_buffer(ctx, S.make_weights(rows, cols, 21), rows, cols, True)
    ys, calls = [], []
    for batch in (4, 64, 256):
        x = upload_new(ctx, S.make_activations(batch * cols, 30 + batch))
        y, y8 = ctx.buffer(batch * rows * 4), ctx.buffer(batch * rows * 4)
        xq = ctx.buffer(H.xq_bytes(cols, batch))
        ys += [(y, batch), (y8, batch)]
        calls.append((x, y, y8, xq, batch))

    # and an F16 matrix with its row lookup
    w16 = upload_new(ctx, (S.make_activations(96 * cols, 5) * np.float32(0.02)).astype(np.float16).view(np.uint8))
    y16, row16 = ctx.buffer(4 * 96 * 4), ctx.buffer(cols * 4)
    ys += [(y16, 4), (row16, 0)]

    def encode():
        for x, y, y8, xq, batch in calls:
            if batch <= H.GEMM_MAX_BATCH:
                ctx.q8_0_gemm(w, x, y, rows, cols, batch)
            else:
                ctx.q8_0_gemm_mma(w, x, y, rows, cols, batch)
            ctx.q8_0_quantize_act(x, xq, cols, batch)
            ctx.q8_0_gemm_i8(w, xq, y8, rows, cols, batch)
        ctx.f16_gemm(w16, calls[0][0], y16, 96, cols, 4)
        ctx.f16_row(w16, row16, 7, cols, 0)

    def outputs():
        return [bits(b.download_f32(0, len(b) // 4)).copy() for b, n in ys]

    ctx.begin_group()
    encode()
    ctx.end_group()
    ctx.fence()
    want = outputs()
    assert all(np.any(o) for o in want)
    ctx.begin_group()
    encode()
    step = ctx.end_group_recorded()
    for replay in range(3):
        for b, n in ys:
            b.zero(0, len(b))
        step.run()
        ctx.fence()
        got = outputs()
        assert all(np.array_equal(g, o) for g, o in zip(got, want)), f"replay {replay}"
    step.free()


def test_a_step_keeps_its_buffers_alive(ctx):
    rows, cols = 512, 1024
    raw = S.make_weights(rows, cols, 61)
    x = S.make_activations(cols, 62)
    w, xb, yb = weights_buffer(ctx, raw, rows, cols, True), upload_new(ctx, x), ctx.buffer(rows * 4)
    ctx.begin_group()
    ctx.q8_0_gemv(w, xb, yb, rows, cols)
    step = ctx.end_group_recorded()
    w.free()  # the handle goes, the step's reference keeps the weights
    filler = [ctx.buffer(len(raw)) for _ in range(4)]  # would reuse the freed memory
    step.run()
    ctx.fence()
    got = yb.download_f32(0, rows)
    want = O.gemv_q8_0_f32(raw, rows, cols, x)
    assert np.max(np.abs(got - want)) <= 1e-5 * np.max(np.abs(want))
    step.free()
    del filler


def test_recording_refusals(ctx):
    with pytest.raises(H.TuckmillError) as e:
        ctx.end_group_recorded()
    assert e.value.abi_code == H.TM_HIP_ERR_UNSUPPORTED
    ctx.begin_group()
    with pytest.raises(H.TuckmillError):
        ctx.end_group_recorded()  # an empty group cannot be recorded
    with pytest.raises(H.TuckmillError):
        ctx.end_group()  # and the refusal closed it
    a, b = upload_new(ctx, np.ones(64, np.float32)), ctx.buffer(256)
    ctx.begin_group()
    ctx.f32_scale(a, b, 2.0, 64)
    step = ctx.end_group_recorded()
    ctx.begin_group()
    with pytest.raises(H.TuckmillError):
        step.run()  # not inside an open group
    ctx.abort_group()
    other = H.HipContext.open()
    try:
        foreign = H.HipStep(other._inner, other._lib, step.raw)
        with pytest.raises(H.TuckmillError):
            foreign.run()
        foreign.raw = None
    finally:
        other.close()
    step.run()
    ctx.fence()
    assert np.array_equal(b.download_f32(0, 64), np.full(64, 2.0, np.float32))
    step.free()
