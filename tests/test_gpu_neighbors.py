"""GPU parity of the small f32 operators either side of a product.

Follows crates/metal/src/tests.rs:585-654 (rmsnorm, silu_mul; the reference's
1e-5 * max(|want|, 1) tolerance) and :1250-1350 (argmax: exact, and the
indirect embedding lookup fed by it).
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


def grid_values(rng, n):
    # the value grid of crates/metal/src/tests.rs:591-593
    return np.array([((rng.next() % 20_001) - 10_000.0) / 1000.0 for _ in range(n)], np.float32)


def close(got, want):
    return np.all(np.abs(got - want) <= 1e-5 * np.maximum(np.abs(want), 1.0))


@pytest.mark.parametrize("rows,cols", [(1, 1024), (16, 128), (8, 128), (1, 7), (3, 1152), (2, 6912)])
def test_rmsnorm_matches_the_scalar_reference(ctx, rows, cols):
    rng = O.Rng(11 + rows + cols)
    x = grid_values(rng, rows * cols)
    w = np.array([0.5 + (rng.next() % 1000) / 1000.0 for _ in range(cols)], np.float32)
    eps = 1e-6
    xb, wb = upload_new(ctx, x), upload_new(ctx, w)
    yb = ctx.buffer(rows * cols * 4)
    ctx.rmsnorm(xb, wb, yb, rows, cols, eps)
    ctx.fence()
    got = yb.download_f32(0, rows * cols).reshape(rows, cols)
    for r in range(rows):
        assert close(got[r], O.rmsnorm(x[r * cols:(r + 1) * cols], w, eps)), f"row {r}"
    # in place
    ctx.rmsnorm(xb, wb, xb, rows, cols, eps)
    ctx.fence()
    assert np.array_equal(bits(xb.download_f32(0, rows * cols)), bits(got.reshape(-1)))


@pytest.mark.parametrize("n", [3072, 3071, 1, 6912 * 3 + 5])
def test_gated_activations_match_the_scalar_reference(ctx, n):
    rng = O.Rng(19 + n)
    gate, up = grid_values(rng, n), grid_values(rng, n)
    gb, ub = upload_new(ctx, gate), upload_new(ctx, up)
    ob = ctx.buffer(n * 4)
    ctx.silu_mul(gb, ub, ob, n)
    ctx.fence()
    assert close(ob.download_f32(0, n), O.silu_mul(gate, up))
    ctx.gelu_tanh_mul(gb, ub, ob, n)
    ctx.fence()
    assert close(ob.download_f32(0, n), O.gelu_tanh_mul(gate, up))
    # the engine's use: the result overwrites the gate (engine/metal.rs:492)
    ctx.gelu_tanh_mul(gb, ub, gb, n)
    ctx.fence()
    assert close(gb.download_f32(0, n), O.gelu_tanh_mul(gate, up))


@pytest.mark.parametrize("n", [1, 255, 1024, 100_003])
def test_axpy_and_scale_are_bit_exact(ctx, n):
    a = S.make_activations(n, 5)
    y = S.make_activations(n, 6)
    ab, yb = upload_new(ctx, a), upload_new(ctx, y)
    ctx.f32_axpy(ab, yb, 0.37, n)
    ctx.fence()
    assert np.array_equal(bits(yb.download_f32(0, n)), bits(O.axpy(a, 0.37, y)))
    sb = ctx.buffer(n * 4)
    ctx.f32_scale(ab, sb, -1.25e-3, n)
    ctx.fence()
    assert np.array_equal(bits(sb.download_f32(0, n)), bits(O.scale(a, -1.25e-3)))


def test_argmax_matches_the_cpu_greedy_rule_exactly(ctx):
    # crates/metal/src/tests.rs:1250-1320
    nan, inf = np.nan, np.inf
    cases = [np.array(c, np.float32) for c in (
        [1.0, 3.0, 2.0], [3.0, 3.0], [nan, 1.0], [nan, inf], [nan, nan, nan], [-inf, -inf],
        [-0.0, 0.0], [0.0, -0.0], [7.5])]
    rng = O.Rng(0xA11CE)
    n = 248_320
    big = np.array([((rng.next() >> 40) / float(1 << 24)) * 20.0 - 10.0 for _ in range(n)],
                   np.float32)
    for k in (200_000, 77_777, 131_071, 77_776):
        big[k] = 42.0
    big[5] = nan
    cases.append(big)
    for ln in (255, 256, 16_384, 16_385, 70_001):
        v = np.ones(ln, np.float32)
        v[ln - 1] = 2.0
        v[ln // 2] = 2.0
        cases.append(v)
    for ln in (5, 6, 7, 70_003):  # the only maximum among the last n % 4 elements
        v = np.ones(ln, np.float32)
        v[ln - 1] = 3.0
        cases.append(v)
    partial = ctx.buffer(H.ARGMAX_PARTIAL_BYTES)
    out = ctx.buffer(8)
    for c, x in enumerate(cases):
        xb = upload_new(ctx, x)
        ctx.argmax_f32(xb, x.size, partial, out, 1)
        ctx.fence()
        got = int(out.download(4, 4).view(np.uint32)[0])
        assert got == O.argmax(x), f"case {c} (len {x.size})"
        xb.free()
    empty = ctx.buffer(4)
    with pytest.raises(H.TuckmillError) as e:
        ctx.argmax_f32(empty, 0, partial, out, 0)
    assert e.value.abi_code == H.TM_HIP_ERR_BOUNDS
    with pytest.raises(H.TuckmillError):
        ctx.argmax_f32(empty, 1, partial, out, 2)  # out_index past the buffer
    with pytest.raises(H.TuckmillError):
        ctx.argmax_f32(empty, 1, ctx.buffer(256), out, 0)  # partial too small


def test_a_decode_tail_runs_in_one_group(ctx):
    # norm -> lm_head GEMV -> argmax -> embedding row of the chosen token, one
    # commit (the shape of crates/tuckcore/src/engine/metal.rs decode tail).
    rows, cols = 4096, 1024
    w = S.make_weights(rows, cols, 77)
    x = S.make_activations(cols, 78)
    g = (0.5 + np.abs(S.make_activations(cols, 79))).astype(np.float32)
    wb = weights_buffer(ctx, w, rows, cols, True)
    xb, gb = upload_new(ctx, x), upload_new(ctx, g)
    hb, yb = ctx.buffer(cols * 4), ctx.buffer(rows * 4)
    partial, ids, emb = ctx.buffer(H.ARGMAX_PARTIAL_BYTES), ctx.buffer(8), ctx.buffer(cols * 4)
    commits = ctx.committed_dispatches()
    ctx.begin_group()
    ctx.rmsnorm(xb, gb, hb, 1, cols, 1e-6)
    ctx.q8_0_gemv(wb, hb, yb, rows, cols)
    ctx.argmax_f32(yb, rows, partial, ids, 0)
    ctx.row_indirect_f32(wb, 8, rows, cols, ids, 0, emb)
    ctx.end_group()
    assert ctx.committed_dispatches() == commits + 1
    ctx.fence()
    h = hb.download_f32(0, cols)
    assert close(h, O.rmsnorm(x, g, 1e-6))
    logits = yb.download_f32(0, rows)
    want_logits = O.gemv_q8_0_f32(w, rows, cols, h)
    assert np.max(np.abs(logits - want_logits)) <= 1e-5 * np.max(np.abs(want_logits))
    token = int(ids.download(0, 4).view(np.uint32)[0])
    assert token == O.argmax(logits)
    row_bytes = (cols // 32) * 34
    want_row = O.dequant_q8_0(w[token * row_bytes:(token + 1) * row_bytes])
    assert np.array_equal(bits(emb.download_f32(0, cols)), bits(want_row))


def test_neighbor_argument_refusals(ctx):
    b = ctx.buffer(64)
    small = ctx.buffer(8)
    for call in (lambda: ctx.silu_mul(b, b, b, 0), lambda: ctx.f32_axpy(b, b, 1.0, 0),
                 lambda: ctx.gelu_tanh_mul(b, small, b, 16), lambda: ctx.f32_scale(b, small, 1.0, 16)):
        with pytest.raises(H.TuckmillError) as e:
            call()
        assert e.value.abi_code == H.TM_HIP_ERR_BOUNDS
    with pytest.raises(H.TuckmillError) as e:
        ctx.rmsnorm(b, b, b, 0, 16, 1e-6)
    assert e.value.abi_code == H.TM_HIP_ERR_UNSUPPORTED
    with pytest.raises(H.TuckmillError) as e:
        ctx.rmsnorm(b, small, b, 1, 16, 1e-6)  # weight shorter than cols
    assert e.value.abi_code == H.TM_HIP_ERR_BOUNDS


@pytest.mark.parametrize("packed", [True, False])
def test_residual_update_behind_its_product_shares_the_launch(ctx, packed):
    # o-projection followed by h += t, as in every layer of a decode step: inside
    # a group the update rides in the product's epilogue (one launch instead of
    # two) and must give the bits of the two separate operators.
    rows, cols = 1024, 2048
    w = S.make_weights(rows, cols, 91)
    x = S.make_activations(cols, 92)
    h0 = S.make_activations(rows, 93)
    wb = weights_buffer(ctx, w, rows, cols, packed)
    xb = upload_new(ctx, x)
    results = []
    for grouped in (False, True):
        hb, tb = upload_new(ctx, h0), ctx.buffer(rows * 4)
        launches = ctx.kernel_launches()
        if grouped:
            ctx.begin_group()
        ctx.q8_0_gemv(wb, xb, tb, rows, cols)
        ctx.f32_axpy(tb, hb, 0.5, rows)
        if grouped:
            ctx.end_group()
        ctx.fence()
        assert ctx.kernel_launches() - launches == (1 if grouped else 2)
        results.append((tb.download_f32(0, rows).copy(), hb.download_f32(0, rows).copy()))
    assert np.array_equal(bits(results[0][0]), bits(results[1][0]))
    assert np.array_equal(bits(results[0][1]), bits(results[1][1]))
    t = O.gemv_q8_0_f32(w, rows, cols, x)
    assert np.max(np.abs(results[1][0] - t)) <= 1e-5 * np.max(np.abs(t))
    assert np.array_equal(bits(results[1][1]), bits(O.axpy(results[1][0], 0.5, h0)))


@pytest.mark.parametrize("packed", [True, False])
@pytest.mark.parametrize("batch,rows", [(5, 1024), (8, 1024), (20, 1024), (32, 1024), (2, 2048),
                                        (4, 1536)])
def test_residual_update_behind_a_small_batch_product_shares_the_launch(ctx, packed, batch, rows):
    # the same behind the exact small-batch product at more tokens than the one-token
    # kernel takes: the token-split kernel has the same epilogue (20 tokens: two
    # descriptors of up to 16, each updating its own rows of h; 2 and 4 tokens over
    # enough rows stay on that kernel as well)
    cols = 2048
    w = S.make_weights(rows, cols, 96)
    x = S.make_activations(batch * cols, 97)
    h0 = S.make_activations(batch * rows, 98)
    wb = weights_buffer(ctx, w, rows, cols, packed)
    xb = upload_new(ctx, x)
    results = []
    for grouped in (False, True):
        hb, tb = upload_new(ctx, h0), ctx.buffer(batch * rows * 4)
        launches = ctx.kernel_launches()
        if grouped:
            ctx.begin_group()
        ctx.q8_0_gemm(wb, xb, tb, rows, cols, batch)
        ctx.f32_axpy(tb, hb, -0.25, batch * rows)
        if grouped:
            ctx.end_group()
        ctx.fence()
        assert ctx.kernel_launches() - launches == (1 if grouped else 2)
        results.append((tb.download_f32(0, batch * rows).copy(),
                        hb.download_f32(0, batch * rows).copy()))
    assert np.array_equal(bits(results[0][0]), bits(results[1][0]))
    assert np.array_equal(bits(results[0][1]), bits(results[1][1]))
    assert np.array_equal(bits(results[1][1]), bits(O.axpy(results[1][0], -0.25, h0)))
    t0 = O.gemv_q8_0_f32(w, rows, cols, x[:cols])
    assert np.max(np.abs(results[1][0][:rows] - t0)) <= 1e-5 * np.max(np.abs(t0))


def test_residual_update_is_not_fused_when_it_would_reorder_accesses(ctx):
    # h is also the product's input: the update must wait for the whole product.
    rows = cols = 1024
    w = S.make_weights(rows, cols, 94)
    h0 = S.make_activations(cols, 95)
    wb = weights_buffer(ctx, w, rows, cols, True)
    hb, tb = upload_new(ctx, h0), ctx.buffer(rows * 4)
    launches = ctx.kernel_launches()
    ctx.begin_group()
    ctx.q8_0_gemv(wb, hb, tb, rows, cols)
    ctx.f32_axpy(tb, hb, 1.0, rows)
    ctx.end_group()
    ctx.fence()
    assert ctx.kernel_launches() - launches == 2
    t = tb.download_f32(0, rows)
    want_t = O.gemv_q8_0_f32(w, rows, cols, h0)
    assert np.max(np.abs(t - want_t)) <= 1e-5 * np.max(np.abs(want_t))
    assert np.array_equal(bits(hb.download_f32(0, rows)), bits(O.axpy(t, 1.0, h0)))


@pytest.mark.parametrize("hidden,qdim,kvdim,ffn", [(1024, 2048, 1024, 3072),     # Qwen3-0.6B
                                                   (1152, 1024, 256, 6912)])     # Gemma-3-1B
def test_rmsnorm_in_front_of_its_products_is_fused_into_their_launch(ctx, hidden, qdim, kvdim, ffn):
    # norm -> q, k, v (one launch) -> o with its residual update -> norm -> gate, up:
    # grouped, the norms ride in the launches of the products that read them and the
    # update in the epilogue of o; every buffer must hold the bits of the separate run.
    # (Gemma's hidden width leaves a column tail of 128 behind the 1024-column chunk.)
    mats = {}
    for i, (name, rows, cols) in enumerate([("q", qdim, hidden), ("k", kvdim, hidden),
                                            ("v", kvdim, hidden), ("o", hidden, qdim),
                                            ("gate", ffn, hidden), ("up", ffn, hidden)]):
        w = S.make_weights(rows, cols, 300 + i)
        mats[name] = (w, rows, cols, weights_buffer(ctx, w, rows, cols, True))
    h0 = S.make_activations(hidden, 310)
    g1 = (0.5 + np.abs(S.make_activations(hidden, 311))).astype(np.float32)
    g2 = (0.5 + np.abs(S.make_activations(hidden, 312))).astype(np.float32)
    attn = S.make_activations(qdim, 313)
    g1b, g2b, attnb = upload_new(ctx, g1), upload_new(ctx, g2), upload_new(ctx, attn)
    runs = []
    for grouped in (False, True):
        hb = upload_new(ctx, h0)
        nb, n2b, tb = ctx.buffer(hidden * 4), ctx.buffer(hidden * 4), ctx.buffer(hidden * 4)
        out = {k: ctx.buffer(mats[k][1] * 4) for k in ("q", "k", "v", "gate", "up")}
        launches = ctx.kernel_launches()
        if grouped:
            ctx.begin_group()
        ctx.rmsnorm(hb, g1b, nb, 1, hidden, 1e-6)
        for k in ("q", "k", "v"):
            ctx.q8_0_gemv(mats[k][3], nb, out[k], mats[k][1], hidden)
        ctx.q8_0_gemv(mats["o"][3], attnb, tb, hidden, qdim)
        ctx.f32_axpy(tb, hb, 1.0, hidden)
        ctx.rmsnorm(hb, g2b, n2b, 1, hidden, 1e-6)
        for k in ("gate", "up"):
            ctx.q8_0_gemv(mats[k][3], n2b, out[k], mats[k][1], hidden)
        if grouped:
            ctx.end_group()
        ctx.fence()
        used = ctx.kernel_launches() - launches
        # grouped: {norm, q, k, v} + {o with its update} + {norm, gate, up}
        assert used == (3 if grouped else 9), used
        got = {k: out[k].download_f32(0, mats[k][1]).copy() for k in out}
        got.update(n=nb.download_f32(0, hidden).copy(), n2=n2b.download_f32(0, hidden).copy(),
                   h=hb.download_f32(0, hidden).copy(), t=tb.download_f32(0, hidden).copy())
        runs.append(got)
    for k in runs[0]:
        assert np.array_equal(bits(runs[0][k]), bits(runs[1][k])), k
    n = O.rmsnorm(h0, g1, 1e-6)
    assert close(runs[1]["n"], n)
    q = O.gemv_q8_0_f32(mats["q"][0], qdim, hidden, runs[1]["n"])
    assert np.max(np.abs(runs[1]["q"] - q)) <= 1e-5 * np.max(np.abs(q))
    assert np.array_equal(bits(runs[1]["h"]), bits(O.axpy(runs[1]["t"], 1.0, h0)))
    assert close(runs[1]["n2"], O.rmsnorm(runs[1]["h"], g2, 1e-6))


def test_a_norm_nobody_reads_still_runs(ctx):
    hidden = 2048
    h = S.make_activations(hidden, 320)
    g = np.ones(hidden, np.float32)
    w = S.make_weights(64, hidden, 321)
    wb = weights_buffer(ctx, w, 64, hidden, True)
    hb, gb, nb, yb = upload_new(ctx, h), upload_new(ctx, g), ctx.buffer(hidden * 4), ctx.buffer(256)
    ctx.begin_group()
    ctx.rmsnorm(hb, gb, nb, 1, hidden, 1e-5)
    ctx.q8_0_gemv(wb, hb, yb, 64, hidden)  # reads h, not the norm's output
    ctx.end_group()
    ctx.fence()
    assert close(nb.download_f32(0, hidden), O.rmsnorm(h, g, 1e-5))
    want = O.gemv_q8_0_f32(w, 64, hidden, h)
    assert np.max(np.abs(yb.download_f32(0, 64) - want)) <= 1e-5 * np.max(np.abs(want))


@pytest.mark.parametrize("hidden,ffn", [(1024, 3072 + 8), (1152, 3072 + 8), (2048 + 128, 3072 + 6),
                                        (1024, 8192 + 12)])
@pytest.mark.parametrize("act,in_place,with_norm", [("silu", True, True), ("silu", False, False),
                                                    ("gelu", True, False), ("gelu", False, True)])
def test_gated_activation_behind_gate_and_up_is_fused(ctx, act, in_place, with_norm, hidden, ffn):
    # [norm ->] gate, up -> act(gate) * up -> down with its residual update: grouped,
    # one wave computes a row of gate and of up and applies the activation itself.
    # Every buffer must hold the bits of the separate operators. (Widths with a column
    # tail of 128 behind the 1024-column chunks too: Gemma-3-1B's 1152. Row counts that
    # leave a partial last tile; few rows go in tiles of 2 rows of each matrix, 8204 rows
    # in tiles of 4.)
    wg, wu = S.make_weights(ffn, hidden, 401), S.make_weights(ffn, hidden, 402)
    wd = S.make_weights(hidden, 1024 * 3, 403)
    wgb, wub = weights_buffer(ctx, wg, ffn, hidden, True), weights_buffer(ctx, wu, ffn, hidden, True)
    h0 = S.make_activations(hidden, 404)
    gw = (0.5 + np.abs(S.make_activations(hidden, 405))).astype(np.float32)
    gwb = upload_new(ctx, gw)
    runs = []
    for grouped in (False, True):
        hb, nb = upload_new(ctx, h0), ctx.buffer(hidden * 4)
        gb, ub = ctx.buffer(ffn * 4), ctx.buffer(ffn * 4)
        ob = gb if in_place else ctx.buffer(ffn * 4)
        launches = ctx.kernel_launches()
        if grouped:
            ctx.begin_group()
        xin = hb
        if with_norm:
            ctx.rmsnorm(hb, gwb, nb, 1, hidden, 1e-6)
            xin = nb
        ctx.q8_0_gemv(wgb, xin, gb, ffn, hidden)
        ctx.q8_0_gemv(wub, xin, ub, ffn, hidden)
        (ctx.silu_mul if act == "silu" else ctx.gelu_tanh_mul)(gb, ub, ob, ffn)
        if grouped:
            ctx.end_group()
        ctx.fence()
        used = ctx.kernel_launches() - launches
        assert used == (1 if grouped else 3 + int(with_norm)), used
        runs.append({"gate": gb.download_f32(0, ffn).copy(), "up": ub.download_f32(0, ffn).copy(),
                     "out": ob.download_f32(0, ffn).copy(), "n": nb.download_f32(0, hidden).copy()})
    for k in runs[0]:
        assert np.array_equal(bits(runs[0][k]), bits(runs[1][k])), k
    x = O.rmsnorm(h0, gw, 1e-6) if with_norm else h0
    if with_norm:
        assert close(runs[1]["n"], x)
        x = runs[1]["n"]
    g, u = O.gemv_q8_0_f32(wg, ffn, hidden, x), O.gemv_q8_0_f32(wu, ffn, hidden, x)
    assert np.max(np.abs(runs[1]["up"] - u)) <= 1e-5 * np.max(np.abs(u))
    if not in_place:
        assert np.max(np.abs(runs[1]["gate"] - g)) <= 1e-5 * np.max(np.abs(g))
    want = (O.silu_mul if act == "silu" else O.gelu_tanh_mul)(g, u)
    assert np.all(np.abs(runs[1]["out"] - want) <= 2e-5 * np.maximum(np.abs(want), 1.0))
    del wd


@pytest.mark.parametrize("tokens", [2, 3, 4])
@pytest.mark.parametrize("hidden,qdim,kvdim,ffn,act", [(1024, 2048, 1024, 3072, "silu"),   # Qwen3-0.6B
                                                       (1152, 1024, 256, 6912, "gelu")])   # Gemma-3-1B
def test_a_few_tokens_take_the_same_fusions_as_one(ctx, tokens, hidden, qdim, kvdim, ffn, act):
    # A speculative step verifies [token, draft] with a small batch through the exact
    # product (crates/tuckcore/src/engine/metal.rs:2170-2192). A whole layer at 2 to 4
    # tokens: norm -> q, k, v -> o with its update -> norm -> gate, up -> activation ->
    # down with its update. Grouped, every token is a descriptor of the one-token kernel
    # and the operators ride along as they do for one token (4 launches for 12); every
    # buffer must hold the bits of the separate run.
    T = tokens
    mats = {}
    for i, (name, rows, cols) in enumerate([("q", qdim, hidden), ("k", kvdim, hidden),
                                            ("v", kvdim, hidden), ("o", hidden, qdim),
                                            ("gate", ffn, hidden), ("up", ffn, hidden),
                                            ("down", hidden, ffn)]):
        w = S.make_weights(rows, cols, 500 + i)
        mats[name] = (w, rows, cols, weights_buffer(ctx, w, rows, cols, True))
    h0 = S.make_activations(T * hidden, 510)
    g1 = (0.5 + np.abs(S.make_activations(hidden, 511))).astype(np.float32)
    g2 = (0.5 + np.abs(S.make_activations(hidden, 512))).astype(np.float32)
    attn = S.make_activations(T * qdim, 513)
    g1b, g2b, attnb = upload_new(ctx, g1), upload_new(ctx, g2), upload_new(ctx, attn)
    runs = []
    for grouped in (False, True):
        hb = upload_new(ctx, h0)
        nb, n2b, tb = (ctx.buffer(T * hidden * 4) for _ in range(3))
        out = {k: ctx.buffer(T * mats[k][1] * 4) for k in ("q", "k", "v", "gate", "up")}
        launches = ctx.kernel_launches()
        if grouped:
            ctx.begin_group()
        ctx.rmsnorm(hb, g1b, nb, T, hidden, 1e-6)
        for k in ("q", "k", "v"):
            ctx.q8_0_gemm(mats[k][3], nb, out[k], mats[k][1], hidden, T)
        ctx.q8_0_gemm(mats["o"][3], attnb, tb, hidden, qdim, T)
        ctx.f32_axpy(tb, hb, 1.0, T * hidden)
        ctx.rmsnorm(hb, g2b, n2b, T, hidden, 1e-6)
        for k in ("gate", "up"):
            ctx.q8_0_gemm(mats[k][3], n2b, out[k], mats[k][1], hidden, T)
        (ctx.silu_mul if act == "silu" else ctx.gelu_tanh_mul)(out["gate"], out["up"], out["gate"],
                                                               T * ffn)
        ctx.q8_0_gemm(mats["down"][3], out["gate"], tb, hidden, ffn, T)
        ctx.f32_axpy(tb, hb, 1.0, T * hidden)
        if grouped:
            ctx.end_group()
        ctx.fence()
        used = ctx.kernel_launches() - launches
        assert used == (4 if grouped else 12), used
        got = {k: out[k].download_f32(0, T * mats[k][1]).copy() for k in out}
        got.update(n=nb.download_f32(0, T * hidden).copy(), n2=n2b.download_f32(0, T * hidden).copy(),
                   h=hb.download_f32(0, T * hidden).copy(), t=tb.download_f32(0, T * hidden).copy())
        runs.append(got)
    for k in runs[0]:
        assert np.array_equal(bits(runs[0][k]), bits(runs[1][k])), k
    # and the separate run is the oracle's, token by token
    for t in range(T):
        n = O.rmsnorm(h0[t * hidden:(t + 1) * hidden], g1, 1e-6)
        assert close(runs[1]["n"][t * hidden:(t + 1) * hidden], n)
        q = O.gemv_q8_0_f32(mats["q"][0], qdim, hidden, runs[1]["n"][t * hidden:(t + 1) * hidden])
        assert np.max(np.abs(runs[1]["q"][t * qdim:(t + 1) * qdim] - q)) <= 1e-5 * np.max(np.abs(q))


def test_fusions_of_a_few_tokens_need_matching_token_counts(ctx):
    # a norm over 2 rows in front of a product of 3 tokens over the same buffer: the
    # product reads a third row that the norm does not write, nothing may be fused
    hidden, rows = 1024, 256
    w = S.make_weights(rows, hidden, 520)
    wb = weights_buffer(ctx, w, rows, hidden, True)
    h = S.make_activations(3 * hidden, 521)
    g = (0.5 + np.abs(S.make_activations(hidden, 522))).astype(np.float32)
    hb, gb = upload_new(ctx, h), upload_new(ctx, g)
    nb, yb = upload_new(ctx, h), ctx.buffer(3 * rows * 4)
    launches = ctx.kernel_launches()
    ctx.begin_group()
    ctx.rmsnorm(hb, gb, nb, 2, hidden, 1e-6)
    ctx.q8_0_gemm(wb, nb, yb, rows, hidden, 3)
    ctx.end_group()
    ctx.fence()
    assert ctx.kernel_launches() - launches == 2
    x = nb.download_f32(0, 3 * hidden)
    assert np.array_equal(bits(x[2 * hidden:]), bits(h[2 * hidden:]))
    for t in range(3):
        want = O.gemv_q8_0_f32(w, rows, hidden, x[t * hidden:(t + 1) * hidden])
        got = yb.download_f32(0, 3 * rows)[t * rows:(t + 1) * rows]
        assert np.max(np.abs(got - want)) <= 1e-5 * np.max(np.abs(want))


def test_a_norm_over_a_few_rows_that_nobody_reads_still_runs(ctx):
    hidden, rows, T = 2048, 64, 2
    h = S.make_activations(T * hidden, 530)
    g = (0.5 + np.abs(S.make_activations(hidden, 531))).astype(np.float32)
    w = S.make_weights(rows, hidden, 532)
    wb = weights_buffer(ctx, w, rows, hidden, True)
    hb, gb = upload_new(ctx, h), upload_new(ctx, g)
    nb, yb = ctx.buffer(T * hidden * 4), ctx.buffer(T * rows * 4)
    ctx.begin_group()
    ctx.rmsnorm(hb, gb, nb, T, hidden, 1e-5)
    ctx.q8_0_gemm(wb, hb, yb, rows, hidden, T)  # reads h, not the norm's output
    ctx.end_group()
    ctx.fence()
    for t in range(T):
        ht = h[t * hidden:(t + 1) * hidden]
        assert close(nb.download_f32(0, T * hidden)[t * hidden:(t + 1) * hidden],
                     O.rmsnorm(ht, g, 1e-5))
        want = O.gemv_q8_0_f32(w, rows, hidden, ht)
        got = yb.download_f32(0, T * rows)[t * rows:(t + 1) * rows]
        assert np.max(np.abs(got - want)) <= 1e-5 * np.max(np.abs(want))


def test_large_products_of_a_few_tokens_are_not_read_once_per_token(ctx):
    # gate and up of more than 16 M weights each at 2 tokens: fused with their
    # activation they would go through the one-token kernel, every token reading the
    # weights again; they stay one launch of the token-split kernel, the activation
    # behind them on its own.
    rows, hidden, T = 16400, 1024, 2
    wg, wu = S.make_weights(rows, hidden, 540), S.make_weights(rows, hidden, 541)
    wgb, wub = weights_buffer(ctx, wg, rows, hidden, True), weights_buffer(ctx, wu, rows, hidden, True)
    x = S.make_activations(T * hidden, 542)
    xb = upload_new(ctx, x)
    runs = []
    for grouped in (False, True):
        gb, ub = ctx.buffer(T * rows * 4), ctx.buffer(T * rows * 4)
        launches = ctx.kernel_launches()
        if grouped:
            ctx.begin_group()
        ctx.q8_0_gemm(wgb, xb, gb, rows, hidden, T)
        ctx.q8_0_gemm(wub, xb, ub, rows, hidden, T)
        ctx.silu_mul(gb, ub, gb, T * rows)
        if grouped:
            ctx.end_group()
        ctx.fence()
        assert ctx.kernel_launches() - launches == (2 if grouped else 3)
        runs.append((gb.download_f32(0, T * rows).copy(), ub.download_f32(0, T * rows).copy()))
    for a, b in zip(runs[0], runs[1]):
        assert np.array_equal(bits(a), bits(b))
    u = O.gemv_q8_0_f32(wu, rows, hidden, x[hidden:])
    assert np.max(np.abs(runs[1][1][rows:] - u)) <= 1e-5 * np.max(np.abs(u))


def test_gated_activation_is_not_fused_when_out_is_the_up_buffer(ctx):
    hidden, ffn = 1024, 256
    wg, wu = S.make_weights(ffn, hidden, 411), S.make_weights(ffn, hidden, 412)
    wgb, wub = weights_buffer(ctx, wg, ffn, hidden, True), weights_buffer(ctx, wu, ffn, hidden, True)
    x = S.make_activations(hidden, 413)
    xb, gb, ub = upload_new(ctx, x), ctx.buffer(ffn * 4), ctx.buffer(ffn * 4)
    launches = ctx.kernel_launches()
    ctx.begin_group()
    ctx.q8_0_gemv(wgb, xb, gb, ffn, hidden)
    ctx.q8_0_gemv(wub, xb, ub, ffn, hidden)
    ctx.silu_mul(gb, ub, ub, ffn)
    ctx.end_group()
    ctx.fence()
    assert ctx.kernel_launches() - launches == 2
    g, u = O.gemv_q8_0_f32(wg, ffn, hidden, x), O.gemv_q8_0_f32(wu, ffn, hidden, x)
    want = O.silu_mul(g, u)
    assert np.all(np.abs(ub.download_f32(0, ffn) - want) <= 2e-5 * np.maximum(np.abs(want), 1.0))


@pytest.mark.parametrize("rows,cols", [(128, 1024), (37, 1152), (5, 1000), (3, 7), (512, 1024)])
@pytest.mark.parametrize("in_place", [False, True])
def test_a_norm_takes_the_residual_update_of_its_input_in_front_of_itself(ctx, rows, cols, in_place):
    # h += alpha * t; xn = rmsnorm(h): between two blocks of a layer at prefill
    # sizes. Inside a group the norm does the update on its way (one launch), with
    # the same bits in h and in xn as the two launched one after the other.
    # Aligned and unaligned widths, rows the size of a prefill chunk and a few.
    n = rows * cols
    h0 = S.make_activations(n, 5)
    t = S.make_activations(n, 6)
    w = (1.0 + 0.25 * S.make_activations(cols, 7)).astype(np.float32)
    hb, tb, wb = upload_new(ctx, h0), upload_new(ctx, t), upload_new(ctx, w)
    yb = hb if in_place else ctx.buffer(n * 4)
    alpha, eps = 0.5, 1e-6

    def run(grouped):
        hb.upload(0, h0)
        before = ctx.kernel_launches()
        if grouped:
            ctx.begin_group()
        ctx.f32_axpy(tb, hb, alpha, n)
        ctx.rmsnorm(hb, wb, yb, rows, cols, eps)
        if grouped:
            ctx.end_group()
        ctx.fence()
        return (hb.download_f32(0, n).copy(), yb.download_f32(0, n).copy(),
                ctx.kernel_launches() - before)

    h_apart, y_apart, n_apart = run(False)
    assert n_apart == 2
    if not in_place:
        assert np.array_equal(bits(h_apart), bits(h0 + np.float32(alpha) * t))
        for r in range(0, rows, max(1, rows // 7)):
            want = O.rmsnorm(h_apart[r * cols:(r + 1) * cols], w, eps)
            assert close(y_apart[r * cols:(r + 1) * cols], want), f"row {r}"
    for attempt in range(2):
        h_fused, y_fused, n_fused = run(True)
        assert n_fused == 1
        assert np.array_equal(bits(h_fused), bits(h_apart)), f"attempt {attempt}"
        assert np.array_equal(bits(y_fused), bits(y_apart)), f"attempt {attempt}"

    # an update of only part of the norm's input, or of another buffer, stays a launch of its own
    hb.upload(0, h0)
    before = ctx.kernel_launches()
    ctx.begin_group()
    ctx.f32_axpy(tb, hb, alpha, n - 1 if n > 1 else 1)
    ctx.rmsnorm(hb, wb, yb, rows, cols, eps)
    ctx.end_group()
    ctx.fence()
    assert ctx.kernel_launches() - before == (2 if n > 1 else 1)
    for b in {hb, tb, wb, yb}:
        b.free()
