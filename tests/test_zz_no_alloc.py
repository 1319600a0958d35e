"""GPU test of tm_hip_q8_0_gemm_mma_noalloc, the entry point that allocates
nothing: its results against tm_hip_q8_0_gemm_mma's (same kernels, so bit for
bit) and against the CPU oracle, on calls in a row that share the library's
static device workspace, the second smaller than the first; its refusals; its
leases; that the device's free memory does not move; and calls from two contexts,
which the library orders on the one workspace.
"""
import ctypes

import numpy as np
import pytest

import oracle as O
from tuckmill_amd import hip as H
from tuckmill_amd import synth as S

from q8util import bits, norm_err, require_gpu, upload_new, weights_buffer

pytestmark = pytest.mark.gpu


@pytest.fixture()
def ctx():
    c = require_gpu()
    yield c
    c.close()


def device_free_bytes() -> int:
    hip = ctypes.CDLL("libamdhip64.so")
    free, total = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return int(free.value)


def problem(ctx, rows, cols, batch, seed, x_off=0):
    w = S.make_weights(rows, cols, seed)
    x = S.make_activations(batch * cols, seed + 1)
    xs = np.zeros(x_off + batch * cols, np.float32)
    xs[x_off:] = x
    return {"rows": rows, "cols": cols, "batch": batch, "x_off": x_off, "w": w, "x": x,
            "wb": weights_buffer(ctx, w, rows, cols, True), "xb": upload_new(ctx, xs),
            "y_new": ctx.buffer((3 + batch * rows) * 4), "y_old": ctx.buffer((3 + batch * rows) * 4)}


def token_sample(batch, n=6):
    return sorted({int(round(i * (batch - 1) / (n - 1))) for i in range(n)}) if batch > 1 else [0]


# (first call, second call with a smaller input): rows, cols, batch, x_off
PAIRS = [
    # bf16 matrix cores, K cut into chunks (split activations, partial tiles, arrival
    # counters all come from the static workspace), then a smaller product of the same kind
    ((6144, 2048, 512, 0), (4096, 1024, 200, 0)),
    # K whole on the large tile, then the 64-token tile
    ((33000, 1024, 384, 0), (16500, 1056, 40, 0)),
    # activations off a 16-byte boundary: the f32 matrix cores (the work-queue form
    # on the large product), then a small product
    ((33000, 1024, 512, 1), (3000, 1024, 100, 1)),
    # small batches: the vector kernels, no workspace at all
    ((3072, 1024, 8, 0), (3072, 1024, 1, 0)),
]


@pytest.mark.parametrize("first,second", PAIRS)
def test_two_calls_in_a_row_match_the_allocating_entry_point(ctx, first, second):
    probs = [problem(ctx, *first[:3], 900 + first[0] % 97, first[3]),
             problem(ctx, *second[:3], 950 + second[0] % 89, second[3])]
    ctx.fence()
    commits = ctx.committed_dispatches()
    free_before = device_free_bytes()
    for p in probs:  # back to back, nothing between them
        ctx.q8_0_gemm_mma_noalloc(p["wb"], p["xb"], p["y_new"], p["rows"], p["cols"], p["batch"],
                                  p["x_off"], 3)
    assert ctx.committed_dispatches() == commits, "the call is not a commit"
    assert ctx.in_flight_bytes() >= sum(p["wb"].len() + p["xb"].len() + p["y_new"].len()
                                        for p in probs)
    ctx.fence()
    assert device_free_bytes() == free_before, "device memory was allocated or freed"
    assert ctx.in_flight_bytes() == 0
    for p in probs:
        ctx.q8_0_gemm_mma(p["wb"], p["xb"], p["y_old"], p["rows"], p["cols"], p["batch"],
                          p["x_off"], 3)
    ctx.fence()
    for p in probs:
        rows, cols, batch = p["rows"], p["cols"], p["batch"]
        new = p["y_new"].download_f32(0, 3 + batch * rows)
        old = p["y_old"].download_f32(0, 3 + batch * rows)
        assert not new[:3].any(), "nothing before y_off"
        assert np.array_equal(bits(new), bits(old)), (rows, cols, batch)
        picked = token_sample(batch)
        xs = np.ascontiguousarray(p["x"].reshape(batch, cols)[picked]).reshape(-1)
        want = O.gemm_q8_0_f32(p["w"], rows, cols, xs, len(picked), threads=8)
        got = new[3:].reshape(batch, rows)[picked]
        assert norm_err(got, want) <= 1e-5
    # once more in the opposite order, after ordinary commits have used their own
    # workspace: the static one is stale from the first round
    for p in reversed(probs):
        p["y_new"].zero(0, p["y_new"].len())
        ctx.q8_0_gemm_mma_noalloc(p["wb"], p["xb"], p["y_new"], p["rows"], p["cols"], p["batch"],
                                  p["x_off"], 3)
    ctx.fence()
    for p in probs:
        n = 3 + p["batch"] * p["rows"]
        assert np.array_equal(bits(p["y_new"].download_f32(0, n)), bits(p["y_old"].download_f32(0, n)))


def test_buffers_may_be_freed_right_after_the_call(ctx):
    rows, cols, batch = 6144, 2048, 256
    p = problem(ctx, rows, cols, batch, 77)
    keep = ctx.buffer(batch * rows * 4)
    ctx.fence()
    ctx.q8_0_gemm_mma_noalloc(p["wb"], p["xb"], p["y_new"], rows, cols, batch, 0, 0)
    ctx.copy_f32(p["y_new"], 0, keep, 0, batch * rows)  # a commit: adopts the leases
    for name in ("wb", "xb", "y_new"):
        p[name].free()
    spoil = [ctx.buffer(n) for n in (S.q8_0_bytes(rows, cols), batch * cols * 4, batch * rows * 4)]
    ctx.fence()
    picked = token_sample(batch)
    xs = np.ascontiguousarray(p["x"].reshape(batch, cols)[picked]).reshape(-1)
    want = O.gemm_q8_0_f32(p["w"], rows, cols, xs, len(picked), threads=8)
    got = keep.download_f32(0, batch * rows).reshape(batch, rows)[picked]
    assert norm_err(got, want) <= 1e-5
    assert ctx.in_flight_bytes() == 0
    for b in spoil + [keep, p["y_old"]]:
        b.free()
    assert ctx.allocated_bytes() == 0


def test_refusals(ctx):
    # too large for the static workspace: 512 x 8192 activations split into 24 MiB
    rows, cols, batch = 4096, 8192, 512
    assert H.gemm_mma_on_bf16(rows, cols, batch) and batch * cols * 6 > H.NOALLOC_XS_BYTES
    wb = weights_buffer(ctx, np.zeros(S.q8_0_bytes(rows, cols), np.uint8), rows, cols, True)
    xb, yb = ctx.buffer(batch * cols * 4), ctx.buffer(batch * rows * 4)
    launches = ctx.kernel_launches()
    with pytest.raises(H.TuckmillError) as e:
        ctx.q8_0_gemm_mma_noalloc(wb, xb, yb, rows, cols, batch)
    assert e.value.abi_code == H.TM_HIP_ERR_UNSUPPORTED and "static workspace" in e.value.message
    assert ctx.kernel_launches() == launches and ctx.in_flight_bytes() == 0
    ctx.q8_0_gemm_mma(wb, xb, yb, rows, cols, batch)  # the allocating entry point takes it
    ctx.q8_0_gemm_mma_noalloc(wb, xb, yb, rows, cols, 128)  # and fewer tokens fit
    # the argument contract of q8_0_gemm_mma
    with pytest.raises(H.TuckmillError) as e:
        ctx.q8_0_gemm_mma_noalloc(wb, xb, yb, rows, cols, H.GEMM_MMA_MAX_BATCH + 1)
    assert e.value.abi_code == H.TM_HIP_ERR_UNSUPPORTED
    with pytest.raises(H.TuckmillError) as e:
        ctx.q8_0_gemm_mma_noalloc(wb, xb, ctx.buffer(64), rows, cols, 128)
    assert e.value.abi_code == H.TM_HIP_ERR_BOUNDS
    # not inside a dispatch group
    ctx.begin_group()
    with pytest.raises(H.TuckmillError) as e:
        ctx.q8_0_gemm_mma_noalloc(wb, xb, yb, rows, cols, 128)
    assert e.value.abi_code == H.TM_HIP_ERR_UNSUPPORTED and "group" in e.value.message
    ctx.abort_group()
    ctx.fence()


def test_two_contexts_share_the_static_workspace_in_order(ctx):
    """Every context of a GPU uses that GPU's one static workspace, each on its own
    stream: calls from two contexts with no fence between them are ordered by the
    library (the later call's stream waits for the earlier context's), so each
    product has the bits of the allocating entry point."""
    other = H.HipContext.open()
    try:
        pa = [problem(ctx, 6144, 2048, 512, 300 + i) for i in range(2)]
        pb = [problem(other, 4096, 3072, 384, 310 + i) for i in range(2)]
        ctx.fence()
        other.fence()
        for round_ in range(3):  # A B A B ..., nothing in between
            for c, p in ((ctx, pa[round_ % 2]), (other, pb[round_ % 2]),
                         (ctx, pa[(round_ + 1) % 2]), (other, pb[(round_ + 1) % 2])):
                c.q8_0_gemm_mma_noalloc(p["wb"], p["xb"], p["y_new"], p["rows"], p["cols"],
                                        p["batch"], 0, 3)
        ctx.fence()
        other.fence()
        for c, probs in ((ctx, pa), (other, pb)):
            for p in probs:
                c.q8_0_gemm_mma(p["wb"], p["xb"], p["y_old"], p["rows"], p["cols"], p["batch"], 0, 3)
            c.fence()
            for p in probs:
                n = 3 + p["batch"] * p["rows"]
                assert np.array_equal(bits(p["y_new"].download_f32(0, n)),
                                      bits(p["y_old"].download_f32(0, n)))
                for name in ("wb", "xb", "y_new", "y_old"):
                    p[name].free()
    finally:
        other.close()
