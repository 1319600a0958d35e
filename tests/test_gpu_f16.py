"""GPU parity of the F16-weight twins of the products.

Follows crates/metal/src/tests.rs:682-725 (f16_gemv) and :924-975 (f16_gemm):
weights on the grid ((rng % 20001) - 10000) / 1000 rounded to f16, activations
from boundary_input, compared with the sequential scalar sum. The reference
accepts 1e-4 * max(|want|, 1); the bar here is 1e-5 of the largest output.
"""
import numpy as np
import pytest

import oracle as O
from tuckmill_amd import hip as H

from q8util import bits, norm_err, require_gpu, upload_new

pytestmark = pytest.mark.gpu

TOL = 1e-5


@pytest.fixture(scope="module")
def ctx():
    c = require_gpu()
    yield c
    c.close()


def grid_f16(rows, cols, seed):
    """f16 bytes of the reference's weight grid; numpy rounds to nearest even
    like f32_to_f16_bits on these finite values (checked against the oracle
    on a sample)."""
    rng = np.random.default_rng(seed)
    v = ((rng.integers(0, 20001, rows * cols) - 10000) / 1000.0).astype(np.float32)
    h = v.astype(np.float16)
    sample = rng.integers(0, v.size, 64)
    assert np.array_equal(O.f16_bytes(v[sample]).view("<u2"), h[sample].view("<u2"))
    return h.view(np.uint8)


@pytest.mark.parametrize("rows,cols", [
    (1, 32), (17, 64), (1024, 1024),          # crates/metal/src/tests.rs:688
    (3, 1), (5, 7), (9, 33), (40, 520), (8, 513), (33, 1030),   # rows that are not 16-byte aligned
    (4096, 2048), (1000, 3072), (151936 // 8, 1024),
])
def test_f16_gemv_matches_the_scalar_reference(ctx, rows, cols):
    w = grid_f16(rows, cols, rows * 31 + cols)
    x = O.boundary_input(cols, 3)
    wb, xb, yb = upload_new(ctx, w), upload_new(ctx, x), ctx.buffer(rows * 4)
    ctx.f16_gemv(wb, xb, yb, rows, cols)
    ctx.fence()
    got = yb.download_f32(0, rows)
    want = O.gemm_f16_f32(w, rows, cols, x)
    assert norm_err(got, want) <= TOL
    for b in (wb, xb, yb):
        b.free()


@pytest.mark.parametrize("rows,cols,batch,x_off,y_off", [
    (128, 256, 8, 0, 0),                      # crates/metal/src/tests.rs:928-950
    (128, 256, 32, 0, 0), (64, 1024, 2, 0, 0), (64, 1024, 3, 5, 9), (200, 520, 5, 3, 1),
    (33, 70, 7, 1, 2), (2048, 2048, 4, 0, 0), (1024, 3072, 31, 0, 0),
])
def test_f16_gemm_is_the_gemv_token_by_token(ctx, rows, cols, batch, x_off, y_off):
    w = grid_f16(rows, cols, 7 * rows + cols + batch)
    x = np.concatenate([O.boundary_input(cols, 41 + b) for b in range(batch)])
    wb = upload_new(ctx, w)
    xb = ctx.buffer((x_off + batch * cols) * 4)
    xb.upload(x_off * 4, x)
    yb = ctx.buffer((y_off + batch * rows) * 4)
    ctx.f16_gemm(wb, xb, yb, rows, cols, batch, x_off, y_off)
    ctx.fence()
    got = yb.download_f32(y_off, batch * rows).reshape(batch, rows)
    want = O.gemm_f16_f32(w, rows, cols, x, batch).reshape(batch, rows)
    assert norm_err(got, want) <= TOL
    if y_off:
        assert not np.any(yb.download_f32(0, y_off))  # nothing written in front of the slice
    # bit-identical to the one-token product on each token
    x1, y1 = ctx.buffer(cols * 4), ctx.buffer(rows * 4)
    for b in (0, batch // 2, batch - 1):
        x1.upload(0, x[b * cols:(b + 1) * cols])
        ctx.f16_gemv(wb, x1, y1, rows, cols)
        ctx.fence()
        assert np.array_equal(bits(y1.download_f32(0, rows)), bits(got[b])), f"token {b}"
    for buf in (wb, xb, yb, x1, y1):
        buf.free()


def test_f16_rows_are_exact(ctx):
    rows, cols = 37, 131
    w = grid_f16(rows, cols, 5)
    # every special encoding goes through the row conversion too
    special = np.array([0x0000, 0x8000, 0x0001, 0x83FF, 0x0400, 0x7BFF, 0xFBFF, 0x7C00, 0xFC00,
                        0x3C00, 0xC000], dtype="<u2")
    w16 = w.view("<u2").copy()
    w16[:special.size] = special
    w = w16.view(np.uint8)
    want = w16.view(np.float16).astype(np.float32).reshape(rows, cols)
    assert want[0, 2] == O.f16_to_f32(0x0001)
    wb = upload_new(ctx, w)
    out = ctx.buffer((cols + 3) * 4)
    for row in (0, 17, rows - 1):
        ctx.f16_row(wb, out, row, cols, 3)
        ctx.fence()
        assert np.array_equal(bits(out.download_f32(3, cols)), bits(want[row]))
    ids = upload_new(ctx, np.array([5, rows, 36], np.uint32))
    dst = ctx.buffer(cols * 4)
    for slot, row in ((0, 5), (2, 36)):
        ctx.row_indirect_f32(wb, 1, rows, cols, ids, slot, dst)
        ctx.fence()
        assert np.array_equal(bits(dst.download_f32(0, cols)), bits(want[row]))
    ctx.row_indirect_f32(wb, 1, rows, cols, ids, 1, dst)  # id == rows: zeros
    ctx.fence()
    assert not np.any(dst.download_f32(0, cols))


def test_f16_matrix_handle_and_groups(ctx):
    # the Matrix handle with type 1 (crates/tuckcore/src/engine/metal.rs:157-226)
    rows, cols, batch = 96, 160, 40   # batch above 32: sliced into two calls
    w = grid_f16(rows, cols, 9)
    m = H.Matrix.load(ctx, w, cols, rows, type_id=1)
    assert len(m.buf) == H.Matrix.plan(cols, rows, 1) == rows * cols * 2
    x = np.concatenate([O.boundary_input(cols, 60 + b) for b in range(batch)])
    xb, yb, y1, emb = upload_new(ctx, x), ctx.buffer(batch * rows * 4), ctx.buffer(rows * 4), ctx.buffer(cols * 4)
    launches = ctx.kernel_launches()
    ctx.begin_group()
    m.gemm(ctx, xb, yb, batch, exact=False)
    m.gemv(ctx, xb, y1)
    m.row_into(ctx, 3, emb, 0)
    ctx.end_group()
    ctx.fence()
    assert ctx.kernel_launches() == launches + 4
    want = O.gemm_f16_f32(w, rows, cols, x, batch).reshape(batch, rows)
    got = yb.download_f32(0, batch * rows).reshape(batch, rows)
    assert norm_err(got, want) <= TOL
    assert np.array_equal(bits(y1.download_f32(0, rows)), bits(got[0]))
    assert np.array_equal(emb.download_f32(0, cols), w.view(np.float16)[3 * cols:4 * cols].astype(np.float32))
    with pytest.raises(H.TuckmillError) as e:
        H.Matrix.load(ctx, w, cols, rows, type_id=2)
    assert e.value.code == "UnsupportedQuantization"


def test_f16_refusals(ctx):
    w, x, y = ctx.buffer(64 * 32 * 2), ctx.buffer(32 * 4 * 32), ctx.buffer(64 * 4 * 32)
    for args in ((0, 32), (64, 0)):
        with pytest.raises(H.TuckmillError) as e:
            ctx.f16_gemv(w, x, y, *args)
        assert e.value.abi_code == H.TM_HIP_ERR_UNSUPPORTED
    for batch in (0, 33):
        with pytest.raises(H.TuckmillError) as e:
            ctx.f16_gemm(w, x, y, 64, 32, batch)
        assert e.value.abi_code == H.TM_HIP_ERR_UNSUPPORTED
    with pytest.raises(H.TuckmillError) as e:
        ctx.f16_gemv(w, x, y, 65, 32)   # weights too short
    assert e.value.abi_code == H.TM_HIP_ERR_BOUNDS
    with pytest.raises(H.TuckmillError) as e:
        ctx.f16_gemm(w, x, y, 64, 32, 32, 1, 0)   # x slice past the end
    assert e.value.abi_code == H.TM_HIP_ERR_BOUNDS
    with pytest.raises(H.TuckmillError) as e:
        ctx.f16_row(w, y, 64, 32, 0)   # row past the table
    assert e.value.abi_code == H.TM_HIP_ERR_BOUNDS
    with pytest.raises(H.TuckmillError):
        ctx.f16_row(w, y, 0, 0, 0)
    ids = ctx.buffer(4)
    with pytest.raises(H.TuckmillError) as e:
        ctx.row_indirect_f32(w, 2, 64, 32, ids, 0, y)   # neither F16 nor Q8_0
    assert e.value.abi_code == H.TM_HIP_ERR_UNSUPPORTED
    with pytest.raises(H.TuckmillError):
        ctx.row_indirect_f32(w, 1, 64, 32, ids, 1, y)   # slot past the ids
