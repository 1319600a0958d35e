"""GPU tests of the C ABI's lifetime, ordering and accounting contract, the
row dequantization kernels and the seal (pack) step.

Follows crates/metal/src/tests.rs:409-574 and :657-678, :789-832, with Q8_0
operations standing in for the f32 utility kernels the reference uses there.
"""
import numpy as np
import pytest

import oracle as O
from tuckmill_amd import hip as H
from tuckmill_amd import synth as S

from q8util import bits, gemv, norm_err, require_gpu, upload_new, weights_buffer

pytestmark = pytest.mark.gpu


@pytest.fixture()
def ctx():
    c = require_gpu()
    yield c
    c.close()


def ones_problem(ctx, rows=4, cols=64, xval=1.0):
    """d = 1, q = 1 weights: y[r] = cols * xval exactly."""
    blk = O.f32_to_f16_bits(1.0).to_bytes(2, "little") + bytes([1] * 32)
    w = np.frombuffer(blk * (rows * cols // 32), np.uint8)
    wb = upload_new(ctx, w)
    xb = upload_new(ctx, np.full(cols, xval, np.float32))
    yb = ctx.buffer(rows * 4)
    return wb, xb, yb


def test_probe_reports_device_presence():
    p = H.probe()
    assert p.info
    assert p.available and "gfx950" in p.info


def test_buffers_are_context_scoped_and_accounted(ctx):
    assert ctx.allocated_bytes() == 0
    a = ctx.buffer(1024, True)
    b = ctx.buffer(2048, False)
    assert ctx.allocated_bytes() == 3072
    assert a.len() == 1024 and b.len() == 2048
    other = H.HipContext.open()
    foreign = other.buffer(64 * 34, True)
    # the typed wrapper refuses first ...
    with pytest.raises(H.TuckmillError) as e:
        ctx.q8_0_gemv(foreign, foreign, a, 1, 32)
    assert "different context" in str(e.value)
    # ... and so does the C ABI itself when called directly
    import ctypes
    err = ctypes.create_string_buffer(H.ERR_CAP)
    rc = H.load_library().tm_hip_q8_0_gemv(ctx.raw, foreign.raw, foreign.raw, a.raw, 1, 32, err,
                                           H.ERR_CAP)
    assert rc == H.TM_HIP_ERR_UNSUPPORTED and b"different context" in err.value
    with pytest.raises(H.TuckmillError):
        b.download(0, 8)  # private buffers have no host copy
    with pytest.raises(H.TuckmillError):
        b.upload(0, bytes(8))
    a.free()
    b.free()
    assert ctx.allocated_bytes() == 0
    assert other.allocated_bytes() == 64 * 34
    foreign.free()
    assert other.allocated_bytes() == 0
    other.close()


def test_an_allocation_the_device_cannot_hold_is_refused_and_leaves_the_context_usable(ctx):
    # crates/metal/src/lib.rs:732-745: an allocation failure is "Unavailable", not a crash
    before = ctx.allocated_bytes()
    with pytest.raises(H.TuckmillError) as e:
        ctx.buffer(1 << 40)  # 1 TiB: more than the device has
    assert e.value.abi_code == H.TM_HIP_ERR_ALLOC and e.value.code == "Unavailable"
    assert ctx.allocated_bytes() == before
    b = ctx.buffer(64)
    b.upload(0, np.arange(16, dtype=np.float32))
    assert np.array_equal(b.download_f32(0, 16), np.arange(16, dtype=np.float32))
    b.free()
    assert ctx.allocated_bytes() == before


def test_dispatch_completion_accounting_is_exact(ctx):
    wb, xb, yb = ones_problem(ctx, xval=2.0)
    base = ctx.committed_dispatches()
    for _ in range(5):
        ctx.q8_0_gemv(wb, xb, yb, 4, 64)
    assert ctx.committed_dispatches() == base + 5
    ctx.fence()
    assert ctx.completed_dispatches() == base + 5
    assert ctx.last_gpu_ms() >= 0.0
    assert ctx.gpu_nanos_total() > 0
    assert np.all(yb.download_f32(0, 4) == 128.0)


def test_gpu_times_are_read_when_asked_for_and_the_commit_log_keeps_them_apart(ctx):
    # A fence retires commits without reading their events; the measurement
    # entry points read them. The per-commit log (no counterpart in the
    # reference) holds one entry per commit completed while it was on.
    wb, xb, yb = ones_problem(ctx, rows=64, cols=1024)
    ctx.q8_0_gemv(wb, xb, yb, 64, 1024)      # before the log is on: must stay out of it
    ctx.fence()
    total0 = ctx.gpu_nanos_total()
    ctx.set_commit_log(True)
    n = 37
    for _ in range(n):
        ctx.q8_0_gemv(wb, xb, yb, 64, 1024)
    ctx.fence()
    assert ctx.completed_dispatches() == ctx.committed_dispatches()
    log = ctx.read_commit_log()
    assert log.size == n and (log > 0).all()
    assert int(log.sum()) == ctx.gpu_nanos_total() - total0
    assert ctx.last_gpu_ms() == pytest.approx(float(log[-1]) / 1e6)
    assert ctx.read_commit_log().size == 0, "read drains the log"
    ctx.set_commit_log(False)
    ctx.q8_0_gemv(wb, xb, yb, 64, 1024)
    ctx.fence()
    assert ctx.read_commit_log().size == 0
    # far more commits than the library keeps unmeasured: nothing is lost
    total1 = ctx.gpu_nanos_total()
    ctx.set_commit_log(True)
    for _ in range(2500):
        ctx.q8_0_gemv(wb, xb, yb, 64, 1024)
    ctx.fence()
    log = ctx.read_commit_log()
    assert log.size == 2500 and int(log.sum()) == ctx.gpu_nanos_total() - total1
    ctx.set_commit_log(False)


def test_a_fence_waits_for_work_issued_outside_commits(ctx):
    # zero fills and the allocation-free launches are not commits: the fence must
    # not take the last commit's event for the whole stream
    rows, cols = 151_936, 1024
    w = S.make_weights(rows, cols, 21)
    x = S.make_activations(cols, 22)
    wb = weights_buffer(ctx, w, rows, cols, True)
    xb, yb = upload_new(ctx, x), ctx.buffer(rows * 4)
    big = upload_new(ctx, np.full(64 << 20, 0xAB, np.uint8))
    for _ in range(5):
        ctx.q8_0_gemv(wb, xb, yb, rows, cols)   # commits
    big.zero(0, 64 << 20)                       # behind them, not a commit
    ctx.fence()
    assert not big.download(0, 64 << 20).any()
    assert norm_err(yb.download_f32(0, rows), O.gemv_q8_0_f32(w, rows, cols, x, threads=8)) <= 1e-5


def test_upload_download_respect_bounds_and_offsets(ctx):
    buf = ctx.buffer(16, True)
    buf.upload(8, bytes([9] * 8))
    out = buf.download(0, 16)
    assert bytes(out[8:]) == bytes([9] * 8) and not out[:8].any()
    with pytest.raises(H.TuckmillError):
        buf.upload(12, bytes(8))
    with pytest.raises(H.TuckmillError):
        buf.download(16, 1)
    buf.zero(8, 4)
    out = buf.download(0, 16)
    assert not out[8:12].any() and bytes(out[12:]) == bytes([9] * 4)
    with pytest.raises(H.TuckmillError):
        buf.zero(12, 8)
    with pytest.raises(H.TuckmillError):
        buf.zero(0, 0)


def test_copy_contract_synchronizes_with_in_flight_compute(ctx):
    wb, xb, yb = ones_problem(ctx, xval=3.0)
    ctx.q8_0_gemv(wb, xb, yb, 4, 64)
    assert np.all(yb.download_f32(0, 4) == 192.0)  # no explicit fence
    xb.upload(0, np.full(64, 5.0, np.float32))
    ctx.q8_0_gemv(wb, xb, yb, 4, 64)
    assert np.all(yb.download_f32(0, 4) == 320.0)


def test_copy_f32_moves_exact_slices_and_refuses_out_of_range(ctx):
    # crates/metal/src/tests.rs:1076-1115
    src = (np.sin(np.arange(64, dtype=np.float32)) * np.float32(1e-30)
           + np.arange(64, dtype=np.float32)).astype(np.float32)
    a, b = ctx.buffer(64 * 4), ctx.buffer(64 * 4)
    a.upload(0, src)
    ctx.copy_f32(a, 8, b, 40, 16)
    ctx.fence()
    out = b.download_f32(0, 64)
    assert np.array_equal(bits(out[40:56]), bits(src[8:24])), "bit-exact slice"
    assert not out[:40].view(np.uint32).any() and not out[56:].view(np.uint32).any()
    for args in [(a, 60, b, 0, 8), (a, 0, b, 60, 8), (a, 0, b, 0, 0)]:
        with pytest.raises(H.TuckmillError) as e:
            ctx.copy_f32(*args)
        assert e.value.abi_code == H.TM_HIP_ERR_BOUNDS
    # every bit pattern survives (NaN payloads, infinities, subnormals, -0), at
    # odd offsets and a ragged length that spans many workgroups
    n = (1 << 20) + 3
    raw = np.random.default_rng(9).integers(0, 1 << 32, n + 5, dtype=np.uint64).astype(np.uint32)
    big, dst = ctx.buffer((n + 5) * 4), ctx.buffer((n + 7) * 4)
    big.upload(0, raw.view(np.float32))
    ctx.copy_f32(big, 5, dst, 7, n)
    got = dst.download_f32(0, n + 7).view(np.uint32)
    assert np.array_equal(got[7:], raw[5:]) and not got[:7].any()


def test_xor_checksum_reads_every_word_once(ctx):
    """The read-only streaming kernel (the HBM read-bandwidth calibration): its
    partial words XOR to numpy's XOR of the same words, on lengths around its
    8 KiB tiles and 16-byte pieces, at an offset, inside a group, and over a
    sealed weight buffer (whose device bytes are the host statement of the
    sealed layout)."""
    rng = np.random.default_rng(31)
    n_max = (17 << 20) + 777  # past one sweep of the grid: 8192 waves x 2048 words
    raw = rng.integers(0, 1 << 32, n_max, dtype=np.uint64).astype(np.uint32)
    buf = ctx.buffer(n_max * 4)
    buf.upload(0, raw.view(np.uint8))
    part = ctx.buffer(H.CHECKSUM_PARTIAL_BYTES)
    for off, n in [(0, 1), (0, 3), (0, 4), (4, 2047), (0, 2048), (8, 2049), (0, 2048 * 4 * 2048),
                   (12, 2048 * 4 * 2048 + 2048 * 3 + 5), (0, n_max), (n_max - 777 - 1, 777)]:
        off -= off % 4
        ctx.xor_checksum_u32(buf, off, n, part)
        ctx.fence()
        want = int(np.bitwise_xor.reduce(raw[off:off + n]))
        assert H.HipContext.checksum_of(part) == want, (off, n)
    # inside a group, behind the copy that writes what it reads
    dst = ctx.buffer(4096 * 4)
    ctx.begin_group()
    ctx.copy_f32(buf, 64, dst, 0, 4096)
    ctx.xor_checksum_u32(dst, 0, 4096, part)
    ctx.end_group()
    ctx.fence()
    assert H.HipContext.checksum_of(part) == int(np.bitwise_xor.reduce(raw[64:64 + 4096]))
    # a sealed matrix: the checksum of the device layout, no download needed
    rows, cols = 96, 1152
    w = S.make_weights(rows, cols, 5)
    m = H.Matrix.load(ctx, w, cols, rows)
    ctx.xor_checksum_u32(m.buf, 0, w.nbytes // 4, part)
    ctx.fence()
    sealed = S.pack_q8_0(w, rows, cols)
    assert H.HipContext.checksum_of(part) == int(np.bitwise_xor.reduce(sealed.view(np.uint32)))
    for args, code in [((buf, 2, 8, part), H.TM_HIP_ERR_UNSUPPORTED),
                       ((buf, 0, 0, part), H.TM_HIP_ERR_BOUNDS),
                       ((buf, 0, n_max + 1, part), H.TM_HIP_ERR_BOUNDS),
                       ((buf, 0, 8, dst if False else ctx.buffer(64)), H.TM_HIP_ERR_BOUNDS),
                       ((part, 0, 8, part), H.TM_HIP_ERR_UNSUPPORTED)]:
        with pytest.raises(H.TuckmillError) as e:
            ctx.xor_checksum_u32(*args)
        assert e.value.abi_code == code


def test_copy_f32_inside_a_group_follows_the_product_that_wrote_its_source(ctx):
    wb, xb, yb = ones_problem(ctx, xval=3.0)
    keep = ctx.buffer(8 * 4)
    ctx.begin_group()
    ctx.q8_0_gemv(wb, xb, yb, 4, 64)
    ctx.copy_f32(yb, 0, keep, 2, 4)
    ctx.end_group()
    ctx.fence()
    out = keep.download_f32(0, 8)
    assert np.all(out[2:6] == 192.0) and not out[:2].any() and not out[6:].any()


def test_dropping_buffers_before_fence_is_safe(ctx):
    wb, xb, yb = ones_problem(ctx, xval=7.0)
    ctx.q8_0_gemv(wb, xb, yb, 4, 64)
    xb.free()  # GPU work on x may still be pending
    wb.free()
    ctx.fence()
    assert np.all(yb.download_f32(0, 4) == 448.0)
    yb.free()
    assert ctx.allocated_bytes() == 0
    assert ctx.in_flight_bytes() == 0


def test_buffers_freed_inside_an_open_group_stay_alive_until_the_commit_completes(ctx):
    # native/metal/tm_metal.m:673, :707-739: a group leases every buffer when the
    # operation is encoded, so handles may be dropped before end_group.
    rows, cols = 151_936, 1024
    w = S.make_weights(rows, cols, 12)
    x = S.make_activations(cols, 13)
    want = O.gemv_q8_0_f32(w, rows, cols, x, threads=8)
    for recorded in (False, True):
        wb = weights_buffer(ctx, w, rows, cols, True)
        xb = upload_new(ctx, x)
        tb = ctx.buffer(rows * 4)   # written by the first product, read by the copy
        keep = ctx.buffer(rows * 4)
        ctx.fence()
        total = wb.len() + xb.len() + tb.len()
        ctx.begin_group()
        ctx.q8_0_gemv(wb, xb, tb, rows, cols)
        ctx.copy_f32(tb, 0, keep, 0, rows)
        wb.free()
        xb.free()
        tb.free()
        assert ctx.allocated_bytes() == rows * 4, "only the kept output is handle-live"
        # fresh (zero-filled) allocations of the same sizes must not land on the
        # group's memory
        spoil = [ctx.buffer(n) for n in (total - rows * 4 - cols * 4, cols * 4, rows * 4)]
        if recorded:
            step = ctx.end_group_recorded()
            step.run()
        else:
            ctx.end_group()
            assert ctx.in_flight_bytes() >= total or ctx.completed_dispatches() == \
                ctx.committed_dispatches()
        ctx.fence()
        assert norm_err(keep.download_f32(0, rows), want) <= 1e-5
        if recorded:
            step.free()
        assert ctx.in_flight_bytes() == 0
        for b in spoil + [keep]:
            b.free()
        assert ctx.allocated_bytes() == 0
    # an aborted group gives its references back
    wb, xb, yb = ones_problem(ctx)
    ctx.begin_group()
    ctx.q8_0_gemv(wb, xb, yb, 4, 64)
    for b in (wb, xb, yb):
        b.free()
    ctx.abort_group()
    assert ctx.allocated_bytes() == 0 and ctx.in_flight_bytes() == 0


def test_in_flight_bytes_stay_visible_until_completion(ctx):
    # crates/metal/src/tests.rs:789-832, with a product large enough that the
    # GPU is still busy when the handles are dropped.
    rows, cols = 151_936, 1024
    w = np.zeros(S.q8_0_bytes(rows, cols), np.uint8)
    wb = upload_new(ctx, w)
    xb = upload_new(ctx, np.ones(cols, np.float32))
    yb = ctx.buffer(rows * 4)
    assert ctx.in_flight_bytes() == 0
    for _ in range(200):
        ctx.q8_0_gemv(wb, xb, yb, rows, cols)
    total = wb.len() + xb.len() + yb.len()
    wb.free()
    xb.free()
    assert ctx.allocated_bytes() == rows * 4, "only y is still handle-live"
    yb.free()
    assert ctx.allocated_bytes() == 0
    leased = ctx.in_flight_bytes()
    assert leased >= total, f"dropped-but-leased buffers must remain visible: {leased}"
    live = ctx.live_gpu_bytes()  # leases only shrink as commits complete
    assert live >= ctx.in_flight_bytes()
    ctx.fence()
    assert ctx.in_flight_bytes() == 0, "leases release at completion"


def test_grouped_encoding_matches_individual_dispatch_and_aborts_cleanly(ctx):
    rows, cols = 96, 256
    w = S.make_weights(rows, cols, 1)
    x = S.make_activations(cols, 2)
    wb = weights_buffer(ctx, w, rows, cols, True)
    xb = upload_new(ctx, x)
    y1, y2 = ctx.buffer(rows * 4), ctx.buffer(rows * 4)
    before = ctx.committed_dispatches()
    launches = ctx.kernel_launches()
    ctx.begin_group()
    ctx.q8_0_gemv(wb, xb, y1, rows, cols)
    ctx.q8_0_gemv(wb, xb, y2, rows, cols)
    ctx.end_group()
    assert ctx.committed_dispatches() == before + 1
    assert ctx.kernel_launches() == launches + 1, "independent products share one launch"
    ctx.fence()
    grouped = y1.download_f32(0, rows).copy()
    assert np.array_equal(bits(grouped), bits(y2.download_f32(0, rows)))
    individual = gemv(ctx, wb, x, rows, cols)
    assert np.array_equal(bits(grouped), bits(individual))
    # abort: never commits, never writes
    y1.zero(0, rows * 4)
    before = ctx.committed_dispatches()
    ctx.begin_group()
    ctx.q8_0_gemv(wb, xb, y1, rows, cols)
    ctx.abort_group()
    assert ctx.committed_dispatches() == before
    assert not y1.download(0, rows * 4).any()
    # fence / copies with an open group are refused rather than guessed
    ctx.begin_group()
    with pytest.raises(H.TuckmillError):
        ctx.fence()
    with pytest.raises(H.TuckmillError):
        y1.download(0, 4)
    with pytest.raises(H.TuckmillError):
        ctx.begin_group()
    ctx.abort_group()
    with pytest.raises(H.TuckmillError):
        ctx.end_group()
    with pytest.raises(H.TuckmillError):
        ctx.abort_group()


def test_dependent_products_in_a_group_run_in_order(ctx):
    # y of the first product is x of the second: the group must not merge them.
    n = 64
    blk = O.f32_to_f16_bits(0.5).to_bytes(2, "little") + bytes([1] * 32)
    w = np.frombuffer(blk * (n * n // 32), np.uint8)  # every entry 0.5
    wb = weights_buffer(ctx, w, n, n, True)
    a = upload_new(ctx, np.ones(n, np.float32))
    b, c = ctx.buffer(n * 4), ctx.buffer(n * 4)
    launches = ctx.kernel_launches()
    ctx.begin_group()
    ctx.q8_0_gemv(wb, a, b, n, n)   # b = 32
    ctx.q8_0_gemv(wb, b, c, n, n)   # c = 32 * 32 = 1024
    ctx.q8_0_gemv(wb, c, a, n, n)   # a = 32768 (overwrites the first input)
    ctx.end_group()
    assert ctx.kernel_launches() == launches + 3
    assert np.all(b.download_f32(0, n) == 32.0)
    assert np.all(c.download_f32(0, n) == 1024.0)
    assert np.all(a.download_f32(0, n) == 32768.0)


def test_download_after_waits_only_for_its_target(ctx):
    wb, xb, yb = ones_problem(ctx, xval=2.0)
    ctx.q8_0_gemv(wb, xb, yb, 4, 64)
    target = ctx.committed_dispatches()
    y2 = ctx.buffer(16)
    ctx.q8_0_gemv(wb, xb, y2, 4, 64)
    out = yb.download_after(0, 16, target).view(np.float32)
    assert np.all(out == 128.0)
    with pytest.raises(H.TuckmillError):
        yb.download_after(0, 16, ctx.committed_dispatches() + 1)
    ctx.fence()


def test_profile_table_labels_products_by_shape(ctx):
    wb, xb, yb = ones_problem(ctx)
    ctx.set_profiling(True)
    ctx.q8_0_gemv(wb, xb, yb, 4, 64)
    ctx.q8_0_gemv(wb, xb, yb, 4, 64)
    ctx.begin_group()
    ctx.q8_0_gemv(wb, xb, yb, 4, 64)
    ctx.end_group()
    ctx.fence()
    table = {name: (nanos, count) for name, nanos, count in ctx.profile_table()}
    assert table["q8_0_gemv:4x64"][1] == 2
    assert table["group"][1] == 1
    ctx.set_profiling(False)
    assert ctx.profile_table() == []


# ------------------------------------------------------------------ rows --

@pytest.mark.parametrize("packed", [False, True])
def test_row_dequantization_is_exact_on_boundary_weights(ctx, packed):
    # crates/metal/src/tests.rs:657-678
    rows, cols = 8, 64
    w = O.boundary_weights(rows, cols, 23)
    wb = weights_buffer(ctx, w, rows, cols, packed)
    ob = ctx.buffer((cols + 5) * 4)
    want = O.dequant_q8_0(w).reshape(rows, cols)
    for row in (0, 5, 7):
        ctx.q8_0_row(wb, ob, row, cols, 5)
        ctx.fence()
        got = ob.download_f32(0, cols + 5)
        assert not got[:5].any()
        assert np.array_equal(bits(got[5:]), bits(want[row]))
    with pytest.raises(H.TuckmillError):
        ctx.q8_0_row(wb, ob, 0, 48, 0)
    with pytest.raises(H.TuckmillError):
        ctx.q8_0_row(wb, ob, rows, cols, 0)  # row past the buffer
    with pytest.raises(H.TuckmillError):
        ctx.q8_0_row(wb, ob, 0, cols, 6)     # out range past the end


@pytest.mark.parametrize("packed", [False, True])
def test_row_indirect_reads_the_id_on_the_device(ctx, packed):
    rows, cols = 37, 1152
    w = S.make_weights(rows, cols, 3)
    wb = weights_buffer(ctx, w, rows, cols, packed)
    want = O.dequant_q8_0(w).reshape(rows, cols)
    ids = upload_new(ctx, np.array([4, 36, 37, 0xFFFFFFFF], np.uint32))
    ob = ctx.buffer(cols * 4)
    for slot, row in ((0, 4), (1, 36)):
        ctx.row_indirect_f32(wb, 8, rows, cols, ids, slot, ob)
        ctx.fence()
        assert np.array_equal(bits(ob.download_f32(0, cols)), bits(want[row]))
    for slot in (2, 3):  # an id >= rows writes zeros
        ctx.row_indirect_f32(wb, 8, rows, cols, ids, slot, ob)
        ctx.fence()
        assert not ob.download(0, cols * 4).any()
    # Type 1 (F16) on this buffer: it is too short for rows x cols halves
    # (BOUNDS); with few enough rows to fit, a sealed buffer is still refused,
    # because it holds Q8_0 in the device layout (UNSUPPORTED).
    with pytest.raises(H.TuckmillError) as e:
        ctx.row_indirect_f32(wb, 1, rows, cols, ids, 0, ob)
    assert e.value.abi_code == H.TM_HIP_ERR_BOUNDS
    if packed:
        with pytest.raises(H.TuckmillError) as e:
            ctx.row_indirect_f32(wb, 1, 19, cols, ids, 0, ob)
        assert e.value.abi_code == H.TM_HIP_ERR_UNSUPPORTED
    with pytest.raises(H.TuckmillError) as e:
        ctx.row_indirect_f32(wb, 2, rows, cols, ids, 0, ob)   # neither Q8_0 nor F16
    assert e.value.abi_code == H.TM_HIP_ERR_UNSUPPORTED
    with pytest.raises(H.TuckmillError):
        ctx.row_indirect_f32(wb, 8, rows, cols, ids, 4, ob)   # slot past ids
    with pytest.raises(H.TuckmillError):
        ctx.row_indirect_f32(wb, 8, 0, cols, ids, 0, ob)


def test_matrix_serves_lm_head_and_embedding_from_one_buffer(ctx):
    # crates/tuckcore/src/engine/metal.rs:1778-1780: the tied output matrix
    # is both the vocabulary projection and the embedding table.
    rows, cols = 515, 1024
    w = S.make_weights(rows, cols, 8)
    before = ctx.allocated_bytes()
    m = H.Matrix.load(ctx, w, cols, rows)
    assert ctx.allocated_bytes() - before == H.Matrix.plan(cols, rows), "ledger equals the plan"
    x = S.make_activations(cols, 9)
    xb, yb, ob = upload_new(ctx, x), ctx.buffer(rows * 4), ctx.buffer(cols * 4)
    m.gemv(ctx, xb, yb)
    m.row_into(ctx, 514, ob, 0)
    ctx.fence()
    want = O.gemv_q8_0_f32(w, rows, cols, x)
    got = yb.download_f32(0, rows)
    assert np.max(np.abs(got - want)) / np.max(np.abs(want)) <= 1e-5
    assert np.array_equal(bits(ob.download_f32(0, cols)),
                          bits(O.dequant_q8_0(w).reshape(rows, cols)[514]))
    # the same bytes declared as F16: the length does not match rows x cols halves
    with pytest.raises(H.TuckmillError) as e:
        H.Matrix.load(ctx, w, cols, rows, type_id=1)
    assert e.value.code == "InvalidArtifact"
    with pytest.raises(H.TuckmillError) as e:  # crates/tuckcore/src/engine/metal.rs:126-131
        H.Matrix.load(ctx, w, cols, rows, type_id=2)
    assert e.value.code == "UnsupportedQuantization"


# ------------------------------------------------------------------ seal --

def test_sealed_buffers_keep_the_ledger_and_refuse_host_access(ctx):
    rows, cols = 40, 96
    w = O.boundary_weights(rows, cols, 5)
    wb = upload_new(ctx, np.concatenate([w, np.arange(7, dtype=np.uint8)]))  # 7 spare bytes
    allocated = ctx.allocated_bytes()
    ctx.q8_0_pack(wb, rows, cols)
    ctx.fence()
    assert ctx.allocated_bytes() == allocated
    assert wb.len() == w.size + 7
    for call in (lambda: wb.download(0, 4), lambda: wb.upload(0, bytes(4)), lambda: wb.zero(0, 4),
                 lambda: ctx.q8_0_pack(wb, rows, cols)):
        with pytest.raises(H.TuckmillError) as e:
            call()
        assert e.value.abi_code == H.TM_HIP_ERR_UNSUPPORTED
    xb, yb = ctx.buffer(cols * 4), ctx.buffer(rows * 4)
    with pytest.raises(H.TuckmillError):
        ctx.q8_0_gemv(wb, xb, yb, rows - 1, cols)  # dims must match the seal
    with pytest.raises(H.TuckmillError):
        ctx.q8_0_gemv(xb, xb, wb, 1, 32)           # a sealed buffer is never an output
    with pytest.raises(H.TuckmillError):
        ctx.q8_0_pack(ctx.buffer(33), 1, 32)       # too short
    with pytest.raises(H.TuckmillError):
        ctx.q8_0_pack(ctx.buffer(64), 1, 48)
