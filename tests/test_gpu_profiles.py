"""GPU parity: the numerical profiles on the `Matrix` handles
(crates/tuckcore/src/forward.rs:284-311, :606-645). `oracle-f32` against
dot_q8_0_x_f32 within 1e-5; `llama-cpu` (activations quantized per 32 on the
device, int8 block dots) against dot_q8_0_q8_0 bit for bit, through the Python
mirror and through the C++ one (libtm_host.so)."""
import ctypes
import os

import numpy as np
import pytest

import oracle as O
from tuckmill_amd import hip as H
from tuckmill_amd import synth as S

from q8util import bits, norm_err, require_gpu, upload_new

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def ctx():
    c = require_gpu()
    yield c
    c.close()


SHAPES = [(3072, 1024, 1), (1024, 3072, 1), (300, 1152, 4), (6912, 1152, 33), (2048, 2048, 128),
          (515, 1024, 512)]


@pytest.mark.parametrize("rows,cols,batch", SHAPES)
def test_both_profiles_through_matrix(ctx, rows, cols, batch):
    raw = S.make_weights(rows, cols, rows + 3 * cols)
    x = S.make_activations(batch * cols, batch + cols)
    xb = upload_new(ctx, x)
    results = {}
    for profile in (H.NumericalProfile.ORACLE_F32, H.NumericalProfile.LLAMA_CPU):
        m = H.Matrix.load(ctx, raw, cols, rows, profile=profile)
        yb = ctx.buffer(batch * rows * 4)
        ctx.begin_group()   # the way an engine step issues it
        if batch == 1:
            m.gemv(ctx, xb, yb)
        else:
            m.gemm(ctx, xb, yb, batch, exact=False)
        ctx.end_group()
        ctx.fence()
        results[profile] = yb.download_f32(0, batch * rows).reshape(batch, rows).copy()
        m.buf.free()
        yb.free()
    want_f32 = O.gemm_q8_0_f32(raw, rows, cols, x, batch, threads=8)
    want_i8 = O.gemm_q8_0_q8_0(raw, rows, cols, x, batch, threads=8)
    assert norm_err(results[H.NumericalProfile.ORACLE_F32], want_f32) <= 1e-5
    assert np.array_equal(bits(results[H.NumericalProfile.LLAMA_CPU]), bits(want_i8))
    # the two profiles are different numerical contracts: they must not be confused
    assert not np.array_equal(bits(want_f32), bits(want_i8))
    xb.free()


def test_llama_cpu_matrix_reuses_and_grows_its_quantized_activations(ctx):
    rows, cols = 640, 1024
    raw = S.make_weights(rows, cols, 5)
    m = H.Matrix.load(ctx, raw, cols, rows, profile=H.NumericalProfile.LLAMA_CPU)
    base = ctx.allocated_bytes()
    for batch in (1, 40, 8, 2100):  # the last one goes in slices of GEMM_I8_MAX_BATCH tokens
        x = S.make_activations(batch * cols, 60 + batch)
        xb, yb = upload_new(ctx, x), ctx.buffer(batch * rows * 4)
        ctx.begin_group()
        m.gemm(ctx, xb, yb, batch, exact=True)
        m.gemv(ctx, xb, yb)     # token 0 again, through the buffer the group still holds
        ctx.end_group()
        ctx.fence()
        want = O.gemm_q8_0_q8_0(raw, rows, cols, x, batch, threads=8)
        assert np.array_equal(bits(yb.download_f32(0, batch * rows)), bits(want.reshape(-1)))
        xb.free()
        yb.free()
    # the matrix holds one quantized-activation buffer, sized for the largest slice
    assert ctx.allocated_bytes() - base == H.xq_bytes(cols, H.GEMM_I8_MAX_BATCH)
    m.buf.free()


def host_lib():
    H.load_library()
    lib = ctypes.CDLL(os.path.join(ROOT, "tuckmill_amd", "libtm_host.so"))
    lib.tmh_matrix_roundtrip_profile.restype = ctypes.c_int
    lib.tmh_matrix_roundtrip_profile.argtypes = [
        ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_char_p,
        ctypes.c_void_p, ctypes.c_uint32, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
        ctypes.c_uint32, ctypes.c_char_p, ctypes.c_size_t]
    return lib


@pytest.mark.parametrize("rows,cols,batch", [(515, 1024, 1), (300, 1152, 40), (2048, 2048, 2100)])
def test_both_profiles_through_the_cpp_matrix(rows, cols, batch):
    lib = host_lib()
    raw = S.make_weights(rows, cols, rows + cols)
    x = S.make_activations(batch * cols, batch)
    row = np.empty(cols, np.float32)
    err = ctypes.create_string_buffer(512)
    out = {}
    for profile in ("oracle-f32", "llama-cpu"):
        y = np.empty((batch, rows), np.float32)
        rc = lib.tmh_matrix_roundtrip_profile(raw.ctypes.data, rows, cols, 8, profile.encode(),
                                              x.ctypes.data, batch, 0, y.ctypes.data,
                                              row.ctypes.data, rows - 1, err, 512)
        assert rc == 0, err.value.decode()
        out[profile] = y
    assert norm_err(out["oracle-f32"], O.gemm_q8_0_f32(raw, rows, cols, x, batch, threads=8)) <= 1e-5
    want = O.gemm_q8_0_q8_0(raw, rows, cols, x, batch, threads=8)
    assert np.array_equal(bits(out["llama-cpu"]), bits(want))


def test_cpp_matrix_refuses_unknown_and_unsupported_profiles():
    lib = host_lib()
    rows, cols = 4, 64
    half = np.zeros(rows * cols, np.float16)
    x = np.zeros(cols, np.float32)
    y = np.zeros(rows, np.float32)
    err = ctypes.create_string_buffer(512)
    # F16 weights under llama-cpu: no device kernel, refused at load
    rc = lib.tmh_matrix_roundtrip_profile(half.ctypes.data, rows, cols, 1, b"llama-cpu",
                                          x.ctypes.data, 1, 0, y.ctypes.data, x.ctypes.data, 0,
                                          err, 512)
    assert rc == H.TM_HIP_ERR_UNSUPPORTED and b"llama-cpu" in err.value
    # ... and run under oracle-f32
    rc = lib.tmh_matrix_roundtrip_profile(half.ctypes.data, rows, cols, 1, b"oracle-f32",
                                          x.ctypes.data, 1, 0, y.ctypes.data, x.ctypes.data, 0,
                                          err, 512)
    assert rc == 0, err.value.decode()
    rc = lib.tmh_matrix_roundtrip_profile(half.ctypes.data, rows, cols, 8, b"fp8", x.ctypes.data,
                                          1, 0, y.ctypes.data, x.ctypes.data, 0, err, 512)
    assert rc == H.TM_HIP_ERR_UNSUPPORTED and b"unknown numerical profile" in err.value
