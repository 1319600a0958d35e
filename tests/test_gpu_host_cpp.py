"""The C++ host layer (tuckmill_amd/host/tm_hip.hpp): typed handles, the
`Matrix` projection abstraction with its staged upload and seal, grouped
encoding, and the native step runner, exercised through libtm_host.so."""
import ctypes
import os

import numpy as np
import pytest

import oracle as O
from tuckmill_amd import hip as H
from tuckmill_amd import synth as S

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def host_lib():
    H.load_library()
    lib = ctypes.CDLL(os.path.join(ROOT, "tuckmill_amd", "libtm_host.so"))
    lib.tmh_matrix_roundtrip.restype = ctypes.c_int
    lib.tmh_matrix_roundtrip.argtypes = [ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint32,
                                         ctypes.c_void_p, ctypes.c_uint32, ctypes.c_int,
                                         ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint32,
                                         ctypes.c_char_p, ctypes.c_size_t]
    return lib


@pytest.mark.parametrize("rows,cols,batch,exact", [(515, 1024, 1, 0), (300, 1152, 40, 1),
                                                   (300, 1152, 40, 0), (4_200_000 // 1088, 1024, 3, 1)])
def test_matrix_load_gemv_gemm_row_through_the_cpp_handles(rows, cols, batch, exact):
    # rows * row_bytes > 4 MiB in the last case: the staged upload crosses a
    # slice boundary that is not a multiple of 34 bytes.
    lib = host_lib()
    w = S.make_weights(rows, cols, rows + cols)
    x = S.make_activations(batch * cols, batch)
    y = np.empty((batch, rows), np.float32)
    row = np.empty(cols, np.float32)
    err = ctypes.create_string_buffer(512)
    rc = lib.tmh_matrix_roundtrip(w.ctypes.data, rows, cols, x.ctypes.data, batch, exact,
                                  y.ctypes.data, row.ctypes.data, rows - 1, err, 512)
    assert rc == 0, err.value.decode()
    want = O.gemm_q8_0_f32(w, rows, cols, x, batch, threads=4)
    assert np.max(np.abs(y - want)) / np.max(np.abs(want)) <= 1e-5
    assert np.array_equal(row.view(np.uint32),
                          O.dequant_q8_0(w).reshape(rows, cols)[rows - 1].view(np.uint32))


def test_cpp_handles_surface_typed_errors():
    lib = host_lib()
    w = np.zeros(34, np.uint8)
    x = np.zeros(32, np.float32)
    y = np.zeros(1, np.float32)
    err = ctypes.create_string_buffer(512)
    # a one-row matrix is refused like engine/metal.rs:124-129 refuses 1-D tensors
    rc = lib.tmh_matrix_roundtrip(w.ctypes.data, 1, 32, x.ctypes.data, 1, 0, y.ctypes.data,
                                  x.ctypes.data, 0, err, 512)
    assert rc != 0 and b"1-D" in err.value
