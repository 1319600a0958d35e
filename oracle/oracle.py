"""ctypes/numpy front end of ``libq8_oracle.so`` (the C restatement of
TuckCore's scalar Q8_0 path). TEST INFRASTRUCTURE ONLY.

Each wrapper keeps the reference's argument meaning and error behaviour:
the checked dot entry points raise ``OracleError`` with the reference's
error-code name where `crates/tuckcore/src/kernels.rs:368-400` returns
``Err``.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libq8_oracle.so")

__all__ = [
    "OracleError", "build", "lib", "f16_to_f32", "f32_to_f16_bits", "f16_to_f32_array",
    "f32_to_f16_bits_array", "dequant_q8_0",
    "quantize_row_q8_0", "dot_q8_0_x_f32", "dot_q8_0_q8_0", "gemv_q8_0_f32",
    "gemv_q8_0_q8_0", "gemm_q8_0_f32", "gemm_q8_0_q8_0", "gemv_q8_0_f32_dequant_first",
    "gemv_q8_0_f64", "Rng", "boundary_weights", "boundary_input", "KRng",
    "random_q8_0_row", "block_sumi", "rmsnorm", "silu_mul", "gelu_tanh_mul", "axpy", "scale",
    "argmax", "ARGMAX_NONE", "dot_f16_x_f32", "gemm_f16_f32", "f16_bytes",
]


class OracleError(Exception):
    """Mirrors a ``TuckmillError``: ``code`` is the reference's ErrorCode name."""

    def __init__(self, code: str, message: str):
        super().__init__(f"{code}: {message}")
        self.code = code


def build(force: bool = False) -> str:
    """Compile the oracle with its Makefile (gcc only, no GPU needed)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        c = ctypes
        u8p, f32p, i8p = c.c_void_p, c.c_void_p, c.c_void_p
        L.q8o_f16_to_f32.restype = c.c_float
        L.q8o_f16_to_f32.argtypes = [c.c_uint16]
        L.q8o_f32_to_f16_bits.restype = c.c_uint16
        L.q8o_f32_to_f16_bits.argtypes = [c.c_float]
        L.q8o_f16_to_f32_n.restype = None
        L.q8o_f16_to_f32_n.argtypes = [c.c_void_p, c.c_size_t, f32p]
        L.q8o_f32_to_f16_bits_n.restype = None
        L.q8o_f32_to_f16_bits_n.argtypes = [f32p, c.c_size_t, c.c_void_p]
        L.q8o_dequant_q8_0.argtypes = [u8p, c.c_size_t, f32p]
        L.q8o_quantize_row_q8_0.argtypes = [f32p, c.c_size_t, i8p, f32p]
        L.q8o_validate_q8_0_row.argtypes = [c.c_size_t, c.c_size_t]
        L.q8o_validate_q8_0_q8_0.argtypes = [c.c_size_t, c.c_size_t, c.c_size_t]
        L.q8o_dot_q8_0_x_f32.restype = c.c_float
        L.q8o_dot_q8_0_x_f32.argtypes = [u8p, c.c_size_t, f32p]
        L.q8o_dot_q8_0_q8_0.restype = c.c_float
        L.q8o_dot_q8_0_q8_0.argtypes = [u8p, c.c_size_t, i8p, f32p, c.c_void_p]
        for name in ("q8o_gemv_q8_0_f32", "q8o_gemv_q8_0_q8_0"):
            getattr(L, name).argtypes = [u8p, c.c_size_t, c.c_size_t, f32p, f32p, c.c_int]
        for name in ("q8o_gemm_q8_0_f32", "q8o_gemm_q8_0_q8_0"):
            getattr(L, name).argtypes = [u8p, c.c_size_t, c.c_size_t, f32p, c.c_size_t,
                                         f32p, c.c_int]
        L.q8o_validate_f16_row.argtypes = [c.c_size_t, c.c_size_t]
        L.q8o_dot_f16_x_f32.restype = c.c_float
        L.q8o_dot_f16_x_f32.argtypes = [u8p, c.c_size_t, f32p]
        L.q8o_gemm_f16_f32.argtypes = [u8p, c.c_size_t, c.c_size_t, f32p, c.c_size_t, f32p]
        L.q8o_gemv_q8_0_f32_dequant_first.argtypes = [u8p, c.c_size_t, c.c_size_t, f32p, f32p]
        L.q8o_gemv_q8_0_f64.argtypes = [u8p, c.c_size_t, c.c_size_t, f32p, c.c_void_p]
        L.q8o_rng_next.restype = c.c_uint64
        L.q8o_rng_next.argtypes = [c.POINTER(c.c_uint64)]
        L.q8o_boundary_weights.argtypes = [c.c_size_t, c.c_size_t, c.c_uint64, u8p]
        L.q8o_boundary_input.argtypes = [c.c_size_t, c.c_uint64, f32p]
        L.q8o_krng_next_f32.restype = c.c_float
        L.q8o_krng_next_f32.argtypes = [c.POINTER(c.c_uint64), c.c_float]
        L.q8o_random_q8_0_row.argtypes = [c.POINTER(c.c_uint64), c.c_size_t, u8p]
        L.q8o_rmsnorm.argtypes = [f32p, f32p, c.c_size_t, c.c_float, f32p]
        L.q8o_silu_mul.argtypes = [f32p, f32p, c.c_size_t, f32p]
        L.q8o_gelu_tanh_mul.argtypes = [f32p, f32p, c.c_size_t, f32p]
        L.q8o_axpy.argtypes = [f32p, c.c_float, c.c_size_t, f32p]
        L.q8o_scale.argtypes = [f32p, c.c_float, c.c_size_t, f32p]
        L.q8o_argmax.restype = c.c_uint32
        L.q8o_argmax.argtypes = [f32p, c.c_size_t]
        _lib = L
    return _lib


def _ptr(a: np.ndarray) -> int:
    return a.ctypes.data


def _u8(a) -> np.ndarray:
    a = np.ascontiguousarray(np.frombuffer(a, dtype=np.uint8) if isinstance(a, (bytes, bytearray))
                             else a)
    if a.dtype != np.uint8:
        a = a.view(np.uint8)
    return a


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


# ---------------------------------------------------------------- scalars --

def f16_to_f32(bits: int) -> np.float32:
    return np.float32(lib().q8o_f16_to_f32(int(bits) & 0xFFFF))


def f32_to_f16_bits(value) -> int:
    return int(lib().q8o_f32_to_f16_bits(float(np.float32(value))))


def f16_to_f32_array(bits) -> np.ndarray:
    b = np.ascontiguousarray(bits, dtype=np.uint16).ravel()
    out = np.empty(b.size, dtype=np.float32)
    lib().q8o_f16_to_f32_n(_ptr(b), b.size, _ptr(out))
    return out


def f32_to_f16_bits_array(values) -> np.ndarray:
    v = _f32(values).ravel()
    out = np.empty(v.size, dtype=np.uint16)
    lib().q8o_f32_to_f16_bits_n(_ptr(v), v.size, _ptr(out))
    return out


def dequant_q8_0(raw) -> np.ndarray:
    raw = _u8(raw)
    if raw.size % 34 != 0:
        raise OracleError("InvalidArtifact", "Q8_0 bytes are not block aligned")
    out = np.empty(raw.size // 34 * 32, dtype=np.float32)
    lib().q8o_dequant_q8_0(_ptr(raw), raw.size // 34, _ptr(out))
    return out


def quantize_row_q8_0(x):
    """Returns (qs int8 [blocks, 32], d float32 [blocks]) like the reference's
    ``quantize_row_q8_0`` fills its two vectors."""
    x = _f32(x).ravel()
    if x.size % 32 != 0:
        raise OracleError("Internal", "activation length is not a multiple of 32")
    qs = np.empty(x.size, dtype=np.int8)
    d = np.empty(x.size // 32, dtype=np.float32)
    lib().q8o_quantize_row_q8_0(_ptr(x), x.size, _ptr(qs), _ptr(d))
    return qs.reshape(-1, 32), d


# ------------------------------------------------------------------- dots --

def dot_q8_0_x_f32(row, x) -> np.float32:
    row = _u8(row)
    x = _f32(x).ravel()
    rc = lib().q8o_validate_q8_0_row(row.size, x.size)
    if rc == -1:
        raise OracleError("InvalidArtifact", f"packed Q8_0 row length {row.size} is not a "
                          "positive multiple of 34 bytes")
    if rc == -2:
        raise OracleError("Internal", f"Q8_0 x f32 dot expects {row.size // 34 * 32} "
                          f"activation elements, got {x.size}")
    return np.float32(lib().q8o_dot_q8_0_x_f32(_ptr(row), row.size // 34, _ptr(x)))


def dot_f16_x_f32(row, x) -> np.float32:
    """kernels.rs:402-410 over scalar::dot_f16_x_f32, with its checked boundary."""
    row = _u8(row)
    x = _f32(x).ravel()
    rc = lib().q8o_validate_f16_row(row.size, x.size)
    if rc == -1:
        raise OracleError("InvalidArtifact", f"packed F16 row length {row.size} is not a "
                          "positive multiple of 2 bytes")
    if rc == -2:
        raise OracleError("Internal", f"F16 x f32 dot expects {row.size // 2} activation "
                          f"elements, got {x.size}")
    return np.float32(lib().q8o_dot_f16_x_f32(_ptr(row), row.size // 2, _ptr(x)))


def gemm_f16_f32(w, rows, cols, x, batch=1) -> np.ndarray:
    """y[b, r] = dot_f16_x_f32(row r of w, x[b]); w holds rows*cols f16 values."""
    w = _u8(w)
    x = _f32(x).ravel()
    if rows <= 0 or cols <= 0 or w.size != rows * cols * 2:
        raise OracleError("InvalidArtifact", f"weight bytes {w.size} != {rows}x{cols} F16")
    if x.size != batch * cols:
        raise OracleError("Internal", f"expects {batch * cols} activation elements, got {x.size}")
    y = np.empty(batch * rows, dtype=np.float32)
    lib().q8o_gemm_f16_f32(_ptr(w), rows, cols, _ptr(x), batch, _ptr(y))
    return y.reshape(batch, rows) if batch > 1 else y


def f16_bytes(values) -> np.ndarray:
    """f32 values -> little-endian f16 bytes through f32_to_f16_bits (the
    fixture construction of crates/metal/src/tests.rs:688-695)."""
    v = _f32(values).ravel()
    out = np.empty(v.size, dtype="<u2")
    for i, f in enumerate(v):
        out[i] = f32_to_f16_bits(f)
    return out.view(np.uint8)


def dot_q8_0_q8_0(row, x_qs, x_d) -> np.float32:
    row = _u8(row)
    x_qs = np.ascontiguousarray(x_qs, dtype=np.int8).reshape(-1, 32)
    x_d = _f32(x_d).ravel()
    rc = lib().q8o_validate_q8_0_q8_0(row.size, x_qs.shape[0], x_d.size)
    if rc == -1:
        raise OracleError("InvalidArtifact", f"packed Q8_0 row length {row.size} is not a "
                          "positive multiple of 34 bytes")
    if rc == -2:
        raise OracleError("Internal", "Q8_0 x q8_0 block/scale count mismatch")
    return np.float32(lib().q8o_dot_q8_0_q8_0(_ptr(row), row.size // 34, _ptr(x_qs),
                                              _ptr(x_d), None))


def block_sumi(row, x_qs) -> np.ndarray:
    """The exact i32 block dots of one weight row against quantized activations."""
    row = _u8(row)
    x_qs = np.ascontiguousarray(x_qs, dtype=np.int8).reshape(-1, 32)
    blocks = row.size // 34
    out = np.empty(blocks, dtype=np.int32)
    d = np.ones(blocks, dtype=np.float32)
    lib().q8o_dot_q8_0_q8_0(_ptr(row), blocks, _ptr(x_qs), _ptr(d), _ptr(out))
    return out


def _check_matrix(w, rows, cols):
    if rows <= 0 or cols <= 0 or cols % 32 != 0:
        raise OracleError("InvalidArtifact", f"rows {rows}, cols {cols}")
    if w.size != rows * (cols // 32) * 34:
        raise OracleError("InvalidArtifact", f"weight bytes {w.size} != {rows}x{cols} Q8_0")


def gemv_q8_0_f32(w, rows, cols, x, threads: int = 1) -> np.ndarray:
    w = _u8(w)
    x = _f32(x).ravel()
    _check_matrix(w, rows, cols)
    if x.size != cols:
        raise OracleError("Internal", f"expects {cols} activation elements, got {x.size}")
    y = np.empty(rows, dtype=np.float32)
    lib().q8o_gemv_q8_0_f32(_ptr(w), rows, cols, _ptr(x), _ptr(y), threads)
    return y


def gemv_q8_0_q8_0(w, rows, cols, x, threads: int = 1) -> np.ndarray:
    w = _u8(w)
    x = _f32(x).ravel()
    _check_matrix(w, rows, cols)
    if x.size != cols:
        raise OracleError("Internal", f"expects {cols} activation elements, got {x.size}")
    y = np.empty(rows, dtype=np.float32)
    lib().q8o_gemv_q8_0_q8_0(_ptr(w), rows, cols, _ptr(x), _ptr(y), threads)
    return y


def gemm_q8_0_f32(w, rows, cols, x, batch, threads: int = 1) -> np.ndarray:
    w = _u8(w)
    x = _f32(x).ravel()
    _check_matrix(w, rows, cols)
    if x.size != batch * cols:
        raise OracleError("Internal", "activation size mismatch")
    y = np.empty((batch, rows), dtype=np.float32)
    lib().q8o_gemm_q8_0_f32(_ptr(w), rows, cols, _ptr(x), batch, _ptr(y), threads)
    return y


def gemm_q8_0_q8_0(w, rows, cols, x, batch, threads: int = 1) -> np.ndarray:
    w = _u8(w)
    x = _f32(x).ravel()
    _check_matrix(w, rows, cols)
    if x.size != batch * cols:
        raise OracleError("Internal", "activation size mismatch")
    y = np.empty((batch, rows), dtype=np.float32)
    lib().q8o_gemm_q8_0_q8_0(_ptr(w), rows, cols, _ptr(x), batch, _ptr(y), threads)
    return y


def gemv_q8_0_f32_dequant_first(w, rows, cols, x) -> np.ndarray:
    w = _u8(w)
    x = _f32(x).ravel()
    _check_matrix(w, rows, cols)
    y = np.empty(rows, dtype=np.float32)
    lib().q8o_gemv_q8_0_f32_dequant_first(_ptr(w), rows, cols, _ptr(x), _ptr(y))
    return y


def gemv_q8_0_f64(w, rows, cols, x) -> np.ndarray:
    w = _u8(w)
    x = _f32(x).ravel()
    _check_matrix(w, rows, cols)
    y = np.empty(rows, dtype=np.float64)
    lib().q8o_gemv_q8_0_f64(_ptr(w), rows, cols, _ptr(x), _ptr(y))
    return y


# ------------------------------------------ operators around the products --

def rmsnorm(x, w, eps) -> np.ndarray:
    """One row (crates/tuckcore/src/forward.rs:911-927)."""
    x, w = _f32(x).ravel(), _f32(w).ravel()
    if x.size == 0 or x.size != w.size:
        raise OracleError("Internal", "rmsnorm: x and weight lengths differ or are zero")
    y = np.empty_like(x)
    lib().q8o_rmsnorm(_ptr(x), _ptr(w), x.size, float(eps), _ptr(y))
    return y


def silu_mul(gate, up) -> np.ndarray:
    gate, up = _f32(gate).ravel(), _f32(up).ravel()
    out = np.empty_like(gate)
    lib().q8o_silu_mul(_ptr(gate), _ptr(up), gate.size, _ptr(out))
    return out


def gelu_tanh_mul(gate, up) -> np.ndarray:
    gate, up = _f32(gate).ravel(), _f32(up).ravel()
    out = np.empty_like(gate)
    lib().q8o_gelu_tanh_mul(_ptr(gate), _ptr(up), gate.size, _ptr(out))
    return out


def axpy(a, alpha, y) -> np.ndarray:
    a = _f32(a).ravel()
    out = _f32(y).ravel().copy()
    lib().q8o_axpy(_ptr(a), float(alpha), a.size, _ptr(out))
    return out


def scale(x, factor) -> np.ndarray:
    x = _f32(x).ravel()
    out = np.empty_like(x)
    lib().q8o_scale(_ptr(x), float(factor), x.size, _ptr(out))
    return out


ARGMAX_NONE = 0xFFFFFFFF


def argmax(x) -> int:
    """Greedy rule of crates/backend/src/sampling.rs:69-83; ARGMAX_NONE when all NaN."""
    x = _f32(x).ravel()
    return int(lib().q8o_argmax(_ptr(x), x.size))


# ------------------------------------------------------------- generators --

class Rng:
    """xorshift64* stream of the reference's operator tests."""

    def __init__(self, seed: int):
        self._s = ctypes.c_uint64(seed)

    def next(self) -> int:
        return int(lib().q8o_rng_next(ctypes.byref(self._s)))


def boundary_weights(rows: int, cols: int, seed: int) -> np.ndarray:
    out = np.empty(rows * (cols // 32) * 34, dtype=np.uint8)
    lib().q8o_boundary_weights(rows, cols, seed, _ptr(out))
    return out


def boundary_input(n: int, seed: int) -> np.ndarray:
    out = np.empty(n, dtype=np.float32)
    lib().q8o_boundary_input(n, seed, _ptr(out))
    return out


class KRng:
    """The xorshift stream of the reference's CPU-kernel tests."""

    def __init__(self, seed: int):
        self._s = ctypes.c_uint64(seed)

    def next_f32(self, scale: float) -> np.float32:
        return np.float32(lib().q8o_krng_next_f32(ctypes.byref(self._s), scale))

    def row(self, blocks: int) -> np.ndarray:
        out = np.empty(blocks * 34, dtype=np.uint8)
        lib().q8o_random_q8_0_row(ctypes.byref(self._s), blocks, _ptr(out))
        return out


def random_q8_0_row(rng: KRng, blocks: int) -> np.ndarray:
    return rng.row(blocks)
