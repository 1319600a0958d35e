"""Helpers shared by the GPU parity tests (not collected by pytest)."""
from __future__ import annotations

import numpy as np
import pytest

import oracle as O
from tuckmill_amd import hip as H


def require_gpu() -> H.HipContext:
    p = H.probe()
    if not p.available:
        pytest.fail(f"-m gpu tests need an MI355X: {p.info}")
    return H.HipContext.open()


def upload_new(ctx: H.HipContext, data, shared: bool = True) -> H.HipBuffer:
    arr = np.ascontiguousarray(data)
    buf = ctx.buffer(arr.nbytes, shared)
    buf.upload(0, arr)
    return buf


def weights_buffer(ctx: H.HipContext, raw: np.ndarray, rows: int, cols: int, packed: bool):
    buf = upload_new(ctx, raw)
    if packed:
        ctx.q8_0_pack(buf, rows, cols)
    return buf


def gemv(ctx, wbuf, x: np.ndarray, rows: int, cols: int) -> np.ndarray:
    xb = upload_new(ctx, x.astype(np.float32))
    yb = ctx.buffer(rows * 4)
    ctx.q8_0_gemv(wbuf, xb, yb, rows, cols)
    ctx.fence()
    y = yb.download_f32(0, rows).copy()
    xb.free()
    yb.free()
    return y


def norm_err(got: np.ndarray, want: np.ndarray) -> float:
    """max_i |got - want| / ||want||_inf: the parity metric of the f32 path."""
    scale = float(np.max(np.abs(want)))
    if scale == 0.0:
        return float(np.max(np.abs(got)))
    return float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64))) / scale)


def ref_scale(want: np.ndarray) -> float:
    """max(||want||_inf, 1): the reference's own normalisation
    (crates/metal/src/tests.rs:367)."""
    return max(float(np.max(np.abs(want))), 1.0)


def bits(a: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
