"""Seeded synthetic inputs of the benchmark's shape: Q8_0 weights quantized
from N(0, 0.02) source weights with the ggml rule, and N(0, 1) activations.

The quantization rule is the one the reference applies to activations
(crates/tuckcore/src/tensor.rs:184-206): per block of 32, d = amax/127,
id = 1/d (0 when d == 0), q = clamp(round_ties_even(w*id), -127, 127), and the
stored scale is the binary16 rounding of d.
"""
from __future__ import annotations

import zlib

import numpy as np

BLOCK = 32
BLOCK_BYTES = 34

# Shapes (rows N, cols K) of the benchmark configurations.
QWEN3_0_6B_LAYER = (
    ("q", 2048, 1024), ("k", 1024, 1024), ("v", 1024, 1024), ("o", 1024, 2048),
    ("gate", 3072, 1024), ("up", 3072, 1024), ("down", 1024, 3072),
)
QWEN3_0_6B_LAYERS = 28
QWEN3_0_6B_LM_HEAD = ("lm_head", 151936, 1024)
GEMMA3_1B = (("gate", 6912, 1152), ("up", 6912, 1152), ("down", 1152, 6912),
             ("lm_head", 262144, 1152))
SWEEP_2B = (("gate", 6144, 2048), ("down", 2048, 6144))


def tensor_seed(config: int, layer: int, name: str) -> int:
    """Documented per-tensor seed: config 0 uses seed 0 for its one tensor."""
    if config == 0:
        return 0
    return zlib.crc32(f"{config}/{layer}/{name}".encode()) & 0x7FFFFFFF


def q8_0_bytes(rows: int, cols: int) -> int:
    return rows * (cols // BLOCK) * BLOCK_BYTES


def gemv_bytes(rows: int, cols: int) -> int:
    """Algorithmic bytes of one GEMV: weights once, x, y."""
    return q8_0_bytes(rows, cols) + 4 * cols + 4 * rows


def quantize_q8_0(w: np.ndarray) -> np.ndarray:
    """f32 [rows, cols] -> raw GGUF Q8_0 bytes (uint8, rows*(cols/32)*34)."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    rows, cols = w.shape
    assert cols % BLOCK == 0
    blk = w.reshape(rows * (cols // BLOCK), BLOCK)
    amax = np.abs(blk).max(axis=1)
    d = (amax / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, np.float32(1.0) / d, np.float32(0.0)).astype(np.float32)
    q = np.rint(blk * inv[:, None])
    np.clip(q, -127, 127, out=q)
    out = np.empty((blk.shape[0], BLOCK_BYTES), dtype=np.uint8)
    with np.errstate(over="ignore"):
        out[:, 0:2] = d.astype(np.float16).view(np.uint8).reshape(-1, 2)
    out[:, 2:] = q.astype(np.int8).view(np.uint8)
    return out.reshape(-1)


def _weights_chunk(args):
    seed, chunk, n, cols, std = args
    rng = np.random.default_rng([seed, chunk])
    w = rng.standard_normal((n, cols), dtype=np.float32)
    w *= np.float32(std)
    return quantize_q8_0(w)


def make_weights(rows: int, cols: int, seed: int, std: float = 0.02,
                 chunk_rows: int = 4096, threads: int = 8) -> np.ndarray:
    """Raw Q8_0 bytes of a [rows, cols] matrix drawn N(0, std), seeded. Row
    chunk c is drawn from its own stream (seed, c), so the bytes do not depend
    on the thread count."""
    from concurrent.futures import ThreadPoolExecutor

    out = np.empty(q8_0_bytes(rows, cols), dtype=np.uint8)
    row_bytes = (cols // BLOCK) * BLOCK_BYTES
    jobs = [(seed, c, min(chunk_rows, rows - r0), cols, std)
            for c, r0 in enumerate(range(0, rows, chunk_rows))]
    if len(jobs) == 1 or threads <= 1:
        parts = map(_weights_chunk, jobs)
    else:
        pool = ThreadPoolExecutor(max_workers=threads)
        parts = pool.map(_weights_chunk, jobs)
    r0 = 0
    for job, part in zip(jobs, parts):
        out[r0 * row_bytes:(r0 + job[2]) * row_bytes] = part
        r0 += job[2]
    return out


def make_activations(n: int, seed: int) -> np.ndarray:
    return np.random.default_rng(seed ^ 0x5EED).standard_normal(n, dtype=np.float32)


def pack_q8_0(raw: np.ndarray, rows: int, cols: int) -> np.ndarray:
    """Host statement of the sealed device layout (quants, then scales)."""
    blk = np.ascontiguousarray(raw).view(np.uint8).reshape(rows * (cols // BLOCK), BLOCK_BYTES)
    return np.concatenate([blk[:, 2:].reshape(-1), blk[:, :2].reshape(-1)])
