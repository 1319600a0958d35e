"""Pins the oracle's restatements of the small f32 operators around the products.

Known answers come from the reference's own tests (cited per case); what those
leave open is fixed by mathematics: float64 closed forms, exact special cases
and an independent brute-force argmax.
"""
import math

import numpy as np
import pytest

import oracle as O


def test_rmsnorm_reference_known_answer():
    # crates/tuckcore/src/forward.rs:1016-1023: x = [3, 4], w = [1, 1], eps = 0.
    y = O.rmsnorm([3.0, 4.0], [1.0, 1.0], 0.0)
    rms = math.sqrt((9.0 + 16.0) / 2.0)
    assert abs(y[0] - 3.0 / rms) < 1e-6 and abs(y[1] - 4.0 / rms) < 1e-6


def test_rmsnorm_against_float64_and_exact_cases():
    rng = np.random.default_rng(5)
    for n in (1, 7, 128, 1024, 1152):
        x = rng.standard_normal(n).astype(np.float32) * np.float32(3.0)
        w = (0.5 + rng.random(n)).astype(np.float32)
        for eps in (0.0, 1e-6, 1e-5):
            y = O.rmsnorm(x, w, eps)
            x64 = x.astype(np.float64)
            want = x64 / np.sqrt(np.mean(x64 * x64) + eps) * w.astype(np.float64)
            assert np.max(np.abs(y - want)) <= 2e-6 * max(1.0, np.max(np.abs(want)))
    # exact: all-equal powers of two normalise to exactly +-1 times the weight
    y = O.rmsnorm(np.full(64, -4.0, np.float32), np.full(64, 0.75, np.float32), 0.0)
    assert np.array_equal(y, np.full(64, -0.75, np.float32))
    # the sum of squares is sequential f32: a transposed accumulation order differs here
    x = np.array([4096.0] + [0.25] * 4095, np.float32)
    seq = np.float32(0.0)
    for v in x:
        seq = np.float32(seq + np.float32(v * v))
    inv = np.float32(1.0) / np.sqrt(np.float32(seq / np.float32(x.size) + np.float32(1e-6)))
    want = (x * inv) * np.ones_like(x)
    assert np.array_equal(O.rmsnorm(x, np.ones_like(x), 1e-6), want.astype(np.float32))
    with pytest.raises(O.OracleError):
        O.rmsnorm([1.0, 2.0], [1.0], 0.0)


def test_silu_mul_reference_bounds_and_float64():
    # crates/tuckcore/src/forward.rs:1044-1048
    s = O.silu_mul([0.0, 10.0, -10.0], [1.0, 1.0, 1.0])
    assert abs(s[0]) < 1e-8 and s[1] > 9.9 and -0.001 < s[2] < 0.0
    rng = np.random.default_rng(19)
    g = ((rng.integers(0, 20001, 4097) - 10000) / 1000.0).astype(np.float32)  # tests.rs:631-637 grid
    u = ((rng.integers(0, 20001, 4097) - 10000) / 1000.0).astype(np.float32)
    got = O.silu_mul(g, u)
    g64, u64 = g.astype(np.float64), u.astype(np.float64)
    want = g64 / (1.0 + np.exp(-g64)) * u64
    assert np.max(np.abs(got - want)) <= 1e-6 * max(1.0, np.max(np.abs(want)))
    # up scales linearly and exactly by powers of two
    assert np.array_equal(O.silu_mul(g, 2.0 * u), 2.0 * got)


def test_gelu_tanh_mul_closed_form():
    # native/metal/kernels.metal:382-396 is the only definition the reference holds.
    assert O.gelu_tanh_mul([0.0], [3.0])[0] == 0.0
    big = O.gelu_tanh_mul([12.0, -12.0], [1.0, 1.0])
    assert big[0] == np.float32(12.0) and big[1] == 0.0  # tanh saturates to +-1 exactly
    rng = np.random.default_rng(23)
    g = (rng.standard_normal(4096) * 3.0).astype(np.float32)
    u = rng.standard_normal(4096).astype(np.float32)
    got = O.gelu_tanh_mul(g, u)
    x = g.astype(np.float64)
    want = 0.5 * x * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * x * (1.0 + 0.044715 * x * x)))
    want = want * u.astype(np.float64)
    assert np.max(np.abs(got - want)) <= 2e-6 * max(1.0, np.max(np.abs(want)))
    # odd-symmetric part: gelu(x) - gelu(-x) = x
    pos = O.gelu_tanh_mul(np.abs(g), np.ones_like(g))
    neg = O.gelu_tanh_mul(-np.abs(g), np.ones_like(g))
    assert np.max(np.abs((pos - neg) - np.abs(g))) <= 1e-5


def test_axpy_and_scale_are_single_rounded_operations():
    rng = np.random.default_rng(3)
    a = rng.standard_normal(1000).astype(np.float32)
    y = rng.standard_normal(1000).astype(np.float32)
    alpha = np.float32(0.37)
    want = (y + (alpha * a).astype(np.float32)).astype(np.float32)  # two roundings, no fma
    assert np.array_equal(O.axpy(a, alpha, y), want)
    assert np.array_equal(O.scale(a, alpha), (a * alpha).astype(np.float32))
    # a case where a fused multiply-add would round differently
    a1, y1, al = np.float32(1.0 + 2.0 ** -12), np.float32(-1.0), np.float32(1.0 + 2.0 ** -12)
    unfused = np.float32(y1 + np.float32(al * a1))
    fused = np.float32(np.float64(al) * np.float64(a1) + np.float64(y1))
    assert unfused != fused
    assert O.axpy([a1], al, [y1])[0] == unfused


def brute_argmax(x):
    best = None
    for i, v in enumerate(x):
        if v != v:
            continue
        if best is None or v > x[best]:
            best = i
    return O.ARGMAX_NONE if best is None else best


def test_argmax_reference_cases():
    # crates/metal/src/tests.rs:1271-1281
    nan, inf = float("nan"), float("inf")
    cases = [([1.0, 3.0, 2.0], 1), ([3.0, 3.0], 0), ([nan, 1.0], 1), ([nan, inf], 1),
             ([nan, nan, nan], O.ARGMAX_NONE), ([-inf, -inf], 0), ([-0.0, 0.0], 0),
             ([0.0, -0.0], 0), ([7.5], 0)]
    for x, want in cases:
        assert O.argmax(x) == want, x
    # crates/metal/src/tests.rs:1284-1299: planted maxima resolve to the lowest index
    rng = np.random.default_rng(0xA11CE)
    big = (rng.random(248_320) * 20.0 - 10.0).astype(np.float32)
    for k in (200_000, 77_777, 131_071, 77_776):
        big[k] = 42.0
    big[5] = np.nan
    assert O.argmax(big) == 77_776
    for n in (255, 256, 16_384, 16_385, 70_001):
        v = np.ones(n, np.float32)
        v[n - 1] = 2.0
        v[n // 2] = 2.0
        assert O.argmax(v) == n // 2
    small = (rng.standard_normal(300)).astype(np.float32)
    small[::7] = np.nan
    assert O.argmax(small) == brute_argmax(small.tolist())
