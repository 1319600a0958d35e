"""Pins the oracle's F16-weight dot product (the reference's F16 twin of the
Q8_0 product, crates/tuckcore/src/kernels.rs:223-232).

Known answers from the reference's tests where it has them; the rest from what
the arithmetic fixes: exact integer cases, a case only the sequential order
satisfies, and a float64 evaluation within the rounding bound.
"""
import numpy as np
import pytest

import oracle as O


def f16(values):
    return np.asarray(values, dtype=np.float16).view(np.uint8)


def test_reference_zero_row_and_error_cases():
    # crates/tuckcore/src/kernels.rs:596-598: a zero row gives exactly 0.0
    x = np.arange(64, dtype=np.float32)
    assert O.dot_f16_x_f32(np.zeros(128, np.uint8), x) == 0.0
    # kernels.rs:583-586: odd byte length, short and over-long activations
    with pytest.raises(O.OracleError) as e:
        O.dot_f16_x_f32(np.zeros(5, np.uint8), np.zeros(2, np.float32))
    assert e.value.code == "InvalidArtifact"
    for n in (1, 3):
        with pytest.raises(O.OracleError) as e:
            O.dot_f16_x_f32(np.zeros(4, np.uint8), np.zeros(n, np.float32))
        assert e.value.code == "Internal"
    with pytest.raises(O.OracleError):
        O.dot_f16_x_f32(np.zeros(0, np.uint8), np.zeros(0, np.float32))


def test_exact_integer_cases():
    # ones times twos (the shape of crates/metal/src/tests.rs:310-330 for Q8_0)
    assert O.dot_f16_x_f32(f16(np.ones(64)), np.full(64, 2.0, np.float32)) == 128.0
    # small integers: every product and partial sum is an integer below 2^24
    rng = np.random.default_rng(3)
    w = rng.integers(-64, 65, 999)
    x = rng.integers(-100, 101, 999)
    assert O.dot_f16_x_f32(f16(w), x.astype(np.float32)) == float(np.dot(w, x))
    # a transposed operand or an off-by-one index fails this one
    w = np.arange(1, 9)
    x = np.array([1, 10, 100, 1000, 1, 10, 100, 1000], np.float32)
    assert O.dot_f16_x_f32(f16(w), x) == float(1 + 20 + 300 + 4000 + 5 + 60 + 700 + 8000)
    # f16 decoding goes through f16_to_f32: a subnormal and a negative value
    row = np.array([0x0001, 0xC000], dtype="<u2").view(np.uint8)
    assert O.dot_f16_x_f32(row, np.array([2.0 ** 24, 0.5], np.float32)) == 1.0 - 1.0


def test_sequential_order_from_zero():
    # 2^24 + 1 + 1 + ... stays 2^24 only when summed left to right in f32;
    # pairwise or reversed orders give 2^24 + n.
    n = 16
    w = f16([1.0] * (n + 1))
    x = np.array([2.0 ** 24] + [1.0] * n, np.float32)
    assert O.dot_f16_x_f32(w, x) == 2.0 ** 24
    x_rev = x[::-1].copy()
    assert O.dot_f16_x_f32(w, x_rev) == 2.0 ** 24 + n
    # products are rounded to f32 before the addition (no fused multiply-add):
    # w*x = (1 + 2^-10)(1 + 2^-23) rounds to 1 + 2^-10 + 2^-23 (the tail 2^-33 is
    # lost), so adding -(1 + 2^-10 + 2^-23) gives 0; a fused form keeps 2^-33.
    w = f16([1.0 + 2.0 ** -10, 1.0])
    a = np.float32(1.0 + 2.0 ** -23)
    prod = np.float32(np.float32(1.0 + 2.0 ** -10) * a)
    got = O.dot_f16_x_f32(w[[2, 3, 0, 1]], np.array([-prod, a], np.float32))
    assert got == 0.0


def test_against_float64_within_the_rounding_bound():
    rng = np.random.default_rng(11)
    for cols in (1, 2, 31, 32, 33, 1024, 3072):
        w = rng.standard_normal(cols).astype(np.float16)
        x = rng.standard_normal(cols).astype(np.float32)
        got = float(O.dot_f16_x_f32(w.view(np.uint8), x))
        terms = w.astype(np.float64) * x.astype(np.float64)
        bound = (cols + 1) * 2.0 ** -24 * float(np.sum(np.abs(terms))) + 1e-30
        assert abs(got - float(np.sum(terms))) <= bound


def test_gemm_is_the_row_loop_of_the_dot():
    rng = np.random.default_rng(13)
    rows, cols, batch = 5, 40, 3
    w = rng.standard_normal(rows * cols).astype(np.float16).view(np.uint8)
    x = rng.standard_normal(batch * cols).astype(np.float32)
    y = O.gemm_f16_f32(w, rows, cols, x, batch)
    assert y.shape == (batch, rows)
    for b in range(batch):
        for r in range(rows):
            want = O.dot_f16_x_f32(w[r * cols * 2:(r + 1) * cols * 2], x[b * cols:(b + 1) * cols])
            assert y[b, r] == want
    assert np.array_equal(O.gemm_f16_f32(w, rows, cols, x[:cols]), y[0])
    with pytest.raises(O.OracleError):
        O.gemm_f16_f32(w[:-2], rows, cols, x, batch)


def test_f16_bytes_uses_the_reference_rounding():
    # crates/tuckcore/src/tensor.rs:358-370 known values through the helper
    got = O.f16_bytes([0.0, 1.0, -2.0, 65504.0, 1e5]).view("<u2")
    assert list(got) == [0x0000, 0x3C00, 0xC000, 0x7BFF, 0x7C00]
