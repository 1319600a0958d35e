"""Pins the CPU oracle (oracle/q8_oracle.c) before anything is compared to it.

Sources of truth used here, none of which is the oracle's own formula:
  * the known answers held by the reference's tests
    (crates/tuckcore/src/tensor.rs:263-392, crates/tuckcore/src/kernels.rs:560-599,
    crates/metal/src/tests.rs:257-330),
  * numpy's float16 conversions (an independent IEEE implementation),
  * exact rational arithmetic with an explicit round-to-nearest-even step
    (detects a fused multiply-add, a reassociated sum or a wrong loop order),
  * integer brute force and closed forms that are exact in f32.
"""
from fractions import Fraction

import numpy as np
import pytest

import oracle as O

MASK64 = (1 << 64) - 1


# ------------------------------------------------------------ f16 decode --

def test_f16_known_values():
    # crates/tuckcore/src/tensor.rs:264-272
    assert O.f16_to_f32(0x3C00) == 1.0
    assert O.f16_to_f32(0xC000) == -2.0
    assert O.f16_to_f32(0x0000) == 0.0
    assert np.isinf(O.f16_to_f32(0x7C00))
    assert np.isnan(O.f16_to_f32(0x7C01))
    assert O.f16_to_f32(0x0001) == np.float32(2.0 ** -24)


def test_f16_to_f32_exhaustive_against_numpy():
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([O.f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


# ------------------------------------------------------------ f16 encode --

def test_f32_to_f16_known_values():
    # crates/tuckcore/src/tensor.rs:358-370
    assert O.f32_to_f16_bits(0.0) == 0x0000
    assert O.f32_to_f16_bits(1.0) == 0x3C00
    assert O.f32_to_f16_bits(-2.0) == 0xC000
    assert O.f32_to_f16_bits(65504.0) == 0x7BFF
    assert O.f32_to_f16_bits(100000.0) == 0x7C00
    assert O.f32_to_f16_bits(5.96e-8) == 0x0001
    assert O.f32_to_f16_bits(1.0 + 2.0 ** -11) == 0x3C00
    assert O.f32_to_f16_bits(1.0 + 2.0 ** -11 + 2.0 ** -13) == 0x3C01


def _np_f16_bits(values: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        return values.astype(np.float32).astype(np.float16).view(np.uint16)


def test_f32_to_f16_reference_gpu_test_values():
    # crates/metal/src/tests.rs:257-275 (finite and infinite entries)
    values = np.array([0.0, -0.0, 1.0, -1.0, 0.1, 65504.0, 65520.0, 100000.0, -100000.0,
                       5.9604645e-8, 2.9802322e-8, 1.0e-7, -6.0e-8, 44.856, np.pi,
                       np.inf, -np.inf], dtype=np.float32)
    want = _np_f16_bits(values)
    got = np.array([O.f32_to_f16_bits(v) for v in values], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_f32_to_f16_every_f16_value_and_every_midpoint():
    bits = np.arange(0x7C00, dtype=np.uint16)  # all finite non-negative f16
    vals = bits.view(np.float16).astype(np.float32)
    # exact values round-trip
    for sign in (1.0, -1.0):
        got = np.array([O.f32_to_f16_bits(sign * v) for v in vals], dtype=np.uint16)
        assert np.array_equal(got, _np_f16_bits(np.float32(sign) * vals))
    # midpoints between neighbours (exact in f32) and one f32 ulp either side
    mids = (vals[:-1].astype(np.float64) + vals[1:].astype(np.float64)) / 2
    mids = mids.astype(np.float32)
    for arr in (mids, np.nextafter(mids, np.float32(np.inf)),
                np.nextafter(mids, np.float32(-np.inf))):
        got = np.array([O.f32_to_f16_bits(v) for v in arr], dtype=np.uint16)
        assert np.array_equal(got, _np_f16_bits(arr))
    # top of the range: 65520 is the midpoint to 2^16 and rounds to inf
    for v in (65519.996, 65520.0, 65536.0, 1e30):
        assert O.f32_to_f16_bits(v) == int(_np_f16_bits(np.array([v]))[0])


def test_f32_to_f16_dense_random_finite_sample():
    rng = np.random.default_rng(1234)
    raw = rng.integers(0, 1 << 32, size=200_000, dtype=np.uint64).astype(np.uint32)
    vals = raw.view(np.float32)
    vals = vals[np.isfinite(vals)]
    want = _np_f16_bits(vals)
    got = np.array([O.f32_to_f16_bits(v) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)
    # exponents near the f16 range, where most of the branches live
    e = rng.integers(96, 146, size=100_000, dtype=np.uint64).astype(np.uint32)
    m = rng.integers(0, 1 << 23, size=100_000, dtype=np.uint64).astype(np.uint32)
    s = rng.integers(0, 2, size=100_000, dtype=np.uint64).astype(np.uint32)
    vals = ((s << 31) | (e << 23) | m).view(np.float32)
    got = np.array([O.f32_to_f16_bits(v) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, _np_f16_bits(vals))


def test_f32_to_f16_nan_becomes_infinity():
    # crates/tuckcore/src/tensor.rs:150-153: exp >= 0x1f returns sign|0x7c00
    # before looking at the mantissa. A documented divergence from IEEE.
    assert O.f32_to_f16_bits(np.float32(np.nan)) in (0x7C00, 0xFC00)
    neg_nan = np.array([0xFFC00001], dtype=np.uint32).view(np.float32)[0]
    assert O.f32_to_f16_bits(neg_nan) == 0xFC00
    assert O.f32_to_f16_bits(np.float32(np.inf)) == 0x7C00
    assert O.f32_to_f16_bits(np.float32(-np.inf)) == 0xFC00


def test_array_forms_are_the_scalar_functions_element_by_element():
    enc = np.arange(1 << 16, dtype=np.uint16)
    want = np.array([O.f16_to_f32(int(b)) for b in enc], dtype=np.float32)
    assert np.array_equal(O.f16_to_f32_array(enc).view(np.uint32), want.view(np.uint32))
    # a wide sample of f32, with all finite ones against numpy's IEEE rounding too
    rng = np.random.default_rng(77)
    vals = rng.integers(0, 1 << 32, size=2_000_000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    got = O.f32_to_f16_bits_array(vals)
    some = np.array([O.f32_to_f16_bits(v) for v in vals[:50_000]], dtype=np.uint16)
    assert np.array_equal(got[:50_000], some)
    finite = np.isfinite(vals)
    assert np.array_equal(got[finite], _np_f16_bits(vals[finite]))


# ---------------------------------------------------------------- dequant --

def test_q8_0_layout_and_scaling():
    # crates/tuckcore/src/tensor.rs:302-314
    block = bytearray()
    block += (0x3800).to_bytes(2, "little")
    block += bytes([0xFF, 2]) + bytes(30)
    out = O.dequant_q8_0(bytes(block))
    assert out.size == 32
    assert out[0] == -0.5 and out[1] == 1.0 and out[2] == 0.0


def fixture_q8_0(elems: int) -> np.ndarray:
    """The synthetic-GGUF Q8_0 pattern of crates/manifest/src/testing.rs:679-691."""
    blocks = elems // 32
    out = np.zeros(blocks * 34, dtype=np.uint8)
    d = O.f32_to_f16_bits(0.0078125)
    for b in range(blocks):
        out[b * 34] = d & 0xFF
        out[b * 34 + 1] = d >> 8
        for j in range(32):
            q = ((b * 32 + j) * 11 + 5) % 128 - 64
            out[b * 34 + 2 + j] = q & 0xFF
    return out


def test_fixture_pattern_dequant_closed_form():
    raw = fixture_q8_0(4 * 32)
    out = O.dequant_q8_0(raw)
    want = np.array([(((i * 11 + 5) % 128) - 64) / 128.0 for i in range(128)], dtype=np.float32)
    assert np.array_equal(out, want)
    assert out.min() >= -0.5 and out.max() < 0.5


# -------------------------------------------------------------- quantizer --

def test_quantize_matches_ggml_rules_known_answer():
    # crates/tuckcore/src/tensor.rs:373-392
    x = np.zeros(32, dtype=np.float32)
    x[0], x[1], x[2] = 127.0, -63.5, 1.0
    qs, ds = O.quantize_row_q8_0(x)
    assert qs.shape == (1, 32)
    assert ds.tolist() == [1.0]
    assert qs[0, 0] == 127 and qs[0, 1] == -64 and qs[0, 2] == 1 and qs[0, 3] == 0
    x2 = np.array([(i - 32.0) / 10.0 for i in range(64)], dtype=np.float32)
    qs, ds = O.quantize_row_q8_0(x2)
    assert qs.shape == (2, 32) and ds.shape == (2,)
    # blocks quantize independently: quantizing each half alone gives the same
    q0, d0 = O.quantize_row_q8_0(x2[:32])
    q1, d1 = O.quantize_row_q8_0(x2[32:])
    assert np.array_equal(qs[0], q0[0]) and np.array_equal(qs[1], q1[0])
    assert ds[0] == d0[0] and ds[1] == d1[0]


def _quantize_f32_stepwise(x: np.ndarray):
    """The same rule written with numpy float32 scalar steps (no fusing)."""
    x = x.astype(np.float32).reshape(-1, 32)
    amax = np.max(np.abs(x), axis=1).astype(np.float32)
    d = (amax / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        idv = np.where(d != 0, np.float32(1.0) / d, np.float32(0.0)).astype(np.float32)
    q = np.rint((x * idv[:, None]).astype(np.float32))
    q = np.clip(q, -127, 127).astype(np.int8)
    d16 = d.astype(np.float16).astype(np.float32)
    return q, d16


def test_quantize_invariants_and_independent_evaluation():
    rng = np.random.default_rng(7)
    for scale in (1e-6, 0.02, 1.0, 37.5, 6e4):
        x = (rng.standard_normal(32 * 64) * scale).astype(np.float32)
        x[5 * 32:6 * 32] = 0.0  # an all-zero block
        qs, ds = O.quantize_row_q8_0(x)
        q_np, d_np = _quantize_f32_stepwise(x)
        assert np.array_equal(qs, q_np)
        assert np.array_equal(ds.view(np.uint32), d_np.view(np.uint32))
        assert np.abs(qs.astype(np.int32)).max() <= 127
        assert ds[5] == 0.0 and not qs[5].any()
        # |x - d*q| <= d/2 (+ rounding slack) with the unrounded scale
        xb = x.reshape(-1, 32).astype(np.float64)
        d = np.abs(xb).max(axis=1) / 127.0
        err = np.abs(xb - d[:, None] * qs.astype(np.float64))
        assert np.all(err <= d[:, None] * (0.5 + 1e-5) + 1e-30)
        # the extreme element of each block maps to +-127
        nz = d > 0
        assert np.all(np.abs(qs.astype(np.int32)).max(axis=1)[nz] == 127)


def test_quantize_is_idempotent_on_its_own_grid():
    rng = np.random.default_rng(11)
    q = rng.integers(-127, 128, size=(8, 32)).astype(np.float32)
    q[:, 0] = 127.0  # amax = 127*d, so d is recovered exactly for power-of-two d
    for d in (1.0, 0.5, 2.0 ** -10, 8.0):
        x = (q * np.float32(d)).astype(np.float32)
        qs, ds = O.quantize_row_q8_0(x)
        assert np.array_equal(qs, q.astype(np.int8))
        assert np.all(ds == np.float32(d))


def test_quantize_non_finite_inputs_follow_rust_casts():
    x = np.zeros(32, dtype=np.float32)
    x[0], x[1] = np.inf, 3.0
    qs, ds = O.quantize_row_q8_0(x)
    # amax = inf -> d = inf, id = 0 -> inf*0 = NaN -> `as i8` = 0; 3*0 = 0
    assert not qs.any() and np.isinf(ds[0])
    x[0] = np.nan
    qs, ds = O.quantize_row_q8_0(x)
    # f32::max skips NaN: amax = 3 -> q[1] = 127, q[0] = NaN as i8 = 0
    assert qs[0, 1] == 127 and qs[0, 0] == 0


# ------------------------------------------------------------------- dots --

def _block(d_bits: int, qs) -> bytes:
    return d_bits.to_bytes(2, "little") + bytes((int(q) & 0xFF) for q in qs)


def test_dot_ones_case_is_64():
    # crates/metal/src/tests.rs:310-330
    row = _block(O.f32_to_f16_bits(1.0), [1] * 32)
    assert O.dot_q8_0_x_f32(row, np.full(32, 2.0, np.float32)) == 64.0


def test_zero_rows_and_zero_x_are_zero():
    # crates/tuckcore/src/kernels.rs:590-599
    row = bytes(34)
    x = np.zeros(32, np.float32)
    assert O.dot_q8_0_x_f32(row, x) == 0.0
    qs, ds = O.quantize_row_q8_0(x)
    assert O.dot_q8_0_q8_0(row, qs, ds) == 0.0


def test_malformed_shapes_are_rejected():
    # crates/tuckcore/src/kernels.rs:560-587
    row34, row68 = bytes(34), bytes(68)
    with pytest.raises(O.OracleError) as e:
        O.dot_q8_0_x_f32(row34, np.zeros(0, np.float32))
    assert e.value.code == "Internal"
    for row, n in ((row34, 31), (row68, 32)):
        with pytest.raises(O.OracleError):
            O.dot_q8_0_x_f32(row, np.zeros(n, np.float32))
    with pytest.raises(O.OracleError) as e:
        O.dot_q8_0_x_f32(bytes(33), np.zeros(32, np.float32))
    assert e.value.code == "InvalidArtifact"
    with pytest.raises(O.OracleError):
        O.dot_q8_0_x_f32(b"", np.zeros(0, np.float32))
    qs, ds = O.quantize_row_q8_0(np.zeros(64, np.float32))
    assert qs.shape[0] == 2
    with pytest.raises(O.OracleError):
        O.dot_q8_0_q8_0(row68, qs[:1], ds)
    with pytest.raises(O.OracleError):
        O.dot_q8_0_q8_0(row68, qs, ds[:1])
    with pytest.raises(O.OracleError):
        O.dot_q8_0_q8_0(row34, qs, ds)


def test_dot_closed_form_on_fixture_pattern():
    # d = 1/128, x = 1: every partial sum is an integer below 2^24 scaled by a
    # power of two, so the f32 evaluation is exact whatever the order.
    blocks = 32
    raw = fixture_q8_0(blocks * 32)
    x = np.ones(blocks * 32, np.float32)
    want = sum((((i * 11 + 5) % 128) - 64) for i in range(blocks * 32)) / 128.0
    assert O.dot_q8_0_x_f32(raw, x) == np.float32(want)
    # x = j within each block: still exact integers
    xj = np.tile(np.arange(32, dtype=np.float32), blocks)
    want = sum(((((b * 32 + j) * 11 + 5) % 128) - 64) * j
               for b in range(blocks) for j in range(32)) / 128.0
    assert O.dot_q8_0_x_f32(raw, xj) == np.float32(want)


def rne_f32(v: Fraction) -> Fraction:
    """Round an exact rational to the nearest binary32 value, ties to even
    (normal range only; the tests stay inside it)."""
    if v == 0:
        return v
    sign = -1 if v < 0 else 1
    a = abs(v)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    if Fraction(2) ** (e + 1) <= a:
        e += 1
    assert -126 <= e <= 127
    ulp = Fraction(2) ** (e - 23)
    n = a / ulp
    fl = n.numerator // n.denominator
    rem = n - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    return sign * fl * ulp


def _exact_dot_kernels_order(d_vals, qs, x):
    """kernels.rs:193-203 in exact arithmetic with one rounding per f32 op."""
    acc = Fraction(0)
    for b, d in enumerate(d_vals):
        block_sum = Fraction(0)
        for l in range(32):
            prod = rne_f32(Fraction(int(qs[b][l])) * Fraction(float(x[b * 32 + l])))
            block_sum = rne_f32(block_sum + prod)
        acc = rne_f32(acc + rne_f32(Fraction(float(d)) * block_sum))
    return acc


def _exact_dot_dequant_first(d_vals, qs, x):
    """crates/metal/src/tests.rs:108-112 in exact arithmetic."""
    acc = Fraction(0)
    for b, d in enumerate(d_vals):
        for l in range(32):
            dq = rne_f32(Fraction(float(d)) * int(qs[b][l]))
            acc = rne_f32(acc + rne_f32(dq * Fraction(float(x[b * 32 + l]))))
    return acc


def test_dot_follows_kernels_rs_order_exactly_and_not_the_other_orders():
    rng = np.random.default_rng(5)
    differs = 0
    for trial in range(40):
        blocks = 1 + trial % 3
        dbits = [O.f32_to_f16_bits(v) for v in rng.uniform(0.01, 0.3, blocks)]
        d_vals = [O.f16_to_f32(b) for b in dbits]
        qs = rng.integers(-127, 128, size=(blocks, 32))
        x = rng.standard_normal(blocks * 32).astype(np.float32)
        row = b"".join(_block(dbits[b], qs[b]) for b in range(blocks))
        got = Fraction(float(O.dot_q8_0_x_f32(row, x)))
        want = _exact_dot_kernels_order(d_vals, qs, x)
        assert got == want, f"trial {trial}: oracle deviates from kernels.rs order"
        other = _exact_dot_dequant_first(d_vals, qs, x)
        y2 = O.gemv_q8_0_f32_dequant_first(row, 1, blocks * 32, x)
        assert Fraction(float(y2[0])) == other
        differs += int(other != want)
    # the two orders must be distinguishable on this data, otherwise the test
    # above would not tell them apart
    assert differs >= 10


def test_dot_within_f64_error_bound():
    rng = O.KRng(0x1234_5678_9ABC_DEF0)
    for blocks in (1, 3, 32, 96):
        row = rng.row(blocks)
        x = np.array([rng.next_f32(2.0) for _ in range(blocks * 32)], np.float32)
        got = float(O.dot_q8_0_x_f32(row, x))
        exact = O.gemv_q8_0_f64(row, 1, blocks * 32, x)[0]
        w = O.dequant_q8_0(row).astype(np.float64)
        bound = (blocks * 32) * 2.0 ** -24 * np.sum(np.abs(w * x.astype(np.float64)))
        assert abs(got - exact) <= bound + 1e-30


def test_q8_q8_block_dots_match_integer_brute_force():
    rng = np.random.default_rng(3)
    for blocks in (1, 8, 40):
        wq = rng.integers(-128, 128, size=(blocks, 32))
        xq = rng.integers(-127, 128, size=(blocks, 32)).astype(np.int8)
        if blocks >= 8:
            wq[0, :] = -128
            xq[0, :] = 127
            wq[1, :] = -128
            xq[1, :] = -127
        dbits = [O.f32_to_f16_bits(v) for v in rng.uniform(0.001, 0.1, blocks)]
        row = b"".join(_block(dbits[b], wq[b]) for b in range(blocks))
        sumi = O.block_sumi(row, xq)
        want = (wq.astype(np.int64) * xq.astype(np.int64)).sum(axis=1)
        assert np.array_equal(sumi.astype(np.int64), want)
        if blocks >= 8:
            assert sumi[0] == -520192 and sumi[1] == 520192
        xd = rng.uniform(0.001, 0.1, blocks).astype(np.float32)
        got = Fraction(float(O.dot_q8_0_q8_0(row, xq, xd)))
        acc = Fraction(0)
        for b in range(blocks):
            s = rne_f32(Fraction(float(O.f16_to_f32(dbits[b]))) * Fraction(float(xd[b])))
            acc = rne_f32(acc + rne_f32(s * int(want[b])))
        assert got == acc


def test_reference_randomized_cases_scalar_is_self_consistent():
    # crates/tuckcore/src/kernels.rs:517-523 (forced scalar == scalar) and
    # :526-541 (q8 x q8 within 1e-5 of the scalar value): here both sides are
    # the oracle, so these hold trivially; kept as a smoke check of the
    # reference's generators at the reference's seeds and sizes.
    rng = O.KRng(0x5511_2233_4455_6677)
    row = rng.row(4)
    x = np.array([rng.next_f32(1.0) for _ in range(128)], np.float32)
    assert O.dot_q8_0_x_f32(row, x) == O.gemv_q8_0_f32(row, 1, 128, x)[0]
    rng = O.KRng(0xFEED_BEEF_CAFE_1234)
    for blocks in (1, 8, 40):
        row = rng.row(blocks)
        x = np.array([rng.next_f32(1.5) for _ in range(blocks * 32)], np.float32)
        qs, ds = O.quantize_row_q8_0(x)
        a = O.dot_q8_0_q8_0(row, qs, ds)
        b = O.gemv_q8_0_q8_0(row, 1, blocks * 32, x)[0]
        assert a == b


# ------------------------------------------------------------- row loops --

def test_gemm_is_one_gemv_per_token_and_threads_do_not_change_bits():
    rows, cols, batch = 37, 96, 5
    w = O.boundary_weights(rows, cols, 17)
    x = O.boundary_input(cols * batch, 23)
    y = O.gemm_q8_0_f32(w, rows, cols, x, batch)
    assert y.shape == (batch, rows)
    for b in range(batch):
        yb = O.gemv_q8_0_f32(w, rows, cols, x[b * cols:(b + 1) * cols])
        assert np.array_equal(y[b].view(np.uint32), yb.view(np.uint32))
        for r in (0, 1, rows - 1):
            one = O.dot_q8_0_x_f32(w[r * 3 * 34:(r + 1) * 3 * 34], x[b * cols:(b + 1) * cols])
            assert one == yb[r] or (np.isnan(one) and np.isnan(yb[r]))
    y4 = O.gemm_q8_0_f32(w, rows, cols, x, batch, threads=4)
    assert np.array_equal(y.view(np.uint32), y4.view(np.uint32))


# ------------------------------------------------------------- generators --

def _xorshift64star(state: int):
    state ^= state >> 12
    state ^= (state << 25) & MASK64
    state ^= state >> 27
    return state, (state * 0x2545F4914F6CDD1D) & MASK64


def test_rng_matches_big_integer_xorshift64star():
    for seed in (1, 3, 5, 7, 11, 13, 0x9E37, 2 ** 63 + 12345):
        r = O.Rng(seed)
        s = seed
        for _ in range(64):
            s, want = _xorshift64star(s)
            assert r.next() == want
    # first output for seed 1 by hand: the state becomes 0x2000001
    assert O.Rng(1).next() == (0x2000001 * 0x2545F4914F6CDD1D) & MASK64


def test_boundary_generators_follow_the_reference_recipe():
    rows, cols, seed = 17, 64, 3
    raw = O.boundary_weights(rows, cols, seed)
    assert raw.size == rows * 2 * 34
    scales = [1.0, -0.5, 2.0 ** -12, 65504.0, -65504.0, 5.96e-8, 0.0, -0.0, 448.0, 6e-5]
    s = seed
    for blk in range(rows * 2):
        s, v = _xorshift64star(s)
        want_d = int(_np_f16_bits(np.array([scales[v % 10]], np.float32))[0])
        got_d = int(raw[blk * 34]) | (int(raw[blk * 34 + 1]) << 8)
        assert got_d == want_d
        for l in range(32):
            s, v = _xorshift64star(s)
            sel = v % 8
            if sel == 0:
                q = -128
            elif sel == 1:
                q = 127
            elif sel == 2:
                q = 0
            else:
                s, v = _xorshift64star(s)
                q = (v % 256) - 256 if (v % 256) >= 128 else (v % 256)
            assert int(np.int8(raw[blk * 34 + 2 + l])) == q
    x = O.boundary_input(50, seed ^ 0x9E37)
    s = seed ^ 0x9E37
    for i in range(50):
        if i % 7 == 0:
            want = 0.0
        elif i % 7 == 1:
            want = -1.0
        elif i % 7 == 2:
            want = 1e3
        elif i % 7 == 3:
            want = -1e3
        else:
            s, v = _xorshift64star(s)
            want = (np.float32(v % 20001) - np.float32(10000.0)) / np.float32(1000.0)
        assert x[i] == np.float32(want)


def test_kernel_test_rng_matches_big_integer_form():
    seed = 0x1234_5678_9ABC_DEF0
    r = O.KRng(seed)
    s = seed
    for _ in range(32):
        s ^= s >> 12
        s ^= (s << 25) & MASK64
        s ^= s >> 27
        u = np.float32(((s * 0x2545F4914F6CDD1D) & MASK64) >> 40)
        want = ((u / np.float32(1 << 24)) * np.float32(2.0) - np.float32(1.0)) * np.float32(0.7)
        assert r.next_f32(0.7) == want
    row = O.KRng(seed).row(3)
    d = O.dequant_q8_0(row)
    for b in range(3):
        dv = O.f16_to_f32(int(row[b * 34]) | (int(row[b * 34 + 1]) << 8))
        assert 1e-4 <= dv <= 0.0501
    assert np.abs(row.reshape(3, 34)[:, 2:].view(np.int8).astype(np.int32)).max() <= 127
    assert d.size == 96
