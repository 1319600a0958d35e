"""GPU: the two cast operators, f16 -> f32 and f32 -> f16
(native/metal/kernels.metal:38-58, host native/metal/tm_metal.m:950-960),
bit for bit against the CPU conversions of crates/tuckcore/src/tensor.rs:12-28
and :145-178, as the reference's own test does (crates/metal/src/tests.rs:250-305)
- here over every binary16 encoding and every binary32 one.
"""
import numpy as np
import pytest

import oracle as O
from tuckmill_amd import hip as H

from q8util import bits, require_gpu, upload_new

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = require_gpu()
    yield c
    c.close()


def to_f16(ctx, values):
    v = np.ascontiguousarray(values, dtype=np.float32)
    xb = upload_new(ctx, v)
    hb = ctx.buffer(v.size * 2)
    ctx.cast_f32_to_f16(xb, hb, v.size)
    ctx.fence()
    out = hb.download(0, v.size * 2).view(np.uint16).copy()
    xb.free()
    hb.free()
    return out


def to_f32(ctx, half_bits):
    h = np.ascontiguousarray(half_bits, dtype=np.uint16)
    hb = upload_new(ctx, h)
    yb = ctx.buffer(h.size * 4)
    ctx.cast_f16_to_f32(hb, yb, h.size)
    ctx.fence()
    out = yb.download_f32(0, h.size).copy()
    hb.free()
    yb.free()
    return out


def test_the_values_the_reference_casts(ctx):
    # crates/metal/src/tests.rs:257-275: representable range, subnormals, ties, overflow
    values = np.array([0.0, -0.0, 1.0, -1.0, 0.1, 65504.0, 65520.0, 100_000.0, -100_000.0,
                       5.960_464_5e-8, 2.980_232_2e-8, 1.0e-7, -6.0e-8, 44.856, np.pi,
                       np.inf, -np.inf], dtype=np.float32)
    half = to_f16(ctx, values)
    for v, got in zip(values, half):
        assert int(got) == O.f32_to_f16_bits(v), v
    # the closed forms among them, so that this does not lean on the oracle alone
    assert list(half[:4]) == [0x0000, 0x8000, 0x3C00, 0xBC00]
    assert half[5] == 0x7BFF and half[6] == 0x7C00 and half[7] == 0x7C00 and half[8] == 0xFC00
    assert half[9] == 0x0001 and half[10] == 0x0000 and half[12] == 0x8001
    back = to_f32(ctx, half)
    want = np.array([O.f16_to_f32(int(h)) for h in half], np.float32)
    assert np.array_equal(bits(back), bits(want))


def test_every_binary16_encoding_to_f32(ctx):
    enc = np.arange(1 << 16, dtype=np.uint16)
    got = to_f32(ctx, enc)
    want = O.f16_to_f32_array(enc)
    nan = (enc & 0x7C00 == 0x7C00) & (enc & 0x03FF != 0)
    assert np.array_equal(bits(got)[~nan], bits(want)[~nan])
    assert np.array_equal(bits(got)[~nan], bits(enc.view(np.float16).astype(np.float32))[~nan])
    # a NaN stays a NaN of the same sign
    assert np.all(np.isnan(got[nan]))
    assert np.array_equal(bits(got)[nan] >> 31, (enc[nan] >> 15).astype(np.uint32))


@pytest.mark.parametrize("n", [1, 7, 8, 9, 2047, 2048, 2049, 100_003])
def test_lengths_around_the_eight_element_step(ctx, n):
    rng = np.random.default_rng(n)
    # random bit patterns: every exponent, both signs
    v = rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32).view(np.float32)
    v = np.where(np.isnan(v), np.float32(1.5), v).astype(np.float32)
    # what lies behind the n elements must stay as it was
    xb = upload_new(ctx, v)
    hb = upload_new(ctx, np.full(n + 16, 0xABCD, np.uint16))
    ctx.cast_f32_to_f16(xb, hb, n)
    ctx.fence()
    half = hb.download(0, (n + 16) * 2).view(np.uint16)
    assert np.array_equal(half[:n], O.f32_to_f16_bits_array(v))
    assert np.all(half[n:] == 0xABCD)
    yb = upload_new(ctx, np.full(n + 16, 7.0, np.float32))
    ctx.cast_f16_to_f32(hb, yb, n)
    ctx.fence()
    back = yb.download_f32(0, n + 16)
    assert np.array_equal(bits(back[:n]), bits(O.f16_to_f32_array(half[:n])))
    assert np.all(back[n:] == 7.0)
    for b in (xb, hb, yb):
        b.free()


def test_every_binary32_encoding_to_f16(ctx):
    """All 2^32 inputs, in slabs: the rounding of tensor.rs:145-178 on every
    number; a NaN becomes the quiet NaN of its sign (the Metal kernel converts in
    hardware, which keeps a NaN a NaN; tensor.rs:150-153 alone would turn it
    into an infinity, and the reference's test holds no NaN)."""
    slab = 1 << 27
    xb = ctx.buffer(slab * 4)
    hb = ctx.buffer(slab * 2)
    for s in range((1 << 32) // slab):
        pattern = np.arange(s * slab, (s + 1) * slab, dtype=np.uint32)
        xb.upload(0, pattern)
        ctx.cast_f32_to_f16(xb, hb, slab)
        ctx.fence()
        got = hb.download(0, slab * 2).view(np.uint16)
        want = O.f32_to_f16_bits_array(pattern.view(np.float32))
        nan = (pattern & 0x7FFFFFFF) > 0x7F800000
        if nan.any():
            sign = ((pattern >> 16) & 0x8000).astype(np.uint16)
            want = np.where(nan, sign | 0x7E00, want).astype(np.uint16)
        bad = np.flatnonzero(got != want)
        assert bad.size == 0, f"f32 bits {int(pattern[bad[0]]):#010x}: {int(got[bad[0]]):#06x} " \
                              f"!= {int(want[bad[0]]):#06x}"
    xb.free()
    hb.free()


def test_casts_inside_a_group_keep_their_order(ctx):
    n = 4096
    v = np.linspace(-3.0, 3.0, n, dtype=np.float32)
    xb, hb, yb = upload_new(ctx, v), ctx.buffer(n * 2), ctx.buffer(n * 4)
    ctx.begin_group()
    ctx.f32_scale(xb, xb, 2.0, n)      # x <- 2x
    ctx.cast_f32_to_f16(xb, hb, n)     # reads the scaled x
    ctx.cast_f16_to_f32(hb, yb, n)     # reads the halves just written
    ctx.end_group()
    ctx.fence()
    want = O.f16_to_f32_array(O.f32_to_f16_bits_array(v * np.float32(2.0)))
    assert np.array_equal(bits(yb.download_f32(0, n)), bits(want))
    for b in (xb, hb, yb):
        b.free()


def test_cast_refusals(ctx):
    # native/metal/tm_metal.m:777-786: zero length and short buffers are bounds errors
    f32 = ctx.buffer(64)       # 16 floats
    f16 = ctx.buffer(32)       # 16 halves
    for call in (lambda: ctx.cast_f32_to_f16(f32, f16, 0), lambda: ctx.cast_f16_to_f32(f16, f32, 0),
                 lambda: ctx.cast_f32_to_f16(f32, f16, 17), lambda: ctx.cast_f16_to_f32(f16, f32, 17),
                 lambda: ctx.cast_f16_to_f32(f16, f16, 16)):
        with pytest.raises(H.TuckmillError) as e:
            call()
        assert e.value.abi_code == H.TM_HIP_ERR_BOUNDS
    ctx.cast_f32_to_f16(f32, f16, 16)
    ctx.cast_f16_to_f32(f16, f32, 16)
    ctx.fence()
    f32.free()
    f16.free()


def test_lengths_just_below_two_to_the_32(ctx):
    """n = 2^32 - 5 elements: the last workgroup is partly beyond the end and
    `n + (elements per workgroup) - 1` does not fit 32 bits. Only the ends are
    looked at (16 GiB of input stay zero)."""
    n = (1 << 32) - 5
    tail = np.array([1.0, -2.5, 65504.0, 1e-7, 3.0, -0.0, 70000.0, 0.5, 0.1, -1.0, 2.0],
                    dtype=np.float32)
    xb = ctx.buffer(n * 4)
    xb.zero(0, n * 4)
    xb.upload((n - tail.size) * 4, tail)
    xb.upload(0, np.array([4.0, -8.0], np.float32))
    hb = ctx.buffer(n * 2 + 32)
    hb.upload(n * 2, np.full(16, 0xABCD, np.uint16))
    ctx.cast_f32_to_f16(xb, hb, n)
    ctx.fence()
    assert list(hb.download(0, 8).view(np.uint16)) == [0x4400, 0xC800, 0, 0]
    got = hb.download((n - tail.size) * 2, tail.size * 2 + 32).view(np.uint16)
    assert np.array_equal(got[:tail.size], O.f32_to_f16_bits_array(tail))
    assert np.all(got[tail.size:] == 0xABCD)
    # the way back over the same length, and an f32 operator with one element per lane
    yb = ctx.buffer(n * 4 + 64)
    yb.upload(n * 4, np.full(16, 7.0, np.float32))
    ctx.cast_f16_to_f32(hb, yb, n)
    ctx.fence()
    back = yb.download_f32(n - tail.size, tail.size + 16)
    assert np.array_equal(bits(back[:tail.size]),
                          bits(O.f16_to_f32_array(O.f32_to_f16_bits_array(tail))))
    assert np.all(back[tail.size:] == 7.0)
    ctx.f32_scale(xb, yb, 2.0, n)
    ctx.fence()
    doubled = yb.download_f32(n - tail.size, tail.size + 16)
    assert np.array_equal(bits(doubled[:tail.size]), bits(tail * np.float32(2.0)))
    assert np.all(doubled[tail.size:] == 7.0)
    assert list(yb.download_f32(0, 3)) == [8.0, -16.0, 0.0]
    for b in (xb, hb, yb):
        b.free()
