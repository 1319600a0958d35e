"""The synthetic-input generator against the oracle's quantizer, and the host
statement of the sealed layout."""
import numpy as np

import oracle as O
from tuckmill_amd import synth as S


def test_weight_quantizer_agrees_with_the_oracle_rule():
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((24, 96)) * 0.02).astype(np.float32)
    w[3, 32:64] = 0.0
    raw = S.quantize_q8_0(w)
    assert raw.size == S.q8_0_bytes(24, 96)
    qs, ds = O.quantize_row_q8_0(w.reshape(-1))
    blk = raw.reshape(-1, 34)
    assert np.array_equal(blk[:, 2:].view(np.int8), qs)
    got_d = np.array([O.f16_to_f32(int(b[0]) | (int(b[1]) << 8)) for b in blk], np.float32)
    assert np.array_equal(got_d.view(np.uint32), ds.view(np.uint32))


def test_generator_is_seeded_and_shaped():
    a = S.make_weights(50, 64, 7, chunk_rows=16, threads=1)
    b = S.make_weights(50, 64, 7, chunk_rows=16)
    c = S.make_weights(50, 64, 8, chunk_rows=16)
    assert np.array_equal(a, b) and not np.array_equal(a, c)
    x = S.make_activations(4096, 0)
    assert abs(float(x.mean())) < 0.1 and abs(float(x.std()) - 1.0) < 0.1
    w = O.dequant_q8_0(S.make_weights(256, 1024, 0))
    assert abs(float(w.std()) - 0.02) < 0.002
    assert S.tensor_seed(0, 0, "gate") == 0
    assert S.gemv_bytes(3072, 1024) == 3_358_720
    step = sum(S.gemv_bytes(r, c) for _, r, c in S.QWEN3_0_6B_LAYER) * S.QWEN3_0_6B_LAYERS \
        + S.gemv_bytes(*S.QWEN3_0_6B_LM_HEAD[1:])
    assert step == 636_368_384


def test_host_pack_layout():
    rows, cols = 3, 64
    raw = O.boundary_weights(rows, cols, 1)
    p = S.pack_q8_0(raw, rows, cols)
    assert p.size == raw.size
    blk = raw.reshape(-1, 34)
    assert np.array_equal(p[:rows * cols].reshape(-1, 32), blk[:, 2:])
    assert np.array_equal(p[rows * cols:].reshape(-1, 2), blk[:, :2])
