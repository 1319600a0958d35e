"""The committed golden vectors (tests/golden/q8_golden.npz) against the CPU
oracle (always) and against the HIP path (with -m gpu)."""
import os

import numpy as np
import pytest

import oracle as O

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "q8_golden.npz"),
            allow_pickle=False)
NCASES = 4


def test_oracle_reproduces_the_reference_known_answers():
    for bits, val in zip(G["known_f16_bits"], G["known_f16_values"]):
        assert O.f16_to_f32(int(bits)) == val
    for x, bits in zip(G["known_f32_inputs"], G["known_f32_to_f16"]):
        assert O.f32_to_f16_bits(x) == int(bits)
    qs, ds = O.quantize_row_q8_0(G["known_quant_x"])
    assert np.array_equal(qs[0], G["known_quant_q"]) and np.array_equal(ds, G["known_quant_d"])


def test_oracle_reproduces_the_generator_streams():
    for seed in (1, 3, 5, 7, 11, 13):
        r = O.Rng(seed)
        assert np.array_equal(np.array([r.next() for _ in range(64)], np.uint64), G[f"rng_{seed}"])
    assert np.array_equal(O.boundary_weights(17, 64, 3), G["boundary_weights_17_64_3"])
    assert np.array_equal(O.boundary_input(64, 3 ^ 0x9E37), G["boundary_input_64_3"])


@pytest.mark.parametrize("i", range(NCASES))
def test_oracle_reproduces_the_seeded_products(i):
    rows, cols, batch = (int(v) for v in G[f"case{i}_dims"])
    w, x = G[f"case{i}_w"], G[f"case{i}_x"]
    y = O.gemm_q8_0_f32(w, rows, cols, x, batch)
    assert np.array_equal(y.view(np.uint32), G[f"case{i}_y_f32"].view(np.uint32))
    yq = O.gemm_q8_0_q8_0(w, rows, cols, x, batch)
    assert np.array_equal(yq.view(np.uint32), G[f"case{i}_y_q8"].view(np.uint32))
    qs, ds = O.quantize_row_q8_0(x)
    assert np.array_equal(qs, G[f"case{i}_xq"])
    assert np.array_equal(ds.view(np.uint32), G[f"case{i}_xd"].view(np.uint32))


@pytest.mark.gpu
@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("i", range(NCASES))
def test_hip_path_reproduces_the_golden_products(i, packed):
    from q8util import require_gpu, upload_new, weights_buffer

    ctx = require_gpu()
    rows, cols, batch = (int(v) for v in G[f"case{i}_dims"])
    w, x = G[f"case{i}_w"], G[f"case{i}_x"]
    wb = weights_buffer(ctx, w, rows, cols, packed)
    xb = upload_new(ctx, x)
    want = G[f"case{i}_y_f32"]
    scale = float(np.max(np.abs(want)))
    for fn in (ctx.q8_0_gemm, ctx.q8_0_gemm_mma):
        yb = ctx.buffer(batch * rows * 4)
        fn(wb, xb, yb, rows, cols, batch, 0, 0)
        ctx.fence()
        got = yb.download_f32(0, batch * rows).reshape(batch, rows)
        assert np.max(np.abs(got - want)) / scale <= 1e-5
    from tuckmill_amd import hip as H

    xq = ctx.buffer(H.xq_bytes(cols, batch))
    yb = ctx.buffer(batch * rows * 4)
    ctx.q8_0_quantize_act(xb, xq, cols, batch)
    ctx.q8_0_gemm_i8(wb, xq, yb, rows, cols, batch)
    ctx.fence()
    qs, ds = H.xq_split(xq.download(0, H.xq_bytes(cols, batch)), cols, batch)
    assert np.array_equal(qs.reshape(-1, 32), G[f"case{i}_xq"])
    assert np.array_equal(ds.reshape(-1).view(np.uint32), G[f"case{i}_xd"].view(np.uint32))
    got = yb.download_f32(0, batch * rows).reshape(batch, rows)
    assert np.array_equal(got.view(np.uint32), G[f"case{i}_y_q8"].view(np.uint32))
    ctx.close()


@pytest.mark.gpu
def test_hip_path_on_the_golden_boundary_case():
    from q8util import gemv, require_gpu, weights_buffer

    ctx = require_gpu()
    w, x = G["boundary_weights_17_64_3"], G["boundary_input_64_3"]
    for packed in (False, True):
        got = gemv(ctx, weights_buffer(ctx, w, 17, 64, packed), x, 17, 64)
        for key in ("boundary_y_kernels_order", "boundary_y_dequant_first"):
            want = G[key]
            assert np.max(np.abs(got - want)) <= 1e-4 * max(float(np.max(np.abs(want))), 1.0)
    ctx.close()
