"""The documented rule for which prefill GEMMs run on the bf16 matrix cores
(tuckmill_amd.hip mirrors the library's choice; the GPU tests check the mirror
against the library's launch counts)."""
from tuckmill_amd import hip as H
from tuckmill_amd import synth as S


def test_work_units_of_the_bf16_gemm():
    plan = H.gemm_mma_bf16_plan
    # tiles of 128 tokens x 256 rows; K whole when the tiles alone give 192 units
    assert plan(14336, 4096, 512) == (128, 4 * 56, True)
    # else in chunks of 512 columns or more, at most eight, about 192 units
    assert plan(6144, 2048, 512) == (128, 4 * 24 * 2, True)
    assert plan(2048, 6144, 512) == (128, 4 * 8 * 6, True)
    # 33 blocks in two chunks of 17 and 16
    assert plan(8300, 1056, 500) == (128, 4 * 33 * 2, True)
    # fewer than 192 such units: tiles of 64 tokens, if 4 chunks are enough ...
    assert plan(4096, 1024, 512) == (64, 8 * 16 * 2, True)
    assert plan(2048, 2048, 512) == (64, 8 * 8 * 3, True)
    assert plan(33000, 96, 65) == (64, 2 * 129, True)
    # ... in however many K chunks (six here) ...
    assert plan(1024, 4096, 512) == (64, 8 * 4 * 6, True)
    assert plan(1152, 6912, 512) == (64, 8 * 5 * 5, True)
    assert plan(1024, 3072, 512) == (64, 8 * 4 * 6, True)
    # ... else none (the large tile's figures are what the plan reports then)
    assert plan(1024, 2048, 512) == (128, 4 * 4 * 4, False)
    assert plan(1024, 1024, 512) == (128, 4 * 4 * 2, False)


def test_which_products_take_the_bf16_matrix_cores():
    # the 0.6B attention and down projections are too small on their own,
    # the vocabulary projections and the 2B-class FFN are not
    for name, rows, cols in S.QWEN3_0_6B_LAYER:
        if name in ("q", "k", "v", "o"):
            assert not H.gemm_mma_on_bf16(rows, cols, 512)
    _, rows, cols = S.QWEN3_0_6B_LM_HEAD
    assert H.gemm_mma_on_bf16(rows, cols, H.GEMM_MMA_BF16_MIN_BATCH)  # 155 M weights: from 5 tokens
    assert not H.gemm_mma_on_bf16(rows, cols, H.GEMM_MMA_BF16_MIN_BATCH - 1)
    assert not H.gemm_mma_on_bf16(33000, 1024, 8) and H.gemm_mma_on_bf16(33000, 1024, 9)  # 34 M: from 9
    assert not H.gemm_mma_on_bf16(6144, 2048, 16)  # 13 M: the vector kernel up to 16 tokens
    for _, rows, cols in S.SWEEP_2B:
        assert H.gemm_mma_on_bf16(rows, cols, 256)
    # 192 units of the small tile are the least that pays: q (128 units) stays on
    # the f32 kernels; gate, up and down (six K chunks) do not
    assert not H.gemm_mma_on_bf16(2048, 1024, 512)
    assert H.gemm_mma_on_bf16(1024, 3072, 512)
    assert H.gemm_mma_on_bf16(3072, 1024, 512)
    # up to 64 tokens: matrices of 16 M weights and more
    assert H.gemm_mma_on_bf16(4096, 4096, 64) and not H.gemm_mma_on_bf16(6144, 2048, 64)
    # activations must start on a 16-byte boundary
    assert not H.gemm_mma_on_bf16(8192, 1024, 512, x_off=3)
    assert H.gemm_mma_on_bf16(8192, 1024, 512, x_off=32)


def test_products_that_share_a_launch_decide_together():
    tile = H.gemm_mma_launch_tile
    M = 512
    layer = {name: (rows, cols, M) for name, rows, cols in S.QWEN3_0_6B_LAYER}
    # alone, only gate, up and down are large enough (tiles of 64 tokens) ...
    assert [tile([layer[n]]) for n in ("q", "k", "v", "o", "gate", "up", "down")] == \
        [0, 0, 0, 0, 64, 64, 64]
    # ... all seven in one launch have 480 units of the large tile between them
    assert tile(list(layer.values())) == 128
    # the dependent layer's launches: q, k, v together and gate, up together take
    # the small and the large tile, down alone the small one; o, alone in its
    # launch, stays on the f32 matrix cores
    assert tile([layer["q"], layer["k"], layer["v"]]) == 64
    assert tile([layer["gate"], layer["up"]]) == 128
    assert tile([layer["o"]]) == 0 and tile([layer["down"]]) == 64
    # the engine's prefill chunk of 128 tokens: all seven on the small tile
    assert tile([(r, c, 128) for _, r, c in S.QWEN3_0_6B_LAYER]) == 64
    # ... and alone there: few tiles under a deep K (3072 columns and more) take the small
    # tile where the f32 kernel is estimated slower. It is not where it can share its output
    # tiles between workgroups (up to 128 tiles) or still fills the chip in one round ...
    assert tile([(1024, 3072, 128)]) == 0 and tile([(1152, 6912, 96)]) == 0
    assert tile([(1024, 4096, 192)]) == 0 and tile([(1024, 4096, 256)]) == 0
    # ... and is with more tiles than that under a deeper K
    assert tile([(1152, 6912, 128)]) == 64 and tile([(2048, 6144, 65)]) == 64
    assert tile([(2048, 8192, 96)]) == 64 and tile([(1030, 4096, 256)]) == 64
    assert tile([(1024, 2048, 128)]) == 0 and tile([(4096, 1024, 128)]) == 0
    # up to 64 tokens: 16 M weights between them
    assert tile([(6144, 2048, 64)]) == 0 and tile([(6144, 2048, 64), (6144, 2048, 64)]) == 64
    assert tile([]) == 0
