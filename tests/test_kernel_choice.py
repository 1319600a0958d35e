"""The documented rule for which prefill GEMMs run on the bf16 matrix cores
(tuckmill_amd.hip mirrors the library's choice; the GPU tests check the mirror
against the library's launch counts)."""
from tuckmill_amd import hip as H
from tuckmill_amd import synth as S


def test_work_units_of_the_bf16_gemm():
    # tiles of 128 tokens x 256 rows; K whole when the tiles alone give 192 units
    assert H.gemm_mma_bf16_units(14336, 4096, 512) == 4 * 56
    # else in chunks of 512 columns or more, at most eight, about 192 units
    assert H.gemm_mma_bf16_units(6144, 2048, 512) == 4 * 24 * 2
    assert H.gemm_mma_bf16_units(2048, 6144, 512) == 4 * 8 * 6
    assert H.gemm_mma_bf16_units(1024, 4096, 512) == 4 * 4 * 8
    assert H.gemm_mma_bf16_units(1024, 1024, 512) == 4 * 4 * 2
    assert H.gemm_mma_bf16_units(33000, 96, 65) == 129
    # 33 blocks in two chunks of 17 and 16
    assert H.gemm_mma_bf16_units(8300, 1056, 500) == 4 * 33 * 2


def test_which_products_take_the_bf16_matrix_cores():
    # the 0.6B projections are too small on their own at any batch ...
    for _, rows, cols in S.QWEN3_0_6B_LAYER:
        assert not H.gemm_mma_on_bf16(rows, cols, 512)
    # ... the vocabulary projections and the 2B-class FFN are not
    _, rows, cols = S.QWEN3_0_6B_LM_HEAD
    assert H.gemm_mma_on_bf16(rows, cols, H.GEMM_MMA_BF16_MIN_BATCH)
    assert not H.gemm_mma_on_bf16(rows, cols, H.GEMM_MMA_BF16_MIN_BATCH - 1)
    for _, rows, cols in S.SWEEP_2B:
        assert H.gemm_mma_on_bf16(rows, cols, 256)
        assert not H.gemm_mma_on_bf16(rows, cols, 128)
    # activations must start on a 16-byte boundary
    assert not H.gemm_mma_on_bf16(8192, 1024, 512, x_off=3)
    assert H.gemm_mma_on_bf16(8192, 1024, 512, x_off=32)
