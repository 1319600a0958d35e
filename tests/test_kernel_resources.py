"""Register budget of the decode kernel, checked at compile time (no GPU).

The decode path streams weights with four waves per SIMD; that needs the whole
kernel, including the general-shape code that shares it, to stay within 128
vector registers. A change elsewhere in the kernel once doubled the count and
cost a quarter of the decode bandwidth without failing any parity test.
"""
import os
import re
import shutil
import subprocess

import pytest

from tuckmill_amd import build as B

# gemv_list_kernel<PACKED, 8 rows, 1 token, aligned x, no tail set, any list capacity, no fused norm,
# no steps of several chunks>
DECODE_KERNEL = re.compile(r"Function Name: _ZN2q816gemv_list_kernelILi1ELi8ELi1ELb1ELi0ELi\d+ELb0ELb0EEE")


@pytest.fixture(scope="module")
def resource_remarks(tmp_path_factory):
    """The compiler's per-kernel resource remarks for the whole library, as lines."""
    hipcc = shutil.which(B.HIPCC) or (B.HIPCC if os.path.exists(B.HIPCC) else None)
    if hipcc is None:
        pytest.skip("hipcc not available")
    out = tmp_path_factory.mktemp("resources") / "device.o"
    cmd = [hipcc, "-x", "hip", "-std=c++17", "-O3", *B.DEVICE_FLAGS, "--cuda-device-only",
           "-I", os.path.join(B.ROOT, "include"), "-I", B.CSRC,
           "-Rpass-analysis=kernel-resource-usage", "-c", os.path.join(B.CSRC, "tm_launch.cpp"),
           "-o", str(out)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    return res.stderr.splitlines()


def _blocks(lines, pattern):
    start = [i for i, l in enumerate(lines) if pattern.search(l)]
    return ["\n".join(lines[at:at + 14]) for at in start]


def test_decode_kernel_keeps_four_waves_per_simd(resource_remarks):
    blocks = _blocks(resource_remarks, DECODE_KERNEL)
    assert blocks, "decode kernel not found in the resource remarks"
    for block in blocks:  # the long- and the short-list instantiation
        vgprs = int(re.search(r" VGPRs: (\d+)", block).group(1))
        spill = int(re.search(r"VGPRs Spill: (\d+)", block).group(1))
        occupancy = int(re.search(r"Occupancy \[waves/SIMD\]: (\d+)", block).group(1))
        assert spill == 0
        assert vgprs <= 128 and occupancy >= 4, f"{vgprs} VGPRs, {occupancy} waves/SIMD"


# gemv_list_kernel<RAW, 8 rows, 1 token, ...>: one token over weights as uploaded
RAW_DECODE_KERNEL = re.compile(r"Function Name: _ZN2q816gemv_list_kernelILi0ELi8ELi1ELb[01]ELi0ELi\d+ELb0ELb0EEE")


def test_raw_decode_kernel_keeps_four_waves_per_simd(resource_remarks):
    """It stages a wave's 8 x 1088 bytes per step in LDS: four workgroups of
    four waves must fit a CU's 160 KiB, and the registers four waves per SIMD."""
    blocks = _blocks(resource_remarks, RAW_DECODE_KERNEL)
    assert blocks, "raw decode kernel not found in the resource remarks"
    for block in blocks:
        vgprs = int(re.search(r" VGPRs: (\d+)", block).group(1))
        spill = int(re.search(r"VGPRs Spill: (\d+)", block).group(1))
        lds = int(re.search(r"LDS Size \[bytes/block\]: (\d+)", block).group(1))
        assert spill == 0 and vgprs <= 128, f"{vgprs} VGPRs, {spill} spilled"
        assert lds == 4 * 8 * 1088 and 4 * lds <= 160 * 1024


# the same with the Gemma column tails: a pass of eight 1152-column rows is staged whole
RAW_DECODE_TAILS_KERNEL = re.compile(
    r"Function Name: _ZN2q816gemv_list_kernelILi0ELi8ELi1ELb[01]ELi1ELi\d+ELb0ELb0EEE")


def test_raw_decode_kernel_with_column_tails_fits_three_workgroups_per_cu(resource_remarks):
    blocks = _blocks(resource_remarks, RAW_DECODE_TAILS_KERNEL)
    assert blocks, "raw decode kernel with tails not found in the resource remarks"
    for block in blocks:
        vgprs = int(re.search(r" VGPRs: (\d+)", block).group(1))
        spill = int(re.search(r"VGPRs Spill: (\d+)", block).group(1))
        lds = int(re.search(r"LDS Size \[bytes/block\]: (\d+)", block).group(1))
        assert spill == 0 and vgprs <= 168, f"{vgprs} VGPRs, {spill} spilled"  # three waves per SIMD
        assert lds == 4 * 8 * 1224 and 3 * lds <= 160 * 1024


# gemm_bf16x3_kernel<WM, 4, 2, NS>: the 128-token and the 64-token tile
BF16_KERNEL = re.compile(r"Function Name: _ZN2q818gemm_bf16x3_kernelILi[12]ELi4ELi2ELi[34]ELb[01]EEE")


def test_bf16_gemm_keeps_its_results_in_vector_registers(resource_remarks):
    """Both tiles run two waves per SIMD and rescale every MFMA result once per
    Q8_0 block: the results must sit in ordinary vector registers (no
    accumulation registers, which cost a move per result), unspilled."""
    blocks = _blocks(resource_remarks, BF16_KERNEL)
    assert len(blocks) >= 2, "bf16 GEMM kernels not found in the resource remarks"
    for block in blocks:
        agprs = int(re.search(r"AGPRs: (\d+)", block).group(1))
        spill = int(re.search(r"VGPRs Spill: (\d+)", block).group(1))
        occupancy = int(re.search(r"Occupancy \[waves/SIMD\]: (\d+)", block).group(1))
        assert agprs == 0 and spill == 0 and occupancy >= 2, block


# gemm_mma_kernel<sealed, 1 token tile, row tiles, K split, aligned, shared tiles, split-form input = true, gated pair>
SPLIT_FORM_KERNEL = re.compile(
    r"Function Name: _ZN2q815gemm_mma_kernelILi1ELi1ELi[12]ELi[124]ELb1ELb[01]ELb1ELb[01]EEE")


def test_split_form_tiles_keep_two_workgroups_per_cu_without_spills(resource_remarks):
    """The small tiles fed from the split form are bound by waiting for operands:
    what hides it is waves side by side, not a deeper queue per wave. With two blocks
    of activations and two weight groups held, the forms with two accumulator tiles
    took all 256 registers and spilled (the gated pair at 128 tokens 17.7 us
    against 15.3 with one of each)."""
    blocks = _blocks(resource_remarks, SPLIT_FORM_KERNEL)
    assert len(blocks) >= 8, "split-form instantiations of gemm_mma_kernel not found"
    for block in blocks:
        vgprs = int(re.search(r" VGPRs: (\d+)", block).group(1))
        spill = int(re.search(r"VGPRs Spill: (\d+)", block).group(1))
        scratch = int(re.search(r"ScratchSize \[bytes/lane\]: (\d+)", block).group(1))
        occupancy = int(re.search(r"Occupancy \[waves/SIMD\]: (\d+)", block).group(1))
        assert spill == 0 and scratch == 0 and vgprs <= 224 and occupancy >= 2, block


# gemm_split_list_kernel<layout, waves, tokens per wave, aligned x, column tails, rows per step>
SMALL_BATCH_KERNEL = re.compile(
    r"Function Name: _ZN2q822gemm_split_list_kernelILi[01]ELi\d+ELi\d+ELb[01]ELb[01]ELi[48]EEE")


def test_small_batch_gemm_keeps_two_waves_per_simd(resource_remarks):
    """The exact small-batch GEMM is bound by vector issue and by its waits for
    LDS: a second wave per SIMD hides them (the 8-token variant with column
    tails ran alone on its SIMD once, a quarter slower)."""
    blocks = _blocks(resource_remarks, SMALL_BATCH_KERNEL)
    assert len(blocks) >= 60  # every waves x tokens form, both layouts, and the 4-row steps
    for block in blocks:
        occupancy = int(re.search(r"Occupancy \[waves/SIMD\]: (\d+)", block).group(1))
        spill = int(re.search(r"VGPRs Spill: (\d+)", block).group(1))
        assert occupancy >= 2 and spill == 0, block


def test_two_token_form_of_the_small_batch_gemm_fits_sixteen_workgroups_per_cu(resource_remarks):
    """One wave with two tokens over sealed weights without column tails stages
    half of a step's rows in LDS and loads the other half directly: 8 KB of LDS and
    at most 128 registers, so that 16 one-wave workgroups (4 waves per SIMD) keep
    128 KB per CU on their way instead of the 80 KB that 16 KB of LDS each allow."""
    pattern = re.compile(r"Function Name: _ZN2q822gemm_split_list_kernelILi1ELi1ELi2ELb[01]ELb0ELi8EEE")
    blocks = _blocks(resource_remarks, pattern)
    assert len(blocks) == 2
    for block in blocks:
        assert int(re.search(r"Occupancy \[waves/SIMD\]: (\d+)", block).group(1)) >= 4, block
        assert int(re.search(r"LDS Size \[bytes/block\]: (\d+)", block).group(1)) == 8192, block
        assert int(re.search(r"VGPRs Spill: (\d+)", block).group(1)) == 0, block
