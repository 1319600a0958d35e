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

# gemv_list_kernel<PACKED, 8 rows, 1 token, aligned x, no tail set, any list capacity, no fused norm>
DECODE_KERNEL = re.compile(r"Function Name: _ZN2q816gemv_list_kernelILi1ELi8ELi1ELb1ELi0ELi\d+ELb0EEE")


def test_decode_kernel_keeps_four_waves_per_simd(tmp_path):
    hipcc = shutil.which(B.HIPCC) or (B.HIPCC if os.path.exists(B.HIPCC) else None)
    if hipcc is None:
        pytest.skip("hipcc not available")
    cmd = [hipcc, "-x", "hip", "-std=c++17", "-O3", *B.DEVICE_FLAGS, "--cuda-device-only",
           "-I", os.path.join(B.ROOT, "include"), "-I", B.CSRC,
           "-Rpass-analysis=kernel-resource-usage", "-c", os.path.join(B.CSRC, "tm_hip.cpp"),
           "-o", str(tmp_path / "device.o")]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    lines = res.stderr.splitlines()
    start = [i for i, l in enumerate(lines) if DECODE_KERNEL.search(l)]
    assert start, "decode kernel not found in the resource remarks"
    for at in start:  # the long- and the short-list instantiation
        block = "\n".join(lines[at:at + 14])
        vgprs = int(re.search(r" VGPRs: (\d+)", block).group(1))
        spill = int(re.search(r"VGPRs Spill: (\d+)", block).group(1))
        occupancy = int(re.search(r"Occupancy \[waves/SIMD\]: (\d+)", block).group(1))
        assert spill == 0
        assert vgprs <= 128 and occupancy >= 4, f"{vgprs} VGPRs, {occupancy} waves/SIMD"
