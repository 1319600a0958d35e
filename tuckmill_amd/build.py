"""Builds the HIP library in-tree for gfx950 (hipcc cross-compiles without a GPU)."""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libtm_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -packed-fp32-ops is switched off on purpose: v_pk_*_f32 forms are not used
# by this library (the flag is for the device pass; the host pass warns that
# it does not know the feature, which is harmless).
DEVICE_FLAGS = [
    "--offload-arch=gfx950",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-ffp-contract=off",
]


# The library is two translation units: the host logic (tm_hip.cpp: no device
# code, seconds to compile) and the kernels with their launchers (tm_launch.cpp).
SOURCES = ("tm_hip.cpp", "tm_launch.cpp")


def build_library(verbose: bool = False, extra: list[str] | None = None) -> str:
    from concurrent.futures import ThreadPoolExecutor

    common = [HIPCC, "-x", "hip", "-std=c++17", "-O3", "-fPIC",
              "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
              *DEVICE_FLAGS,
              "-I", os.path.join(ROOT, "include"), "-I", CSRC,
              *(extra or [])]
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)

    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, capture_output=True, text=True)
        out = "\n".join(l for l in (res.stdout + res.stderr).splitlines()
                        if "packed-fp32-ops" not in l and l.strip())
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed ({res.returncode}):\n{out}")
        return out

    objs = [os.path.join(objdir, src.replace(".cpp", ".o")) for src in SOURCES]
    with ThreadPoolExecutor(max_workers=len(SOURCES)) as pool:
        outs = list(pool.map(run, [[*common, "-c", "-o", obj, os.path.join(CSRC, src)]
                                   for src, obj in zip(SOURCES, objs)]))
    outs.append(run([HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB, *objs]))
    if verbose:
        for out in outs:
            if out:
                print(out)
    return LIB


HOST_LIB = os.path.join(HERE, "libtm_host.so")
CXX = os.environ.get("CXX", "g++")


def build_host(verbose: bool = False) -> str:
    """The C++ host layer above the C ABI (typed handles + native step runner)."""
    cmd = [CXX, "-std=c++17", "-O2", "-fPIC", "-shared", "-Wall", "-Wextra",
           "-I", os.path.join(ROOT, "include"), "-I", os.path.join(HERE, "host"),
           "-o", HOST_LIB, os.path.join(HERE, "host", "workloads.cpp"),
           "-L", HERE, "-ltm_hip", "-Wl,-rpath,$ORIGIN"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"host build failed ({res.returncode}):\n{res.stdout}{res.stderr}")
    if verbose and (res.stdout or res.stderr):
        print(res.stdout + res.stderr)
    return HOST_LIB


def build_all(verbose: bool = False) -> None:
    build_library(verbose)
    build_host(verbose)


if __name__ == "__main__":
    build_library(verbose=True, extra=sys.argv[1:])
    build_host(verbose=True)
    print("built", LIB, HOST_LIB)
