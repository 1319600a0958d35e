"""Kernel selection and numerical profile on the host handles, without a GPU:
`--kernels hip` beside auto / scalar / neon / metal
(crates/tuckcore/src/kernels.rs:36-113), the profile names
(crates/tuckcore/src/forward.rs:284-311) and the load-time checks of
crates/tuckcore/src/executor.rs:294-314. The C++ types (host/tm_hip.hpp) are
reached through libtm_host.so, the Python mirror directly; both must agree."""
import ctypes
import os
import platform

import pytest

from tuckmill_amd import hip as H

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
AARCH64 = platform.machine() in ("aarch64", "arm64")
# error classes of the C surface: 1 unknown name, 2 InvalidRequest, 3 Unavailable,
# 4 UnsupportedArchitecture
CLASS = {2: "InvalidRequest", 3: "Unavailable", 4: "UnsupportedArchitecture"}


@pytest.fixture(scope="module")
def host():
    H.load_library()
    lib = ctypes.CDLL(os.path.join(ROOT, "tuckmill_amd", "libtm_host.so"))
    lib.tmh_resolve_kernels.restype = ctypes.c_int
    lib.tmh_resolve_kernels.argtypes = [ctypes.c_char_p, ctypes.c_int, ctypes.c_char_p,
                                        ctypes.c_size_t, ctypes.c_char_p, ctypes.c_size_t]
    lib.tmh_check_engine_options.restype = ctypes.c_int
    lib.tmh_check_engine_options.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_int,
                                             ctypes.c_char_p, ctypes.c_size_t]
    return lib


def resolve_cpp(host, name, device):
    out, err = ctypes.create_string_buffer(32), ctypes.create_string_buffer(512)
    rc = host.tmh_resolve_kernels(name.encode(), device, out, 32, err, 512)
    return rc, out.value.decode(), err.value.decode()


def resolve_py(name, available):
    sel = H.KernelSelection.parse(name)
    if sel is None:
        return 1, "", "unknown"
    try:
        return 0, sel.resolve(H.Probe(available, "test device" if available else "no device")), ""
    except H.TuckmillError as e:
        return {v: k for k, v in CLASS.items()}[e.code], "", e.message


def test_parse_knows_the_five_names_and_nothing_else():
    # kernels.rs:46-54 plus "hip"
    for name in ("auto", "scalar", "neon", "metal", "hip"):
        assert H.KernelSelection.parse(name) == H.KernelSelection(name)
    for name in ("", "Hip", "cuda", "rocm", "gpu", "metal "):
        assert H.KernelSelection.parse(name) is None


@pytest.mark.parametrize("name,device,want", [
    ("scalar", 0, (0, "scalar")), ("scalar", 1, (0, "scalar")),
    # auto never chooses a GPU path unasked (kernels.rs:61, :95-101)
    ("auto", 1, (0, "neon" if AARCH64 else "scalar")),
    ("hip", 1, (0, "hip")),
    # a forced selection never falls back silently (kernels.rs:38-41)
    ("hip", 0, (3, "")),
    ("metal", 1, (3, "")),          # requires macOS: Unavailable (kernels.rs:62-72)
    ("neon", 1, (0, "neon") if AARCH64 else (2, "")),  # InvalidRequest (kernels.rs:73-83)
    ("vulkan", 1, (1, "")),
])
def test_resolve_in_both_mirrors(host, name, device, want):
    rc, resolved, err = resolve_cpp(host, name, device)
    assert (rc, resolved) == want, err
    rc_py, resolved_py, _ = resolve_py(name, bool(device))
    assert (rc_py, resolved_py) == want
    if rc in CLASS:
        assert "--kernels" in err  # the refusal names what to select instead


def test_hip_without_a_device_is_refused_here(host):
    # this container has no GPU: the library's own probe must say so
    if H.probe().available:
        pytest.skip("a device is present")
    rc, _, err = resolve_cpp(host, "hip", -1)
    assert rc == 3 and "gfx950" in err
    with pytest.raises(H.TuckmillError) as e:
        H.KernelSelection.parse("hip").resolve()
    assert e.value.code == "Unavailable" and e.value.abi_code == H.TM_HIP_ERR_NO_DEVICE


def test_numerical_profile_names():
    # forward.rs:297-311
    assert H.NumericalProfile.parse("oracle-f32") == H.NumericalProfile.ORACLE_F32
    assert H.NumericalProfile.parse("llama-cpu") == H.NumericalProfile.LLAMA_CPU
    for name in ("", "oracle", "llama_cpu", "f32"):
        assert H.NumericalProfile.parse(name) is None


@pytest.mark.parametrize("kernels,profile,prefill,want", [
    ("hip", "oracle-f32", 1, 0), ("hip", "llama-cpu", 1, 0), ("hip", "llama-cpu", 0, 0),
    ("metal", "oracle-f32", 1, 0),
    # executor.rs:308-314: the Metal path is oracle-f32 only
    ("metal", "llama-cpu", 0, 4),
    # executor.rs:296-301: prefill_batch must not be silently ignored by CPU kernels
    ("scalar", "oracle-f32", 1, 2), ("neon", "llama-cpu", 1, 2),
    ("scalar", "llama-cpu", 0, 0),
    ("hip", "fp8", 0, 1),
])
def test_engine_option_checks_in_both_mirrors(host, kernels, profile, prefill, want):
    err = ctypes.create_string_buffer(512)
    rc = host.tmh_check_engine_options(kernels.encode(), profile.encode(), prefill, err, 512)
    assert rc == want, err.value.decode()
    if want == 0:
        H.check_engine_options(kernels, profile, bool(prefill))
    else:
        with pytest.raises(H.TuckmillError) as e:
            H.check_engine_options(kernels, profile, bool(prefill))
        assert e.value.code == CLASS.get(want, "InvalidRequest")


def test_matrix_refuses_an_unsupported_profile_before_touching_the_device():
    class NoContext:  # load must refuse before it allocates anything
        def buffer(self, *a, **k):
            raise AssertionError("allocated")

    with pytest.raises(H.TuckmillError) as e:
        H.Matrix.load(NoContext(), bytes(64 * 2 * 2), 64, 2, type_id=1,
                      profile=H.NumericalProfile.LLAMA_CPU)
    assert e.value.code == "UnsupportedArchitecture"
    with pytest.raises(H.TuckmillError) as e:
        H.Matrix.load(NoContext(), bytes(68), 32, 2, profile="bf16")
    assert e.value.code == "InvalidRequest"
