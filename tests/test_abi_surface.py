"""CPU-only checks of the drop-in boundary: the library loads, exports every
symbol that include/tm_hip.h declares, refuses to run without a device, and
validates null handles before touching one. No compute is called here."""
import ctypes
import os
import re

import pytest

from tuckmill_amd import hip as H

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "tm_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tm_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree_on_the_symbol_list():
    assert declared_symbols() == sorted(H.ABI_SYMBOLS)


def test_library_exports_every_declared_symbol():
    lib = H.load_library()
    for name in declared_symbols():
        assert getattr(lib, name) is not None, name


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(H, "_lib", None)
    monkeypatch.setattr(H, "LIB_PATH", os.path.join(ROOT, "tuckmill_amd", "nope.so"))
    with pytest.raises(H.TuckmillError) as e:
        H.load_library()
    assert e.value.code == "Unavailable" and "no CPU fallback" in str(e.value)


def test_null_context_is_refused_by_every_operation():
    lib = H.load_library()
    err = ctypes.create_string_buffer(H.ERR_CAP)
    U = H.TM_HIP_ERR_UNSUPPORTED
    assert lib.tm_hip_q8_0_gemv(None, None, None, None, 1, 32, err, H.ERR_CAP) == U
    assert b"null context" in err.value
    assert lib.tm_hip_q8_0_gemm(None, None, None, None, 1, 32, 1, 0, 0, err, H.ERR_CAP) == U
    assert lib.tm_hip_q8_0_gemm_mma(None, None, None, None, 1, 32, 1, 0, 0, err, H.ERR_CAP) == U
    assert lib.tm_hip_q8_0_row_f32(None, None, None, 0, 32, 0, err, H.ERR_CAP) == U
    assert lib.tm_hip_row_indirect_f32(None, None, 8, 1, 32, None, 0, None, err, H.ERR_CAP) == U
    assert lib.tm_hip_q8_0_pack(None, None, 1, 32, err, H.ERR_CAP) == U
    assert lib.tm_hip_q8_0_quantize_act(None, None, None, 32, 1, 0, err, H.ERR_CAP) == U
    assert lib.tm_hip_q8_0_gemm_i8(None, None, None, None, None, 1, 32, 1, 0, err, H.ERR_CAP) == U
    assert lib.tm_hip_fence(None, err, H.ERR_CAP) == U
    assert lib.tm_hip_begin_group(None, err, H.ERR_CAP) == U
    assert lib.tm_hip_upload(None, None, 0, None, 1, err, H.ERR_CAP) == U
    assert lib.tm_hip_buffer_new(None, 16, 1, err, H.ERR_CAP) is None
    assert lib.tm_hip_buffer_len(None, None) == 0
    assert lib.tm_hip_committed_dispatches(None) == 0
    assert lib.tm_hip_allocated_bytes(None) == 0
    # a NULL err buffer is allowed
    assert lib.tm_hip_fence(None, None, 0) == U


def test_error_mapping_follows_the_reference():
    # crates/metal/src/lib.rs:732-745
    assert H.hip_error(H.TM_HIP_ERR_BOUNDS, "", "x").code == "InvalidRequest"
    assert H.hip_error(H.TM_HIP_ERR_UNSUPPORTED, "", "x").code == "InvalidRequest"
    assert H.hip_error(H.TM_HIP_ERR_NO_DEVICE, "", "x").code == "Unavailable"
    assert H.hip_error(H.TM_HIP_ERR_ALLOC, "", "x").code == "Unavailable"
    assert H.hip_error(H.TM_HIP_ERR_INTERNAL, "", "x").code == "Internal"
    assert H.hip_error(H.TM_HIP_ERR_SOURCE, "", "x").code == "Internal"


def test_without_a_device_creation_is_refused_not_emulated():
    p = H.probe()
    if p.available:
        pytest.skip("a device is present; covered by the gpu tests")
    assert "no HIP device" in p.info
    with pytest.raises(H.TuckmillError) as e:
        H.HipContext.open()
    assert e.value.code == "Unavailable"
