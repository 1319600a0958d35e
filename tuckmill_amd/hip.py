"""Typed handles over the ``tm_hip_*`` C ABI (``include/tm_hip.h``).

The shape of this module follows the reference's Rust wrapper over its Metal
ABI (``crates/metal/src/lib.rs``): ``HipContext`` / ``HipBuffer`` carry the
same method names, argument meaning and error mapping as ``MetalContext`` /
``MetalBuffer``, and ``Matrix`` is the projection abstraction of
``crates/tuckcore/src/engine/metal.rs:106-226``.

There is no CPU fallback: loading fails loudly when ``libtm_hip.so`` has not
been built, and every operation runs on the GPU through the C ABI.
"""
from __future__ import annotations

import ctypes
import os
import threading
from dataclasses import dataclass

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtm_hip.so")

ERR_CAP = 512  # crates/metal/src/lib.rs:32
GEMM_MAX_BATCH = 32  # crates/metal/src/lib.rs:28-30
GEMM_MMA_MAX_BATCH = 512
PREFILL_BATCH = 128  # crates/tuckcore/src/engine/metal.rs:25 (the engine's prefill chunk)
# From this batch on tm_hip_q8_0_gemm_mma over sealed weights with 16-byte aligned
# activations may run on the bf16 matrix cores (activations split into three exact bf16
# pieces), when the products of its launch are large enough together (gemm_mma_launch_tile);
# below 17 tokens only a product that is large on its own (gemm_mma_small_batch_on_tiles),
# the others take the vector kernels there.
GEMM_MMA_BF16_MIN_BATCH = 5


def _bf16_units(rows: int, cols: int, batch: int, tokens: int):
    """(work units, K chunks) of a product on the bf16 matrix-core GEMM with tiles
    of `tokens` tokens x 256 rows: K is cut into at most eight chunks of 512
    columns or more, as many as give the product about 192 units of its own
    (mirror of q8::bx3_plan_with, csrc/q8_gemm_bf16x3.hpp)."""
    tiles = -(-batch // tokens) * -(-rows // 256)
    blocks = cols // 32
    chunks = min(-(-192 // tiles), -(-blocks // 16), 8)
    per_chunk = -(-blocks // chunks)
    chunks = -(-blocks // per_chunk)
    return tiles * chunks, chunks


def gemm_mma_launch_tile(shapes) -> int:
    """Tokens per tile (128 or 64) with which the products `shapes` = [(rows, cols,
    batch), ...] that share one launch run on the bf16 matrix cores, or 0 when they
    stay on the f32 ones (mirror of q8::bx3_launch_tile). All batches up to 32, all
    from 33 to 64, or all above. Up to 64 tokens: 16 M weights (32 M up to 32 tokens) and 128 units of
    the small tile between them. Above, in order of preference: 192 units or more of the large tile; 192 or
    more of the small tile; 128 or more of the large tile; the small tile for products of 3072
    columns and more with 32 units or more where the f32 kernel is estimated slower."""
    shapes = list(shapes)
    if not shapes:
        return 0
    small = sum(_bf16_units(r, c, b, 64)[0] for r, c, b in shapes)
    large = sum(_bf16_units(r, c, b, 128)[0] for r, c, b in shapes)
    if shapes[0][2] <= 32:  # half of the one token tile is padding: twice the weights
        return 64 if sum(r * c for r, c, _ in shapes) >= 1 << 25 and small >= 128 else 0
    if shapes[0][2] <= 64:
        return 64 if sum(r * c for r, c, _ in shapes) >= 1 << 24 and small >= 128 else 0
    if large >= 192:
        return 128
    if small >= 192:
        return 64
    if large >= 128:
        return 128
    # few output tiles under a deep K: the cheaper of two estimates (hundredths of a microsecond)
    if min(c for _, c, _ in shapes) < 3072 or small < 32:
        return 0
    shapes = shapes[:64]
    tmw, tiles, z = _f32_launch_shape(shapes)
    max_blocks = max(c // 32 for _, c, _ in shapes)
    per_wave = -(-max_blocks // (4 * z))
    f32_us = 450 + 72 * tmw * per_wave * (-(-(tiles * z) // 256))
    here_us = 2250 + 230 * (max_blocks * 32) // 1024
    return 64 if here_us < f32_us else 0


def _f32_launch_shape(shapes):
    """(tokens per wave tile / 32, output tiles, workgroups per tile) of a launch of
    `shapes` on the f32 matrix cores (mirror of q8::pick_mma_config, q8::mma_tiles and
    q8::mma_shared_parts)."""
    tiles64 = sum(-(-b // 64) * -(-r // 32) for r, _, b in shapes)
    short_last_round = tiles64 <= 128 or 256 < tiles64 <= 384
    tmw = 2 if max(b for _, _, b in shapes) > 32 and not short_last_round else 1
    tiles = sum(-(-b // (32 * tmw)) * -(-r // 32) for r, _, b in shapes)
    min_blocks = min(c // 32 for _, c, _ in shapes)
    z = 1
    if min_blocks >= 4:  # K split over the four waves of a workgroup
        while z < 8 and tiles * z * 2 <= 256 and min_blocks // (4 * z * 2) >= 4:
            z *= 2
    return tmw, tiles, z


def gemm_mma_bf16_plan(rows: int, cols: int, batch: int):
    """(tokens per tile, work units, worth it) of a product that launches alone."""
    tile = gemm_mma_launch_tile([(rows, cols, batch)])
    tokens = tile or (64 if batch <= 64 else 128)
    return tokens, _bf16_units(rows, cols, batch, tokens)[0], tile != 0


def gemm_mma_on_bf16(rows: int, cols: int, batch: int, x_off: int = 0) -> bool:
    """Whether tm_hip_q8_0_gemm_mma over sealed weights takes the bf16 matrix-core
    kernel for this product when it launches alone (mirror of gemv_key,
    csrc/tm_hip.cpp; the limits on region sizes beyond 4 GiB are left out). In a
    dispatch group the products that share a launch decide together
    (gemm_mma_launch_tile)."""
    if batch <= 16 and cols >= 1024 and not gemm_mma_small_batch_on_tiles(rows, cols, batch):
        return False
    return (batch >= GEMM_MMA_BF16_MIN_BATCH and x_off % 4 == 0 and
            gemm_mma_bf16_plan(rows, cols, batch)[2])


def gemm_mma_small_batch_on_tiles(rows: int, cols: int, batch: int) -> bool:
    """Whether a sealed product of 5 to 16 tokens leaves the vector kernels for the
    32-token tiles on the bf16 matrix cores (mirror of q8::mma_small_batch_on_tiles):
    32 M weights and more from 9 tokens, 128 M and more from 5. (From 9 tokens the
    products of one launch that are that large together do so as well:
    gemm_mma_launch_tile over the launch's shapes.)"""
    if batch < 5 or batch > 16:
        return False
    return rows * cols >= (1 << 27 if batch <= 8 else 1 << 25) and \
        gemm_mma_launch_tile([(rows, cols, batch)]) != 0


NOALLOC_WORKSPACE_BYTES = 64 << 20  # TM_HIP_NOALLOC_WORKSPACE_BYTES
NOALLOC_XS_BYTES = 20 << 20
GEMM_I8_MAX_BATCH = 2048
ARGMAX_NONE = 0xFFFFFFFF  # crates/metal/src/lib.rs (ARGMAX_NONE), native/metal/kernels.metal:143
ARGMAX_PARTIAL_BYTES = 512
CHECKSUM_PARTIAL_BYTES = 8192  # include/tm_hip.h TM_HIP_CHECKSUM_PARTIAL_BYTES
STAGING_CHUNK_BYTES = 4 << 20  # crates/tuckcore/src/qwen35_gpu.rs:1176

TM_HIP_ERR_NO_DEVICE = -1
TM_HIP_ERR_SOURCE = -2
TM_HIP_ERR_ALLOC = -3
TM_HIP_ERR_BOUNDS = -4
TM_HIP_ERR_UNSUPPORTED = -5
TM_HIP_ERR_INTERNAL = -6


class TuckmillError(Exception):
    """``code`` carries the reference's ErrorCode name."""

    def __init__(self, code: str, message: str, abi_code: int = 0):
        super().__init__(f"{code}: {message}")
        self.code = code
        self.message = message
        self.abi_code = abi_code


def hip_error(abi_code: int, text: str, what: str) -> TuckmillError:
    # crates/metal/src/lib.rs:732-745
    if abi_code in (TM_HIP_ERR_BOUNDS, TM_HIP_ERR_UNSUPPORTED):
        code = "InvalidRequest"
    elif abi_code in (TM_HIP_ERR_NO_DEVICE, TM_HIP_ERR_ALLOC):
        code = "Unavailable"
    else:
        code = "Internal"
    return TuckmillError(code, f"hip {what}: {text}", abi_code)


# ---- kernel selection (crates/tuckcore/src/kernels.rs:36-113) -----------------

class ResolvedKernels:
    """A concrete kernel implementation actually used at runtime."""
    SCALAR, NEON, METAL, HIP = "scalar", "neon", "metal", "hip"

    @staticmethod
    def default_for_target() -> str:
        import platform
        return ResolvedKernels.NEON if platform.machine() in ("aarch64", "arm64") \
            else ResolvedKernels.SCALAR


class KernelSelection:
    """``--kernels`` as the reference parses it, with ``hip`` beside ``metal``. A
    forced selection never falls back silently: ``hip`` without a usable gfx950
    device is a typed refusal at load."""
    NAMES = ("auto", "scalar", "neon", "metal", "hip")

    def __init__(self, name: str):
        self.name = name

    def __eq__(self, other):
        return isinstance(other, KernelSelection) and other.name == self.name

    def __repr__(self):
        return f"KernelSelection({self.name!r})"

    @staticmethod
    def parse(s: str):
        """kernels.rs:46-54: None for an unknown name."""
        return KernelSelection(s) if s in KernelSelection.NAMES else None

    def resolve(self, device: "Probe | None" = None) -> str:
        """kernels.rs:58-86. ``device`` stands in for the library's probe."""
        import platform
        import sys
        if self.name == "scalar":
            return ResolvedKernels.SCALAR
        if self.name == "auto":  # never a GPU path unasked
            return ResolvedKernels.default_for_target()
        if self.name == "metal":
            if sys.platform == "darwin":
                return ResolvedKernels.METAL
            raise TuckmillError("Unavailable", "the Metal kernel implementation requires macOS; "
                                "select --kernels auto, hip, neon, or scalar on this machine")
        if self.name == "neon":
            if platform.machine() in ("aarch64", "arm64"):
                return ResolvedKernels.NEON
            raise TuckmillError("InvalidRequest", "the NEON kernel implementation requires an "
                                "aarch64 target; select --kernels auto or --kernels scalar on this "
                                "machine")
        device = device if device is not None else probe()
        if not device.available:
            raise TuckmillError("Unavailable", "the HIP kernel implementation requires a gfx950 "
                                f"device ({device.info}); select --kernels auto or scalar on this "
                                "machine", TM_HIP_ERR_NO_DEVICE)
        return ResolvedKernels.HIP


# ---- numerical profile (crates/tuckcore/src/forward.rs:284-311) ---------------

class NumericalProfile:
    """``oracle-f32``: f32 activations, weights dequantized exactly. ``llama-cpu``:
    activations quantized per 32 to Q8_0 for Q8_0 weights, int8 block dots."""
    ORACLE_F32, LLAMA_CPU = "oracle-f32", "llama-cpu"

    @staticmethod
    def parse(s: str):
        return s if s in (NumericalProfile.ORACLE_F32, NumericalProfile.LLAMA_CPU) else None


def check_engine_options(kernels: str, profile: str, prefill_batch_given: bool = False):
    """The load-time checks of crates/tuckcore/src/executor.rs:294-314 with a
    device mode that covers Metal and HIP. The Metal path implements oracle-f32
    only (typed refusal); the HIP path also implements llama-cpu for Q8_0 weights."""
    device_mode = kernels in (ResolvedKernels.METAL, ResolvedKernels.HIP)
    if not device_mode and prefill_batch_given:
        raise TuckmillError("InvalidRequest", "prefill_batch applies only to the device kernel "
                            "paths (metal, hip); the resolved CPU kernels execute single-token "
                            "steps and must not silently ignore it")
    if NumericalProfile.parse(profile) is None:
        raise TuckmillError("InvalidRequest", f"unknown numerical profile {profile!r} "
                            "(oracle-f32, llama-cpu)")
    if kernels == ResolvedKernels.METAL and profile != NumericalProfile.ORACLE_F32:
        raise TuckmillError("UnsupportedArchitecture", "the Metal path implements the oracle-f32 "
                            "numerical profile only; select --numerical-profile oracle-f32, or "
                            "--kernels hip for llama-cpu on a GPU")


_lib = None
_lib_lock = threading.Lock()

_SIGS = {
    # name: (restype, argtypes)
    "tm_hip_available": (ctypes.c_int, []),
    "tm_hip_runtime_info": (ctypes.c_char_p, []),
    "tm_hip_create": (ctypes.c_void_p, [ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_destroy": (None, [ctypes.c_void_p]),
    "tm_hip_buffer_new": (ctypes.c_void_p, [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int,
                                            ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_buffer_free": (None, [ctypes.c_void_p, ctypes.c_void_p]),
    "tm_hip_buffer_len": (ctypes.c_size_t, [ctypes.c_void_p, ctypes.c_void_p]),
    "tm_hip_buffer_zero": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                                          ctypes.c_size_t, ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_upload": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                                     ctypes.c_void_p, ctypes.c_size_t, ctypes.c_char_p,
                                     ctypes.c_size_t]),
    "tm_hip_download": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                                       ctypes.c_void_p, ctypes.c_size_t, ctypes.c_char_p,
                                       ctypes.c_size_t]),
    "tm_hip_download_after": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t,
                                             ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint64,
                                             ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_f32_scale": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                         ctypes.c_float, ctypes.c_uint32, ctypes.c_char_p,
                                         ctypes.c_size_t]),
    "tm_hip_cast_f16_f32": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                            ctypes.c_uint32, ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_cast_f32_f16": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                            ctypes.c_uint32, ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_f32_axpy": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                        ctypes.c_float, ctypes.c_uint32, ctypes.c_char_p,
                                        ctypes.c_size_t]),
    "tm_hip_rmsnorm_f32": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                           ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint32,
                                           ctypes.c_float, ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_silu_mul_f32": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                            ctypes.c_void_p, ctypes.c_uint32, ctypes.c_char_p,
                                            ctypes.c_size_t]),
    "tm_hip_gelu_tanh_mul_f32": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                                 ctypes.c_void_p, ctypes.c_uint32, ctypes.c_char_p,
                                                 ctypes.c_size_t]),
    "tm_hip_argmax_f32": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint32,
                                          ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint32,
                                          ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_copy_f32": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint32,
                                       ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint32,
                                       ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_xor_checksum_u32": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint32,
                                               ctypes.c_uint32, ctypes.c_void_p, ctypes.c_char_p,
                                               ctypes.c_size_t]),
    "tm_hip_begin_group": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_end_group": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_abort_group": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_end_group_recorded": (ctypes.c_int, [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p),
                                                 ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_step_run": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_char_p,
                                       ctypes.c_size_t]),
    "tm_hip_step_launches": (ctypes.c_uint32, [ctypes.c_void_p, ctypes.c_void_p]),
    "tm_hip_step_free": (None, [ctypes.c_void_p, ctypes.c_void_p]),
    "tm_hip_fence": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_q8_0_gemv": (ctypes.c_int, [ctypes.c_void_p] * 4 + [ctypes.c_uint32] * 2 +
                         [ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_q8_0_gemm": (ctypes.c_int, [ctypes.c_void_p] * 4 + [ctypes.c_uint32] * 5 +
                         [ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_q8_0_gemm_mma": (ctypes.c_int, [ctypes.c_void_p] * 4 + [ctypes.c_uint32] * 5 +
                             [ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_q8_0_gemm_mma_noalloc": (ctypes.c_int, [ctypes.c_void_p] * 4 + [ctypes.c_uint32] * 5 +
                                     [ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_q8_0_row_f32": (ctypes.c_int, [ctypes.c_void_p] * 3 + [ctypes.c_uint32] * 3 +
                            [ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_f16_gemv": (ctypes.c_int, [ctypes.c_void_p] * 4 + [ctypes.c_uint32] * 2 +
                        [ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_f16_gemm": (ctypes.c_int, [ctypes.c_void_p] * 4 + [ctypes.c_uint32] * 5 +
                        [ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_f16_row_f32": (ctypes.c_int, [ctypes.c_void_p] * 3 + [ctypes.c_uint32] * 3 +
                           [ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_row_indirect_f32": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint32,
                                               ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p,
                                               ctypes.c_uint32, ctypes.c_void_p, ctypes.c_char_p,
                                               ctypes.c_size_t]),
    "tm_hip_q8_0_pack": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint32,
                                        ctypes.c_uint32, ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_q8_0_quantize_act": (ctypes.c_int, [ctypes.c_void_p] * 3 + [ctypes.c_uint32] * 3 +
                                 [ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_q8_0_gemm_i8_fma": (ctypes.c_int, [ctypes.c_void_p] * 4 + [ctypes.c_uint32] * 4 +
                                [ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_q8_0_gemm_i8": (ctypes.c_int, [ctypes.c_void_p] * 5 + [ctypes.c_uint32] * 4 +
                            [ctypes.c_char_p, ctypes.c_size_t]),
    "tm_hip_committed_dispatches": (ctypes.c_uint64, [ctypes.c_void_p]),
    "tm_hip_completed_dispatches": (ctypes.c_uint64, [ctypes.c_void_p]),
    "tm_hip_last_gpu_ms": (ctypes.c_double, [ctypes.c_void_p]),
    "tm_hip_gpu_nanos_total": (ctypes.c_uint64, [ctypes.c_void_p]),
    "tm_hip_kernel_launches": (ctypes.c_uint64, [ctypes.c_void_p]),
    "tm_hip_profile_set": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int]),
    "tm_hip_profile_read": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_uint32, ctypes.c_char_p,
                                           ctypes.c_size_t, ctypes.POINTER(ctypes.c_uint64),
                                           ctypes.POINTER(ctypes.c_uint64)]),
    "tm_hip_commit_log_set": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int]),
    "tm_hip_commit_log_read": (ctypes.c_size_t, [ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint64),
                                                 ctypes.c_size_t]),
    "tm_hip_allocated_bytes": (ctypes.c_uint64, [ctypes.c_void_p]),
    "tm_hip_in_flight_bytes": (ctypes.c_uint64, [ctypes.c_void_p]),
}

ABI_SYMBOLS = tuple(_SIGS)


def load_library() -> ctypes.CDLL:
    """Loads ``libtm_hip.so``; raises when it has not been built."""
    global _lib
    with _lib_lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise TuckmillError(
                    "Unavailable",
                    f"{LIB_PATH} is missing: build it with `python -m tuckmill_amd.build` "
                    "(there is no CPU fallback for the HIP path)")
            lib = ctypes.CDLL(LIB_PATH)
            for name, (restype, argtypes) in _SIGS.items():
                fn = getattr(lib, name)
                fn.restype = restype
                fn.argtypes = argtypes
            _lib = lib
    return _lib


@dataclass
class Probe:
    available: bool
    info: str


def probe() -> Probe:
    """Cheap device probe (crates/metal/src/lib.rs ``probe``)."""
    lib = load_library()
    return Probe(bool(lib.tm_hip_available()), lib.tm_hip_runtime_info().decode())


def _host_view(data):
    """(address, nbytes, keepalive) of a bytes-like object or numpy array."""
    if isinstance(data, np.ndarray):
        arr = np.ascontiguousarray(data)
        return arr.ctypes.data, arr.nbytes, arr
    mv = memoryview(data).cast("B")
    arr = np.frombuffer(mv, dtype=np.uint8)
    return arr.ctypes.data, arr.nbytes, arr


class _Inner:
    def __init__(self, raw):
        self.raw = raw
        self.lock = threading.RLock()
        self.live_buffers = 0

    def close(self):
        if self.raw:
            load_library().tm_hip_destroy(self.raw)
            self.raw = None


class HipContext:
    """One device context; every ABI call is serialized by one lock
    (crates/metal/src/lib.rs:695-708, :983-1005)."""

    def __init__(self, inner: _Inner):
        self._inner = inner
        self._lib = load_library()

    @staticmethod
    def open() -> "HipContext":
        lib = load_library()
        err = ctypes.create_string_buffer(ERR_CAP)
        raw = lib.tm_hip_create(err, ERR_CAP)
        if not raw:
            raise hip_error(TM_HIP_ERR_NO_DEVICE, err.value.decode(), "create")
        return HipContext(_Inner(raw))

    def close(self):
        self._inner.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    @property
    def raw(self):
        return self._inner.raw

    def _operate(self, name: str, fn, *args):
        with self._inner.lock:
            err = ctypes.create_string_buffer(ERR_CAP)
            code = fn(self._inner.raw, *args, err, ERR_CAP)
        if code != 0:
            raise hip_error(code, err.value.decode(), name)

    def _check_owned(self, *buffers):
        for b in buffers:
            if b is not None and b._ctx is not self._inner:
                raise TuckmillError("InvalidRequest",
                                    "buffer belongs to a different context", TM_HIP_ERR_UNSUPPORTED)

    # -- buffers ----------------------------------------------------------
    def buffer(self, nbytes: int, shared: bool = True) -> "HipBuffer":
        if nbytes == 0:
            raise TuckmillError("InvalidRequest", "zero-length HIP buffers are refused "
                                "(allocation must be explicit)", TM_HIP_ERR_BOUNDS)
        with self._inner.lock:
            err = ctypes.create_string_buffer(ERR_CAP)
            raw = self._lib.tm_hip_buffer_new(self._inner.raw, nbytes, 1 if shared else 0, err,
                                              ERR_CAP)
        if not raw:
            raise hip_error(TM_HIP_ERR_ALLOC, err.value.decode(), "buffer")
        return HipBuffer(self._inner, raw)

    # -- grouping / ordering ---------------------------------------------
    def begin_group(self):
        self._operate("begin_group", self._lib.tm_hip_begin_group)

    def end_group(self):
        self._operate("end_group", self._lib.tm_hip_end_group)

    def abort_group(self):
        self._operate("abort_group", self._lib.tm_hip_abort_group)

    def end_group_recorded(self) -> "HipStep":
        """Closes the open group as a replayable step instead of committing it."""
        raw = ctypes.c_void_p()
        self._operate("end_group_recorded", self._lib.tm_hip_end_group_recorded, ctypes.byref(raw))
        return HipStep(self._inner, self._lib, raw)

    def fence(self):
        self._operate("fence", self._lib.tm_hip_fence)

    # -- the Q8_0 products -------------------------------------------------
    def q8_0_gemv(self, w, x, y, rows: int, cols: int):
        self._check_owned(w, x, y)
        self._operate("q8_0_gemv", self._lib.tm_hip_q8_0_gemv, w.raw, x.raw, y.raw, rows, cols)

    def q8_0_gemm(self, w, x, y, rows, cols, batch, x_off=0, y_off=0):
        self._check_owned(w, x, y)
        self._operate("q8_0_gemm", self._lib.tm_hip_q8_0_gemm, w.raw, x.raw, y.raw, rows, cols,
                      batch, x_off, y_off)

    def q8_0_gemm_mma(self, w, x, y, rows, cols, batch, x_off=0, y_off=0):
        self._check_owned(w, x, y)
        self._operate("q8_0_gemm_mma", self._lib.tm_hip_q8_0_gemm_mma, w.raw, x.raw, y.raw, rows,
                      cols, batch, x_off, y_off)

    def q8_0_gemm_mma_noalloc(self, w, x, y, rows, cols, batch, x_off=0, y_off=0):
        """q8_0_gemm_mma launched at once out of the library's static device
        workspace: allocates nothing, is not a commit."""
        self._check_owned(w, x, y)
        self._operate("q8_0_gemm_mma_noalloc", self._lib.tm_hip_q8_0_gemm_mma_noalloc, w.raw, x.raw,
                      y.raw, rows, cols, batch, x_off, y_off)

    def q8_0_row(self, w, out, row: int, cols: int, out_off: int = 0):
        self._check_owned(w, out)
        self._operate("q8_0_row", self._lib.tm_hip_q8_0_row_f32, w.raw, out.raw, row, cols, out_off)

    # -- F16 weight twins ----------------------------------------------------
    def f16_gemv(self, w, x, y, rows: int, cols: int):
        self._check_owned(w, x, y)
        self._operate("f16_gemv", self._lib.tm_hip_f16_gemv, w.raw, x.raw, y.raw, rows, cols)

    def f16_gemm(self, w, x, y, rows, cols, batch, x_off=0, y_off=0):
        self._check_owned(w, x, y)
        self._operate("f16_gemm", self._lib.tm_hip_f16_gemm, w.raw, x.raw, y.raw, rows, cols,
                      batch, x_off, y_off)

    def f16_row(self, w, out, row: int, cols: int, out_off: int = 0):
        self._check_owned(w, out)
        self._operate("f16_row", self._lib.tm_hip_f16_row_f32, w.raw, out.raw, row, cols, out_off)

    def row_indirect_f32(self, w, type_id, rows, cols, ids, slot, out):
        self._check_owned(w, ids, out)
        self._operate("row_indirect", self._lib.tm_hip_row_indirect_f32, w.raw, type_id, rows, cols,
                      ids.raw, slot, out.raw)

    # -- the small f32 operators either side of a product (crates/metal/src/lib.rs:1027-1060,
    #    :2244-2319) --
    def f32_scale(self, x, y, factor, n):
        self._operate("f32_scale", self._lib.tm_hip_f32_scale, x.raw, y.raw, float(factor), n)

    def cast_f16_to_f32(self, x, y, n):
        """y = (f32) x over n binary16 elements (crates/metal/src/lib.rs:1636-1648)."""
        self._check_owned(x, y)
        self._operate("cast_f16_f32", self._lib.tm_hip_cast_f16_f32, x.raw, y.raw, n)

    def cast_f32_to_f16(self, x, y, n):
        """y = (half) x over n f32 elements, round to nearest even
        (crates/metal/src/lib.rs:1650-1662)."""
        self._check_owned(x, y)
        self._operate("cast_f32_f16", self._lib.tm_hip_cast_f32_f16, x.raw, y.raw, n)

    def f32_axpy(self, a, y, alpha, n):
        self._operate("f32_axpy", self._lib.tm_hip_f32_axpy, a.raw, y.raw, float(alpha), n)

    def rmsnorm(self, x, weight, y, rows, cols, eps):
        self._operate("rmsnorm", self._lib.tm_hip_rmsnorm_f32, x.raw, weight.raw, y.raw, rows, cols,
                      float(eps))

    def silu_mul(self, gate, up, out, n):
        self._operate("silu_mul", self._lib.tm_hip_silu_mul_f32, gate.raw, up.raw, out.raw, n)

    def gelu_tanh_mul(self, gate, up, out, n):
        self._operate("gelu_tanh_mul", self._lib.tm_hip_gelu_tanh_mul_f32, gate.raw, up.raw,
                      out.raw, n)

    def argmax_f32(self, x, n, partial, out, out_index):
        self._operate("argmax_f32", self._lib.tm_hip_argmax_f32, x.raw, n, partial.raw, out.raw,
                      out_index)

    def copy_f32(self, src, src_off, dst, dst_off, n):
        self._check_owned(src, dst)
        self._operate("copy_f32", self._lib.tm_hip_copy_f32, src.raw, src_off, dst.raw, dst_off, n)

    def xor_checksum_u32(self, src, src_off, n, partial):
        """Records the XOR of n 32-bit words of `src` as CHECKSUM_PARTIAL_BYTES / 4 partial
        words in `partial` (XOR them after a fence: `checksum_of`)."""
        self._check_owned(src, partial)
        self._operate("xor_checksum_u32", self._lib.tm_hip_xor_checksum_u32, src.raw, src_off, n,
                      partial.raw)

    @staticmethod
    def checksum_of(partial) -> int:
        words = np.frombuffer(partial.download(0, CHECKSUM_PARTIAL_BYTES), dtype=np.uint32)
        return int(np.bitwise_xor.reduce(words))

    # -- additions ---------------------------------------------------------
    def q8_0_pack(self, w, rows: int, cols: int):
        self._check_owned(w)
        self._operate("q8_0_pack", self._lib.tm_hip_q8_0_pack, w.raw, rows, cols)

    def q8_0_quantize_act(self, x, xq, cols, batch, x_off=0):
        self._check_owned(x, xq)
        self._operate("q8_0_quantize_act", self._lib.tm_hip_q8_0_quantize_act, x.raw, xq.raw, cols,
                      batch, x_off)

    def q8_0_gemm_i8(self, w, xq, y, rows, cols, batch, y_off=0, sumi=None):
        self._check_owned(w, xq, y, sumi)
        self._operate("q8_0_gemm_i8", self._lib.tm_hip_q8_0_gemm_i8, w.raw, xq.raw, y.raw,
                      sumi.raw if sumi is not None else None, rows, cols, batch, y_off)

    def q8_0_gemm_i8_fma(self, w, xq, y, rows, cols, batch, y_off=0):
        """The declared fast variant: exact block dots, each term fused into the sum."""
        self._check_owned(w, xq, y)
        self._operate("q8_0_gemm_i8_fma", self._lib.tm_hip_q8_0_gemm_i8_fma, w.raw, xq.raw, y.raw,
                      rows, cols, batch, y_off)

    # -- measurement -------------------------------------------------------
    def committed_dispatches(self) -> int:
        return int(self._lib.tm_hip_committed_dispatches(self._inner.raw))

    def completed_dispatches(self) -> int:
        return int(self._lib.tm_hip_completed_dispatches(self._inner.raw))

    def last_gpu_ms(self) -> float:
        return float(self._lib.tm_hip_last_gpu_ms(self._inner.raw))

    def gpu_nanos_total(self) -> int:
        return int(self._lib.tm_hip_gpu_nanos_total(self._inner.raw))

    def kernel_launches(self) -> int:
        return int(self._lib.tm_hip_kernel_launches(self._inner.raw))

    def allocated_bytes(self) -> int:
        return int(self._lib.tm_hip_allocated_bytes(self._inner.raw))

    def in_flight_bytes(self) -> int:
        return int(self._lib.tm_hip_in_flight_bytes(self._inner.raw))

    def live_gpu_bytes(self) -> int:
        return self.allocated_bytes() + self.in_flight_bytes()

    def set_commit_log(self, enabled: bool):
        """Starts (and clears) or stops the per-commit GPU time log."""
        with self._inner.lock:
            self._lib.tm_hip_commit_log_set(self._inner.raw, 1 if enabled else 0)

    def read_commit_log(self) -> np.ndarray:
        """GPU nanoseconds of the commits completed since the last read, oldest first."""
        out = np.empty(65536, dtype=np.uint64)
        with self._inner.lock:
            n = self._lib.tm_hip_commit_log_read(
                self._inner.raw, out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint64)), out.size)
        return out[:int(n)].copy()

    def set_profiling(self, enabled: bool):
        with self._inner.lock:
            self._lib.tm_hip_profile_set(self._inner.raw, 1 if enabled else 0)

    def profile_table(self):
        out = []
        index = 0
        while True:
            name = ctypes.create_string_buffer(64)
            nanos = ctypes.c_uint64(0)
            count = ctypes.c_uint64(0)
            with self._inner.lock:
                found = self._lib.tm_hip_profile_read(self._inner.raw, index, name, 64,
                                                      ctypes.byref(nanos), ctypes.byref(count))
            if not found:
                break
            out.append((name.value.decode(), int(nanos.value), int(count.value)))
            index += 1
        return out


class HipBuffer:
    """RAII-style handle; ``free()`` (or garbage collection) releases it."""

    def __init__(self, ctx: _Inner, raw):
        self._ctx = ctx
        self.raw = raw
        self._lib = load_library()

    def __len__(self) -> int:
        return self.len()

    def len(self) -> int:
        if not self.raw:
            return 0
        return int(self._lib.tm_hip_buffer_len(self._ctx.raw, self.raw))

    def free(self):
        if self.raw and self._ctx.raw:
            with self._ctx.lock:
                self._lib.tm_hip_buffer_free(self._ctx.raw, self.raw)
        self.raw = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass

    def _copy(self, name, fn, *args):
        with self._ctx.lock:
            err = ctypes.create_string_buffer(ERR_CAP)
            code = fn(self._ctx.raw, self.raw, *args, err, ERR_CAP)
        if code != 0:
            raise hip_error(code, err.value.decode(), name)

    def zero(self, offset: int, length: int):
        self._copy("buffer_zero", self._lib.tm_hip_buffer_zero, offset, length)

    def upload(self, offset: int, data):
        addr, nbytes, keep = _host_view(data)
        self._copy("upload", self._lib.tm_hip_upload, offset, addr, nbytes)
        del keep

    def download(self, offset: int, nbytes: int) -> np.ndarray:
        out = np.empty(nbytes, dtype=np.uint8)
        self._copy("download", self._lib.tm_hip_download, offset, out.ctypes.data, nbytes)
        return out

    def download_into(self, offset: int, out: np.ndarray):
        self._copy("download", self._lib.tm_hip_download, offset, out.ctypes.data, out.nbytes)

    def download_f32(self, offset_elems: int, n: int) -> np.ndarray:
        return self.download(offset_elems * 4, n * 4).view(np.float32)

    def download_after(self, offset: int, nbytes: int, completed_target: int) -> np.ndarray:
        out = np.empty(nbytes, dtype=np.uint8)
        # no lock, like crates/metal/src/lib.rs:2618-2633
        err = ctypes.create_string_buffer(ERR_CAP)
        code = self._lib.tm_hip_download_after(self._ctx.raw, self.raw, offset, out.ctypes.data,
                                               nbytes, completed_target, err, ERR_CAP)
        if code != 0:
            raise hip_error(code, err.value.decode(), "download_after")
        return out


class HipStep:
    """A recorded dispatch group (``HipContext.end_group_recorded``): ``run()``
    replays its launches as one commit; ``free()`` (or garbage collection)
    releases the graph and the buffer references it holds."""

    def __init__(self, ctx: _Inner, lib, raw):
        self._ctx = ctx
        self._lib = lib
        self.raw = raw

    def run(self):
        with self._ctx.lock:
            err = ctypes.create_string_buffer(ERR_CAP)
            code = self._lib.tm_hip_step_run(self._ctx.raw, self.raw, err, ERR_CAP)
        if code != 0:
            raise hip_error(code, err.value.decode(), "step_run")

    @property
    def launches(self) -> int:
        return int(self._lib.tm_hip_step_launches(self._ctx.raw, self.raw))

    def free(self):
        if self.raw and self._ctx.raw:
            with self._ctx.lock:
                self._lib.tm_hip_step_free(self._ctx.raw, self.raw)
        self.raw = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def q8_0_bytes(rows: int, cols: int) -> int:
    return rows * (cols // 32) * 34


def xq_bytes(cols: int, batch: int) -> int:
    """Size of a quantized-activation buffer (see tm_hip_q8_0_quantize_act)."""
    bpad = (batch + 3) & ~3
    return batch * cols + (cols // 32) * bpad * 4


def xq_split(raw: np.ndarray, cols: int, batch: int):
    """(quants int8 [batch, cols/32, 32], scales f32 [batch, cols/32]) of a
    downloaded quantized-activation buffer."""
    blocks = cols // 32
    bpad = (batch + 3) & ~3
    qs = raw[:batch * cols].view(np.int8).reshape(batch, blocks, 32)
    ds = raw[batch * cols:batch * cols + blocks * bpad * 4].view(np.float32).reshape(blocks, bpad)
    return qs, np.ascontiguousarray(ds[:, :batch].T)


class Matrix:
    """A device projection matrix: the HIP form of the reference's ``Matrix``
    (crates/tuckcore/src/engine/metal.rs:106-226): Q8_0 blocks (type 8) or
    F16 halves (type 1), uploaded raw, with the numerical profile its products
    run under (crates/tuckcore/src/forward.rs:606-645 switches per matvec):
    ``oracle-f32`` (default), or ``llama-cpu`` for Q8_0 weights — activations
    quantized per 32 on the device, int8 block dots, the f32 sum of
    kernels.rs:206-221 bit for bit; the matrix owns and sizes the
    quantized-activation buffer. F16 weights under ``llama-cpu`` have no device
    kernel here: a typed refusal at load, never a substitution.
    ``fused_i8_tail`` (llama-cpu only, off unless asked for): the int8 products go
    through ``q8_0_gemm_i8_fma``, whose block dots are the same exact integers but
    whose f32 sum takes each term with a fused multiply-add: faster from 5 tokens,
    within 1e-5 of the CPU's result instead of bit-identical to it."""

    def __init__(self, buf: HipBuffer, type_id: int, in_dim: int, out_dim: int,
                 profile: str = NumericalProfile.ORACLE_F32, fused_i8_tail: bool = False):
        if fused_i8_tail and profile != NumericalProfile.LLAMA_CPU:
            raise TuckmillError("InvalidRequest", "fused_i8_tail names a variant of the llama-cpu "
                                "profile's int8 product; this matrix runs under " + profile,
                                TM_HIP_ERR_UNSUPPORTED)
        self.buf = buf
        self.type_id = type_id
        self.in_dim = in_dim
        self.out_dim = out_dim
        self.profile = profile
        self.fused_i8_tail = fused_i8_tail
        self._xq = None  # quantized activations of the llama-cpu profile

    @staticmethod
    def plan(in_dim: int, out_dim: int, type_id: int = 8) -> int:
        return out_dim * in_dim * 2 if type_id == 1 else q8_0_bytes(out_dim, in_dim)

    @staticmethod
    def load(ctx: HipContext, raw, in_dim: int, out_dim: int, type_id: int = 8,
             seal: bool = True, profile: str = NumericalProfile.ORACLE_F32,
             fused_i8_tail: bool = False) -> "Matrix":
        """Staged raw upload in 4 MiB slices (engine/metal.rs:138-147), then
        the seal step that re-lays the weights out for the device."""
        if out_dim <= 1:
            raise TuckmillError("Internal", "1-D tensors use the f32 path")
        if type_id not in (1, 8):
            raise TuckmillError("UnsupportedQuantization",
                                f"engine matrices must be F16 or Q8_0; got type {type_id}")
        if NumericalProfile.parse(profile) is None:
            raise TuckmillError("InvalidRequest", f"unknown numerical profile {profile!r} "
                                "(oracle-f32, llama-cpu)", TM_HIP_ERR_UNSUPPORTED)
        if fused_i8_tail and profile != NumericalProfile.LLAMA_CPU:
            raise TuckmillError("InvalidRequest", "fused_i8_tail names a variant of the llama-cpu "
                                "profile's int8 product; this matrix runs under " + profile,
                                TM_HIP_ERR_UNSUPPORTED)
        if profile == NumericalProfile.LLAMA_CPU and type_id != 8:
            raise TuckmillError("UnsupportedArchitecture",
                                "the HIP path implements the llama-cpu numerical profile for Q8_0 "
                                "weights only; F16 weights run under oracle-f32",
                                TM_HIP_ERR_UNSUPPORTED)
        raw = np.ascontiguousarray(np.frombuffer(raw, dtype=np.uint8) if not
                                   isinstance(raw, np.ndarray) else raw).view(np.uint8).ravel()
        total = Matrix.plan(in_dim, out_dim, type_id)
        if raw.size != total:
            raise TuckmillError("InvalidArtifact", f"tensor holds {raw.size} bytes, "
                                f"expected {total}")
        buf = ctx.buffer(total, True)
        off = 0
        while off < total:
            n = min(STAGING_CHUNK_BYTES, total - off)
            buf.upload(off, raw[off:off + n])
            off += n
        if seal and type_id == 8:
            ctx.q8_0_pack(buf, out_dim, in_dim)
        return Matrix(buf, type_id, in_dim, out_dim, profile, fused_i8_tail)

    def _gemm_llama_cpu(self, ctx: HipContext, x: HipBuffer, y: HipBuffer, batch: int):
        """forward.rs:783-821 on the device: quantize the activations once per
        product, then the int8 product, in slices of GEMM_I8_MAX_BATCH tokens."""
        rows, cols = self.out_dim, self.in_dim
        t0 = 0
        while t0 < batch:
            n = min(batch - t0, GEMM_I8_MAX_BATCH)
            need = xq_bytes(cols, n)
            if self._xq is None or self._xq.len() < need:
                # (a buffer replaced while an open group still names it stays alive:
                # the group holds its memory)
                self._xq = ctx.buffer(need, True)
            ctx.q8_0_quantize_act(x, self._xq, cols, n, t0 * cols)
            if self.fused_i8_tail:
                ctx.q8_0_gemm_i8_fma(self.buf, self._xq, y, rows, cols, n, t0 * rows)
            else:
                ctx.q8_0_gemm_i8(self.buf, self._xq, y, rows, cols, n, t0 * rows)
            t0 += n

    def gemv(self, ctx: HipContext, x: HipBuffer, y: HipBuffer):
        if self.profile == NumericalProfile.LLAMA_CPU:
            self._gemm_llama_cpu(ctx, x, y, 1)
        elif self.type_id == 1:
            ctx.f16_gemv(self.buf, x, y, self.out_dim, self.in_dim)
        else:
            ctx.q8_0_gemv(self.buf, x, y, self.out_dim, self.in_dim)

    def gemm(self, ctx: HipContext, x: HipBuffer, y: HipBuffer, batch: int, exact: bool):
        rows, cols = self.out_dim, self.in_dim
        if self.profile == NumericalProfile.LLAMA_CPU:
            # exact whatever the batch: the int8 products are bit-identical to the CPU's
            self._gemm_llama_cpu(ctx, x, y, batch)
            return
        if not exact and self.type_id == 8 and 2 <= batch <= GEMM_MMA_MAX_BATCH:
            ctx.q8_0_gemm_mma(self.buf, x, y, rows, cols, batch, 0, 0)
            return
        product = ctx.f16_gemm if self.type_id == 1 else ctx.q8_0_gemm
        t0 = 0
        while t0 < batch:
            n = min(batch - t0, GEMM_MAX_BATCH)
            product(self.buf, x, y, rows, cols, n, t0 * cols, t0 * rows)
            t0 += n

    def row_indirect(self, ctx: HipContext, ids: HipBuffer, slot: int, out: HipBuffer):
        ctx.row_indirect_f32(self.buf, self.type_id, self.out_dim, self.in_dim, ids, slot, out)

    def row_into(self, ctx: HipContext, row: int, out: HipBuffer, out_off: int):
        if self.type_id == 1:
            ctx.f16_row(self.buf, out, row, self.in_dim, out_off)
        else:
            ctx.q8_0_row(self.buf, out, row, self.in_dim, out_off)
