"""MI355X-native Q8_0 matrix-product path for TuckCore (HIP, gfx950).

``tuckmill_amd.hip`` holds the typed handles over the C ABI declared in
``include/tm_hip.h``; ``tuckmill_amd.build`` compiles the library in-tree.
"""
from .hip import (GEMM_MAX_BATCH, GEMM_MMA_MAX_BATCH, HipBuffer, HipContext,  # noqa: F401
                  Matrix, TuckmillError, load_library, probe)
