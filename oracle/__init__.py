"""CPU oracle for the Q8_0 matrix-product path: TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the benchmark's CPU-baseline leg may import
this package. The product (``tuckmill_amd``) never does.
"""
from .oracle import *  # noqa: F401,F403
