"""CPU oracle for the LUT-GEMM hot path -- TEST INFRASTRUCTURE ONLY.

Only the test-suite, the smoke check and the CPU-baseline leg of the benchmark
may import this package.  The shipped package never does; its compute path is
the HIP library and nothing else.
"""
from .oracle import *  # noqa: F401,F403
