"""CPU oracle for the MXFP4 hot path (TEST INFRASTRUCTURE ONLY).

Nothing under ``alto_amd`` may import this package: it exists so that tests,
the smoke check and the benchmark's CPU-baseline leg can compare the HIP
kernels against an independent restatement of the reference arithmetic.
"""
from .mxfp4_oracle import *  # noqa: F401,F403
