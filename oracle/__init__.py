"""CPU checker for the fused MXFP4 MoE path.  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the CPU-baseline leg of the benchmark import
this package; the GPU library never does.
"""
from .pyoracle import *  # noqa: F401,F403
