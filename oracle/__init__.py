"""CPU oracle for the add_m / scan / sgemm / bf16-gemm path.

TEST INFRASTRUCTURE ONLY: import from tests/, __graft_entry__.smoke() and
bench.py's cpu_baseline leg, never from prism_amd/.
"""
from .oracle import *  # noqa: F401,F403
