"""CPU oracle for the fused linear + cross-entropy path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this
directory; only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may use it, and only as the checker.
"""
from .lce_oracle import (  # noqa: F401
    OracleResult,
    lce_forward_fp64,
    lce_forward_backward_fp64,
    lce_bruteforce,
    eager_fp32_step,
    eager_fp32_step_chunked,
)
