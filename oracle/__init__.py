"""CPU oracle for the pipeline-stage hot path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``pippy_amd/`` imports this package; only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do, and only as the
checker.  The reference (pytorch/PiPPy 0.2.0) has no arithmetic of its own on this path: every
number comes from a torch call, so the oracle restates the reference's control flow in plain
Python and uses torch's CPU fp32 kernels for the arithmetic.  Each function cites the reference
lines it follows.
"""
