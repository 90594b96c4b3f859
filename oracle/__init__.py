"""CPU oracle for the single-GPU MoE hot path.

TEST INFRASTRUCTURE ONLY.  This package restates, on the CPU, what the
reference computes on the path this repository accelerates.  Only tests/,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it, and only as the checker; the product package never does.
"""
