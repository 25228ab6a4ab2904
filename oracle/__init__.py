"""CPU restatement of the reference's FP8 GEMM arithmetic.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package imports this; it is the
checker used by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py``.
"""
