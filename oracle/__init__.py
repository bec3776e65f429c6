"""CPU oracle for the attention hot path.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package (``kvax_amd``) imports this; only ``tests/``, the smoke check and
the benchmark's CPU-baseline leg do, and only as the checker.
"""
