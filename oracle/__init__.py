"""CPU parity oracle for the sLSTM forward path.

TEST INFRASTRUCTURE ONLY: importable from ``tests/``, from the smoke check and
from the benchmark's CPU-baseline leg.  The product package never imports it.
"""
