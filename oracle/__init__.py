"""CPU oracle for the Liger hot path: test infrastructure only (parity checker and CPU baseline).

Nothing in the shipped GPU package imports this module; only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py do.
"""
