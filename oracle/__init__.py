"""CPU oracle for the row-wise FP8 GEMM path. TEST INFRASTRUCTURE ONLY.

Nothing under oracle/ is part of the product: only tests/, __graft_entry__.smoke() and
the cpu_baseline leg of bench.py may import it, and only as the checker.
"""
