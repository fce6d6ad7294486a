"""TEST INFRASTRUCTURE ONLY - CPU restatement of the reference's FP8 block-scaled GEMM path.

Nothing under this directory is part of the product: only tests/, __graft_entry__.smoke() and the
``cpu_baseline`` leg of bench.py may import it, and only as the checker.
"""
