"""CPU restatements of the reference path, used only as the checker.

TEST INFRASTRUCTURE: only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg
import this package. The product (chessrl_amd) never does and has no CPU fallback.
"""
