"""TEST INFRASTRUCTURE ONLY.

CPU oracle for the GPU operators: a restatement of what the reference's c-mcpu
backend computes.  Nothing in the shipped package imports this; it is used by
tests/, by __graft_entry__.smoke() as the checker, and by bench.py to time the
CPU baseline.
"""
