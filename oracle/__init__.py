"""CPU oracle for the MoE expert-layer hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package may import, call or
link anything in this directory.  Only `tests/`, `__graft_entry__.smoke()` and
the `cpu_baseline` leg of `bench.py` use it, and only as the checker.
"""
