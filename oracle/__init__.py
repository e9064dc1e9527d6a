"""CPU oracle for the quantized-linear path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package (`xla_amd/`) imports this directory.  Only
`tests/`, `__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py`
may use it, and only as the checker.
"""
