"""CPU oracle for the CLUSTEN ops.  TEST INFRASTRUCTURE ONLY.

Nothing in the product package imports this directory.  It may be used by `tests/`, by
`__graft_entry__.smoke()` and by the `cpu_baseline` leg of `bench.py` — as the checker and as the
timed CPU baseline, never as a fallback for the HIP kernels.
"""
