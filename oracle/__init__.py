"""CPU checkers for the GPU kernels.  TEST INFRASTRUCTURE ONLY.

These modules restate, in numpy, the arithmetic of the reference's generated
kernels (the files and lines each function cites).  Only `tests/`,
`__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py` may import
them; no module under `deca_amd/` does, and the product has no CPU path.

Parity status (what pins each function is listed in its module header):
every function here is pinned by library routines and closed forms in
tests/test_oracle_*.py; none is "parity unpinned".
"""
