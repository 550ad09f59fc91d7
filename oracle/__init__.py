"""CPU oracle for the quantized-linear forward: TEST INFRASTRUCTURE ONLY.

`oracle_np` is the numpy restatement, `oracle_c` loads the C restatement
(`oq_oracle.c`, built by `oracle/build.py`).  Only tests, the smoke check and the
CPU-baseline leg of the benchmark may import this package; the shipped
`orbitquant_amd` package never does.
"""
