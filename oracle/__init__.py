"""CPU parity oracle for the quantized-matmul path.

TEST INFRASTRUCTURE: imported only by tests, by the smoke check and by the
`cpu_baseline` leg of the benchmark.  The product package never imports it.
"""
