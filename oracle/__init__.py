"""CPU oracle for the fused-attention hot path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this directory: it exists so that tests, the smoke check
and the CPU-baseline leg of the benchmark can compare the HIP kernels with an independent fp32/fp64
restatement of the reference's torch math.
"""
