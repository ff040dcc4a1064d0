"""CPU oracle for the raw-block quantized matmul path.

TEST INFRASTRUCTURE ONLY. Nothing in the shipped package imports this directory; it exists so that
tests, the smoke check and the CPU-baseline leg of the benchmark have an independent statement of
what the GPU kernels must compute.
"""
