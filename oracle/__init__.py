"""CPU oracle for the distillation-loss hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
directory; it is the checker that the HIP kernels are compared against (tests,
the smoke check and the CPU-baseline leg of the benchmark).
"""
