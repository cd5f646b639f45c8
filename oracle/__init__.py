"""CPU oracle for the ring-attractor time loop.

TEST INFRASTRUCTURE ONLY.  Nothing under this package is part of the shipped
path: only tests, the smoke check and the benchmark's cpu_baseline leg may
import it, and only as the checker that the HIP kernels are compared against.
"""
