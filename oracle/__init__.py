"""CPU checker for the SpMM / SDDMM kernels.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package imports this directory: the test-suite, the
smoke check and the benchmark's CPU-baseline leg are its only users.
"""
