"""CPU oracle for the training-GEMM path.  TEST INFRASTRUCTURE ONLY.

Nothing under this package is part of the product: only tests/, the smoke check
and the benchmark's cpu_baseline leg may import it.  The product path
(vkgrad_amd/) never falls back to it and fails loudly without its HIP library.
"""
