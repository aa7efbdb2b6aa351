"""CPU oracle for the fused encoder-layer path.  TEST INFRASTRUCTURE ONLY.

Nothing under this package is part of the product: only the test suite, the
smoke check and the benchmark's CPU-baseline leg may import it, and there only
as the checker / the timed CPU baseline.  The HIP path never routes through it.
"""
