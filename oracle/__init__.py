"""CPU oracle (test infrastructure only).

Nothing under this package is part of the shipped product: only the test
suite, the smoke check and the benchmark's CPU-baseline leg may import it,
and only as the checker that the HIP path is compared against.
"""
