"""CPU oracle of the HisCache hot path -- test infrastructure, not part of the product.

Only tests, the smoke check and the benchmark's CPU-baseline leg import this package.
"""
