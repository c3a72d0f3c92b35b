"""TEST INFRASTRUCTURE ONLY: CPU checkers for the PackKV hot path.

Nothing in the product package imports this.  Only tests, the smoke check and
the benchmark's CPU-baseline leg do.
"""
