"""CPU oracle for the block-quantized linear path: test infrastructure only.

Only the test suite, the smoke check and the benchmark's cpu_baseline leg import this package.
"""
