"""CPU oracle for the fused per-layer kernels -- TEST INFRASTRUCTURE ONLY.

Only the test-suite, the smoke check and the benchmark's cpu_baseline leg import this package;
the product (`inferspore_amd`) never does.
"""
from .binding import Oracle, load, build  # noqa: F401
