"""CPU checker for the Stream-K GEMM path.  TEST INFRASTRUCTURE ONLY: imported by tests/, the smoke
check and the benchmark's cpu_baseline leg -- never by the shipped package."""
