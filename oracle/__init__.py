"""CPU oracle: test infrastructure only (tests/, the smoke check and the benchmark's cpu_baseline leg)."""
