"""CPU oracle (test infrastructure).  Only tests, the smoke entry and the benchmark's
cpu_baseline leg import this package; the product package never does."""
