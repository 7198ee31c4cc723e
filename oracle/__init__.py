"""CPU oracle (test infrastructure): see oracle.cpp for what it restates and
what pins it.  Import from tests, the smoke check and the benchmark's
cpu_baseline leg only."""
