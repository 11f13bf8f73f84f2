"""CPU oracle (test infrastructure).  Import from tests/, smoke() and bench.py's cpu_baseline leg only."""
