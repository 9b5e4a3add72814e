"""CPU oracle of the FP8 hot path.  Test infrastructure: imported by tests/, smoke() and the
cpu_baseline leg of bench.py only."""
