"""Workload drivers shared by bench.py and the tests: BASELINE configs[4] (the MLP training step as
ZeNu's op sequence, written once against the Matrix API) and the HIP device it runs on.  Nothing here
touches the CPU oracle; the CPU device of the same step lives beside the oracle (oracle/cpu_dev.py)."""
