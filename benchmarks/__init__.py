"""Workload drivers behind bench.py: the single-op microbenchmarks and the full-shape model runs."""
