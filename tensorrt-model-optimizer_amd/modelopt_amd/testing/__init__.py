"""Synthetic workloads used by the benchmarks and tests (no checkpoints, no datasets)."""
