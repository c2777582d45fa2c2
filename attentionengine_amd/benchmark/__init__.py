"""Benchmark harness of the example scripts (``from benchmark.bench_utils import ...``)."""
