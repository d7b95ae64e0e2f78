"""Benchmark definitions with the axes of the reference's benchmark/ops/*.py files, runnable as
`python -m iris_amd.bench.suites.<name> [--axis_M=...] [--benchmark_format=json]`."""
