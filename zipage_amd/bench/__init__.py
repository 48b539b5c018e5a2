"""Benchmark harness: synthetic workloads at the benchmark shapes and the pool-placement probe.
Nothing in the product (kernel wrappers, compress.py, engine) imports this package."""
