"""Benchmark drivers: YAML shape lists in, CSV rows out (the reference's benchmarks/ and datasets/)."""
