"""Benchmark entry points that mirror the reference's mooncake-ep/benchmarks/."""
