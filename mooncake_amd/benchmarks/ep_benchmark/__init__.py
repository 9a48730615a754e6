"""Dispatch/combine benchmark with the routing modes, flags and JSON schema of
the reference's mooncake-ep/benchmarks/ep_benchmark/."""
