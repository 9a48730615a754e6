"""Writes tests/golden/routing_vectors.npz: what the reference's own routing generators
(mooncake-ep/benchmarks/ep_benchmark/routing.py: uniform, k-hot, Zipf) return for a few seeds and shapes,
so that the generators of mooncake_amd/benchmarks/ep_benchmark/routing.py can be held to them value for
value.  No other check pins a seed's tensors (the definitions - distinct experts, expected loads, error
conditions - are tested separately), which is why this one script loads a file of the reference: the module
needs nothing but torch and is run here, in the build container, where /root/reference exists.  The vectors
travel; the reference does not.

    python tests/golden/make_routing_golden.py            (from the repository root)

The fixture holds data only: per case the arguments (as a JSON string), topk_idx (int32) and topk_weights
(float32 bit patterns)."""
import importlib.util
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REFERENCE = "/root/reference/mooncake-ep/benchmarks/ep_benchmark/routing.py"

# (mode, num_tokens, num_experts, top_k, seed, extra keyword arguments)
CASES = [
    ("uniform", 64, 32, 4, 0, {}),
    ("uniform", 33, 256, 8, 7, {}),
    ("uniform", 128, 8, 2, 2026, {}),
    ("k_hot", 64, 32, 4, 0, {}),                                        # the defaults: 4 hot experts, 0.9
    ("k_hot", 100, 256, 8, 3, {"hot_experts": 32, "hot_fraction": 0.9}),  # the shipped incast configuration
    ("k_hot", 37, 16, 2, 11, {"hot_experts": 2, "hot_fraction": 0.5}),
    ("zipf", 64, 32, 4, 0, {}),
    ("zipf", 100, 256, 8, 5, {"zipf_alpha": 1.0}),
    ("zipf", 50, 64, 6, 9, {"zipf_alpha": 1.2}),
]


def main() -> int:
    spec = importlib.util.spec_from_file_location("reference_ep_benchmark_routing", REFERENCE)
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    out = {"torch_version": np.array(torch.__version__)}
    for i, (mode, tokens, experts, top_k, seed, extra) in enumerate(CASES):
        idx, weights = module.ROUTING_MODES[mode](tokens, experts, top_k, device=torch.device("cpu"), seed=seed, **extra)
        assert idx.dtype == torch.int64 and weights.dtype == torch.float32
        out[f"case{i}_args"] = np.array(json.dumps({"mode": mode, "num_tokens": tokens, "num_experts": experts,
                                                    "top_k": top_k, "seed": seed, "extra": extra}))
        out[f"case{i}_topk_idx"] = idx.numpy().astype(np.int32)
        out[f"case{i}_topk_weights"] = weights.numpy().view(np.int32).copy()
    np.savez_compressed(os.path.join(HERE, "routing_vectors.npz"), **out)
    print(f"wrote {len(CASES)} cases to tests/golden/routing_vectors.npz")
    return 0


if __name__ == "__main__":
    sys.exit(main())
