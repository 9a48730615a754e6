"""Latency percentiles, expert load and the result document of the EP
benchmark, in the schema of the reference's
mooncake-ep/benchmarks/ep_benchmark/metrics.py (percentiles :10-21, expert load
:24-63, document :66-137)."""
from __future__ import annotations

import json
from typing import Any, Dict, Optional, Sequence

import numpy as np
import torch

PERCENTILES = (("p50", 50.0), ("p90", 90.0), ("p99", 99.0), ("p999", 99.9))
EMPTY_LOAD = {"max_tokens_per_expert": 0, "min_tokens_per_expert": 0, "mean_tokens_per_expert": 0,
              "imbalance_ratio": 0}


def compute_percentiles(values) -> Dict[str, float]:
    """p50 / p90 / p99 / p999 (numpy's linear interpolation) and the mean of latencies in ms; zeros when empty."""
    arr = np.asarray(values, dtype=np.float64)
    if arr.size == 0:
        return {**{name: 0.0 for name, _ in PERCENTILES}, "mean": 0.0}
    out = {name: float(np.percentile(arr, q)) for name, q in PERCENTILES}
    out["mean"] = float(arr.mean())
    return out


def compute_global_expert_load(topk_idx: torch.Tensor, num_experts: int, group=None) -> Dict[str, float]:
    """Selections per expert over the whole world, with imbalance_ratio =
    max / mean.  The reference all-reduces each rank's bincount over `group`
    (metrics.py:39-49); here `topk_idx` holds every logical rank's selections
    ([R, T, K] or any shape), so the sum is one bincount.  Entries < 0 (masked
    selections) are not counted."""
    flat = topk_idx.reshape(-1).to(torch.int64)
    flat = flat[flat >= 0]
    counts = torch.bincount(flat, minlength=num_experts).to(torch.float64)
    hi, lo, mean = float(counts.max()), float(counts.min()), float(counts.mean())
    return {
        "max_tokens_per_expert": hi,
        "min_tokens_per_expert": lo,
        "mean_tokens_per_expert": mean,
        "imbalance_ratio": hi / mean if mean > 0 else 0.0,
    }


def assemble_json_output(backend: str, world_size: int, num_experts: int, hidden_size: int, top_k: int,
                         num_tokens: int, dtype: str, routing_mode: str, zero_copy: bool, async_finish: bool,
                         return_recv_hook: bool, warmup_iters: int, iters: int,
                         hot_experts: Optional[int] = None, hot_fraction: Optional[float] = None,
                         zipf_alpha: Optional[float] = None,
                         dispatch_latencies_ms: Optional[Sequence[float]] = None,
                         combine_latencies_ms: Optional[Sequence[float]] = None,
                         e2e_latencies_ms: Optional[Sequence[float]] = None,
                         expert_load: Optional[Dict[str, float]] = None, pg_backend: str = "nccl", *,
                         per_rank_stats: Dict[str, Any]) -> Dict[str, Any]:
    """The result document: run parameters, then `metrics` with the three
    latency distributions, tokens_per_second = world tokens / mean end-to-end
    latency, expert load and per-rank statistics (metrics.py:66-137)."""
    doc: Dict[str, Any] = dict(
        benchmark="mooncake_ep", backend=backend, world_size=world_size, num_experts=num_experts,
        hidden_size=hidden_size, top_k=top_k, num_tokens=num_tokens, dtype=dtype, routing_mode=routing_mode,
        zero_copy=zero_copy, async_finish=async_finish, return_recv_hook=return_recv_hook,
        warmup_iters=warmup_iters, iters=iters, pg_backend=pg_backend)
    if routing_mode == "k_hot":
        doc.update(hot_experts=hot_experts, hot_fraction=hot_fraction)
    elif routing_mode == "zipf":
        doc.update(zipf_alpha=zipf_alpha)
    e2e = compute_percentiles(e2e_latencies_ms or [])
    mean_s = e2e["mean"] / 1000.0
    doc["metrics"] = {
        "dispatch_latency_ms": compute_percentiles(dispatch_latencies_ms or []),
        "combine_latency_ms": compute_percentiles(combine_latencies_ms or []),
        "end_to_end_latency_ms": e2e,
        "tokens_per_second": num_tokens * world_size / mean_s if mean_s > 0 else 0.0,
        "expert_load": expert_load or dict(EMPTY_LOAD),
        "per_rank_stats": per_rank_stats,
    }
    return doc


def write_json_output(data: Dict[str, Any], path: str) -> None:
    with open(path, "w") as f:
        json.dump(data, f, indent=2)
