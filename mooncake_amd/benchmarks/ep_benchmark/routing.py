"""Routing generators of the EP benchmark: which experts each token selects.

Same three modes, signatures, defaults and error conditions as the reference's
mooncake-ep/benchmarks/ep_benchmark/routing.py (uniform :19-44, k-hot :47-103,
Zipf :106-146, table :149-153).  Each generator draws from one seeded
`torch.Generator` in the order the reference's text does (scores, then
weights), so a seed gives the reference's tensors value for value on the CPU:
the tests hold the generators to the definitions (distinct experts, expected
loads, error conditions) and to vectors written by the reference's own
generators (tests/golden/routing_vectors.npz).
"""
from __future__ import annotations

from typing import Callable, Dict, Optional, Tuple

import torch

Routing = Tuple[torch.Tensor, torch.Tensor]   # topk_idx [T, K] int64, topk_weights [T, K] f32


def _generator(device: Optional[torch.device], seed: int) -> Tuple[torch.device, torch.Generator]:
    dev = torch.device("cpu") if device is None else torch.device(device)
    return dev, torch.Generator(device=dev).manual_seed(seed)


def _gaussian_topk(rows: int, columns: int, top_k: int, dev: torch.device, gen: torch.Generator) -> torch.Tensor:
    """Top-k of i.i.d. normal scores: k distinct columns, uniformly distributed."""
    scores = torch.randn(rows, columns, dtype=torch.float32, device=dev, generator=gen)
    return scores.topk(top_k, dim=-1).indices.to(torch.int64)


def generate_topk_weights(num_tokens: int, top_k: int, device: torch.device,
                          generator: torch.Generator) -> torch.Tensor:
    """Softmax of uniform(0, 1) draws: positive weights that sum to one per token (routing.py:10-16)."""
    draws = torch.rand(num_tokens, top_k, dtype=torch.float32, device=device, generator=generator)
    return draws.softmax(dim=-1)


def uniform_routing(num_tokens: int, num_experts: int, top_k: int, device: Optional[torch.device] = None,
                    seed: int = 0, **kwargs) -> Routing:
    """Every expert equally likely (routing.py:19-44)."""
    dev, gen = _generator(device, seed)
    topk_idx = _gaussian_topk(num_tokens, num_experts, top_k, dev, gen)
    return topk_idx, generate_topk_weights(num_tokens, top_k, dev, gen)


def k_hot_routing(num_tokens: int, num_experts: int, top_k: int, device: Optional[torch.device] = None,
                  seed: int = 0, hot_experts: int = 4, hot_fraction: float = 0.9, **kwargs) -> Routing:
    """Incast: int(num_tokens * hot_fraction) tokens take all their experts
    from the first `hot_experts`; the others route uniformly; token order is
    then shuffled (routing.py:47-103).  ValueError for hot_experts outside
    [top_k, num_experts] or hot_fraction outside (0, 1)."""
    if hot_experts > num_experts:
        raise ValueError(f"hot_experts ({hot_experts}) > num_experts ({num_experts})")
    if hot_experts < top_k:
        raise ValueError(f"hot_experts ({hot_experts}) < top_k ({top_k}); cannot pick {top_k} distinct experts "
                         f"from {hot_experts} hot experts")
    if not 0.0 < hot_fraction < 1.0:
        raise ValueError(f"hot_fraction must be in (0, 1), got {hot_fraction}")
    dev, gen = _generator(device, seed)
    hot_tokens = int(num_tokens * hot_fraction)
    hot = _gaussian_topk(hot_tokens, hot_experts, top_k, dev, gen)
    cold = _gaussian_topk(num_tokens - hot_tokens, num_experts, top_k, dev, gen)
    order = torch.randperm(num_tokens, generator=gen, device=dev)
    topk_idx = torch.cat([hot, cold], dim=0)[order]
    return topk_idx, generate_topk_weights(num_tokens, top_k, dev, gen)


def zipfian_routing(num_tokens: int, num_experts: int, top_k: int, device: Optional[torch.device] = None,
                    seed: int = 0, zipf_alpha: float = 1.0, **kwargs) -> Routing:
    """P(expert i) proportional to (i + 1) ** -alpha, k experts per token
    without replacement by the Gumbel top-k trick (routing.py:106-146)."""
    if zipf_alpha <= 0:
        raise ValueError(f"zipf_alpha must be > 0, got {zipf_alpha}")
    dev, gen = _generator(device, seed)
    ranks = torch.arange(1, num_experts + 1, dtype=torch.float32, device=dev)
    log_p = -zipf_alpha * ranks.log()
    log_p = log_p - log_p.logsumexp(dim=0)
    u = torch.rand(num_tokens, num_experts, dtype=torch.float32, device=dev, generator=gen).clamp(min=1e-20)
    gumbel = -torch.log(-torch.log(u))
    topk_idx = (log_p.unsqueeze(0) + gumbel).topk(top_k, dim=-1).indices.to(torch.int64)
    return topk_idx, generate_topk_weights(num_tokens, top_k, dev, gen)


ROUTING_MODES: Dict[str, Callable[..., Routing]] = {
    "uniform": uniform_routing,
    "k_hot": k_hot_routing,
    "zipf": zipfian_routing,
}
