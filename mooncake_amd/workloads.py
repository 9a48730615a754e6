"""Seeded synthetic workloads for the dispatch/combine path.

The five named configurations are the ones the benchmark contract lists; the
routing generators follow the methods of the reference's benchmark harness
(mooncake-ep/benchmarks/ep_benchmark/routing.py:19-146: top-k of Gaussian
scores for uniform routing, Gumbel top-k over Zipf log-probabilities for
skewed routing, softmax weights).  Everything is drawn on the CPU from one
`torch.Generator` so a (config, seed) pair names the same tensors everywhere.
"""
from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Dict, List

import torch


@dataclass(frozen=True)
class EPConfig:
    name: str
    num_ranks: int          # logical EP ranks, all resident in one GPU's HBM
    tokens_per_rank: int
    hidden: int
    num_experts: int
    num_topk: int
    use_fp8: bool
    routing: str = "uniform"        # "uniform" | "zipf"
    zipf_alpha: float = 1.2
    outlier_fraction: float = 0.0   # fraction of token rows scaled x100
    masked_fraction: float = 0.0    # fraction of tokens with every topk_idx = -1

    @property
    def max_tokens(self) -> int:
        return self.tokens_per_rank

    @property
    def num_local_experts(self) -> int:
        return self.num_experts // self.num_ranks

    @property
    def total_tokens(self) -> int:
        return self.num_ranks * self.tokens_per_rank


CONFIGS: Dict[str, EPConfig] = {
    # 0: the case the CPU PyTorch statement of the contract is checked on
    "cpu_check": EPConfig("cpu_check", 4, 128, 2048, 16, 4, False),
    # 1: DeepSeek-V3 decode, the configuration the headline metric is quoted on
    "dsv3_decode": EPConfig("dsv3_decode", 32, 128, 7168, 256, 8, True),
    # 2: Qwen3-MoE decode
    "qwen3_decode": EPConfig("qwen3_decode", 16, 256, 4096, 128, 8, False),
    # 3: DeepSeek-V3 prefill burst: 4096 tokens in total, skewed routing, fp8 outliers
    "dsv3_prefill": EPConfig("dsv3_prefill", 32, 128, 7168, 256, 8, True, routing="zipf",
                             zipf_alpha=1.2, outlier_fraction=0.01),
    # 4: Mixtral: 8192 tokens in total, 10 % of tokens masked
    "mixtral": EPConfig("mixtral", 8, 1024, 4096, 8, 2, False, masked_fraction=0.10),
}
CONFIG_ORDER: List[str] = ["cpu_check", "dsv3_decode", "qwen3_decode", "dsv3_prefill", "mixtral"]


def shrink(cfg: EPConfig, **kw) -> EPConfig:
    """A smaller case of the same family (for oracle-sized parity tests)."""
    return replace(cfg, **kw)


def uniform_routing(num_tokens: int, num_experts: int, top_k: int, gen: torch.Generator) -> torch.Tensor:
    scores = torch.randn(num_tokens, num_experts, dtype=torch.float32, generator=gen)
    return torch.topk(scores, top_k, dim=-1)[1].to(torch.int64)


def zipf_routing(num_tokens: int, num_experts: int, top_k: int, gen: torch.Generator, alpha: float) -> torch.Tensor:
    ids = torch.arange(1, num_experts + 1, dtype=torch.float32)
    log_probs = -alpha * torch.log(ids)
    log_probs = log_probs - log_probs.logsumexp(dim=0)
    u = torch.rand(num_tokens, num_experts, dtype=torch.float32, generator=gen).clamp(min=1e-20)
    gumbel = -torch.log(-torch.log(u))
    return torch.topk(log_probs.unsqueeze(0) + gumbel, top_k, dim=-1)[1].to(torch.int64)


def generate(cfg: EPConfig, seed: int = 0) -> Dict[str, torch.Tensor]:
    """CPU tensors for the whole logical world, rank-major:
    x bf16 [R, T, H], topk_idx int64 [R, T, K], topk_weights f32 [R, T, K]."""
    gen = torch.Generator().manual_seed(seed)
    R, T, H, E, K = cfg.num_ranks, cfg.tokens_per_rank, cfg.hidden, cfg.num_experts, cfg.num_topk
    xs, idxs, ws = [], [], []
    for _ in range(R):
        x = torch.randn(T, H, dtype=torch.float32, generator=gen)
        if cfg.outlier_fraction > 0:
            rows = torch.rand(T, generator=gen) < cfg.outlier_fraction
            x[rows] *= 100.0
        if cfg.routing == "zipf":
            idx = zipf_routing(T, E, K, gen, cfg.zipf_alpha)
        else:
            idx = uniform_routing(T, E, K, gen)
        w = torch.softmax(torch.randn(T, K, dtype=torch.float32, generator=gen), dim=-1)
        if cfg.masked_fraction > 0:
            masked = torch.rand(T, generator=gen) < cfg.masked_fraction
            idx[masked] = -1
        xs.append(x.to(torch.bfloat16))
        idxs.append(idx)
        ws.append(w)
    return {
        "x": torch.stack(xs).contiguous(),
        "topk_idx": torch.stack(idxs).contiguous(),
        "topk_weights": torch.stack(ws).contiguous(),
    }


def algorithmic_bytes(cfg: EPConfig, num_valid_selections: int) -> Dict[str, int]:
    """Bytes the path has to move at minimum (what achieved GB/s is priced on).

    dispatch: read every token row and its K indices once; write one payload
    row (+ per-128 scales in fp8 mode) and one src_info entry per selection,
    plus the per-expert counts and (expert, source rank) ranges.
    combine: read one bf16 row per selection, K (index, weight) pairs per token
    and the src_info entry of each row; write one bf16 row per token.
    """
    N, H, K, E, R = cfg.total_tokens, cfg.hidden, cfg.num_topk, cfg.num_experts, cfg.num_ranks
    S = num_valid_selections
    P = H + H // 128 * 4 if cfg.use_fp8 else 2 * H
    dispatch = N * H * 2 + N * K * 8 + S * (P + 4) + E * 4 + E * R * 8
    combine = S * H * 2 + N * K * 12 + S * 4 + N * H * 2
    return {"dispatch": dispatch, "combine": combine}
