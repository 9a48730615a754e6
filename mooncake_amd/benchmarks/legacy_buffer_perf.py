#!/usr/bin/env python3
"""Native-loop dispatch + combine benchmark: Python owns the tensors, the timed
loop runs inside the HIP library with no Python or torch call in it.

Counterpart of the reference's mooncake-ep/benchmarks/legacy_buffer_perf.py
(flags :21-29, tensors :52-82, report :107-117) and its native loop
`mooncake._ep._benchmark_legacy_buffer` (legacy_buffer_perf.cpp:84-146).  The
reference runs one process per GPU under torchrun; here `--ranks` logical
ranks share one GPU and the loop drives all of them, so there is one report
line for the world instead of one per rank.

    python -m mooncake_amd.benchmarks.legacy_buffer_perf --ranks 32 --tokens 128 --experts 256
"""
from __future__ import annotations

import argparse
from typing import Dict, Sequence

import torch

from mooncake_amd import ep


def parse_args(argv: Sequence[str] | None = None) -> argparse.Namespace:
    parser = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    parser.add_argument("--ranks", type=int, default=8, help="logical ranks (the reference's world size)")
    parser.add_argument("--tokens", type=int, default=128)
    parser.add_argument("--hidden", type=int, default=7168)
    parser.add_argument("--experts", type=int, default=288)
    parser.add_argument("--topk", type=int, default=8)
    parser.add_argument("--warmups", type=int, default=20)
    parser.add_argument("--iterations", type=int, default=30)
    return parser.parse_args(argv)


def run(args: argparse.Namespace, device: str = "cuda") -> Dict[str, float]:
    R = args.ranks
    if args.experts % R:
        raise ValueError("--experts must be divisible by world size")
    if args.hidden % 128:
        raise ValueError("--hidden must be divisible by 128")
    dev = torch.device(device)
    L, RM = args.experts // R, R * args.tokens
    x, topk_idx, topk_weights = [], [], []
    for r in range(R):
        # rank r's inputs from seed r, as each reference process does (:46)
        gen = torch.Generator(device=dev).manual_seed(r)
        x.append(torch.randn((args.tokens, args.hidden), dtype=torch.bfloat16, device=dev, generator=gen))
        scores = torch.randn((args.tokens, args.experts), dtype=torch.float32, device=dev, generator=gen)
        topk_idx.append(scores.topk(args.topk, dim=-1).indices.contiguous())
        topk_weights.append(torch.rand((args.tokens, args.topk), dtype=torch.float32, device=dev, generator=gen))
    active_ranks = torch.ones((R, R), dtype=torch.int32, device=dev)
    expert_x = torch.randn((R, L, RM, args.hidden), dtype=torch.bfloat16, device=dev)
    packed_recv_x = torch.empty_like(expert_x)
    packed_recv_count = torch.empty((R, L), dtype=torch.int32, device=dev)
    packed_recv_src_info = torch.empty((R, L, RM), dtype=torch.int32, device=dev)
    packed_recv_layout_range = torch.empty((R, L, R), dtype=torch.int64, device=dev)
    combined_x = torch.empty((R, args.tokens, args.hidden), dtype=torch.bfloat16, device=dev)
    cache_flush = torch.empty(int(256e6 // 4), dtype=torch.int32, device=dev)

    def per_rank(t) -> list:
        return [t[r].data_ptr() for r in range(R)]

    tensors = {
        "x": per_rank(x), "topk_idx": per_rank(topk_idx), "topk_weights": per_rank(topk_weights),
        "active_ranks": per_rank(active_ranks), "expert_x": per_rank(expert_x),
        "packed_recv_x": per_rank(packed_recv_x), "packed_recv_count": per_rank(packed_recv_count),
        "packed_recv_src_info": per_rank(packed_recv_src_info),
        "packed_recv_layout_range": per_rank(packed_recv_layout_range), "combined_x": per_rank(combined_x),
    }
    world = ep.World(R)
    cache_flush.zero_()
    stream = torch.cuda.current_stream(dev)
    average_us, min_us, max_us = world.legacy_buffer_perf(
        tensors, num_tokens=args.tokens, hidden=args.hidden, num_topk=args.topk, num_local_experts=L,
        num_max_dispatch_tokens_per_rank=args.tokens, num_experts=args.experts, warmups=args.warmups,
        iterations=args.iterations, compute_stream_ptr=int(stream.cuda_stream))
    # the reference's payload figure (:109-110): every selection moves a bf16 row out and a bf16 row back
    selections = sum(int(t.numel()) for t in topk_idx)
    payload_bytes = selections * args.hidden * 4
    return {"bandwidth_gbs": payload_bytes / average_us / 1e3, "average_us": average_us, "min_us": min_us,
            "max_us": max_us, "ranks": R}


def main(argv: Sequence[str] | None = None) -> Dict[str, float]:
    out = run(parse_args(argv))
    print(f"[world of {out['ranks']} ranks] Native dispatch + combine: {out['bandwidth_gbs']:.2f} GB/s, "
          f"avg_t={out['average_us']:.2f} us, min_t={out['min_us']:.2f} us, max_t={out['max_us']:.2f} us",
          flush=True)
    return out


if __name__ == "__main__":
    main()
