#!/usr/bin/env python3
"""Dispatch / combine benchmark with the flags, cycle and result document of
the reference's mooncake-ep/benchmarks/ep_benchmark/run_ep_benchmark.py.

    python -m mooncake_amd.benchmarks.ep_benchmark.run_ep_benchmark \\
        --num-ranks 8 --num-experts 256 --hidden-size 7168 --top-k 8 --num-tokens 1024 \\
        --routing-mode k_hot --hot-experts 32 --hot-fraction 0.9 --async-finish

One measured iteration is the reference's (run_ep_benchmark.py:311-334):
dispatch, mock expert forward (rows times expert_id * 0.1 + 1, :291-301),
combine, with an event pair around dispatch, one around combine, and
end-to-end = dispatch start to combine end.

Where the reference spawns one process per GPU, here the `--num-ranks` ranks
are logical ranks of one world on one GPU.  `--api buffer` (the default) makes
the reference's calls rank by rank on `mooncake_amd.mooncake_ep_buffer.Buffer`
objects: a collective is launched when its last rank has called, so the event
pairs include the host time of the other ranks' calls.  `--api world` makes
one whole-world call per collective and times the kernels alone.  Either way
a collective ends for all ranks at once, so every rank's entry in
`per_rank_stats` is the world's series.
"""
from __future__ import annotations

import argparse
import json
import sys
from typing import Any, Dict, List, Sequence, Tuple

import torch

from mooncake_amd import ep
from mooncake_amd.harness import WorldHarness
from mooncake_amd.mooncake_ep_buffer import Buffer, LogicalGroup
from mooncake_amd.workloads import EPConfig

from .metrics import assemble_json_output, compute_global_expert_load, compute_percentiles, write_json_output
from .routing import ROUTING_MODES

# flag, type, default, help -- the reference's flags (run_ep_benchmark.py:40-171)
_VALUE_FLAGS = (
    ("--backend", str, "hip", "device backend label for the result document"),
    ("--num-ranks", int, 8, "number of EP ranks (logical ranks on this GPU)"),
    ("--num-experts", int, 256, "experts over all ranks"),
    ("--hidden-size", int, 7168, "hidden dimension"),
    ("--top-k", int, 8, "experts per token"),
    ("--num-tokens", int, 1024, "tokens per rank"),
    ("--hot-experts", int, 32, "hot experts (k_hot mode)"),
    ("--hot-fraction", float, 0.9, "fraction of tokens routed to the hot experts (k_hot mode)"),
    ("--zipf-alpha", float, 1.0, "Zipf exponent (zipf mode)"),
    ("--warmup-iters", int, 20, "untimed iterations"),
    ("--iters", int, 100, "measured iterations"),
    ("--seed", int, 0, "base seed; rank r uses seed + r"),
    ("--json-output", str, None, "write the result document here instead of stdout"),
)
_SWITCHES = (
    ("--zero-copy", "zero-copy combine through get_next_combine_buffer"),
    ("--async-finish", "event-based completion of dispatch / combine"),
    ("--return-recv-hook", "hook-based completion of dispatch / combine"),
)


def parse_args(argv: Sequence[str] | None = None) -> argparse.Namespace:
    """A JSON file named by --config supplies defaults; flags given on the command line win (:28-37,:173-176)."""
    first = argparse.ArgumentParser(add_help=False)
    first.add_argument("--config", default=None)
    known, _ = first.parse_known_args(argv)
    parser = argparse.ArgumentParser(description="Mooncake EP dispatch/combine benchmark on one MI355X")
    parser.add_argument("--config", type=str, default=None, help="JSON file of defaults")
    for flag, kind, default, text in _VALUE_FLAGS:
        parser.add_argument(flag, type=kind, default=default, help=text)
    for flag, text in _SWITCHES:
        parser.add_argument(flag, action="store_true", help=text)
    parser.add_argument("--dtype", choices=["bf16", "fp8"], default="bf16", help="dispatch payload type")
    parser.add_argument("--routing-mode", choices=sorted(ROUTING_MODES), default="uniform")
    parser.add_argument("--pg-backend", type=str, default="none",
                        help="recorded in the result document; there is no process group on one GPU")
    parser.add_argument("--api", choices=["buffer", "world"], default="buffer",
                        help="per-rank Buffer calls (reference-shaped) or one whole-world call per collective")
    if known.config:
        with open(known.config) as f:
            parser.set_defaults(**json.load(f))
    return parser.parse_args(argv)


def validate_args(args: argparse.Namespace) -> None:
    """The reference's checks (:181-193) plus what the logical world adds."""
    if args.num_experts % args.num_ranks != 0:
        raise ValueError(f"num_experts ({args.num_experts}) must be divisible by num_ranks ({args.num_ranks})")
    if args.async_finish and args.return_recv_hook:
        raise ValueError("async_finish and return_recv_hook are mutually exclusive")
    if args.dtype == "fp8" and args.hidden_size % 128 != 0:
        raise ValueError(f"hidden_size ({args.hidden_size}) must be divisible by 128 for fp8 dtype")
    if args.api == "world" and args.zero_copy:
        raise ValueError("--zero-copy belongs to --api buffer")
    if args.api == "world" and (args.async_finish or args.return_recv_hook):
        # a whole-world call is one stream-ordered launch sequence: there is nothing to wait on
        print("--api world: --async-finish / --return-recv-hook do not apply and are recorded as off",
              file=sys.stderr)
        args.async_finish = args.return_recv_hook = False


def dequantize_fp8(x_fp8: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """Payload times its group's scale, per 128 elements, to bf16 (:196-203)."""
    hidden = x_fp8.shape[-1]
    groups = x_fp8.reshape(-1, hidden // 128, 128).float() * scales.reshape(-1, hidden // 128, 1).float()
    return groups.reshape(x_fp8.shape).to(torch.bfloat16)


class EPBenchmark:
    """All ranks of the world: inputs, the dispatch -> expert -> combine cycle, timing and the report."""

    def __init__(self, args: argparse.Namespace, device: str = "cuda"):
        self.args = args
        self.device = torch.device(device)
        self.use_fp8 = args.dtype == "fp8"
        R = self.R = args.num_ranks
        self.L = args.num_experts // R
        self.timeout_us = -1
        route = ROUTING_MODES[args.routing_mode]
        # the reference draws routing and x on the GPU; routing is drawn on the host here so that a seed
        # names the same workload on any machine
        routed = [route(num_tokens=args.num_tokens, num_experts=args.num_experts, top_k=args.top_k,
                        device=torch.device("cpu"), seed=args.seed + r, hot_experts=args.hot_experts,
                        hot_fraction=args.hot_fraction, zipf_alpha=args.zipf_alpha) for r in range(R)]
        self.topk_idx = torch.stack([i for i, _ in routed]).to(self.device)
        self.topk_weights = torch.stack([w for _, w in routed]).to(self.device)
        self.x = torch.randn(R, args.num_tokens, args.hidden_size, dtype=torch.bfloat16, device=self.device)
        self.factor = (torch.arange(args.num_experts, dtype=torch.float32, device=self.device) * 0.1 + 1.0)
        if args.api == "buffer":
            self.world = ep.World(R)
            size = Buffer.get_ep_buffer_size_hint(args.num_tokens, args.hidden_size, R, args.num_experts)
            self.bufs = [Buffer(LogicalGroup(self.world, r), size) for r in range(R)]
            self.active = [torch.ones((R,), dtype=torch.int32, device=self.device) for _ in range(R)]
            self.out = torch.zeros_like(self.x)
        else:
            cfg = EPConfig("ep_benchmark", R, args.num_tokens, args.hidden_size, args.num_experts, args.top_k,
                           self.use_fp8)
            self.harness = WorldHarness(cfg, device=device)
            self.harness.load({"x": self.x, "topk_idx": self.topk_idx, "topk_weights": self.topk_weights})
            self.harness.alloc_dispatch_outputs()
            self.harness.alloc_combine_io()

    # ---- per-rank Buffer calls ------------------------------------------------
    def _finish(self, results: List[Tuple]) -> None:
        for *_, event, hook in results:
            if self.args.return_recv_hook:
                hook()
            elif self.args.async_finish:
                event.current_stream_wait()

    def _buffer_dispatch(self) -> List[Tuple]:
        a = self.args
        results = [self.bufs[r].dispatch(self.x[r], self.topk_idx[r], self.active[r],
                                         num_max_dispatch_tokens_per_rank=a.num_tokens, num_experts=a.num_experts,
                                         timeout_us=self.timeout_us, use_fp8=self.use_fp8,
                                         async_finish=a.async_finish, return_recv_hook=a.return_recv_hook)
                   for r in range(self.R)]
        self._finish(results)
        return results

    def _buffer_expert(self, results: List[Tuple]) -> List[torch.Tensor]:
        outs = []
        for r, (recv_x, _count, _handle, _event, _hook) in enumerate(results):
            rows = dequantize_fp8(recv_x[0], recv_x[1]) if self.use_fp8 else recv_x
            scale = self.factor[r * self.L:(r + 1) * self.L].view(self.L, 1, 1)
            outs.append((rows * scale).to(torch.bfloat16))
        return outs

    def _buffer_combine(self, results: List[Tuple], expert_out: List[torch.Tensor]) -> None:
        a = self.args
        done = []
        for r in range(self.R):
            handle = results[r][2]
            rows = expert_out[r]
            if a.zero_copy:
                staged = self.bufs[r].get_next_combine_buffer(handle)
                staged.copy_(rows)
                rows = staged
            done.append(self.bufs[r].combine(rows.contiguous(), self.topk_idx[r], self.topk_weights[r],
                                             self.active[r], timeout_us=self.timeout_us, handle=handle,
                                             zero_copy=a.zero_copy, async_finish=a.async_finish,
                                             return_recv_hook=a.return_recv_hook, out=self.out[r]))
        self._finish(done)

    # ---- one cycle, optionally timed -------------------------------------------
    def cycle(self, events: Tuple[torch.cuda.Event, ...] | None = None) -> None:
        mark = (lambda i: events[i].record()) if events is not None else (lambda i: None)
        if self.args.api == "buffer":
            mark(0)
            results = self._buffer_dispatch()
            mark(1)
            expert_out = self._buffer_expert(results)
            mark(2)
            self._buffer_combine(results, expert_out)
            mark(3)
        else:
            mark(0)
            self.harness.dispatch()
            mark(1)
            self.harness.cast_back(self.factor)     # the mock expert, valid rows only, by the consumer kernel
            mark(2)
            self.harness.combine()
            mark(3)

    def run(self) -> Dict[str, Any]:
        a = self.args
        for _ in range(a.warmup_iters):
            self.cycle()
        torch.cuda.synchronize(self.device)
        events = [tuple(torch.cuda.Event(enable_timing=True) for _ in range(4)) for _ in range(a.iters)]
        for marks in events:
            self.cycle(marks)
        torch.cuda.synchronize(self.device)
        dispatch_ms = [m[0].elapsed_time(m[1]) for m in events]
        combine_ms = [m[2].elapsed_time(m[3]) for m in events]
        e2e_ms = [m[0].elapsed_time(m[3]) for m in events]
        return self.report(dispatch_ms, combine_ms, e2e_ms)

    def report(self, dispatch_ms: List[float], combine_ms: List[float], e2e_ms: List[float]) -> Dict[str, Any]:
        a = self.args
        per_rank = {}
        for name, series in (("dispatch", dispatch_ms), ("combine", combine_ms), ("e2e", e2e_ms)):
            stats = compute_percentiles(series)
            per_rank[f"{name}_latency_ms"] = {f"rank{r}": dict(stats) for r in range(self.R)}
        k_hot, zipf = a.routing_mode == "k_hot", a.routing_mode == "zipf"
        return assemble_json_output(
            backend=a.backend, world_size=self.R, num_experts=a.num_experts, hidden_size=a.hidden_size,
            top_k=a.top_k, num_tokens=a.num_tokens, dtype=a.dtype, routing_mode=a.routing_mode,
            zero_copy=a.zero_copy, async_finish=a.async_finish, return_recv_hook=a.return_recv_hook,
            warmup_iters=a.warmup_iters, iters=a.iters, hot_experts=a.hot_experts if k_hot else None,
            hot_fraction=a.hot_fraction if k_hot else None, zipf_alpha=a.zipf_alpha if zipf else None,
            dispatch_latencies_ms=dispatch_ms, combine_latencies_ms=combine_ms, e2e_latencies_ms=e2e_ms,
            expert_load=compute_global_expert_load(self.topk_idx.cpu(), a.num_experts), pg_backend=a.pg_backend,
            per_rank_stats=per_rank)


def main(argv: Sequence[str] | None = None) -> Dict[str, Any]:
    args = parse_args(argv)
    validate_args(args)
    result = EPBenchmark(args).run()
    result["api"] = args.api
    if args.json_output:
        write_json_output(result, args.json_output)
        print(f"Results written to {args.json_output}", file=sys.stderr)
    else:
        print(json.dumps(result, indent=2))
    return result


if __name__ == "__main__":
    main()
