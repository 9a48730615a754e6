"""The benchmark harness on the GPU: the native dispatch + combine loop of the
C ABI (the reference's _benchmark_legacy_buffer) and the ep_benchmark cycle,
checked for what they leave in the output tensors as well as for the shape of
what they report."""
import argparse

import pytest
import torch

from mooncake_amd.benchmarks import legacy_buffer_perf
from mooncake_amd.benchmarks.ep_benchmark import run_ep_benchmark as runner
from mooncake_amd.harness import WorldHarness
from mooncake_amd.workloads import EPConfig, generate
from tests.gpu_util import announce, compare_dispatch

pytestmark = pytest.mark.gpu


def _loop_tensors(h: WorldHarness):
    R = h.cfg.num_ranks
    p = lambda t: [t[r].data_ptr() for r in range(R)]
    return {"x": p(h.x), "topk_idx": p(h.topk_idx), "topk_weights": p(h.topk_weights),
            "active_ranks": p(h.active_ranks), "expert_x": p(h.expert_out), "packed_recv_x": p(h.recv_x),
            "packed_recv_count": p(h.recv_count), "packed_recv_src_info": p(h.src_info),
            "packed_recv_layout_range": p(h.layout_range), "combined_x": p(h.combined)}


def _loop_harness():
    cfg = EPConfig("native_loop", 4, 48, 1024, 16, 4, False)
    data = generate(cfg, seed=21)
    h = WorldHarness(cfg)
    h.load(data)
    h.alloc_dispatch_outputs(poison=True)
    h.alloc_combine_io()
    gen = torch.Generator().manual_seed(5)
    h.expert_out.copy_(torch.randn(h.expert_out.shape, generator=gen).to(torch.bfloat16))
    return cfg, data, h


def test_native_loop_leaves_oracle_results(gpu_device, oracle):
    cfg, data, h = _loop_harness()
    announce(f"native loop {cfg}")
    kw = dict(num_tokens=cfg.tokens_per_rank, hidden=cfg.hidden, num_topk=cfg.num_topk,
              num_local_experts=cfg.num_local_experts, num_max_dispatch_tokens_per_rank=cfg.max_tokens,
              num_experts=cfg.num_experts, compute_stream_ptr=int(torch.cuda.current_stream().cuda_stream))
    avg, lo, hi = h.world.legacy_buffer_perf(_loop_tensors(h), warmups=2, iterations=5, **kw)
    torch.cuda.synchronize()
    assert 0 < lo <= avg <= hi < 1e6
    nt = [cfg.tokens_per_rank] * cfg.num_ranks
    ref = oracle.dispatch(data["x"], data["topk_idx"], nt, cfg.max_tokens, cfg.num_experts, False)
    compare_dispatch(h, ref, check_poison=True)
    want = oracle.combine(h.expert_out.cpu(), data["topk_idx"], data["topk_weights"], ref["src_info"],
                          ref["layout_range"], nt, cfg.max_tokens, cfg.num_experts)
    assert torch.equal(h.combined.cpu().view(torch.int16), want.view(torch.int16))


def test_native_loop_rejects_what_the_reference_rejects(gpu_device):
    cfg, _, h = _loop_harness()
    announce("native loop validation")
    good = dict(num_tokens=cfg.tokens_per_rank, hidden=cfg.hidden, num_topk=cfg.num_topk,
                num_local_experts=cfg.num_local_experts, num_max_dispatch_tokens_per_rank=cfg.max_tokens,
                num_experts=cfg.num_experts, warmups=1, iterations=2)
    for bad in (dict(iterations=1), dict(num_tokens=0), dict(warmups=-1), dict(num_topk=0),
                dict(num_max_dispatch_tokens_per_rank=cfg.tokens_per_rank - 1), dict(num_local_experts=0)):
        # std::invalid_argument in the reference (legacy_buffer_perf.cpp:58-82): ValueError through pybind11
        with pytest.raises(ValueError, match="invalid legacy EP benchmark configuration"):
            h.world.legacy_buffer_perf(_loop_tensors(h), **{**good, **bad})
    t = _loop_tensors(h)
    t["expert_x"] = list(t["expert_x"])
    t["expert_x"][2] = 0
    with pytest.raises(ValueError, match="null tensor pointer"):
        h.world.legacy_buffer_perf(t, **good)
    t = _loop_tensors(h)
    del t["combined_x"]
    with pytest.raises(ValueError, match="null tensor pointer"):
        h.world.legacy_buffer_perf(t, **good)


def test_legacy_buffer_perf_script(gpu_device):
    announce("legacy_buffer_perf script")
    args = legacy_buffer_perf.parse_args(["--ranks", "4", "--tokens", "32", "--hidden", "1024", "--experts", "16",
                                          "--topk", "4", "--warmups", "2", "--iterations", "4"])
    out = legacy_buffer_perf.run(args)
    assert out["ranks"] == 4 and 0 < out["min_us"] <= out["average_us"] <= out["max_us"]
    # 4 ranks x 32 tokens x 4 selections, a bf16 row each way
    assert out["bandwidth_gbs"] == pytest.approx(4 * 32 * 4 * 1024 * 4 / out["average_us"] / 1e3)
    with pytest.raises(ValueError, match="divisible by world size"):
        legacy_buffer_perf.run(legacy_buffer_perf.parse_args(["--ranks", "5", "--experts", "16"]))
    with pytest.raises(ValueError, match="divisible by 128"):
        legacy_buffer_perf.run(legacy_buffer_perf.parse_args(["--ranks", "4", "--experts", "16", "--hidden", "192"]))


def _bench_args(*extra):
    return runner.parse_args(["--num-ranks", "4", "--num-experts", "16", "--hidden-size", "1024", "--top-k", "4",
                              "--num-tokens", "40", "--warmup-iters", "2", "--iters", "6", "--seed", "9", *extra])


@pytest.mark.parametrize("extra", [(), ("--async-finish",), ("--return-recv-hook",), ("--dtype", "fp8"),
                                   ("--routing-mode", "k_hot", "--hot-experts", "8", "--hot-fraction", "0.5",
                                    "--async-finish"),
                                   ("--routing-mode", "zipf", "--zipf-alpha", "1.3", "--dtype", "fp8",
                                    "--return-recv-hook"),
                                   ("--api", "world"), ("--api", "world", "--dtype", "fp8", "--routing-mode", "zipf")])
def test_ep_benchmark_cycle(gpu_device, extra):
    announce(f"ep_benchmark {extra}")
    args = _bench_args(*extra)
    runner.validate_args(args)
    bench = runner.EPBenchmark(args)
    doc = bench.run()
    assert doc["world_size"] == 4 and doc["routing_mode"] == args.routing_mode and doc["dtype"] == args.dtype
    m = doc["metrics"]
    for key in ("dispatch_latency_ms", "combine_latency_ms", "end_to_end_latency_ms"):
        assert 0 < m[key]["p50"] <= m[key]["p90"] <= m[key]["p99"] <= m[key]["p999"]
    assert m["end_to_end_latency_ms"]["mean"] >= m["dispatch_latency_ms"]["mean"] + m["combine_latency_ms"]["mean"]
    assert m["tokens_per_second"] == pytest.approx(4 * 40 / (m["end_to_end_latency_ms"]["mean"] / 1e3))
    assert m["expert_load"]["mean_tokens_per_expert"] == 4 * 40 * 4 / 16
    assert sorted(m["per_rank_stats"]["e2e_latency_ms"]) == ["rank0", "rank1", "rank2", "rank3"]
    # the last cycle's result is the closed form of the reference's grid test
    # (mooncake-ep/tests/test_ep_grid.py:100-108): x * sum_k factor(e_k) * w_k
    out = bench.out if args.api == "buffer" else bench.harness.combined
    factor = bench.factor[bench.topk_idx]                                   # [R, T, K]
    want = bench.x.float() * (factor * bench.topk_weights).sum(-1, keepdim=True)
    rtol, atol = (0.15, 5e-3) if args.dtype == "fp8" else (5e-2, 1e-3)
    torch.testing.assert_close(out.float(), want, rtol=rtol, atol=atol)


def test_ep_benchmark_zero_copy_is_refused_like_the_reference_build_without_it(gpu_device):
    announce("ep_benchmark zero copy")
    bench = runner.EPBenchmark(_bench_args("--zero-copy"))
    with pytest.raises(NotImplementedError):
        bench.cycle()


def test_native_driver_runs_without_python_in_the_loop(gpu_device):
    """The C++ driver built from the C header alone: the per-rank Buffer calls in the three completion modes, from
    one thread and from a thread per rank (combined rows against the same multiply-add chain on the host, bit for
    bit), the whole-world self-check
    (per-expert row counts against a host count) and both timing loops."""
    import os
    import subprocess
    from mooncake_amd import _lib
    exe = os.path.join(os.path.dirname(_lib.LIB_PATH), "ep_native_bench")
    assert os.path.exists(exe), "build it first (make -C mooncake_amd/csrc)"
    announce("native driver")
    for flags in (["--ranks", "4", "--tokens", "32", "--hidden", "1024", "--experts", "16", "--topk", "4",
                   "--warmups", "2", "--iterations", "4", "--per-rank"],
                  ["--ranks", "2", "--tokens", "17", "--hidden", "256", "--experts", "6", "--topk", "3", "--bf16",
                   "--warmups", "1", "--iterations", "3", "--per-rank"]):
        run = subprocess.run([exe] + flags, capture_output=True, text=True, timeout=100)
        assert run.returncode == 0, run.stderr
        assert "us per step" in run.stdout and "native loop" in run.stdout
        assert "a thread per rank: combined rows equal the host chain" in run.stdout
    bad = subprocess.run([exe, "--ranks", "3", "--experts", "16"], capture_output=True, text=True, timeout=100)
    assert bad.returncode == 2 and "unusable shape" in bad.stderr
