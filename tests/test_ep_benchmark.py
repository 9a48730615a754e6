"""The benchmark harness either side of the hot path: routing generators,
percentile / expert-load metrics and the result document, checked against
what their definitions fix (mooncake-ep/benchmarks/ep_benchmark/routing.py,
metrics.py, run_ep_benchmark.py)."""
import json
import math

import numpy as np
import pytest
import torch

from mooncake_amd.benchmarks.ep_benchmark import metrics, routing
from mooncake_amd.benchmarks.ep_benchmark import run_ep_benchmark as runner


def _distinct_in_range(idx, num_experts):
    assert idx.dtype == torch.int64
    assert int(idx.min()) >= 0 and int(idx.max()) < num_experts
    s = idx.sort(dim=-1).values
    assert bool((s[:, 1:] != s[:, :-1]).all())


@pytest.mark.parametrize("mode", ["uniform", "k_hot", "zipf"])
def test_routing_shapes_distinct_deterministic(mode):
    fn = routing.ROUTING_MODES[mode]
    kw = dict(num_tokens=300, num_experts=64, top_k=8, seed=5, hot_experts=16, hot_fraction=0.75, zipf_alpha=1.1)
    idx, w = fn(**kw)
    assert idx.shape == (300, 8) and w.shape == (300, 8) and w.dtype == torch.float32
    _distinct_in_range(idx, 64)
    # softmax of uniform(0,1) draws: positive, rows sum to one, ratio of any two of a row at most e
    assert torch.allclose(w.sum(-1), torch.ones(300), atol=1e-6)
    assert float(w.min()) > 0 and float((w.max(-1).values / w.min(-1).values).max()) <= math.e + 1e-5
    idx2, w2 = fn(**kw)
    assert torch.equal(idx, idx2) and torch.equal(w, w2)
    idx3, _ = fn(**{**kw, "seed": 6})
    assert not torch.equal(idx, idx3)


def test_uniform_routing_is_topk_of_seeded_normal_scores():
    # the definition, restated with the generator's stream made explicit
    gen = torch.Generator().manual_seed(11)
    scores = torch.randn(50, 32, generator=gen)
    draws = torch.rand(50, 4, generator=gen)
    idx, w = routing.uniform_routing(50, 32, 4, seed=11)
    assert torch.equal(idx, scores.topk(4, dim=-1).indices)
    assert torch.equal(w, torch.softmax(draws, dim=-1))
    # all experts about equally loaded
    idx, _ = routing.uniform_routing(20000, 16, 4, seed=1)
    load = torch.bincount(idx.flatten(), minlength=16).double()
    assert float(load.max() / load.mean()) < 1.05


def test_k_hot_fraction_and_errors():
    T, E, K, hot = 1000, 64, 4, 8
    idx, _ = routing.k_hot_routing(T, E, K, seed=3, hot_experts=hot, hot_fraction=0.9)
    all_hot = (idx < hot).all(dim=-1)
    # 900 hot tokens by construction; a cold token lands entirely in the hot set with probability
    # C(8,4)/C(64,4) ~ 1e-4
    assert 900 <= int(all_hot.sum()) <= 901
    # shuffled: hot tokens are not simply the first 900
    assert not bool(all_hot[:900].all())
    with pytest.raises(ValueError, match="hot_experts .* > num_experts"):
        routing.k_hot_routing(10, 8, 2, hot_experts=9)
    with pytest.raises(ValueError, match="cannot pick 4 distinct experts"):
        routing.k_hot_routing(10, 8, 4, hot_experts=3)
    for bad in (0.0, 1.0, -0.5, 1.5):
        with pytest.raises(ValueError, match="hot_fraction"):
            routing.k_hot_routing(10, 8, 2, hot_experts=4, hot_fraction=bad)


def test_zipf_marginals_follow_power_law():
    # top-1 of log p + Gumbel noise samples expert i with probability p_i exactly
    E, alpha, T = 16, 1.2, 200000
    idx, _ = routing.zipfian_routing(T, E, 1, seed=2, zipf_alpha=alpha)
    freq = torch.bincount(idx.flatten(), minlength=E).double() / T
    p = torch.arange(1, E + 1, dtype=torch.float64) ** -alpha
    p = p / p.sum()
    assert float((freq - p).abs().max()) < 4e-3
    # with k > 1 the load still falls with the expert index
    idx, _ = routing.zipfian_routing(20000, 32, 4, seed=2, zipf_alpha=alpha)
    load = torch.bincount(idx.flatten(), minlength=32)
    assert int(load[0]) > int(load[7]) > int(load[31])
    with pytest.raises(ValueError, match="zipf_alpha"):
        routing.zipfian_routing(10, 8, 2, zipf_alpha=0.0)


def test_percentiles_known_answers():
    assert metrics.compute_percentiles([]) == {"p50": 0.0, "p90": 0.0, "p99": 0.0, "p999": 0.0, "mean": 0.0}
    # 0..1000: the q-th percentile with linear interpolation is 10 q
    got = metrics.compute_percentiles(list(range(1001)))
    assert got == pytest.approx({"p50": 500.0, "p90": 900.0, "p99": 990.0, "p999": 999.0, "mean": 500.0})
    # two points: interpolated between them
    got = metrics.compute_percentiles([1.0, 3.0])
    assert got["p50"] == pytest.approx(2.0) and got["p90"] == pytest.approx(2.8) and got["mean"] == 2.0
    assert metrics.compute_percentiles(torch.tensor([4.0]))["p999"] == 4.0


def test_expert_load_counts_world_selections():
    idx = torch.tensor([[[0, 1], [0, 2]], [[0, 3], [-1, -1]]])   # two ranks, two tokens, top-2
    load = metrics.compute_global_expert_load(idx, 8)
    assert load == {"max_tokens_per_expert": 3.0, "min_tokens_per_expert": 0.0,
                    "mean_tokens_per_expert": 6 / 8, "imbalance_ratio": 4.0}


def _document(**over):
    kw = dict(backend="hip", world_size=4, num_experts=16, hidden_size=2048, top_k=4, num_tokens=100, dtype="bf16",
              routing_mode="uniform", zero_copy=False, async_finish=True, return_recv_hook=False, warmup_iters=2,
              iters=3, dispatch_latencies_ms=[1.0, 2.0, 3.0], combine_latencies_ms=[2.0, 2.0, 2.0],
              e2e_latencies_ms=[4.0, 4.0, 4.0], per_rank_stats={"dispatch_latency_ms": {}})
    kw.update(over)
    return metrics.assemble_json_output(**kw)


def test_result_document_schema():
    doc = _document()
    assert list(doc) == ["benchmark", "backend", "world_size", "num_experts", "hidden_size", "top_k", "num_tokens",
                         "dtype", "routing_mode", "zero_copy", "async_finish", "return_recv_hook", "warmup_iters",
                         "iters", "pg_backend", "metrics"]
    assert doc["benchmark"] == "mooncake_ep" and doc["pg_backend"] == "nccl"
    m = doc["metrics"]
    assert list(m) == ["dispatch_latency_ms", "combine_latency_ms", "end_to_end_latency_ms", "tokens_per_second",
                       "expert_load", "per_rank_stats"]
    assert m["dispatch_latency_ms"]["mean"] == 2.0
    # 4 ranks x 100 tokens every 4 ms
    assert m["tokens_per_second"] == pytest.approx(100000.0)
    assert m["expert_load"]["imbalance_ratio"] == 0
    assert "hot_experts" not in doc and "zipf_alpha" not in doc
    doc = _document(routing_mode="k_hot", hot_experts=8, hot_fraction=0.5, zipf_alpha=2.0)
    assert doc["hot_experts"] == 8 and doc["hot_fraction"] == 0.5 and "zipf_alpha" not in doc
    doc = _document(routing_mode="zipf", hot_experts=8, zipf_alpha=2.0)
    assert doc["zipf_alpha"] == 2.0 and "hot_experts" not in doc
    assert _document(e2e_latencies_ms=[])["metrics"]["tokens_per_second"] == 0.0
    json.dumps(doc)


def test_cli_defaults_config_file_and_validation(tmp_path):
    a = runner.parse_args([])
    assert (a.num_ranks, a.num_experts, a.hidden_size, a.top_k, a.num_tokens) == (8, 256, 7168, 8, 1024)
    assert (a.dtype, a.routing_mode, a.warmup_iters, a.iters, a.seed) == ("bf16", "uniform", 20, 100, 0)
    assert (a.hot_experts, a.hot_fraction, a.zipf_alpha) == (32, 0.9, 1.0)
    assert not (a.zero_copy or a.async_finish or a.return_recv_hook)
    cfg = tmp_path / "c.json"
    cfg.write_text(json.dumps({"num_ranks": 4, "routing_mode": "zipf", "zipf_alpha": 1.5, "async_finish": True}))
    a = runner.parse_args(["--config", str(cfg), "--num-ranks", "2"])
    assert a.num_ranks == 2 and a.routing_mode == "zipf" and a.zipf_alpha == 1.5 and a.async_finish
    runner.validate_args(a)
    with pytest.raises(ValueError, match="divisible by num_ranks"):
        runner.validate_args(runner.parse_args(["--num-ranks", "3", "--num-experts", "16"]))
    with pytest.raises(ValueError, match="mutually exclusive"):
        runner.validate_args(runner.parse_args(["--async-finish", "--return-recv-hook"]))
    with pytest.raises(ValueError, match="divisible by 128"):
        runner.validate_args(runner.parse_args(["--dtype", "fp8", "--hidden-size", "192"]))
    with pytest.raises(ValueError, match="--api buffer"):
        runner.validate_args(runner.parse_args(["--api", "world", "--zero-copy"]))
    a = runner.parse_args(["--api", "world", "--async-finish"])
    runner.validate_args(a)
    assert not a.async_finish


def test_shipped_configs_parse():
    import glob
    import os
    here = os.path.dirname(runner.__file__)
    paths = sorted(glob.glob(os.path.join(here, "configs", "*.json")))
    assert len(paths) == 3
    for p in paths:
        a = runner.parse_args(["--config", p])
        runner.validate_args(a)
        assert a.backend == "hip" and a.routing_mode in routing.ROUTING_MODES


def test_dequantize_fp8_is_payload_times_group_scale():
    x = torch.arange(-128, 128, dtype=torch.float32).view(1, 256).to(torch.float8_e4m3fn).view(1, 1, 256)
    s = torch.tensor([0.5, 2.0]).view(1, 1, 2)
    out = runner.dequantize_fp8(x, s)
    assert out.dtype == torch.bfloat16 and out.shape == x.shape
    want = torch.cat([x.float()[..., :128] * 0.5, x.float()[..., 128:] * 2.0], dim=-1).to(torch.bfloat16)
    assert torch.equal(out, want)


def test_routing_generators_reproduce_the_reference_value_for_value():
    """tests/golden/routing_vectors.npz holds what the reference's own generators return for nine
    (mode, shape, seed) cases (written by tests/golden/make_routing_golden.py, the one place a file of the
    reference is run); the generators here must give the same indices and the same weight bits on the CPU."""
    import json
    import os

    import numpy as np
    fixture = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "routing_vectors.npz"))
    cases = sorted(k for k in fixture.files if k.endswith("_args"))
    assert len(cases) == 9
    modes = set()
    for key in cases:
        args = json.loads(str(fixture[key]))
        prefix = key[:-len("_args")]
        idx, weights = routing.ROUTING_MODES[args["mode"]](args["num_tokens"], args["num_experts"], args["top_k"],
                                                           device=torch.device("cpu"), seed=args["seed"],
                                                           **args["extra"])
        assert idx.dtype == torch.int64 and weights.dtype == torch.float32
        assert np.array_equal(idx.numpy().astype(np.int32), fixture[prefix + "_topk_idx"]), args
        assert np.array_equal(weights.numpy().view(np.int32), fixture[prefix + "_topk_weights"]), args
        modes.add(args["mode"])
    assert modes == {"uniform", "k_hot", "zipf"}
