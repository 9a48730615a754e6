"""Whole-world calls recorded into HIP graphs: every replay, on fresh input
values, must give what the oracle gives - also with eager calls of the same
world between the replays, which rewrite the world's shared tables and routing
state.  (Serving loops run dispatch / combine from graphs; the reference's
low-latency kernels are written to be capturable for that reason.)"""
import pytest
import torch

from mooncake_amd import ep
from mooncake_amd.harness import WorldHarness
from mooncake_amd.mooncake_ep_buffer import Buffer, LogicalGroup
from mooncake_amd.workloads import EPConfig, generate
from tests.gpu_util import announce, compare_dispatch

pytestmark = pytest.mark.gpu


def _reference(oracle, cfg, data, factor):
    nt = [cfg.tokens_per_rank] * cfg.num_ranks
    ref = oracle.dispatch(data["x"], data["topk_idx"], nt, cfg.max_tokens, cfg.num_experts, cfg.use_fp8)
    rows = oracle.cast_back(ref["recv_x"], ref["scales"] if cfg.use_fp8 else None, ref["recv_count"], factor)
    out = oracle.combine(rows, data["topk_idx"], data["topk_weights"], ref["src_info"], ref["layout_range"], nt,
                         cfg.max_tokens, cfg.num_experts)
    return ref, out


def _load_in_place(h, data):
    h.x.copy_(data["x"])
    h.topk_idx.copy_(data["topk_idx"])
    h.topk_weights.copy_(data["topk_weights"])


def _harness(cfg, world, seed):
    h = WorldHarness(cfg, world=world)
    h.load(generate(cfg, seed=seed))
    h.alloc_dispatch_outputs(poison=False)
    h.alloc_combine_io()
    return h


@pytest.mark.parametrize("use_fp8", [True, False])
@pytest.mark.parametrize("one_graph", [True, False])
def test_replays_match_the_oracle(gpu_device, oracle, use_fp8, one_graph):
    cfg = EPConfig("graph", 4, 48, 1024, 16, 4, use_fp8, masked_fraction=0.2)
    announce(f"graph capture {cfg} one_graph={one_graph}")
    world = ep.World(cfg.num_ranks)
    h = _harness(cfg, world, seed=100)
    other = _harness(cfg, world, seed=200)          # eager traffic on the same world
    factor = (torch.arange(cfg.num_experts, dtype=torch.float32) * 0.1 + 1.0).to(gpu_device)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                   # sizes the world's scratch; nothing may grow while recording
        h.dispatch()
        h.cast_back(factor)
        h.combine()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graphs = []
    if one_graph:                                   # combine reuses the routing state of the dispatch beside it
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            h.dispatch()
            h.cast_back(factor)
            h.combine()
        graphs = [g]
    else:                                           # a combine recorded on its own resolves its handle
        for part in (lambda: (h.dispatch(), h.cast_back(factor)), h.combine):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                part()
            graphs.append(g)

    for seed in (1, 2, 3):
        data = generate(cfg, seed=seed)
        _load_in_place(h, data)
        h.combined.zero_()
        other.dispatch()                            # overwrites the shared tables and the routing state
        other.cast_back(None)
        other.combine()
        torch.cuda.synchronize()
        for g in graphs:
            g.replay()
        torch.cuda.synchronize()
        ref, want = _reference(oracle, cfg, data, factor.cpu())
        compare_dispatch(h, ref, check_poison=False)
        assert torch.equal(h.combined.cpu().view(torch.int16), want.view(torch.int16)), f"replay with seed {seed}"

    # eager calls of the world are still right after its graphs ran
    data = generate(cfg, seed=200)
    ref, want = _reference(oracle, cfg, data, None)
    other.dispatch()
    other.cast_back(None)
    other.combine()
    torch.cuda.synchronize()
    compare_dispatch(other, ref, check_poison=False)
    assert torch.equal(other.combined.cpu().view(torch.int16), want.view(torch.int16))


def test_recording_refuses_to_grow_scratch_and_per_rank_calls(gpu_device):
    cfg = EPConfig("graph_refusals", 2, 16, 256, 4, 2, False)
    announce(f"graph refusals {cfg}")
    world = ep.World(cfg.num_ranks)
    h = _harness(cfg, world, seed=1)                # never called eagerly: its scratch does not exist yet
    buf = Buffer(LogicalGroup(world, 0), Buffer.get_ep_buffer_size_hint(16, 256, 2, 4))
    marker = torch.zeros(8, device=gpu_device)
    g = torch.cuda.CUDAGraph()
    errors = []
    with torch.cuda.graph(g):
        marker.add_(1.0)                            # so that the graph is not empty
        try:
            h.dispatch()
        except RuntimeError as e:
            errors.append(str(e))
        try:
            buf.dispatch(h.x[0], h.topk_idx[0], None, cfg.max_tokens, cfg.num_experts, -1, use_fp8=False)
        except NotImplementedError as e:
            errors.append(str(e))
    assert len(errors) == 2
    assert "outside the capture first" in errors[0]
    assert "cannot be recorded into a graph" in errors[1]
    g.replay()
    torch.cuda.synchronize()
    assert float(marker[0]) == 1.0
    # the refused calls left the world usable
    h.dispatch()
    torch.cuda.synchronize()
    assert int(h.recv_count.sum()) == int((h.topk_idx >= 0).sum())
