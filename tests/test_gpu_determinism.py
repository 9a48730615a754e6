"""Run-to-run determinism (the reference's tests hash the outputs of repeated
runs, mooncake-wheel/tests/test_mooncake_ep.py:175-181; there the row order
inside an expert's block may differ between runs, here it is fixed), and two
worlds working at the same time on different streams."""
import pytest
import torch

from mooncake_amd.harness import WorldHarness
from mooncake_amd.workloads import EPConfig, generate
from tests.gpu_util import announce, compare_dispatch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("use_fp8", [True, False])
def test_repeated_runs_are_bit_identical(gpu_device, use_fp8):
    cfg = EPConfig("repeat", 8, 96, 2048, 64, 8, use_fp8, routing="zipf", masked_fraction=0.1)
    announce(f"determinism {cfg}")
    data = generate(cfg, seed=11)
    factor = torch.arange(cfg.num_experts, dtype=torch.float32) * 0.1 + 1.0
    snapshots = []
    for _ in range(5):
        h = WorldHarness(cfg)
        h.load(data)
        h.alloc_dispatch_outputs(poison=True)
        h.alloc_combine_io()
        h.expert_out.view(torch.int16).fill_(0x1111)
        h.combined.fill_(3.0)
        h.dispatch()
        h.cast_back(factor)
        h.combine()
        torch.cuda.synchronize()
        tensors = [h.recv_x, h.recv_count, h.src_info, h.layout_range, h.expert_out.view(torch.int16),
                   h.combined.view(torch.int16)]
        if use_fp8:
            tensors.append(h.recv_scales_phys.view(torch.int32))
        snapshots.append([t.clone() for t in tensors])
    for other in snapshots[1:]:
        for a, b in zip(snapshots[0], other):
            assert torch.equal(a, b)          # whole tensors: the padding is as untouched as the first time


def test_two_worlds_on_two_streams(gpu_device, oracle):
    cfgs = [EPConfig("world_a", 4, 64, 2048, 32, 4, True), EPConfig("world_b", 8, 48, 1024, 16, 2, False)]
    announce(f"two worlds {cfgs}")
    datas = [generate(c, seed=20 + i) for i, c in enumerate(cfgs)]
    hs, streams = [], [torch.cuda.Stream(), torch.cuda.Stream()]
    for c, d in zip(cfgs, datas):
        h = WorldHarness(c)
        h.load(d)
        h.alloc_dispatch_outputs(poison=True)
        h.alloc_combine_io()
        hs.append(h)
    torch.cuda.synchronize()
    for _ in range(4):                         # interleaved launches, no synchronisation in between
        for h, s in zip(hs, streams):
            h.dispatch(stream=s)
            h.cast_back(None, stream=s)
            h.combine(stream=s)
    torch.cuda.synchronize()
    for c, d, h in zip(cfgs, datas, hs):
        nt = [c.tokens_per_rank] * c.num_ranks
        ref = oracle.dispatch(d["x"], d["topk_idx"], nt, c.max_tokens, c.num_experts, c.use_fp8)
        compare_dispatch(h, ref, check_poison=True)
        rows = oracle.cast_back(ref["recv_x"], ref["scales"] if c.use_fp8 else None, ref["recv_count"], None)
        want = oracle.combine(rows, d["topk_idx"], d["topk_weights"], ref["src_info"], ref["layout_range"], nt,
                              c.max_tokens, c.num_experts)
        assert torch.equal(h.combined.cpu().view(torch.int16), want.view(torch.int16))
