"""The packed combine (`mc_ep_world_combine_packed`: dispatch's payload -> the
weighted sum, with the consumer's cast and the per-expert factor applied in
registers) against the oracle's two-step statement,
oracle.combine(oracle.cast_back(...)), bit for bit, and against the library's
own two-kernel path.  fp8 and bf16 payloads, with and without a factor, rows
from the last dispatch's routing state and from the handle, masked tokens,
ragged ranks, inactive ranks, and the DeepSeek-V3 decode world at full size."""
import pytest
import torch

from mooncake_amd.harness import WorldHarness
from mooncake_amd.workloads import CONFIGS, EPConfig, generate
from tests.gpu_util import announce, run_dispatch

pytestmark = pytest.mark.gpu

CASES = [
    EPConfig("tiny_fp8", 2, 4, 128, 4, 2, True),
    EPConfig("odd_hidden_fp8", 4, 24, 2560, 16, 3, True),
    EPConfig("odd_hidden_bf16", 4, 24, 2560, 16, 3, False),
    EPConfig("h3072_fp8", 4, 20, 3072, 16, 4, True),
    EPConfig("h5120_fp8", 4, 20, 5120, 32, 6, True),
    EPConfig("k11", 4, 40, 2048, 32, 11, True),
    EPConfig("k16_bf16", 2, 20, 1024, 32, 16, False),
    EPConfig("one_rank", 1, 36, 1024, 6, 2, True),
    # bf16 payloads with few rows per token: two 512-element chunks per lane, the second one partly or wholly
    # beyond the hidden size in the last slab
    EPConfig("k2_bf16", 8, 40, 4096, 8, 2, False, masked_fraction=0.1),
    EPConfig("k4_h1536_bf16", 4, 20, 1536, 16, 4, False),
    EPConfig("k1_h640_bf16", 2, 12, 640, 4, 1, False),
    EPConfig("masked_fp8", 8, 64, 1024, 8, 2, True, masked_fraction=0.3),
    EPConfig("zipf_outliers", 8, 32, 2048, 64, 8, True, routing="zipf", outlier_fraction=0.05),
    # slab counts on either side of the 8 XCDs the kernel's block order deals slabs to: 8, 9, 10 and 16 slabs of
    # 1024 elements (the cases above have 1, 2, 3 and 5; the full-size test below has 7)
    EPConfig("h8192_fp8", 4, 12, 8192, 16, 4, True),
    EPConfig("h9216_fp8", 2, 14, 9216, 8, 3, True),
    EPConfig("h10240_fp8", 4, 9, 10240, 8, 2, True),
    EPConfig("h16384_fp8", 2, 10, 16384, 8, 4, True),
]


def ragged(cfg, on):
    if not on:
        return None
    return [max(0, cfg.tokens_per_rank - (r * 5) % (cfg.tokens_per_rank + 1)) for r in range(cfg.num_ranks)]


def oracle_two_step(oracle, cfg, data, nt, factor, active=None):
    ref = oracle.dispatch(data["x"], data["topk_idx"], nt, cfg.max_tokens, cfg.num_experts, cfg.use_fp8)
    rows = oracle.cast_back(ref["recv_x"], ref["scales"] if cfg.use_fp8 else None, ref["recv_count"], factor)
    return oracle.combine(rows, data["topk_idx"], data["topk_weights"], ref["src_info"], ref["layout_range"], nt,
                          cfg.max_tokens, cfg.num_experts, active=active)


@pytest.mark.parametrize("cfg", CASES, ids=[c.name for c in CASES])
@pytest.mark.parametrize("is_ragged", [False, True], ids=["full", "ragged"])
@pytest.mark.parametrize("with_factor", [True, False], ids=["factor", "nofactor"])
@pytest.mark.parametrize("direct,packed_map", [(1, 1), (0, 1), (1, 0)], ids=["direct", "handle", "direct_rank_groups"])
def test_packed_combine_matches_oracle(gpu_device, oracle, cfg, is_ragged, with_factor, direct, packed_map):
    """packed_map: how the kernel's blocks are dealt to the XCDs (slabs owned by XCDs, or (rank, slab) groups)."""
    nt = ragged(cfg, is_ragged)
    announce(f"packed combine {cfg} ragged={nt} factor={with_factor} direct={direct} packed_map={packed_map}")
    data = generate(cfg, seed=21)
    h = run_dispatch(cfg, data, num_tokens=nt, poison=True,
                     options={"combine_direct": direct, "packed_map": packed_map})
    factor = (torch.arange(cfg.num_experts).float() * 0.1 + 1.0) if with_factor else None
    h.alloc_combine_io()
    h.combined.fill_(7.0)
    h.combine_packed(factor)
    torch.cuda.synchronize()
    got = h.combined.cpu()
    want = oracle_two_step(oracle, cfg, data, h.num_tokens, factor)
    for r, n in enumerate(h.num_tokens):
        assert torch.equal(got[r, :n].view(torch.int16), want[r, :n].view(torch.int16)), f"rank {r}"
        assert bool((got[r, n:] == 7.0).all()), "rows beyond num_tokens written"
    # the library's two-kernel path gives the same bits
    h.cast_back(factor)
    h.combined.fill_(7.0)
    h.combine()
    torch.cuda.synchronize()
    assert torch.equal(h.combined.cpu().view(torch.int16), got.view(torch.int16))


@pytest.mark.parametrize("chunks", [1, 2])
@pytest.mark.parametrize("direct", [1, 0], ids=["direct", "handle"])
def test_packed_combine_bf16_chunks_per_lane(gpu_device, oracle, chunks, direct):
    """One or two 16-byte chunks per lane (option combine_chunks; by default two up to top-4) are the same function."""
    cfg = EPConfig("chunks_bf16", 4, 28, 2560, 16, 3, False, masked_fraction=0.2)
    announce(f"packed combine of a bf16 payload, combine_chunks={chunks} direct={direct}")
    data = generate(cfg, seed=25)
    h = run_dispatch(cfg, data, poison=True, options={"combine_chunks": chunks, "combine_direct": direct})
    factor = torch.arange(cfg.num_experts).float() * 0.1 + 1.0
    h.alloc_combine_io()
    h.combine_packed(factor)
    torch.cuda.synchronize()
    want = oracle_two_step(oracle, cfg, data, h.num_tokens, factor)
    assert torch.equal(h.combined.cpu().view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("direct", [1, 0], ids=["direct", "handle"])
def test_packed_combine_skips_inactive_ranks(gpu_device, oracle, direct):
    cfg = EPConfig("inactive_packed", 4, 16, 1024, 16, 4, True)
    announce(f"packed combine with inactive ranks direct={direct}")
    data = generate(cfg, seed=22)
    h = run_dispatch(cfg, data, poison=True, options={"combine_direct": direct})
    factor = torch.arange(16).float() * 0.1 + 1.0
    h.alloc_combine_io()
    h.active_ranks[:, 2] = 0
    h.active_ranks[3, 1] = 0
    h.combine_packed(factor)
    torch.cuda.synchronize()
    want = oracle_two_step(oracle, cfg, data, h.num_tokens, factor, active=h.active_ranks.cpu())
    assert torch.equal(h.combined.cpu().view(torch.int16), want.view(torch.int16))


def test_packed_combine_of_an_older_handle(gpu_device, oracle):
    cfg = EPConfig("older_packed", 4, 24, 1024, 16, 4, True)
    announce("packed combine with the handle of an older dispatch")
    a = run_dispatch(cfg, generate(cfg, seed=23), poison=True)
    b = WorldHarness(cfg, world=a.world)
    b.load(generate(cfg, seed=24))
    b.alloc_dispatch_outputs(poison=True)
    b.dispatch()
    for h, seed in ((a, 23), (b, 24)):
        h.alloc_combine_io()
        h.combine_packed(None)
        torch.cuda.synchronize()
        want = oracle_two_step(oracle, cfg, generate(cfg, seed=seed), h.num_tokens, None)
        assert torch.equal(h.combined.cpu().view(torch.int16), want.view(torch.int16))


def test_packed_combine_dsv3_decode_full_size(gpu_device, oracle):
    cfg = CONFIGS["dsv3_decode"]
    announce(f"packed combine, full size {cfg}")
    data = generate(cfg, seed=0)
    h = run_dispatch(cfg, data, poison=False)
    factor = torch.arange(cfg.num_experts).float() * 0.1 + 1.0
    h.alloc_combine_io()
    h.combine_packed(factor)
    torch.cuda.synchronize()
    got = h.combined.cpu()
    # two-kernel path on the GPU (itself checked against the oracle at this size elsewhere) ...
    h.cast_back(factor)
    h.combine()
    torch.cuda.synchronize()
    assert torch.equal(h.combined.cpu().view(torch.int16), got.view(torch.int16))
    # ... and the oracle, on a slice of ranks' tokens (its cast_back of the whole 15 GB layout is the slow part)
    nt = [cfg.tokens_per_rank] * cfg.num_ranks
    want = oracle_two_step(oracle, cfg, data, nt, factor)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    w = data["topk_weights"] * (data["topk_idx"].float() * 0.1 + 1.0)
    expect = data["x"].float() * w.sum(dim=2, keepdim=True)
    torch.testing.assert_close(got.float(), expect, rtol=0.15, atol=5e-3 * float(data["x"].float().abs().max()))
