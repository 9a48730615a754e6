"""Combine reads `topk_idx` as it is at combine time, like the reference's kernel
(mooncake-ep/src/mooncake_ep_kernel.cu:719-732: `reg_topk_idx[i] >= 0` decides per call whether
expert i contributes): a caller that masks selections to -1 in place between a dispatch and the
combine of its handle drops those experts' rows.  Checked for both ways combine finds its rows (the
last dispatch's routing state, and the handle), for the packed combine, whole-world and through
the per-rank `Buffer`, bit for bit against the oracle's combine on the masked indices."""
import pytest
import torch

from mooncake_amd import Buffer, LogicalGroup
from mooncake_amd.workloads import EPConfig, generate
from tests.gpu_util import announce, run_dispatch

pytestmark = pytest.mark.gpu

CASES = [
    EPConfig("mask_bf16", 4, 48, 2048, 32, 8, False),
    EPConfig("mask_fp8", 8, 32, 2560, 64, 6, True),
    EPConfig("mask_k2", 8, 64, 1024, 8, 2, False),          # two 16-byte chunks per lane in the reduce kernel
]


def mask_some(idx: torch.Tensor, fraction: float, seed: int) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    return torch.rand(idx.shape, generator=g) < fraction


@pytest.mark.parametrize("cfg", CASES, ids=[c.name for c in CASES])
@pytest.mark.parametrize("direct", [1, 0], ids=["direct", "handle"])
def test_world_combine_after_masking_in_place(gpu_device, oracle, cfg, direct):
    announce(f"mask 20 % of topk_idx between dispatch and combine {cfg} direct={direct}")
    data = generate(cfg, seed=31)
    h = run_dispatch(cfg, data, poison=False, options={"combine_direct": direct})
    nt = h.num_tokens
    ref = oracle.dispatch(data["x"], data["topk_idx"], nt, cfg.max_tokens, cfg.num_experts, cfg.use_fp8)
    factor = torch.arange(cfg.num_experts).float() * 0.1 + 1.0
    h.alloc_combine_io()
    h.cast_back(factor)
    torch.cuda.synchronize()
    # the same device tensor, changed in place: the host still sees "the last dispatch's" pointers
    mask = mask_some(data["topk_idx"], 0.2, 5)
    masked = data["topk_idx"].clone()
    masked[mask] = -1
    h.topk_idx[mask.to(h.topk_idx.device)] = -1
    assert int(mask.sum()) > 0
    rows = oracle.cast_back(ref["recv_x"], ref["scales"] if cfg.use_fp8 else None, ref["recv_count"], factor)
    want = oracle.combine(rows, masked, data["topk_weights"], ref["src_info"], ref["layout_range"], nt,
                          cfg.max_tokens, cfg.num_experts)
    unmasked = oracle.combine(rows, data["topk_idx"], data["topk_weights"], ref["src_info"], ref["layout_range"],
                              nt, cfg.max_tokens, cfg.num_experts)
    assert not torch.equal(want.view(torch.int16), unmasked.view(torch.int16))   # the mask matters
    h.combined.fill_(7.0)
    h.combine()
    torch.cuda.synchronize()
    assert torch.equal(h.combined.cpu().view(torch.int16), want.view(torch.int16)), "combine"
    h.combined.fill_(7.0)
    h.combine_packed(factor)
    torch.cuda.synchronize()
    assert torch.equal(h.combined.cpu().view(torch.int16), want.view(torch.int16)), "packed combine"


@pytest.mark.parametrize("direct", [1, 0], ids=["direct", "handle"])
def test_a_selection_pointed_at_another_expert_has_no_row(gpu_device, oracle, direct):
    """Out of contract in the reference (it would read a slot nobody wrote); here such a selection contributes
    nothing on either path - the handle holds no row of that token for the new expert."""
    cfg = EPConfig("repoint", 4, 32, 1024, 32, 4, False)
    announce(f"re-pointed selections direct={direct}")
    data = generate(cfg, seed=32)
    h = run_dispatch(cfg, data, poison=False, options={"combine_direct": direct})
    nt = h.num_tokens
    ref = oracle.dispatch(data["x"], data["topk_idx"], nt, cfg.max_tokens, cfg.num_experts, False)
    h.alloc_combine_io()
    h.cast_back(None)
    idx = data["topk_idx"].clone()
    # k = 0 of every third token moves to an expert the token did not select
    for r in range(cfg.num_ranks):
        for t in range(0, cfg.tokens_per_rank, 3):
            free = [e for e in range(cfg.num_experts) if e not in idx[r, t].tolist()]
            idx[r, t, 0] = free[(r + t) % len(free)]
    h.topk_idx.copy_(idx)
    h.combine()
    torch.cuda.synchronize()
    want = oracle.combine(ref["recv_x"], idx, data["topk_weights"], ref["src_info"], ref["layout_range"], nt,
                          cfg.max_tokens, cfg.num_experts)
    assert torch.equal(h.combined.cpu().view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("direct", [1, 0], ids=["direct", "handle"])
@pytest.mark.parametrize("use_fp8", [False, True], ids=["bf16", "fp8"])
def test_buffer_combine_after_masking_in_place(gpu_device, oracle, direct, use_fp8):
    R, T, H, E, K = 4, 40, 2048, 32, 6
    announce(f"per-rank Buffer: mask topk_idx in place before combine direct={direct} fp8={use_fp8}")
    world, groups = LogicalGroup.make_world(R)
    world.set_option("combine_direct", direct)
    nbytes = Buffer.get_ep_buffer_size_hint(T, H, R, E)
    bufs = [Buffer(g, nbytes) for g in groups]
    cfg = EPConfig("buffer_mask", R, T, H, E, K, use_fp8)
    data = generate(cfg, seed=33)
    dev = [(data["x"][r].to(gpu_device), data["topk_idx"][r].to(gpu_device), data["topk_weights"][r].to(gpu_device))
           for r in range(R)]
    outs = [bufs[r].dispatch(dev[r][0], dev[r][1], None, T, E, -1, use_fp8=use_fp8) for r in range(R)]
    torch.cuda.synchronize()
    nt = [T] * R
    ref = oracle.dispatch(data["x"], data["topk_idx"], nt, T, E, use_fp8)
    rows = oracle.cast_back(ref["recv_x"], ref["scales"] if use_fp8 else None, ref["recv_count"], None)
    mask = mask_some(data["topk_idx"], 0.2, 6)
    masked = data["topk_idx"].clone()
    masked[mask] = -1
    L = E // R
    res = []
    for r in range(R):
        dev[r][1][mask[r].to(gpu_device)] = -1                      # in place, same tensor as at dispatch
        eo = rows[r].to(gpu_device)                                  # [L, R*T, H] bf16: the consumer's rows
        assert eo.shape == (L, R * T, H)
        res.append(bufs[r].combine(eo, dev[r][1], dev[r][2], None, -1, outs[r][2]))
    torch.cuda.synchronize()
    want = oracle.combine(rows, masked, data["topk_weights"], ref["src_info"], ref["layout_range"], nt, T, E)
    for r in range(R):
        assert torch.equal(res[r][0].cpu().view(torch.int16), want[r].view(torch.int16)), f"rank {r}"
