"""The five named workloads at their full size on the GPU, and two worlds with a payload too large for the
memory-side cache.

Each is compared with the oracle on its valid rows (the oracle finishes a
whole world in about a second) and through size-independent properties:
every selection lands exactly once, per-expert counts are the histogram of
topk_idx, ranges tile [0, count), src_info is ascending inside a range, a
dispatch -> identity expert -> combine round trip returns x * (sum of unmasked
weights), and rows beyond recv_count are never written (sampled)."""
import pytest
import torch

from mooncake_amd.harness import WorldHarness, valid_rows
from mooncake_amd.workloads import CONFIG_ORDER, CONFIGS, EPConfig, generate
from tests import ref_checks as rc
from tests.gpu_util import announce, compare_dispatch

pytestmark = pytest.mark.gpu


# two worlds whose payload (470 and 484 MB) is well past the 256 MB memory-side cache, one per payload type
BEYOND_CACHE = {"beyond_cache_bf16": EPConfig("beyond_cache_bf16", 16, 256, 7168, 128, 8, False),
                "beyond_cache_fp8": EPConfig("beyond_cache_fp8", 16, 512, 7168, 128, 8, True)}


@pytest.mark.parametrize("name,summed", [(n, 1) for n in CONFIG_ORDER] + [("dsv3_decode", 0), ("mixtral", 0)] +
                         [(n, 1) for n in BEYOND_CACHE])
def test_named_config_full_size(gpu_device, oracle, name, summed):
    cfg = CONFIGS[name] if name in CONFIGS else BEYOND_CACHE[name]
    announce(f"full size {cfg} routing_sum={summed}")
    data = generate(cfg, seed=0)
    R, T, E, K, L = cfg.num_ranks, cfg.tokens_per_rank, cfg.num_experts, cfg.num_topk, cfg.num_local_experts
    RM = R * cfg.max_tokens
    h = WorldHarness(cfg)
    h.world.set_option("routing_sum", summed)
    h.load(data)
    h.alloc_dispatch_outputs(poison=False)
    # sentinel in the row right after each block's expected end, to see that padding is not touched
    idx = data["topk_idx"]
    hist = torch.bincount(idx[idx >= 0].flatten(), minlength=E).view(R, L)
    probe = hist.clamp(max=RM - 1).to(gpu_device)
    rr = torch.arange(R, device=gpu_device).view(R, 1).expand(R, L)
    ll = torch.arange(L, device=gpu_device).view(1, L).expand(R, L)
    h.recv_x[rr, ll, probe] = 0x5C if cfg.use_fp8 else 0x5C5C
    h.src_info[rr, ll, probe] = -12345
    h.dispatch()
    torch.cuda.synchronize()

    # properties
    cnt = h.recv_count.cpu()
    assert torch.equal(cnt.to(torch.int64), hist)
    lr = h.layout_range.cpu()
    counts, begins = lr & 0xFFFFFFFF, lr >> 32
    assert torch.equal(counts.sum(dim=2), cnt.to(torch.int64))
    running = torch.zeros(R, L, dtype=torch.int64)
    for r in range(R):
        nz = counts[:, :, r] > 0
        assert torch.equal(begins[:, :, r][nz], running[nz])
        running += counts[:, :, r]
    not_full = (hist < RM).to(gpu_device)
    assert bool((h.src_info[rr, ll, probe][not_full] == -12345).all())
    assert bool((h.recv_x[rr, ll, probe][not_full] == (0x5C if cfg.use_fp8 else 0x5C5C)).all())

    # the oracle, on valid rows
    nt = [T] * R
    ref = oracle.dispatch(data["x"], idx, nt, cfg.max_tokens, E, cfg.use_fp8, poison=None)
    compare_dispatch(h, ref, check_poison=False)

    # round trip with the identity expert (bf16) / dequantising expert (fp8)
    h.alloc_combine_io()
    h.fill_expert_out_from_recv()
    h.combine()
    torch.cuda.synchronize()
    w = data["topk_weights"].masked_fill(idx == -1, 0).sum(dim=2, keepdim=True)
    expect = data["x"].float() * w
    got = h.combined.cpu()
    if cfg.use_fp8:
        torch.testing.assert_close(got.float(), expect, rtol=0.15, atol=5e-3 * float(data["x"].float().abs().max()))
    else:
        assert rc.calc_diff(expect, got.float()) < 1e-5
    assert not bool(torch.isnan(got.float()).any())
    # and bit for bit against the oracle's combine on the same expert outputs (valid rows copied sparsely)
    eo = torch.empty((R, L, RM, cfg.hidden), dtype=torch.bfloat16)
    rows = valid_rows(h.expert_out, h.recv_count).cpu()
    mask = torch.arange(RM).view(1, RM) < cnt.reshape(-1, 1)
    eo.view(R * L, RM, cfg.hidden)[mask] = rows
    want = oracle.combine(eo, idx, data["topk_weights"], ref["src_info"], ref["layout_range"], nt, cfg.max_tokens, E)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_dsv3_decode_full_size_through_the_per_rank_buffer_api(gpu_device, oracle):
    """The headline world driven the way the reference's callers drive it: 32 `Buffer.dispatch` and 32
    `Buffer.combine` calls (the Python wrapper with the reference's signature, async_finish), every rank's
    outputs against the oracle bit for bit."""
    from mooncake_amd import Buffer, LogicalGroup
    cfg = CONFIGS["dsv3_decode"]
    announce(f"full size through Buffer.dispatch / Buffer.combine {cfg}")
    data = generate(cfg, seed=0)
    R, T, E, L, H = cfg.num_ranks, cfg.tokens_per_rank, cfg.num_experts, cfg.num_local_experts, cfg.hidden
    world, groups = LogicalGroup.make_world(R)
    nbytes = Buffer.get_ep_buffer_size_hint(cfg.max_tokens, H, R, E)
    bufs = [Buffer(g, nbytes) for g in groups]
    x = data["x"].to(gpu_device)
    idx = data["topk_idx"].to(gpu_device)
    w = data["topk_weights"].to(gpu_device)
    disp = [bufs[r].dispatch(x[r], idx[r], None, cfg.max_tokens, E, -1, use_fp8=True, async_finish=True)
            for r in range(R)]
    for d in disp:
        d[3].current_stream_wait()
    torch.cuda.synchronize()
    nt = [T] * R
    ref = oracle.dispatch(data["x"], data["topk_idx"], nt, cfg.max_tokens, E, True, poison=None)
    RM = R * cfg.max_tokens
    for r in range(R):
        (recv_x, scales), cnt, handle, _, _ = disp[r]
        cnt_cpu = cnt.cpu()
        assert torch.equal(cnt_cpu, ref["recv_count"][r])
        assert torch.equal(handle[1].cpu(), ref["layout_range"][r])
        assert scales.shape == (L, RM, H // 128) and scales.stride() == (H // 128 * RM, 1, RM)
        mask = torch.arange(RM).view(1, RM) < cnt_cpu.view(L, 1)
        assert torch.equal(handle[0].cpu()[mask], ref["src_info"][r][mask])
        assert torch.equal(recv_x.view(torch.uint8).cpu()[mask], ref["recv_x"][r].view(torch.uint8)[mask])
        assert torch.equal(scales.cpu()[mask].contiguous().view(torch.int32),
                           ref["scales"][r][mask].contiguous().view(torch.int32))
    # the mock expert of the reference's grid test, then combine
    factor = torch.arange(E, dtype=torch.float32) * 0.1 + 1.0
    rows = oracle.cast_back(ref["recv_x"], ref["scales"], ref["recv_count"], factor)
    want = oracle.combine(rows, data["topk_idx"], data["topk_weights"], ref["src_info"], ref["layout_range"], nt,
                          cfg.max_tokens, E)
    outs = []
    for r in range(R):
        (recv_x, scales), cnt, handle, _, _ = disp[r]
        f = factor[r * L:(r + 1) * L].to(gpu_device).view(L, 1, 1)
        once = (recv_x.float().view(L, RM, H // 128, 128) * scales.unsqueeze(-1)).view(L, RM, H).to(torch.bfloat16)
        expert_out = (once.float() * f).to(torch.bfloat16)
        outs.append(bufs[r].combine(expert_out, idx[r], w[r], None, -1, handle, async_finish=True))
        del once, expert_out
    for o in outs:
        o[1].current_stream_wait()
    torch.cuda.synchronize()
    for r in range(R):
        assert torch.equal(outs[r][0].cpu().view(torch.int16), want[r].view(torch.int16)), f"rank {r}"
