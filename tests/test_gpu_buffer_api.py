"""The per-rank `Buffer` API (the drop-in boundary) on logical ranks, checked
the way the reference checks its own Buffer:

* the correctness grid of mooncake-ep/tests/test_ep_grid.py (seeded random
  tokens, a mock expert `recv * (expert_id * 0.1 + 1)`, the closed form
  `x * sum_k factor(e_k) * w_k`, tolerances of :204-210), over fp8 / bf16,
  default / async_finish / return_recv_hook, and a rank that dies before
  dispatch;
* the structured-data smoke test of mooncake-wheel/tests/test_mooncake_ep.py
  (:28-36, :59-75, :92-94);
* against the oracle, bit for bit;
* the reference's host assertions and NotImplementedError paths.
"""
import random

import pytest
import torch

from mooncake_amd import Buffer, LogicalGroup, ep
from tests import ref_checks as rc
from tests.gpu_util import announce

pytestmark = pytest.mark.gpu


def make_world(num_ranks, max_tokens, hidden, num_experts, disable_p2p=False):
    world, groups = LogicalGroup.make_world(num_ranks)
    nbytes = Buffer.get_ep_buffer_size_hint(max_tokens, hidden, num_ranks, num_experts)
    return world, [Buffer(g, nbytes, disable_p2p=disable_p2p) for g in groups]


def grid_inputs(rank, num_ranks, max_tokens, hidden, num_experts, top_k, device):
    # test_ep_grid.py:72-83
    g = torch.Generator().manual_seed(2026 + rank)
    num_tokens = int(max_tokens * (1.0 - 0.05 * (rank / num_ranks)))
    x = torch.randn(num_tokens, hidden, generator=g).to(torch.bfloat16)
    scores = torch.randn(num_tokens, num_experts, generator=g)
    topk_idx = torch.topk(scores, top_k, dim=-1)[1]
    topk_weights = torch.softmax(torch.rand(num_tokens, top_k, generator=g), dim=-1)
    return x.to(device), topk_idx.to(device), topk_weights.to(device)


def dequantize_fp8(x_fp8, scales):
    L, rows, hidden = x_fp8.shape
    v = x_fp8.float().view(L, rows, hidden // 128, 128) * scales.unsqueeze(-1)
    return v.view(L, rows, hidden).to(torch.bfloat16)


MODES = [(False, False), (True, False), (False, True)]      # (async_finish, return_recv_hook)


@pytest.mark.parametrize("use_fp8", [False, True], ids=["bf16", "fp8"])
@pytest.mark.parametrize("async_finish,return_recv_hook", MODES, ids=["default", "async", "hook"])
@pytest.mark.parametrize("fail_rank", [-1, 1], ids=["all_alive", "rank1_dead"])
@pytest.mark.parametrize("disable_p2p", [False, True], ids=["p2p", "no_p2p"])
@pytest.mark.parametrize("comm_stream", [0, 1], ids=["callers_stream", "comm_stream"])
def test_grid_closed_form(gpu_device, oracle, use_fp8, async_finish, return_recv_hook, fail_rank, disable_p2p,
                          comm_stream):
    # the reference's grid (test_ep_grid.py:469-483): fp8 x async x hook x fail_rank {-1, 1} x disable_p2p at its one
    # shape, on 8 ranks (its world is one rank per GPU of a node); use_fallback has no counterpart here
    num_ranks, max_tokens, hidden, num_experts, top_k = 8, 256, 2048, 288, 8
    announce(f"grid fp8={use_fp8} async={async_finish} hook={return_recv_hook} fail_rank={fail_rank} "
             f"disable_p2p={disable_p2p} comm_stream={comm_stream}")
    world, bufs = make_world(num_ranks, max_tokens, hidden, num_experts, disable_p2p)
    assert bufs[0].runtime.p2p_enabled() == (not disable_p2p)
    world.set_option("comm_stream", comm_stream)     # 1: the reference's arrangement, rounds on a stream of their own
    L = num_experts // num_ranks
    alive = [r for r in range(num_ranks) if r != fail_rank]
    timeout_us = 5_000_000 if fail_rank != -1 else -1
    if fail_rank != -1:
        world.set_rank_silent(fail_rank)                 # the process that calls os._exit(0) in the reference test

    inputs = {r: grid_inputs(r, num_ranks, max_tokens, hidden, num_experts, top_k, gpu_device) for r in alive}
    active = {r: torch.ones(num_ranks, dtype=torch.int32, device=gpu_device) for r in alive}
    disp = {}
    for r in alive:
        x, idx, _ = inputs[r]
        disp[r] = bufs[r].dispatch(x, idx, active[r], num_max_dispatch_tokens_per_rank=max_tokens,
                                   num_experts=num_experts, timeout_us=timeout_us, use_fp8=use_fp8,
                                   async_finish=async_finish, return_recv_hook=return_recv_hook)
    for r in alive:
        _, _, _, event, hook = disp[r]
        if return_recv_hook:
            hook()
        if async_finish:
            event.current_stream_wait()
    torch.cuda.synchronize()

    if fail_rank != -1:
        for r in alive:
            assert active[r][fail_rank].item() == 0
            assert active[r].sum().item() == num_ranks - 1

    # bit-exact against the oracle for every live rank's outputs
    Tmax = max_tokens
    xs = torch.zeros(num_ranks, Tmax, hidden, dtype=torch.bfloat16)
    idxs = torch.full((num_ranks, Tmax, top_k), -1, dtype=torch.int64)
    nts = [0] * num_ranks
    for r in alive:
        x, idx, _ = inputs[r]
        nts[r] = x.size(0)
        xs[r, :nts[r]] = x.cpu()
        idxs[r, :nts[r]] = idx.cpu()
    present = [int(r in alive) for r in range(num_ranks)]
    ref = oracle.dispatch(xs, idxs, nts, max_tokens, num_experts, use_fp8, src_present=present)
    for r in alive:
        recv_x, recv_count, handle, _, _ = disp[r]
        cnt = recv_count.cpu()
        assert torch.equal(cnt, ref["recv_count"][r])
        assert torch.equal(handle[1].cpu(), ref["layout_range"][r])
        for le in range(L):
            n = int(cnt[le])
            assert torch.equal(handle[0][le, :n].cpu(), ref["src_info"][r, le, :n])
            if use_fp8:
                assert recv_x[1].shape == (L, num_ranks * max_tokens, hidden // 128)
                assert recv_x[1].stride() == (hidden // 128 * num_ranks * max_tokens, 1, num_ranks * max_tokens)
                assert torch.equal(recv_x[0][le, :n].view(torch.uint8).cpu(), ref["recv_x"][r, le, :n].view(torch.uint8))
                assert torch.equal(recv_x[1][le, :n].cpu().contiguous().view(torch.int32),
                                   ref["scales"][r, le, :n].contiguous().view(torch.int32))
            else:
                assert torch.equal(recv_x[le, :n].view(torch.int16).cpu(), ref["recv_x"][r, le, :n].view(torch.int16))

    # mock expert forward, test_ep_grid.py:160-173
    outs = {}
    for r in alive:
        recv_x, recv_count, handle, _, _ = disp[r]
        recv_bf16 = dequantize_fp8(recv_x[0], recv_x[1]) if use_fp8 else recv_x
        factor = (torch.arange(r * L, (r + 1) * L, device=gpu_device).float() * 0.1 + 1.0).view(L, 1, 1)
        expert_out = (recv_bf16.float() * factor).to(torch.bfloat16).contiguous()
        x, idx, w = inputs[r]
        out_tensor = torch.zeros_like(x)
        outs[r] = bufs[r].combine(expert_out, idx, w, active[r], timeout_us=timeout_us, handle=handle,
                                  zero_copy=False, async_finish=async_finish, return_recv_hook=return_recv_hook,
                                  out=out_tensor)
    for r in alive:
        combined_x, event, hook = outs[r]
        if return_recv_hook:
            hook()
        if async_finish:
            event.current_stream_wait()
    torch.cuda.synchronize()

    for r in alive:
        x, idx, w = inputs[r]
        factors = idx.float() * 0.1 + 1.0
        if fail_rank != -1:
            factors = factors * (idx // L != fail_rank).float()
        expected = (x.float() * (factors * w).sum(dim=1, keepdim=True)).to(torch.bfloat16)
        torch.testing.assert_close(outs[r][0], expected, rtol=0.15 if use_fp8 else 5e-2,
                                   atol=5e-3 if use_fp8 else 1e-3)


@pytest.mark.parametrize("use_fp8", [False, True], ids=["bf16", "fp8"])
def test_structured_data(gpu_device, use_fp8):
    # test_mooncake_ep.py:16-94 at its own shape (128 tokens, hidden 7168, top-8, 288 experts), on 2 ranks
    num_ranks, num_tokens, hidden, num_topk, num_experts = 2, 128, 7168, 8, 288
    announce(f"structured data fp8={use_fp8}")
    world, bufs = make_world(num_ranks, num_tokens, hidden, num_experts)
    L = num_experts // num_ranks
    rnd = random.Random(1)
    xs, idxs, ws = [], [], []
    for rank in range(num_ranks):
        g = torch.Generator().manual_seed(1 + rank)
        x = torch.ones((num_tokens, hidden), dtype=torch.bfloat16) * (rank - 128)
        x[:, -128:] = torch.arange(num_tokens).to(torch.bfloat16).view(-1, 1)
        scores = torch.randn((num_tokens, num_experts), generator=g).abs() + 1
        topk_idx = torch.topk(scores, num_topk, dim=-1, largest=True, sorted=True)[1]
        topk_weights = torch.randn((num_tokens, num_topk), generator=g).abs()
        for _ in range(10):
            topk_idx[rnd.randint(0, num_tokens - 1), rnd.randint(0, num_topk - 1)] = -1
        xs.append(x.to(gpu_device)); idxs.append(topk_idx.to(gpu_device)); ws.append(topk_weights.to(gpu_device))
    # the reference test passes an active_ranks tensor of the wrong length (num_tokens); the wrapper replaces it
    active = torch.ones((num_tokens,), dtype=torch.int32, device=gpu_device)
    disp = [bufs[r].dispatch(xs[r], idxs[r], active, num_tokens, num_experts, -1, use_fp8=use_fp8)
            for r in range(num_ranks)]
    torch.cuda.synchronize()
    all_topk_idx = torch.stack(idxs).cpu()
    recv_rows, counts, infos, ranges = [], [], [], []
    for r in range(num_ranks):
        packed, cnt, handle, _, _ = disp[r]
        if use_fp8:
            rows = rc.reference_cast_back(packed[0].reshape(-1, hidden).cpu(),
                                          packed[1].reshape(-1, hidden // 128).cpu().contiguous())
            rows = rows.view(L, -1, hidden)
        else:
            rows = packed.cpu()
        recv_rows.append(rows); counts.append(cnt.cpu()); infos.append(handle[0].cpu()); ranges.append(handle[1].cpu())
    rc.check_structured_dispatch(torch.stack(recv_rows), torch.stack(counts), torch.stack(infos),
                                 torch.stack(ranges), all_topk_idx, num_tokens)
    # combine: the dispatched rows straight back (:78-94)
    outs = []
    for r in range(num_ranks):
        packed, _, handle, _, _ = disp[r]
        sim = recv_rows[r].to(gpu_device).contiguous()
        out = torch.empty((num_tokens, hidden), dtype=torch.bfloat16, device=gpu_device)
        outs.append(bufs[r].combine(sim, idxs[r], ws[r], active, -1, handle, out=out)[0])
    torch.cuda.synchronize()
    for r in range(num_ranks):
        expect = xs[r].float() * ws[r].masked_fill(idxs[r] == -1, 0).sum(dim=1).view(-1, 1)
        assert torch.isnan(outs[r]).sum().item() == 0
        assert rc.calc_diff(expect.cpu(), outs[r].float().cpu()) < 1e-5


def test_single_rank_group(gpu_device, oracle):
    # group_size == 1 runs the native path with no peers (mooncake_ep_buffer.py:266-270)
    announce("single-rank group")
    world, bufs = make_world(1, 64, 1024, 8)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(50, 1024, generator=g).to(torch.bfloat16)
    idx = torch.topk(torch.randn(50, 8, generator=g), 2, dim=-1)[1]
    w = torch.softmax(torch.randn(50, 2, generator=g), dim=-1)
    recv, cnt, handle, _, _ = bufs[0].dispatch(x.cuda(), idx.cuda(), None, 64, 8, -1, use_fp8=False)
    out, _, _ = bufs[0].combine(recv.clone(), idx.cuda(), w.cuda(), None, -1, handle)
    torch.cuda.synchronize()
    ref = oracle.dispatch(x.unsqueeze(0), idx.unsqueeze(0), [50], 64, 8, False)
    assert torch.equal(cnt.cpu(), ref["recv_count"][0])
    expect = x.float() * w.sum(dim=1, keepdim=True)
    assert rc.calc_diff(expect, out.float().cpu()) < 1e-5


def test_collective_rounds_and_pending_errors(gpu_device):
    """A rank may run ahead (second dispatch before its peers' first); waiting
    on a round that is not complete is an error, not a hang."""
    announce("collective rounds")
    world, bufs = make_world(2, 16, 256, 4)
    g = torch.Generator().manual_seed(0)
    mk = lambda: (torch.randn(16, 256, generator=g).to(torch.bfloat16).cuda(),
                  torch.topk(torch.randn(16, 4, generator=g), 2, dim=-1)[1].cuda())
    (xa0, ia0), (xa1, ia1), (xb0, ib0), (xb1, ib1) = mk(), mk(), mk(), mk()
    ra0 = bufs[0].dispatch(xa0, ia0, None, 16, 4, -1, use_fp8=False, async_finish=True)
    rb0 = bufs[0].dispatch(xb0, ib0, None, 16, 4, -1, use_fp8=False, return_recv_hook=True)   # rank 0 runs ahead
    # MC_EP_ERR_PENDING: a RuntimeError (what the reference's callers catch) of a type of its own
    with pytest.raises(ep.PendingError, match="collective") as failure:
        ra0[3].current_stream_wait()
    assert isinstance(failure.value, RuntimeError)
    with pytest.raises(ep.PendingError, match="collective"):
        rb0[4]()
    ra1 = bufs[1].dispatch(xa1, ia1, None, 16, 4, -1, use_fp8=False)
    ra0[3].current_stream_wait()                                   # round A is complete now
    with pytest.raises(ep.PendingError, match="collective"):
        rb0[4]()
    rb1 = bufs[1].dispatch(xb1, ib1, None, 16, 4, -1, use_fp8=False)
    rb0[4]()
    torch.cuda.synchronize()
    for (ra, rb) in ((ra0, ra1), (rb0, rb1)):
        total = int(ra[1].sum() + rb[1].sum())
        assert total == 2 * 16 * 2                                 # every selection landed exactly once
    # round A and round B routed different tokens
    assert not torch.equal(ra0[0][:, :4], rb0[0][:, :4])


def test_a_round_that_cannot_launch_tells_every_waiter(gpu_device):
    """Ranks that disagree about the shape of a collective: the call that completes the round fails, and the
    rank that was already waiting on it learns why instead of seeing a round that is pending for ever."""
    announce("failed round")
    world, bufs = make_world(2, 16, 256, 4)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(16, 256, generator=g).to(torch.bfloat16).cuda()
    idx = torch.topk(torch.randn(16, 4, generator=g), 2, dim=-1)[1].cuda()
    first = bufs[0].dispatch(x, idx, None, 16, 4, -1, use_fp8=False, async_finish=True)
    with pytest.raises(RuntimeError, match="Failed: Assertion"):
        bufs[1].dispatch(x, idx[:, :1].contiguous(), None, 16, 4, -1, use_fp8=False)       # top-1 against top-2
    with pytest.raises(RuntimeError, match="could not be launched"):
        first[3].current_stream_wait()
    # the world goes on with the next round
    a = bufs[0].dispatch(x, idx, None, 16, 4, -1, use_fp8=False)
    b = bufs[1].dispatch(x, idx, None, 16, 4, -1, use_fp8=False)
    torch.cuda.synchronize()
    assert int(a[1].sum() + b[1].sum()) == 2 * 16 * 2


def test_host_assertions_and_unsupported(gpu_device):
    announce("host assertions")
    world, groups = LogicalGroup.make_world(2)
    x = torch.zeros(8, 256, dtype=torch.bfloat16, device=gpu_device)
    idx = torch.zeros(8, 2, dtype=torch.int64, device=gpu_device)
    w = torch.ones(8, 2, dtype=torch.float32, device=gpu_device)
    small = Buffer(groups[0], num_ep_buffer_bytes=1024)
    with pytest.raises(RuntimeError, match="Failed: Assertion"):   # layout.total_bytes <= num_ep_buffer_bytes
        small.dispatch(x, idx, None, 8, 4, -1, use_fp8=False)
    buf = Buffer(groups[0], Buffer.get_ep_buffer_size_hint(8, 256, 2, 4))
    with pytest.raises(RuntimeError, match="Failed: Assertion"):   # async together with return_recv_hook
        buf.dispatch(x, idx, None, 8, 4, -1, use_fp8=False, async_finish=True, return_recv_hook=True)
    with pytest.raises(AssertionError):                            # hidden % 128
        buf.dispatch(x[:, :200].contiguous(), idx, None, 8, 4, -1, use_fp8=False)
    with pytest.raises(AssertionError):                            # more tokens than the per-rank maximum
        buf.dispatch(x, idx, None, 4, 4, -1, use_fp8=False)
    with pytest.raises(AssertionError):                            # experts not divisible by ranks
        buf.dispatch(x, idx, None, 8, 5, -1, use_fp8=False)
    handle = (torch.zeros(2, 16, dtype=torch.int32, device=gpu_device),
              torch.zeros(2, 2, dtype=torch.int64, device=gpu_device), 8, 256, 4)
    eo = torch.zeros(2, 16, 256, dtype=torch.bfloat16, device=gpu_device)
    with pytest.raises(NotImplementedError, match="zero-copy"):
        buf.combine(eo, idx, w, None, -1, handle, zero_copy=True)
    with pytest.raises(NotImplementedError, match="zero-copy"):
        buf.get_next_combine_buffer(handle)
    assert buf.runtime.ibgda_disabled() and buf.runtime.use_fast_path() and not buf.runtime.is_roce()
    assert buf.runtime.get_local_qpns() == [] and buf.runtime.get_mr_info() == (0, 0)


def test_the_buffer_sees_the_callers_current_stream(gpu_device):
    """Buffer.dispatch / combine run on torch's current stream (reference: mooncake_ep_buffer.py:488-507 passes
    torch.cuda.current_stream().cuda_stream); the wrapper's shortcut to that address must follow stream contexts."""
    from mooncake_amd import mooncake_ep_buffer as mod
    announce("current stream lookup")
    assert mod._native_current_stream_ptr() == torch.cuda.current_stream().cuda_stream
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        assert mod._native_current_stream_ptr() == side.cuda_stream
        assert mod._native_current_stream_ptr() == torch.cuda.current_stream().cuda_stream
    assert mod._native_current_stream_ptr() == torch.cuda.current_stream().cuda_stream
