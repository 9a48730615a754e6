"""Lifetime, ordering and failure scenarios of the per-rank `Buffer` API on
logical ranks:

* a rank that runs several collectives ahead of its peers and drops its
  tensors at once (the round is enqueued later, from raw addresses);
* calls of one world alternating between two streams with no waits;
* the reference's stale-data test (mooncake-ep/tests/test_ep_grid.py:250-369):
  a rank that dies between dispatch and combine, after a full round on the
  same buffers;
* `return_recv_hook` launched in two parts, like the reference's SEND / RECV
  split (mooncake_ep_buffer.cpp:303-305, :330-335);
* a silent rank that comes back (Buffer.update_ep_member);
* a dispatch of which only the layout phase ran, followed by a combine;
* a world whose scratch grows after one of its calls went into a graph.
"""
import gc

import pytest
import torch

from mooncake_amd import Buffer, LogicalGroup, _lib, ep
from mooncake_amd.harness import WorldHarness
from mooncake_amd.workloads import EPConfig, generate
from tests.gpu_util import announce, compare_dispatch

pytestmark = pytest.mark.gpu


def make_world(num_ranks, max_tokens, hidden, num_experts):
    world, groups = LogicalGroup.make_world(num_ranks)
    nbytes = Buffer.get_ep_buffer_size_hint(max_tokens, hidden, num_ranks, num_experts)
    return world, [Buffer(g, nbytes) for g in groups]


def rank_inputs(seed, num_tokens, hidden, num_experts, top_k):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(num_tokens, hidden, generator=g).to(torch.bfloat16)
    idx = torch.topk(torch.randn(num_tokens, num_experts, generator=g), top_k, dim=-1)[1]
    w = torch.softmax(torch.rand(num_tokens, top_k, generator=g), dim=-1)
    return x, idx, w


def oracle_world(oracle, per_rank, max_tokens, num_experts, use_fp8, present=None):
    """Oracle dispatch of a world given {rank: (x, idx, w)} CPU tensors."""
    R = len(per_rank)
    H, K = per_rank[0][0].size(1), per_rank[0][1].size(1)
    xs = torch.zeros(R, max_tokens, H, dtype=torch.bfloat16)
    idxs = torch.full((R, max_tokens, K), -1, dtype=torch.int64)
    ws = torch.zeros(R, max_tokens, K, dtype=torch.float32)
    nts = [0] * R
    for r, (x, idx, w) in enumerate(per_rank):
        if present is not None and not present[r]:
            continue
        nts[r] = x.size(0)
        xs[r, :nts[r]], idxs[r, :nts[r]], ws[r, :nts[r]] = x, idx, w
    ref = oracle.dispatch(xs, idxs, nts, max_tokens, num_experts, use_fp8, src_present=present)
    return ref, xs, idxs, ws, nts


def check_rank_dispatch(ref, r, recv_x, recv_count, handle, use_fp8):
    cnt = recv_count.cpu()
    assert torch.equal(cnt, ref["recv_count"][r])
    assert torch.equal(handle[1].cpu(), ref["layout_range"][r])
    for le in range(cnt.numel()):
        n = int(cnt[le])
        assert torch.equal(handle[0][le, :n].cpu(), ref["src_info"][r, le, :n])
        if use_fp8:
            assert torch.equal(recv_x[0][le, :n].view(torch.uint8).cpu(), ref["recv_x"][r, le, :n].view(torch.uint8))
            assert torch.equal(recv_x[1][le, :n].cpu().contiguous().view(torch.int32),
                               ref["scales"][r, le, :n].contiguous().view(torch.int32))
        else:
            assert torch.equal(recv_x[le, :n].view(torch.int16).cpu(), ref["recv_x"][r, le, :n].view(torch.int16))


def test_rank_runs_four_rounds_ahead_and_drops_its_tensors(gpu_device, oracle):
    R, T, H, E, K = 2, 64, 1024, 16, 4
    announce("rank 0 posts four dispatches with temporaries, rank 1 catches up")
    world, bufs = make_world(R, T, H, E)
    rounds = [[rank_inputs(1000 + 10 * j + r, T, H, E, K) for r in range(R)] for j in range(4)]
    out0 = []
    for j in range(4):
        x, idx, _ = rounds[j][0]
        # the device copies are temporaries: nothing but the Buffer's own bookkeeping keeps them alive
        res = bufs[0].dispatch(x.to(gpu_device), idx.to(gpu_device), None, T, E, -1, use_fp8=False)
        out0.append(res[:3])
        del res
        gc.collect()
        # allocator traffic that would reuse the dropped inputs' memory if it had been freed
        junk = [torch.full((T, H), 7.0, dtype=torch.bfloat16, device=gpu_device) for _ in range(4)]
        junk2 = [torch.full((T, K), 3, dtype=torch.int64, device=gpu_device) for _ in range(4)]
        del junk, junk2
    assert bufs[0].runtime.pending_calls() == (4, 0)
    assert bufs[0].runtime.retained() == (4, 0)            # the runtime holds the four calls' tensors
    out1 = []
    for j in range(4):
        x, idx, _ = rounds[j][1]
        out1.append(bufs[1].dispatch(x.to(gpu_device), idx.to(gpu_device), None, T, E, -1, use_fp8=False)[:3])
    torch.cuda.synchronize()
    assert bufs[0].runtime.pending_calls() == (0, 0)
    for j in range(4):
        ref, *_ = oracle_world(oracle, rounds[j], T, E, False)
        check_rank_dispatch(ref, 0, *out0[j], False)
        check_rank_dispatch(ref, 1, *out1[j], False)
    # the next call of rank 0 lets go of what the finished rounds pinned
    x, idx, _ = rounds[0][0]
    bufs[0].dispatch(x.to(gpu_device), idx.to(gpu_device), None, T, E, -1, use_fp8=False)
    assert bufs[0].runtime.retained() == (1, 0)


@pytest.mark.parametrize("use_fp8", [True, False], ids=["fp8", "bf16"])
def test_two_streams_alternate_on_one_world_without_waits(gpu_device, oracle, use_fp8):
    cfg = EPConfig("two_streams", 8, 96, 2048, 64, 8, use_fp8)
    announce(f"two streams on one world {cfg}")
    world = ep.World(cfg.num_ranks)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    hs = []
    for i in range(4):
        h = WorldHarness(cfg, world=world)
        h.load(generate(cfg, seed=50 + i))
        h.alloc_dispatch_outputs(poison=True)
        h.alloc_combine_io()
        hs.append(h)
    torch.cuda.synchronize()
    # dispatch / consumer / combine of four data sets, every call on the other stream than the one
    # before it, and nothing but the library orders them
    streams = [s1, s2]
    n = 0
    for h in hs:
        for call in (h.dispatch, h.cast_back, h.combine):
            call(stream=streams[n % 2])
            n += 1
    torch.cuda.synchronize()
    nt = [cfg.tokens_per_rank] * cfg.num_ranks
    for i, h in enumerate(hs):
        data = generate(cfg, seed=50 + i)
        ref = oracle.dispatch(data["x"], data["topk_idx"], nt, cfg.max_tokens, cfg.num_experts, use_fp8)
        compare_dispatch(h, ref, check_poison=True)
        rows = oracle.cast_back(ref["recv_x"], ref["scales"] if use_fp8 else None, ref["recv_count"], None)
        want = oracle.combine(rows, data["topk_idx"], data["topk_weights"], ref["src_info"], ref["layout_range"], nt,
                              cfg.max_tokens, cfg.num_experts)
        assert torch.equal(h.combined.cpu().view(torch.int16), want.view(torch.int16)), f"data set {i}"


@pytest.mark.parametrize("mode", ["default", "async", "hook"])
def test_every_rank_on_a_stream_of_its_own(gpu_device, oracle, mode):
    """Callers on different streams: the round runs on the world's communication stream, after what each
    rank's stream holds, and each rank's later work (default: at once; async / hook: after the wait) sees it."""
    R, T, H, E, K = 4, 96, 2048, 32, 4
    announce(f"one stream per rank, {mode}")
    world, bufs = make_world(R, T, H, E)
    streams = [torch.cuda.Stream() for _ in range(R)]
    ins = [rank_inputs(700 + r, T, H, E, K) for r in range(R)]
    host = [tuple(t.pin_memory() for t in i) for i in ins]
    dev, outs, sums = [None] * R, [None] * R, [None] * R
    kw = dict(async_finish=mode == "async", return_recv_hook=mode == "hook")
    for r in range(R):
        with torch.cuda.stream(streams[r]):
            # the inputs arrive on the rank's own stream right before the call: the round must wait for that
            dev[r] = tuple(t.to(gpu_device, non_blocking=True) for t in host[r])
            outs[r] = bufs[r].dispatch(dev[r][0], dev[r][1], None, T, E, -1, use_fp8=True, **kw)
    for r in range(R):
        with torch.cuda.stream(streams[r]):
            if mode == "async":
                outs[r][3].current_stream_wait()
            if mode == "hook":
                outs[r][4]()
            # a consumer on the rank's stream, with nothing but the library between it and the round
            sums[r] = outs[r][1].sum()
    torch.cuda.synchronize()
    ref, *_ = oracle_world(oracle, ins, T, E, True)
    for r in range(R):
        assert int(sums[r]) == int(ref["recv_count"][r].sum())
        check_rank_dispatch(ref, r, outs[r][0], outs[r][1], outs[r][2], True)
    # combine the same way
    factor = torch.arange(E, dtype=torch.float32) * 0.1 + 1.0
    rows = oracle.cast_back(ref["recv_x"], ref["scales"], ref["recv_count"], factor)
    nt = [T] * R
    xs = torch.stack([i[0] for i in ins]); idxs = torch.stack([i[1] for i in ins]); ws = torch.stack([i[2] for i in ins])
    want = oracle.combine(rows, idxs, ws, ref["src_info"], ref["layout_range"], nt, T, E)
    L = E // R
    res = [None] * R
    for r in range(R):
        with torch.cuda.stream(streams[r]):
            (px, ps), cnt, handle, _, _ = outs[r]
            f = factor[r * L:(r + 1) * L].to(gpu_device, non_blocking=True).view(L, 1, 1)
            once = (px.float().view(L, R * T, H // 128, 128) * ps.unsqueeze(-1)).view(L, R * T, H).to(torch.bfloat16)
            eo = (once.float() * f).to(torch.bfloat16)
            res[r] = bufs[r].combine(eo, dev[r][1], dev[r][2], None, -1, handle, **kw)
    copies = [None] * R
    for r in range(R):
        with torch.cuda.stream(streams[r]):
            if mode == "async":
                res[r][1].current_stream_wait()
            if mode == "hook":
                res[r][2]()
            copies[r] = res[r][0].clone()
    torch.cuda.synchronize()
    for r in range(R):
        assert torch.equal(copies[r].cpu().view(torch.int16), want[r].view(torch.int16)), f"rank {r}"


def test_rank_dies_between_dispatch_and_combine(gpu_device, oracle):
    # test_ep_grid.py:250-369 at its shape family: 2 ranks, bf16, async_finish, fail_rank 1
    R, T, H, E, K = 2, 128, 2048, 32, 4
    L, fail = E // R, 1
    announce("stale data: rank 1 dies after dispatch, rank 0 combines with a timeout")
    world, bufs = make_world(R, T, H, E)

    def dispatch_all(seed, nts):
        ins = [tuple(t.to(gpu_device) for t in rank_inputs(seed + r, nts[r], H, E, K)) for r in range(R)]
        act = [torch.ones(R, dtype=torch.int32, device=gpu_device) for _ in range(R)]
        outs = [bufs[r].dispatch(ins[r][0], ins[r][1], act[r], T, E, -1, use_fp8=False, async_finish=True)
                for r in range(R)]
        for o in outs:
            o[3].current_stream_wait()
        return ins, act, outs

    def mock_expert(r, recv_x):
        factor = (torch.arange(r * L, (r + 1) * L, device=gpu_device).float() * 0.1 + 1.0).view(L, 1, 1)
        return (recv_x.float() * factor).to(torch.bfloat16)

    # first cycle: every rank alive, on the buffers the second cycle reuses
    nts = [T, int(T * (1.0 - 0.05 * (1 / R)))]
    ins, act, outs = dispatch_all(2026, nts)
    combined = []
    for r in range(R):
        res = bufs[r].combine(mock_expert(r, outs[r][0]), ins[r][1], ins[r][2], act[r], -1, outs[r][2],
                              async_finish=True, out=torch.zeros_like(ins[r][0]))
        combined.append(res)
    for r in range(R):
        combined[r][1].current_stream_wait()
    torch.cuda.synchronize()
    for r in range(R):
        x, idx, w = ins[r]
        want = (x.float() * ((idx.float() * 0.1 + 1.0) * w).sum(dim=1, keepdim=True)).to(torch.bfloat16)
        torch.testing.assert_close(combined[r][0], want, rtol=5e-2, atol=1e-3)

    # second cycle: both ranks dispatch, rank 1 goes away before combine
    ins, act, outs = dispatch_all(200, nts)
    torch.cuda.synchronize()
    world.set_rank_silent(fail)
    x, idx, w = ins[0]
    out, event, _ = bufs[0].combine(mock_expert(0, outs[0][0]), idx, w, act[0], 5_000, outs[0][2],
                                    async_finish=True, out=torch.zeros_like(x))
    event.current_stream_wait()
    torch.cuda.synchronize()
    assert act[0][fail].item() == 0
    assert not torch.isnan(out).any().item()
    factors = (idx.float() * 0.1 + 1.0) * (idx // L != fail).float()
    want = (x.float() * (factors * w).sum(dim=1, keepdim=True)).to(torch.bfloat16)
    torch.testing.assert_close(out, want, rtol=5e-2, atol=1e-3)
    # and bit for bit: the oracle's combine with rank 0 seeing rank 1 inactive, on rank 0's expert rows only
    cpu = [tuple(t.cpu() for t in ins[r]) for r in range(R)]
    ref, xs, idxs, ws, nt = oracle_world(oracle, cpu, T, E, False)
    eo = torch.zeros(R, L, R * T, H, dtype=torch.bfloat16)
    eo[0] = mock_expert(0, outs[0][0]).cpu()
    active = torch.ones(R, R, dtype=torch.int32)
    active[0, fail] = 0
    got = oracle.combine(eo, idxs, ws, ref["src_info"], ref["layout_range"], nt, T, E, active=active)
    assert torch.equal(out.cpu().view(torch.int16), got[0, :nts[0]].view(torch.int16))


def test_recv_hook_enqueues_the_second_part(gpu_device, oracle):
    R, T, H, E, K = 4, 64, 2048, 32, 4
    announce("return_recv_hook: layout + data at the call, scales at the first hook")
    world, bufs = make_world(R, T, H, E)
    ins = [rank_inputs(300 + r, T, H, E, K) for r in range(R)]
    dev = [tuple(t.to(gpu_device) for t in i) for i in ins]
    outs = [bufs[r].dispatch(dev[r][0], dev[r][1], None, T, E, -1, use_fp8=True, return_recv_hook=True)
            for r in range(R)]
    # poison the scales after the first part has run; the second part has not been enqueued yet
    torch.cuda.synchronize()
    assert bufs[0].runtime.pending_calls() == (1, 0)
    for o in outs:
        o[0][1].fill_(float("nan"))
    torch.cuda.synchronize()
    ref, *_ = oracle_world(oracle, ins, T, E, True)
    for r in range(R):
        cnt = outs[r][1].cpu()
        assert torch.equal(cnt, ref["recv_count"][r])               # counts and payload are there already
        n = int(cnt[0])
        assert torch.equal(outs[r][0][0][0, :n].view(torch.uint8).cpu(), ref["recv_x"][r, 0, :n].view(torch.uint8))
        assert bool(torch.isnan(outs[r][0][1]).all())               # the scales are not
    outs[2][4]()                                                     # any rank's hook enqueues the rest
    torch.cuda.synchronize()
    assert bufs[0].runtime.pending_calls() == (0, 0)
    for r in range(R):
        outs[r][4]()
    torch.cuda.synchronize()
    for r in range(R):
        check_rank_dispatch(ref, r, outs[r][0], outs[r][1], outs[r][2], True)


def test_next_dispatch_enqueues_a_second_part_nobody_asked_for(gpu_device, oracle):
    R, T, H, E, K = 2, 32, 1024, 8, 2
    announce("return_recv_hook: a second dispatch before the first one's hook")
    world, bufs = make_world(R, T, H, E)
    a = [rank_inputs(400 + r, T, H, E, K) for r in range(R)]
    b = [rank_inputs(500 + r, T, H, E, K) for r in range(R)]
    outs_a = [bufs[r].dispatch(a[r][0].cuda(), a[r][1].cuda(), None, T, E, -1, use_fp8=True, return_recv_hook=True)
              for r in range(R)]
    outs_b = [bufs[r].dispatch(b[r][0].cuda(), b[r][1].cuda(), None, T, E, -1, use_fp8=True, return_recv_hook=True)
              for r in range(R)]
    for o in outs_a + outs_b:
        o[4]()
    torch.cuda.synchronize()
    for ins, outs in ((a, outs_a), (b, outs_b)):
        ref, *_ = oracle_world(oracle, ins, T, E, True)
        for r in range(R):
            check_rank_dispatch(ref, r, outs[r][0], outs[r][1], outs[r][2], True)


def test_next_dispatch_after_every_hook_was_dropped(gpu_device, oracle):
    """The hooks of a two-part round are the only other owners of its state once the round has left the
    queue.  Dropped without being called, they leave the world's own reference as the last one - and the
    next dispatch, which has to enqueue the second part itself, must keep the round alive while it does."""
    R, T, H, E, K = 2, 32, 1024, 8, 2
    announce("return_recv_hook: hooks destroyed uncalled, then a second dispatch")
    world, bufs = make_world(R, T, H, E)
    a = [rank_inputs(410 + r, T, H, E, K) for r in range(R)]
    b = [rank_inputs(510 + r, T, H, E, K) for r in range(R)]
    outs_a = [bufs[r].dispatch(a[r][0].cuda(), a[r][1].cuda(), None, T, E, -1, use_fp8=True, return_recv_hook=True)
              for r in range(R)]
    assert bufs[0].runtime.pending_calls() == (1, 0)
    kept_a = [o[:3] for o in outs_a]
    del outs_a                                   # the hook closures go, and the library's hook objects with them
    gc.collect()
    outs_b = [bufs[r].dispatch(b[r][0].cuda(), b[r][1].cuda(), None, T, E, -1, use_fp8=True) for r in range(R)]
    torch.cuda.synchronize()
    assert bufs[0].runtime.pending_calls() == (0, 0)
    for ins, outs in ((a, kept_a), (b, outs_b)):
        ref, *_ = oracle_world(oracle, ins, T, E, True)
        for r in range(R):
            check_rank_dispatch(ref, r, outs[r][0], outs[r][1], outs[r][2], True)


def test_silent_rank_comes_back(gpu_device, oracle):
    R, T, H, E, K = 3, 32, 512, 12, 3
    announce("a silent rank rejoins the world")
    world, bufs = make_world(R, T, H, E)

    def run(seed, alive):
        ins = [rank_inputs(seed + r, T, H, E, K) for r in range(R)]
        outs = {r: bufs[r].dispatch(ins[r][0].cuda(), ins[r][1].cuda(), None, T, E, 1000, use_fp8=False)
                for r in alive}
        torch.cuda.synchronize()
        present = [int(r in alive) for r in range(R)]
        ref, *_ = oracle_world(oracle, ins, T, E, False, present=present)
        for r in alive:
            check_rank_dispatch(ref, r, outs[r][0], outs[r][1], outs[r][2], False)

    run(600, [0, 1, 2])
    world.set_rank_silent(1)
    run(610, [0, 2])
    run(620, [0, 2])
    world.set_rank_silent(1, False)
    run(630, [0, 1, 2])
    run(640, [0, 1, 2])


def test_combine_after_a_dispatch_of_which_only_the_layout_ran(gpu_device, oracle):
    cfg = EPConfig("layout_only", 4, 48, 1024, 16, 4, False)
    announce(f"combine after a layout-only dispatch {cfg}")
    data = generate(cfg, seed=9)
    full = WorldHarness(cfg)                         # a full dispatch produces the handle
    full.load(data)
    full.alloc_dispatch_outputs(poison=True)
    full.alloc_combine_io()
    full.dispatch()
    full.cast_back()
    # another world sees the same tensors, but of its dispatch only the layout phase is issued: its
    # routing state is incomplete, and a combine of the handle must not lean on it
    other = WorldHarness(cfg)
    for name in ("x", "topk_idx", "topk_weights", "recv_x", "recv_count", "src_info", "layout_range", "expert_out"):
        setattr(other, name, getattr(full, name))
    other.alloc_combine_io()
    other.dispatch(phases=_lib.PHASE_LAYOUT)
    other.combine()
    torch.cuda.synchronize()
    nt = [cfg.tokens_per_rank] * cfg.num_ranks
    ref = oracle.dispatch(data["x"], data["topk_idx"], nt, cfg.max_tokens, cfg.num_experts, False)
    want = oracle.combine(ref["recv_x"], data["topk_idx"], data["topk_weights"], ref["src_info"],
                          ref["layout_range"], nt, cfg.max_tokens, cfg.num_experts)
    assert torch.equal(other.combined.cpu().view(torch.int16), want.view(torch.int16))


def test_scratch_grows_after_a_call_went_into_a_graph(gpu_device, oracle):
    small = EPConfig("graph_small", 4, 16, 512, 8, 2, True)
    large = EPConfig("graph_large", 4, 64, 2048, 32, 8, True)
    announce(f"graph of {small}, then eager {large} on the same world")
    world = ep.World(4)

    def harness(cfg, seed):
        h = WorldHarness(cfg, world=world)
        h.load(generate(cfg, seed=seed))
        h.alloc_dispatch_outputs(poison=False)
        h.alloc_combine_io()
        return h

    def expected(cfg, data):
        nt = [cfg.tokens_per_rank] * cfg.num_ranks
        ref = oracle.dispatch(data["x"], data["topk_idx"], nt, cfg.max_tokens, cfg.num_experts, True)
        rows = oracle.cast_back(ref["recv_x"], ref["scales"], ref["recv_count"], None)
        return ref, oracle.combine(rows, data["topk_idx"], data["topk_weights"], ref["src_info"],
                                   ref["layout_range"], nt, cfg.max_tokens, cfg.num_experts)

    hs = harness(small, 1)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        hs.dispatch(); hs.cast_back(); hs.combine()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        hs.dispatch(); hs.cast_back(); hs.combine()
    # the larger shape outgrows every piece of the world's scratch while the graph holds the old addresses
    hl = harness(large, 2)
    hl.dispatch(); hl.cast_back(); hl.combine()
    torch.cuda.synchronize()
    ref, want = expected(large, generate(large, seed=2))
    compare_dispatch(hl, ref, check_poison=False)
    assert torch.equal(hl.combined.cpu().view(torch.int16), want.view(torch.int16))
    for seed in (3, 4):
        data = generate(small, seed=seed)
        hs.x.copy_(data["x"]); hs.topk_idx.copy_(data["topk_idx"]); hs.topk_weights.copy_(data["topk_weights"])
        hs.combined.zero_()
        torch.cuda.synchronize()
        g.replay()
        hl.dispatch(); hl.combine()                   # eager traffic on the grown scratch in between
        torch.cuda.synchronize()
        ref, want = expected(small, data)
        compare_dispatch(hs, ref, check_poison=False)
        assert torch.equal(hs.combined.cpu().view(torch.int16), want.view(torch.int16)), f"replay, seed {seed}"
