"""A thread per rank, each running the reference's per-rank code unchanged: `Buffer(group, ...)`, `dispatch`,
use the results at once, `combine`, use the result at once - what a process of the reference does
(mooncake-ep/tests/test_ep_grid.py:60-119).  With the world's option "blocking" a per-rank call returns only
when its collective has been launched, so whatever the thread does next with its outputs is ordered behind the
kernels; every thread checks its own results against the oracle while the others are still running."""
import time

import pytest
import torch

from mooncake_amd import Buffer, LogicalGroup, ep, spawn_ranks
from tests.gpu_util import announce
from tests.test_gpu_buffer_lifetime import check_rank_dispatch, oracle_world, rank_inputs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("mode", ["default", "async_finish", "return_recv_hook"])
@pytest.mark.parametrize("use_fp8", [True, False], ids=["fp8", "bf16"])
@pytest.mark.parametrize("own_stream", [True, False], ids=["own_streams", "shared_stream"])
def test_thread_per_rank_uses_results_as_soon_as_the_call_returns(gpu_device, oracle, use_fp8, mode, own_stream):
    R, T, H, E, K, steps = 4, 48, 1024, 16, 4, 3
    announce(f"thread per rank, fp8={use_fp8}, {mode}, own_stream={own_stream}")
    shared = torch.cuda.Stream()
    nbytes = Buffer.get_ep_buffer_size_hint(T, H, R, E)
    inputs = [[rank_inputs(7000 + 10 * j + r, T - r, H, E, K) for r in range(R)] for j in range(steps)]
    refs = [oracle_world(oracle, inputs[j], T, E, use_fp8) for j in range(steps)]
    wants = []
    for j in range(steps):
        ref, xs, idxs, ws, nts = refs[j]
        rows = oracle.cast_back(ref["recv_x"], ref["scales"] if use_fp8 else None, ref["recv_count"], None)
        wants.append(oracle.combine(rows, idxs, ws, ref["src_info"], ref["layout_range"], nts, T, E))
    kw = {"async_finish": mode == "async_finish", "return_recv_hook": mode == "return_recv_hook"}

    def worker(r, group):
        assert group.rank() == r and group.size() == R
        buf = Buffer(group, nbytes)
        # every rank on a stream of its own (rounds then run on the world's stream, fenced against each), or
        # all on one stream (rounds run there)
        stream = torch.cuda.Stream() if own_stream else shared
        with torch.cuda.stream(stream):
            for j in range(steps):
                x, idx, w = (t.to(gpu_device, non_blocking=False) for t in inputs[j][r])
                if r == j % R:
                    time.sleep(0.02)                       # one rank is late: the others wait inside their calls
                recv_x, recv_count, handle, event, hook = buf.dispatch(x, idx, None, T, E, -1, use_fp8=use_fp8, **kw)
                if kw["async_finish"]:
                    event.current_stream_wait()
                if kw["return_recv_hook"]:
                    hook()
                # used at once, on this thread's stream, while other ranks may still be inside their calls
                check_rank_dispatch(refs[j][0], r, recv_x, recv_count, handle, use_fp8)
                if use_fp8:
                    payload, scales = recv_x
                    g = scales.size(-1)
                    expert_out = (payload.float().view(*payload.shape[:2], g, 128) * scales.unsqueeze(-1)) \
                        .view(payload.shape).to(torch.bfloat16)
                else:
                    expert_out = recv_x
                out, event, hook = buf.combine(expert_out, idx, w, None, -1, handle, **kw)
                if kw["async_finish"]:
                    event.current_stream_wait()
                if kw["return_recv_hook"]:
                    hook()
                n = x.size(0)
                assert torch.equal(out.cpu().view(torch.int16), wants[j][r, :n].view(torch.int16)), f"step {j}"
        return r * 10

    assert spawn_ranks(worker, R, join_timeout=100) == [0, 10, 20, 30]


def test_a_rank_that_fails_is_reported_and_its_peers_are_not_left_waiting(gpu_device):
    R, T, H, E, K = 3, 16, 256, 6, 2
    announce("spawn_ranks: one rank raises")
    nbytes = Buffer.get_ep_buffer_size_hint(T, H, R, E)

    def worker(r, group):
        buf = Buffer(group, nbytes)
        if r == 1:
            raise ValueError("rank 1 gives up")
        x, idx, _ = (t.to(gpu_device) for t in rank_inputs(7300 + r, T, H, E, K))
        _, recv_count, _, _, _ = buf.dispatch(x, idx, None, T, E, -1, use_fp8=False)
        return int(recv_count.sum())

    t0 = time.perf_counter()
    with pytest.raises(RuntimeError, match="logical rank 1 failed.*rank 1 gives up"):
        spawn_ranks(worker, R, join_timeout=60, block_timeout_ms=20000)
    # the failed rank was taken out of the collective: the others did not sit out the time limit
    assert time.perf_counter() - t0 < 15.0


def test_a_blocked_call_gives_up_after_the_timeout_and_stays_posted(gpu_device, oracle):
    R, T, H, E, K = 2, 32, 512, 8, 2
    announce("blocking call times out, the round completes later")
    world, groups = LogicalGroup.make_world(R)
    world.set_option("blocking", 1)
    world.set_option("block_timeout_ms", 150)
    nbytes = Buffer.get_ep_buffer_size_hint(T, H, R, E)
    bufs = [Buffer(g, nbytes) for g in groups]
    per_rank = [rank_inputs(7100 + r, T, H, E, K) for r in range(R)]
    dev = [tuple(t.to(gpu_device) for t in per_rank[r]) for r in range(R)]
    outs = [dict(recv_x=torch.empty((E // R, R * T, H), dtype=torch.bfloat16, device=gpu_device),
                 recv_count=torch.empty((E // R,), dtype=torch.int32, device=gpu_device),
                 src_info=torch.empty((E // R, R * T), dtype=torch.int32, device=gpu_device),
                 layout_range=torch.empty((E // R, R), dtype=torch.int64, device=gpu_device)) for _ in range(R)]
    active = torch.ones(R, dtype=torch.int32, device=gpu_device)
    stream = torch.cuda.current_stream().cuda_stream

    def post(r):
        x, idx, _ = dev[r]
        o = outs[r]
        return bufs[r].runtime.dispatch(x.data_ptr(), idx.data_ptr(), active.data_ptr(), T, H, K, T, E, -1, False,
                                        o["recv_x"].data_ptr(), 0, o["recv_count"].data_ptr(),
                                        o["src_info"].data_ptr(), o["layout_range"].data_ptr(), False, False, stream,
                                        (x, idx, o))       # keep_alive: what the Python Buffer hands over

    t0 = time.perf_counter()
    with pytest.raises(ep.PendingError, match="waited 150 ms") as failure:
        post(0)                                            # nobody else is calling
    assert isinstance(failure.value, RuntimeError)         # what the reference's callers catch
    assert 0.1 < time.perf_counter() - t0 < 5.0
    assert bufs[0].runtime.pending_calls() == (1, 0)      # the call stays posted
    assert bufs[0].runtime.retained() == (1, 0)           # ... and so do its tensors, although the call failed
    post(1)                                                # completes the round and returns at once
    torch.cuda.synchronize()
    assert bufs[0].runtime.pending_calls() == (0, 0)
    assert bufs[1].runtime.retained() == (0, 0)
    ref, *_ = oracle_world(oracle, per_rank, T, E, False)
    for r in range(R):
        o = outs[r]
        check_rank_dispatch(ref, r, o["recv_x"], o["recv_count"], (o["src_info"], o["layout_range"]), False)


def test_without_the_option_one_thread_still_drives_all_ranks(gpu_device, oracle):
    """The default stays what it was: calls return at once, and the last rank's call launches the round."""
    R, T, H, E, K = 2, 32, 512, 8, 2
    announce("non-blocking default")
    world, groups = LogicalGroup.make_world(R)
    assert world.get_option("blocking") == 0
    nbytes = Buffer.get_ep_buffer_size_hint(T, H, R, E)
    bufs = [Buffer(g, nbytes) for g in groups]
    per_rank = [rank_inputs(7200 + r, T, H, E, K) for r in range(R)]
    t0 = time.perf_counter()
    res = [bufs[r].dispatch(per_rank[r][0].to(gpu_device), per_rank[r][1].to(gpu_device), None, T, E, -1, use_fp8=False)
           for r in range(R)]
    assert time.perf_counter() - t0 < 5.0
    torch.cuda.synchronize()
    ref, *_ = oracle_world(oracle, per_rank, T, E, False)
    for r in range(R):
        check_rank_dispatch(ref, r, res[r][0], res[r][1], res[r][2], False)


@pytest.mark.parametrize("use_fp8", [False, True], ids=["bf16", "fp8"])
@pytest.mark.parametrize("mode", ["default", "async_finish", "return_recv_hook"])
def test_reference_grid_worker_on_threads_with_a_rank_that_dies(gpu_device, use_fp8, mode):
    """The reference's per-rank worker (mooncake-ep/tests/test_ep_grid.py:60-119, :160-173): dispatch, mock expert,
    combine, closed form; two steps, and rank 1 stops calling after the first (the reference's os._exit(0),
    :121-158, forced here from the host), so the survivors' second step runs without it."""
    from tests.test_gpu_buffer_api import dequantize_fp8, grid_inputs
    R, max_tokens, hidden, num_experts, top_k, fail_rank = 4, 64, 1024, 32, 4, 1
    announce(f"grid worker on threads, fp8={use_fp8}, {mode}")
    L = num_experts // R
    nbytes = Buffer.get_ep_buffer_size_hint(max_tokens, hidden, R, num_experts)
    kw = {"async_finish": mode == "async_finish", "return_recv_hook": mode == "return_recv_hook"}

    def worker(rank, group):
        buf = Buffer(group, nbytes)
        x, idx, w = grid_inputs(rank, R, max_tokens, hidden, num_experts, top_k, gpu_device)
        active = torch.ones(R, dtype=torch.int32, device=gpu_device)
        for step in range(2):
            if step == 1 and rank == fail_rank:
                group.world.set_rank_silent(rank)          # this rank's process is gone
                return "dead"
            timeout_us = 5000 if step == 1 else -1
            recv_x, recv_count, handle, event, hook = buf.dispatch(x, idx, active, max_tokens, num_experts, timeout_us,
                                                                   use_fp8=use_fp8, **kw)
            if kw["return_recv_hook"]:
                hook()
            if kw["async_finish"]:
                event.current_stream_wait()
            recv_bf16 = dequantize_fp8(*recv_x) if use_fp8 else recv_x
            factor = (torch.arange(rank * L, (rank + 1) * L, device=gpu_device).float() * 0.1 + 1.0).view(L, 1, 1)
            expert_out = (recv_bf16.float() * factor).to(torch.bfloat16).contiguous()
            out, event, hook = buf.combine(expert_out, idx, w, active, timeout_us, handle, out=torch.zeros_like(x), **kw)
            if kw["return_recv_hook"]:
                hook()
            if kw["async_finish"]:
                event.current_stream_wait()
            factors = idx.float() * 0.1 + 1.0
            if step == 1:
                assert active[fail_rank].item() == 0 and active.sum().item() == R - 1
                factors = factors * (idx // L != fail_rank).float()
            else:
                assert active.sum().item() == R
            expected = (x.float() * (factors * w).sum(dim=1, keepdim=True)).to(torch.bfloat16)
            assert not torch.isnan(out.float()).any()
            torch.testing.assert_close(out, expected, rtol=0.15 if use_fp8 else 5e-2, atol=5e-3 if use_fp8 else 1e-3)
        return "alive"

    assert spawn_ranks(worker, R, join_timeout=100) == ["alive", "dead", "alive", "alive"]
