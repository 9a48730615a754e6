"""The allocation-free dispatch (`mc_ep_world_dispatch_noalloc`, scratch in a
static device array) against `mc_ep_world_dispatch`, through the C ABI: every
output tensor bit for bit, padding included (both start from the same poison),
on two calls in a row of one world, the second on a smaller input - so whatever
the first call left in the shared static scratch must not leak into the second.
Each dispatch is followed by a combine of the handle it produced (the ordinary
one reuses its dispatch's routing state, the allocation-free one resolves the
handle), and the two results must be equal as well.  Then the property the entry point exists for - the
driver's free device memory is the same before and after a call of a shape its world has never seen - and a
recorded call replayed with eager calls of another shape in between, which overwrite the shared array."""
import pytest
import torch

from mooncake_amd import _lib, ep
from mooncake_amd.harness import WorldHarness
from mooncake_amd.workloads import CONFIGS, EPConfig, generate
from tests.gpu_util import announce, compare_dispatch

pytestmark = pytest.mark.gpu


def _run(cfg, world, data, num_tokens, noalloc):
    h = WorldHarness(cfg, world=world, num_tokens=num_tokens)
    h.load(data)
    h.alloc_dispatch_outputs(poison=True)
    h.dispatch(noalloc=noalloc)
    h.alloc_combine_io()
    h.cast_back()
    h.combined.fill_(float("nan"))
    h.combine()
    torch.cuda.synchronize()
    return h


def _compare(cfg, world, data, num_tokens=None):
    a = _run(cfg, world, data, num_tokens, noalloc=False)
    b = _run(cfg, world, data, num_tokens, noalloc=True)
    assert torch.equal(a.recv_count, b.recv_count), "recv_count"
    assert torch.equal(a.layout_range, b.layout_range), "layout_range"
    assert torch.equal(a.src_info, b.src_info), "src_info"
    assert torch.equal(a.recv_x, b.recv_x), "payload"
    if cfg.use_fp8:
        # the poison is NaN: compare bit patterns
        assert torch.equal(a.recv_scales_phys.view(torch.int32), b.recv_scales_phys.view(torch.int32)), "scales"
    selections = sum(int((data["topk_idx"][r, :n] >= 0).sum()) for r, n in enumerate(a.num_tokens))
    assert int(b.recv_count.sum()) == selections
    assert torch.equal(a.combined.view(torch.int16), b.combined.view(torch.int16)), "combine of the handle"
    for r, n in enumerate(b.num_tokens):
        assert not bool(torch.isnan(b.combined[r, :n]).any())


@pytest.mark.parametrize("use_fp8", [True, False], ids=["fp8", "bf16"])
def test_noalloc_dispatch_matches_dispatch_twice_in_a_row(gpu_device, use_fp8):
    big = CONFIGS["dsv3_decode"] if use_fp8 else EPConfig("dsv3_decode_bf16", 32, 128, 7168, 256, 8, False)
    announce(f"noalloc dispatch, first call {big}")
    world = ep.World(big.num_ranks)
    _compare(big, world, generate(big, seed=3))
    torch.cuda.empty_cache()
    # the same world again, on a smaller and ragged input with masked tokens
    small = EPConfig("small_after_big", 32, 24, 1024, 64, 4, use_fp8, masked_fraction=0.2)
    nt = [(5 * r) % 25 for r in range(small.num_ranks)]
    announce(f"noalloc dispatch, second call {small} tokens {nt}")
    _compare(small, world, generate(small, seed=4), num_tokens=nt)
    torch.cuda.empty_cache()


@pytest.mark.parametrize("cfg", [EPConfig("never_seen_small", 4, 40, 2048, 32, 6, True),       # one launch
                                 EPConfig("never_seen_large", 16, 96, 2048, 64, 8, True)],    # count, pack, scales
                         ids=lambda c: c.name)
def test_noalloc_dispatch_leaves_device_memory_as_it_was(gpu_device, oracle, cfg):
    """What the entry point is for: a shape its world has never seen costs no device allocation - the free memory
    the driver reports is the same before and after the call."""
    announce(f"noalloc dispatch allocates nothing {cfg}")
    warm = EPConfig("warm", 2, 8, 256, 4, 2, True)          # loads the library's kernels through another world
    hw = WorldHarness(warm)
    hw.load(generate(warm, seed=1))
    hw.alloc_dispatch_outputs()
    hw.dispatch(noalloc=True)
    hw.world.set_option("fused_small", 0)
    hw.dispatch(noalloc=True)
    torch.cuda.synchronize()
    data = generate(cfg, seed=5)
    h = WorldHarness(cfg)                                   # a fresh world: nothing of this shape has been sized
    h.load(data)
    h.alloc_dispatch_outputs(poison=True)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    h.dispatch(noalloc=True)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before
    ref = oracle.dispatch(data["x"], data["topk_idx"], h.num_tokens, cfg.max_tokens, cfg.num_experts, True)
    compare_dispatch(h, ref, check_poison=True)


@pytest.mark.parametrize("fused_small", [1, 0], ids=["one_launch", "three_launch"])
def test_noalloc_dispatch_in_a_graph_with_other_noalloc_calls_between_replays(gpu_device, oracle, fused_small):
    """A recorded allocation-free dispatch keeps its rank table and scratch in the array every such call on the
    GPU shares.  An eager call of another shape between two replays overwrites all of it; the replay must not
    care (its table travels in the recorded kernels' arguments, its scratch is rewritten before it is read)."""
    cfg = EPConfig("noalloc_graph", 4, 48, 1024, 16, 4, True, masked_fraction=0.2)
    other_cfg = EPConfig("noalloc_other", 8, 64, 2048, 64, 8, False)
    announce(f"noalloc dispatch in a graph {cfg} fused_small={fused_small}, eager {other_cfg} between replays")
    world = ep.World(cfg.num_ranks)
    world.set_option("fused_small", fused_small)
    h = WorldHarness(cfg, world=world)
    h.load(generate(cfg, seed=60))
    h.alloc_dispatch_outputs(poison=False)
    other = WorldHarness(other_cfg)
    other.world.set_option("fused_small", 0)
    other.load(generate(other_cfg, seed=61))
    other.alloc_dispatch_outputs(poison=False)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        h.dispatch(noalloc=True)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        h.dispatch(noalloc=True)
    nt = [cfg.tokens_per_rank] * cfg.num_ranks
    for seed in (62, 63, 64):
        data = generate(cfg, seed=seed)
        h.x.copy_(data["x"])
        h.topk_idx.copy_(data["topk_idx"])
        h.recv_count.fill_(-1)
        other.dispatch(noalloc=True)                        # another shape, another world, the same static array
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        ref = oracle.dispatch(data["x"], data["topk_idx"], nt, cfg.max_tokens, cfg.num_experts, True)
        compare_dispatch(h, ref, check_poison=False)
    # and the eager call's own result, after a replay rewrote the array under it
    other.dispatch(noalloc=True)
    torch.cuda.synchronize()
    data = generate(other_cfg, seed=61)
    ref = oracle.dispatch(data["x"], data["topk_idx"], [other_cfg.tokens_per_rank] * other_cfg.num_ranks,
                          other_cfg.max_tokens, other_cfg.num_experts, False)
    compare_dispatch(other, ref, check_poison=False)


def test_noalloc_dispatch_rejects_what_does_not_fit(gpu_device):
    # 8 ranks x 4096 tokens, 256 experts: row_src alone is 32 MiB.  The check is on the host; nothing is launched.
    announce("noalloc dispatch, shape beyond the static scratch")
    world = ep.World(8)
    ptrs = [256] * 8
    with pytest.raises(RuntimeError, match="allocation-free dispatch holds 16777216"):
        world.dispatch_noalloc(ptrs, ptrs, [1] * 8, 7168, 8, 4096, 256, False, ptrs, None, ptrs, ptrs, ptrs, 0)
    assert _lib.last_error().startswith("Failed: this shape needs ")
