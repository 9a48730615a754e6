"""The allocation-free dispatch (`mc_ep_world_dispatch_noalloc`, scratch in a
static device array) against `mc_ep_world_dispatch`, through the C ABI: every
output tensor bit for bit, padding included (both start from the same poison),
on two calls in a row of one world, the second on a smaller input - so whatever
the first call left in the shared static scratch must not leak into the second.
Each dispatch is followed by a combine of the handle it produced (the ordinary
one reuses its dispatch's routing state, the allocation-free one resolves the
handle), and the two results must be equal as well."""
import pytest
import torch

from mooncake_amd import _lib, ep
from mooncake_amd.harness import WorldHarness
from mooncake_amd.workloads import CONFIGS, EPConfig, generate
from tests.gpu_util import announce

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


def test_noalloc_dispatch_rejects_what_does_not_fit(gpu_device):
    # 8 ranks x 4096 tokens, 256 experts: row_src alone is 32 MiB.  The check is on the host; nothing is launched.
    announce("noalloc dispatch, shape beyond the static scratch")
    world = ep.World(8)
    ptrs = [256] * 8
    with pytest.raises(RuntimeError, match="allocation-free dispatch holds 16777216"):
        world.dispatch_noalloc(ptrs, ptrs, [1] * 8, 7168, 8, 4096, 256, False, ptrs, None, ptrs, ptrs, ptrs, 0)
    assert _lib.last_error().startswith("Failed: this shape needs ")
