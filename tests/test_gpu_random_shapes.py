"""Seeded random worlds: odd rank / expert / top-k / hidden sizes, ragged token
counts (some zero), masked tokens, ranks that take no part, per-rank views of
inactive ranks.  Every case runs dispatch -> cast back -> combine through the C
ABI and is compared with the oracle bit for bit; the packed combine then has to
give the same bits from dispatch's output."""
import os
import random

import pytest
import torch

from mooncake_amd.harness import WorldHarness
from mooncake_amd.workloads import EPConfig, generate
from tests.gpu_util import announce, compare_dispatch

pytestmark = pytest.mark.gpu


def _case(seed: int):
    rng = random.Random(seed)
    R = rng.choice([1, 2, 3, 5, 8, 12])
    L = rng.choice([1, 2, 3, 5, 9, 24])
    E = R * L
    K = rng.randint(1, min(E, 16))
    H = rng.choice([128, 256, 1152, 2048, 4096, 7168])
    use_fp8 = rng.random() < 0.5
    T = rng.randint(1, 70)
    if use_fp8:
        while (R * T) % 4:          # the reference's alignment requirement on the scale layout
            T += 1
    cfg = EPConfig(f"random{seed}", R, T, H, E, K, use_fp8, routing=rng.choice(["uniform", "zipf"]),
                   masked_fraction=rng.choice([0.0, 0.0, 0.15, 0.5]))
    num_tokens = [rng.choice([T, T, rng.randint(0, T), 0 if rng.random() < 0.15 else T]) for _ in range(R)]
    present = [0 if (R > 1 and rng.random() < 0.12) else 1 for _ in range(R)]
    if not any(present):
        present[0] = 1
    active = torch.ones((R, R), dtype=torch.int32)
    for _ in range(rng.randint(0, 2)):
        active[rng.randrange(R), rng.randrange(R)] = 0
    direct = rng.choice([0, 1])
    summed = rng.choice([0, 1])      # both routing plans (prefix pass as its own launch, or inside pack)
    return cfg, num_tokens, present, active, direct, summed


# more seeds for a longer sweep: MC_EP_RANDOM_WORLDS=300 python -m pytest tests/test_gpu_random_shapes.py -m gpu
@pytest.mark.parametrize("seed", range(int(os.environ.get("MC_EP_RANDOM_WORLDS", "32"))))
def test_random_world(gpu_device, oracle, seed):
    cfg, num_tokens, present, active, direct, summed = _case(seed)
    announce(f"random world seed={seed} {cfg} tokens={num_tokens} present={present} direct={direct} summed={summed}")
    data = generate(cfg, seed=1000 + seed)
    h = WorldHarness(cfg, num_tokens=num_tokens)
    h.world.set_option("combine_direct", direct)
    h.world.set_option("routing_sum", summed)
    h.load(data)
    h.alloc_dispatch_outputs(poison=True)
    h.alloc_combine_io()
    h.expert_out.fill_(float("nan"))
    h.combined.fill_(7.0)
    h.active_ranks.copy_(active)
    factor = torch.arange(cfg.num_experts, dtype=torch.float32) * 0.1 + 1.0
    h.dispatch(present=present)
    h.cast_back(factor, present=present)
    h.combine(present=present)
    torch.cuda.synchronize()

    sent = [n if present[r] else 0 for r, n in enumerate(num_tokens)]
    ref = oracle.dispatch(data["x"], data["topk_idx"], sent, cfg.max_tokens, cfg.num_experts, cfg.use_fp8,
                          src_present=present)
    # a rank that takes no part receives nothing either: its outputs keep their poison
    for r in range(cfg.num_ranks):
        if present[r]:
            continue
        assert bool((h.recv_count[r] == -7).all()) and bool((h.src_info[r] == -7).all())
        h.recv_count[r] = 0
        ref["recv_count"][r] = 0
        ref["layout_range"][r] = -7
        ref["src_info"][r] = -7
    compare_dispatch(h, ref, check_poison=True)

    rows = oracle.cast_back(ref["recv_x"], ref["scales"] if cfg.use_fp8 else None, ref["recv_count"], factor)
    # ... and contributes nothing to combine, which is what every rank seeing it as inactive amounts to
    seen = active.clone()
    seen[:, [r for r in range(cfg.num_ranks) if not present[r]]] = 0
    full = oracle.dispatch(data["x"], data["topk_idx"], sent, cfg.max_tokens, cfg.num_experts, cfg.use_fp8,
                           src_present=present)
    want = oracle.combine(rows, data["topk_idx"], data["topk_weights"], full["src_info"], full["layout_range"], sent,
                          cfg.max_tokens, cfg.num_experts, active=seen)
    got = h.combined.cpu()
    for r, n in enumerate(sent):
        assert torch.equal(got[r, :n].view(torch.int16), want[r, :n].view(torch.int16)), f"rank {r}"
        assert bool((got[r, n:] == 7.0).all()), f"rank {r}: rows beyond its tokens written"
    # the combine fused with the consumer gives the same bits from dispatch's packed output
    h.combined.fill_(7.0)
    h.combine_packed(factor, present=present)
    torch.cuda.synchronize()
    fused = h.combined.cpu()
    assert torch.equal(fused.view(torch.int16), got.view(torch.int16)), "packed combine differs from cast back + combine"
