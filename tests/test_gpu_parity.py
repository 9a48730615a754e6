"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle
on the same seeded inputs.  Bit-exact for counts, ranges, source indices, fp8
payload and scales, bf16 payload; combine bit-exact against the oracle's fused
fp32 chain and within one bf16 ulp of a float64 sum."""
import pytest
import torch

from mooncake_amd.workloads import CONFIGS, EPConfig, generate, shrink
from tests import ref_checks as rc
from tests.gpu_util import announce, compare_dispatch, run_dispatch

pytestmark = pytest.mark.gpu

SMALL = [
    EPConfig("tiny_bf16", 2, 4, 128, 4, 2, False),
    EPConfig("tiny_fp8", 2, 4, 128, 4, 2, True),
    EPConfig("odd_hidden_fp8", 4, 24, 2560, 16, 3, True),            # 2.5 slabs of 1024
    EPConfig("odd_hidden_bf16", 4, 24, 2560, 16, 3, False),
    # the hidden sizes the reference instantiates its kernels for (SWITCH_HIDDEN, mooncake_ep_launch.cuh:66-87)
    # beyond the ones other cases use: 1024-element pack slabs and 512-element combine slabs with and without a tail
    EPConfig("h3072_fp8", 4, 20, 3072, 16, 4, True),
    EPConfig("h3072_bf16", 4, 20, 3072, 16, 4, False),
    EPConfig("h5120_fp8", 4, 20, 5120, 32, 6, True),
    EPConfig("h5120_bf16", 4, 20, 5120, 32, 6, False),
    EPConfig("h6144_fp8", 2, 36, 6144, 16, 8, True),
    EPConfig("h6144_bf16", 2, 36, 6144, 16, 8, False),
    EPConfig("h8192_fp8", 4, 24, 8192, 32, 8, True),
    EPConfig("h8192_bf16", 4, 24, 8192, 32, 8, False),
    EPConfig("h4096_fp8", 4, 24, 4096, 32, 8, True),
    EPConfig("h7168_bf16", 4, 24, 7168, 32, 8, False),
    EPConfig("k11", 4, 40, 2048, 32, 11, True),                      # the reference's top-k cap
    EPConfig("k16_bf16", 2, 20, 1024, 32, 16, False),
    EPConfig("one_rank", 1, 36, 1024, 6, 2, True),                   # group_size == 1
    EPConfig("masked", 8, 64, 1024, 8, 2, False, masked_fraction=0.3),
    EPConfig("zipf_outliers", 8, 32, 2048, 64, 8, True, routing="zipf", outlier_fraction=0.05),
    shrink(CONFIGS["cpu_check"]),                                    # the contract's CPU-reference case, full size
    # shapes at the edges of the routing plans: the count kernel's LDS beyond the default 48 KB (summed plan),
    # too many experts for 1024-selection units' LDS, too many units to sum (both: table plan)
    EPConfig("experts768", 8, 16, 256, 768, 8, True),
    EPConfig("experts1024", 8, 16, 256, 1024, 8, False),
    EPConfig("units80", 16, 600, 256, 32, 8, False),
    # more ranks than one table-writer launch carries (384 words): the rank table goes up in pieces
    EPConfig("ranks64", 64, 4, 128, 64, 2, True),
    EPConfig("ranks100", 100, 3, 128, 100, 3, False),
]


def ragged(cfg, on):
    if not on:
        return None
    return [max(0, cfg.tokens_per_rank - (r * 5) % (cfg.tokens_per_rank + 1)) for r in range(cfg.num_ranks)]


@pytest.mark.parametrize("cfg", SMALL, ids=[c.name for c in SMALL])
@pytest.mark.parametrize("is_ragged", [False, True], ids=["full", "ragged"])
def test_dispatch_matches_oracle(gpu_device, oracle, cfg, is_ragged, fused_small):
    nt = ragged(cfg, is_ragged)
    announce(f"dispatch {cfg} ragged={nt} fused_small={fused_small}")
    data = generate(cfg, seed=0)
    h = run_dispatch(cfg, data, num_tokens=nt, poison=True)
    ref = oracle.dispatch(data["x"], data["topk_idx"], h.num_tokens, cfg.max_tokens, cfg.num_experts, cfg.use_fp8)
    compare_dispatch(h, ref, check_poison=True)


@pytest.mark.parametrize("nt", [0, 1, 2, 3])
@pytest.mark.parametrize("uniform", [0, 1])
@pytest.mark.parametrize("arith", [0, 1], ids=["torch_arith", "kernel_arith"])
def test_fp8_pack_variants_match_oracle(gpu_device, oracle, nt, uniform, arith, fused_small):
    """Every tuning variant of the pack path is the same function; the scale arithmetic follows either of the
    reference's two statements of it."""
    cfg = EPConfig("variants", 4, 24, 2560, 16, 3, True)
    announce(f"pack nt={nt} uniform={uniform} fp8_arith={arith}")
    data = generate(cfg, seed=1)
    h = run_dispatch(cfg, data, poison=True, options={"pack_nt": nt, "uniform": uniform, "fp8_arith": arith})
    oracle.set_fp8_arith(arith)
    try:
        ref = oracle.dispatch(data["x"], data["topk_idx"], h.num_tokens, cfg.max_tokens, cfg.num_experts, True)
    finally:
        oracle.set_fp8_arith(0)
    compare_dispatch(h, ref, check_poison=True)


@pytest.mark.parametrize("opts", [{"uniform": 0}, {"pack_waves": 1}, {"pack_waves": 8}, {"pack_nt": 1}, {"pack_nt": 0}, {"pack_nt": 2}, {"pack_nt": 3},
                                  {"routing_sum": 0}, {"routing_sum": 0, "uniform": 0}],
                         ids=lambda o: "-".join(f"{k}{v}" for k, v in o.items()))
def test_dispatch_tuning_options_match_oracle(gpu_device, oracle, opts):
    cfg = EPConfig("opts", 8, 32, 2048, 64, 8, True, routing="zipf", outlier_fraction=0.05)
    announce(f"dispatch options {opts}")
    data = generate(cfg, seed=2)
    nt = ragged(cfg, True)
    # (these are options of the count / pack / scale-transpose launches: the one-launch dispatch is switched off)
    h = run_dispatch(cfg, data, num_tokens=nt, poison=True, options={"fused_small": 0, **opts})
    ref = oracle.dispatch(data["x"], data["topk_idx"], h.num_tokens, cfg.max_tokens, cfg.num_experts, True)
    compare_dispatch(h, ref, check_poison=True)


@pytest.mark.parametrize("arith", [0, 1], ids=["torch_arith", "kernel_arith"])
def test_fp8_every_bf16_value(gpu_device, oracle, arith, fused_small):
    """All finite bf16 bit patterns through the quantiser, in shuffled groups
    (mixed magnitudes) and in sorted groups (tiny amax, subnormal payloads)."""
    bits = torch.arange(0, 65536, dtype=torch.int32)
    vals = (bits << 16).view(torch.float32)
    vals = vals[torch.isfinite(vals)]
    g = torch.Generator().manual_seed(11)
    H = 1024
    pad = (-vals.numel()) % H
    shuffled = torch.cat([vals[torch.randperm(vals.numel(), generator=g)], torch.zeros(pad)])
    ordered = torch.cat([vals.sort().values, torch.zeros(pad)])
    rows = torch.cat([shuffled, ordered]).view(-1, H).to(torch.bfloat16)       # 128 rows
    T = rows.size(0)
    cfg = EPConfig("all_bf16", 1, T, H, 2, 1, True)
    announce(f"every bf16 value: {T} rows of {H}")
    data = {"x": rows.unsqueeze(0).contiguous(),
            "topk_idx": (torch.arange(T) % 2).view(1, T, 1).to(torch.int64),
            "topk_weights": torch.ones(1, T, 1)}
    h = run_dispatch(cfg, data, poison=True, options={"fp8_arith": arith})
    oracle.set_fp8_arith(arith)
    try:
        ref = oracle.dispatch(data["x"], data["topk_idx"], [T], T, 2, True)
    finally:
        oracle.set_fp8_arith(0)
    compare_dispatch(h, ref, check_poison=True)
    if arith == 1:
        return
    # and against the reference's formula executed by torch
    q_ref, s_ref = rc.reference_fp8_cast(rows)
    got = h.recv_x.cpu()[0]                                                    # [2, T, H]
    si = h.src_info.cpu()[0]
    for e in range(2):
        n = int(h.recv_count[0, e])
        assert torch.equal(got[e, :n], q_ref.view(torch.uint8)[si[e, :n].long()])
        assert torch.equal(h.recv_scales()[0, e, :n].cpu().contiguous().view(torch.int32),
                           s_ref[si[e, :n].long()].contiguous().view(torch.int32))


def test_fp8_inf_and_nan_inputs(gpu_device, oracle, fused_small):
    H, T = 1024, 8
    g = torch.Generator().manual_seed(2)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    x[1, 5] = float("inf")
    x[2, 700] = float("-inf")
    x[3, 130] = float("nan")
    cfg = EPConfig("nonfinite", 1, T, H, 1, 1, True)
    announce("fp8 inf / nan inputs")
    data = {"x": x.unsqueeze(0).contiguous(), "topk_idx": torch.zeros(1, T, 1, dtype=torch.int64),
            "topk_weights": torch.ones(1, T, 1)}
    h = run_dispatch(cfg, data, poison=True)
    ref = oracle.dispatch(data["x"], data["topk_idx"], [T], T, 1, True)
    got, want = h.recv_x.cpu()[0, 0, :T], ref["recv_x"].view(torch.uint8)[0, 0, :T]
    # NaN payload bytes: both must be a NaN encoding (0x7F / 0xFF); everything else bit-exact
    nan_w = (want & 0x7F) == 0x7F
    assert torch.equal((got & 0x7F) == 0x7F, nan_w)
    assert torch.equal(got[~nan_w], want[~nan_w])
    assert torch.equal(h.recv_scales()[0, 0, :T].cpu().contiguous().view(torch.int32),
                       ref["scales"][0, 0, :T].contiguous().view(torch.int32))


def test_duplicate_experts_follow_the_oracle(gpu_device, oracle, fused_small):
    """Out of contract, but defined: one row per (token, k) occurrence; rows that
    would overflow a block's capacity are dropped."""
    cfg = EPConfig("dups", 2, 16, 1024, 4, 4, True)
    announce("dispatch with repeated experts in a token")
    data = generate(cfg, seed=6)
    data["topk_idx"][:, ::3, 1] = data["topk_idx"][:, ::3, 0]          # k=1 repeats k=0 on every third token
    data["topk_idx"][0, :, :] = 1                                      # rank 0: every token names expert 1 four times
    h = run_dispatch(cfg, data, poison=True)
    ref = oracle.dispatch(data["x"], data["topk_idx"], h.num_tokens, cfg.max_tokens, cfg.num_experts, True)
    assert int(ref["recv_count"].max()) == cfg.num_ranks * cfg.max_tokens   # the overflow case is exercised
    compare_dispatch(h, ref, check_poison=True)


COMBINE_CASES = [
    EPConfig("tiny_c", 2, 4, 128, 4, 2, False),
    EPConfig("odd_hidden_c", 4, 24, 2560, 16, 3, False),
    EPConfig("h3072_c", 4, 20, 3072, 16, 4, False),
    EPConfig("h5120_c", 4, 20, 5120, 32, 6, True),
    EPConfig("h6144_c", 2, 36, 6144, 16, 8, False),
    EPConfig("h8192_c", 4, 24, 8192, 32, 8, True),
    EPConfig("k11_c", 4, 40, 2048, 32, 11, False),
    EPConfig("k16_c", 2, 20, 1024, 32, 16, False),
    EPConfig("masked_c", 8, 64, 1024, 8, 2, False, masked_fraction=0.3),
    EPConfig("fp8_c", 8, 32, 2048, 64, 8, True, routing="zipf", outlier_fraction=0.05),
    EPConfig("ranks64_c", 64, 4, 128, 64, 2, True),                  # rank table in two pieces
    shrink(CONFIGS["cpu_check"]),
]


@pytest.mark.parametrize("cfg", COMBINE_CASES, ids=[c.name for c in COMBINE_CASES])
@pytest.mark.parametrize("is_ragged", [False, True], ids=["full", "ragged"])
@pytest.mark.parametrize("chunks,cnt,direct", [(1, 3, 1), (2, 3, 1), (1, 0, 1), (1, 3, 0), (2, 0, 0)])
def test_combine_matches_oracle(gpu_device, oracle, cfg, is_ragged, chunks, cnt, direct, fused_small):
    """direct=1: the handle is the last dispatch's, rows come from its routing
    state; direct=0: the general path that re-derives rows from the handle."""
    nt = ragged(cfg, is_ragged)
    announce(f"combine {cfg} ragged={nt} chunks={chunks} nt={cnt} direct={direct} fused_small={fused_small}")
    data = generate(cfg, seed=3)
    h = run_dispatch(cfg, data, num_tokens=nt, poison=False,
                     options={"combine_chunks": chunks, "combine_nt": cnt, "combine_direct": direct})
    factor = torch.arange(cfg.num_experts).float() * 0.1 + 1.0
    h.alloc_combine_io()
    h.expert_out.fill_(float("nan"))                       # rows outside the handle must never be read
    h.fill_expert_out_from_recv(factor)
    # keep NaN in every padding row
    RM = cfg.num_ranks * cfg.max_tokens
    pad = torch.arange(RM, device=h.recv_count.device).view(1, 1, RM) >= h.recv_count.unsqueeze(-1)
    h.expert_out[pad] = float("nan")
    h.combined.fill_(7.0)
    h.combine()
    torch.cuda.synchronize()
    eo = h.expert_out.cpu()
    ref_d = oracle.dispatch(data["x"], data["topk_idx"], h.num_tokens, cfg.max_tokens, cfg.num_experts, cfg.use_fp8)
    want = oracle.combine(eo, data["topk_idx"], data["topk_weights"], ref_d["src_info"], ref_d["layout_range"],
                          h.num_tokens, cfg.max_tokens, cfg.num_experts, use_fma=True)
    got = h.combined.cpu()
    exact = rc.combine_fp64(torch.nan_to_num(eo.float()).to(torch.bfloat16), data["topk_idx"], data["topk_weights"],
                            ref_d["slot_map"], h.num_tokens, cfg.max_tokens, cfg.num_experts)
    for r, n in enumerate(h.num_tokens):
        assert torch.equal(got[r, :n].view(torch.int16), want[r, :n].view(torch.int16)), f"rank {r}"
        assert bool(rc.within_one_ulp_of(got[r, :n], exact[r, :n]).all()), f"rank {r} vs float64"
        assert bool((got[r, n:] == 7.0).all()), "rows beyond num_tokens written"


@pytest.mark.parametrize("waves,occupancy", [(4, 0), (4, 20), (4, 8), (1, 20), (8, 20), (8, 4), (3, 200)])
def test_combine_launch_shapes_match_oracle(gpu_device, oracle, waves, occupancy):
    """Waves per block and the cap on waves per CU (imposed with unused dynamic LDS; by default 20 from top-7 up)
    change how the combine kernel is launched, not what it computes."""
    cfg = EPConfig("launch_shapes", 8, 48, 3072, 64, 8, False, masked_fraction=0.1)
    announce(f"combine with combine_waves={waves} combine_occupancy={occupancy}")
    data = generate(cfg, seed=6)
    h = run_dispatch(cfg, data, poison=False, options={"combine_waves": waves, "combine_occupancy": occupancy})
    h.alloc_combine_io()
    h.fill_expert_out_from_recv(torch.arange(cfg.num_experts).float() * 0.1 + 1.0)
    h.combined.fill_(7.0)
    h.combine()
    torch.cuda.synchronize()
    ref_d = oracle.dispatch(data["x"], data["topk_idx"], h.num_tokens, cfg.max_tokens, cfg.num_experts, False)
    want = oracle.combine(h.expert_out.cpu(), data["topk_idx"], data["topk_weights"], ref_d["src_info"],
                          ref_d["layout_range"], h.num_tokens, cfg.max_tokens, cfg.num_experts, use_fma=True)
    assert torch.equal(h.combined.cpu().view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("direct", [1, 0])
def test_combine_skips_inactive_ranks(gpu_device, oracle, direct, fused_small):
    cfg = EPConfig("inactive", 4, 16, 1024, 16, 4, False)
    announce(f"combine with an inactive rank direct={direct}")
    data = generate(cfg, seed=4)
    h = run_dispatch(cfg, data, poison=False, options={"combine_direct": direct})
    h.alloc_combine_io()
    h.fill_expert_out_from_recv(torch.arange(16).float() * 0.1 + 1.0)
    h.active_ranks[:, 2] = 0
    h.active_ranks[3, 1] = 0                              # views differ per rank
    h.combine()
    torch.cuda.synchronize()
    want = oracle.combine(h.expert_out.cpu(), data["topk_idx"], data["topk_weights"], h.src_info.cpu(),
                          h.layout_range.cpu(), h.num_tokens, cfg.max_tokens, cfg.num_experts,
                          active=h.active_ranks.cpu())
    assert torch.equal(h.combined.cpu().view(torch.int16), want.view(torch.int16))


def test_combine_with_an_older_handle(gpu_device, oracle):
    """dispatch A, dispatch B into other buffers, then combine A: the routing
    state on the device is B's, so A's rows must be re-derived from A's handle."""
    from mooncake_amd.harness import WorldHarness
    cfg = EPConfig("older", 4, 24, 1024, 16, 4, False)
    announce("combine with the handle of an older dispatch")
    a = run_dispatch(cfg, generate(cfg, seed=7), poison=False)
    b = WorldHarness(cfg, world=a.world)
    b.load(generate(cfg, seed=8))
    b.alloc_dispatch_outputs()
    b.dispatch()
    torch.cuda.synchronize()
    for h, seed in ((a, 7), (b, 8)):
        data = generate(cfg, seed=seed)
        h.alloc_combine_io()
        h.fill_expert_out_from_recv(torch.arange(16).float() * 0.1 + 1.0)
        h.combine()
        torch.cuda.synchronize()
        want = oracle.combine(h.expert_out.cpu(), data["topk_idx"], data["topk_weights"], h.src_info.cpu(),
                              h.layout_range.cpu(), h.num_tokens, cfg.max_tokens, cfg.num_experts)
        # rows outside the handle hold garbage in expert_out; the oracle never reads them either
        assert torch.equal(h.combined.cpu().view(torch.int16), want.view(torch.int16))


def test_dispatch_with_silent_rank(gpu_device, oracle, fused_small):
    cfg = EPConfig("silent", 4, 16, 1024, 16, 4, True)
    announce("dispatch with a silent rank")
    data = generate(cfg, seed=5)
    present = [1, 1, 0, 1]
    h = run_dispatch(cfg, data, poison=True, present=present)
    ref = oracle.dispatch(data["x"], data["topk_idx"], h.num_tokens, cfg.max_tokens, cfg.num_experts, True,
                          src_present=present)
    # the silent rank's own outputs are never written
    assert bool((h.recv_count[2] == -7).all()) and bool((h.src_info[2] == -7).all())
    for k in ("recv_count", "layout_range", "src_info"):
        ref[k][2] = -7
    h.recv_count[2] = 0
    ref["recv_count"][2] = 0
    compare_dispatch(h, ref, check_poison=False)


@pytest.mark.parametrize("direct", [1, 0])
def test_ids_outside_the_expert_range_name_no_expert(gpu_device, oracle, direct, fused_small):
    """The reference asserts nothing about top-k ids; here anything outside [0, E) is treated like -1 by every
    kernel (and by the oracle), instead of indexing out of bounds."""
    cfg = EPConfig("stray_ids", 4, 24, 512, 8, 4, True)
    announce(f"stray expert ids direct={direct}")
    data = generate(cfg, seed=9)
    idx = data["topk_idx"]
    gen = torch.Generator().manual_seed(1)
    stray = torch.rand(idx.shape, generator=gen)
    idx[stray < 0.1] = cfg.num_experts + 3
    idx[(stray >= 0.1) & (stray < 0.2)] = -5
    idx[(stray >= 0.2) & (stray < 0.25)] = 2 ** 40
    clean = idx.clone()
    clean[(idx < 0) | (idx >= cfg.num_experts)] = -1
    h = run_dispatch(cfg, data, poison=True, options={"combine_direct": direct})
    nt = [cfg.tokens_per_rank] * cfg.num_ranks
    ref = oracle.dispatch(data["x"], idx, nt, cfg.max_tokens, cfg.num_experts, True)
    same = oracle.dispatch(data["x"], clean, nt, cfg.max_tokens, cfg.num_experts, True)
    assert torch.equal(ref["recv_count"], same["recv_count"]) and torch.equal(ref["layout_range"], same["layout_range"])
    compare_dispatch(h, ref, check_poison=True)
    h.alloc_combine_io()
    h.cast_back(None)
    h.combine()
    torch.cuda.synchronize()
    rows = oracle.cast_back(ref["recv_x"], ref["scales"], ref["recv_count"], None)
    want = oracle.combine(rows, idx, data["topk_weights"], ref["src_info"], ref["layout_range"], nt, cfg.max_tokens,
                          cfg.num_experts)
    want_clean = oracle.combine(rows, clean, data["topk_weights"], ref["src_info"], ref["layout_range"], nt,
                                cfg.max_tokens, cfg.num_experts)
    assert torch.equal(want.view(torch.int16), want_clean.view(torch.int16))
    assert torch.equal(h.combined.cpu().view(torch.int16), want.view(torch.int16))
