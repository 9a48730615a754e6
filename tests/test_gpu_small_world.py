"""The one-launch dispatch of small worlds (`dispatch_small_kernel`: at most 8 ranks and, by default, 4096
selections; every wave rebuilds the routing it needs from the ranks' index lists) against the CPU oracle, bit
for bit, and against the library's own count / pack / scale-transpose path: shapes at the edges of what it
takes (list lengths around the 128- and 512-entry steps of its counting loop, odd list lengths, the most ranks
and selections it accepts, every top-k bracket), ragged and silent ranks, a rank that receives nothing,
repeated experts, stray ids, index lists at either alignment, and the shapes it must leave to the other path."""
import pytest
import torch

from mooncake_amd.harness import WorldHarness
from mooncake_amd.workloads import EPConfig, generate
from tests import gpu_util
from tests.gpu_util import announce, compare_dispatch, run_dispatch

pytestmark = pytest.mark.gpu

CASES = [
    # name, R, T, H, E, K, fp8
    EPConfig("one_rank_decode", 1, 128, 7168, 256, 8, True),         # one rank of the DeepSeek-V3 decode world
    EPConfig("one_rank_decode_bf16", 1, 128, 7168, 256, 8, False),
    EPConfig("odd_list", 4, 21, 1024, 12, 3, True),                  # 63 entries per list: odd, below one step
    EPConfig("list_127", 2, 127, 256, 16, 1, False),
    EPConfig("list_129", 4, 43, 256, 16, 3, True),                   # 129 entries: one past a 128-entry step
    EPConfig("list_513", 2, 57, 512, 32, 9, False),                  # 513: one past a 512-entry round
    EPConfig("most_ranks", 8, 64, 1024, 64, 8, True),                # 8 ranks x 512 = 4096 selections
    EPConfig("most_ranks_bf16", 8, 64, 1536, 64, 8, False),
    EPConfig("k16", 4, 32, 2048, 64, 16, True),
    EPConfig("k2", 8, 100, 640, 8, 2, True),
    EPConfig("k5", 4, 50, 2560, 40, 5, False),
    EPConfig("many_experts", 4, 16, 256, 2048, 8, True),             # more experts than the count kernel's LDS holds
    EPConfig("hot_expert", 4, 64, 1024, 16, 4, True, routing="zipf"),
    EPConfig("masked", 8, 64, 1024, 8, 2, False, masked_fraction=0.3),
]


def ragged(cfg, on):
    if not on:
        return None
    return [max(0, cfg.tokens_per_rank - (r * 5) % (cfg.tokens_per_rank + 1)) for r in range(cfg.num_ranks)]


def launches(h):
    return h.world.get_option("last_dispatch_launches")


@pytest.fixture(autouse=True)
def any_number_of_list_rounds(request):
    """The default takes the one-launch dispatch only where it pays (few rounds of index-list entries); these
    tests are about its results on every shape it accepts, so the rule is lifted - except where it is the subject."""
    if "default_size_rule" in request.node.name:
        yield
        return
    gpu_util.DEFAULT_OPTIONS["fused_small_rounds"] = 1 << 20
    yield
    gpu_util.DEFAULT_OPTIONS.pop("fused_small_rounds", None)


def test_default_size_rule(gpu_device, oracle):
    """One launch while the ranks' index lists make at most 6 rounds of 512 entries (fp8 payload: two launches
    saved) or 4 (bf16: one), each rank's list counted by itself; the option moves the limit."""
    announce("one-launch dispatch: the default size rule")
    cases = [(EPConfig("fp8_6_rounds", 1, 384, 256, 16, 8, True), 1), (EPConfig("fp8_7_rounds", 1, 448, 256, 16, 8, True), 3),
             (EPConfig("fp8_6_lists", 6, 8, 256, 12, 2, True), 1), (EPConfig("fp8_7_lists", 7, 8, 256, 14, 2, True), 3),
             (EPConfig("bf16_4_rounds", 2, 128, 256, 16, 8, False), 1), (EPConfig("bf16_5_rounds", 5, 4, 256, 10, 2, False), 2)]
    for cfg, want in cases:
        data = generate(cfg, seed=47)
        h = run_dispatch(cfg, data, poison=True)
        assert (launches(h) == 1) == (want == 1), cfg.name
        assert launches(h) >= want, cfg.name
        ref = oracle.dispatch(data["x"], data["topk_idx"], h.num_tokens, cfg.max_tokens, cfg.num_experts, cfg.use_fp8)
        compare_dispatch(h, ref, check_poison=True)
    cfg = cases[1][0]
    h = run_dispatch(cfg, generate(cfg, seed=47), poison=True, options={"fused_small_rounds": 7})
    assert launches(h) == 1
    cfg = cases[0][0]
    h = run_dispatch(cfg, generate(cfg, seed=47), poison=True, options={"fused_small_rounds": 5})
    assert launches(h) >= 3


@pytest.mark.parametrize("cfg", CASES, ids=[c.name for c in CASES])
@pytest.mark.parametrize("is_ragged", [False, True], ids=["full", "ragged"])
def test_one_launch_dispatch_matches_oracle(gpu_device, oracle, cfg, is_ragged):
    nt = ragged(cfg, is_ragged)
    announce(f"one-launch dispatch {cfg} ragged={nt}")
    data = generate(cfg, seed=41)
    h = run_dispatch(cfg, data, num_tokens=nt, poison=True)
    assert launches(h) == 1
    ref = oracle.dispatch(data["x"], data["topk_idx"], h.num_tokens, cfg.max_tokens, cfg.num_experts, cfg.use_fp8)
    compare_dispatch(h, ref, check_poison=True)
    # the same world through the other path: the same bits everywhere, padding included
    g = run_dispatch(cfg, data, num_tokens=nt, poison=True, options={"fused_small": 0})
    assert launches(g) >= 2
    for name in ("recv_x", "recv_count", "src_info", "layout_range"):
        assert torch.equal(getattr(h, name), getattr(g, name)), name
    if cfg.use_fp8:
        assert torch.equal(h.recv_scales_phys.view(torch.int32), g.recv_scales_phys.view(torch.int32))
    # and a combine of the handle finds its rows in what the launch left (no resolve launch)
    factor = torch.arange(cfg.num_experts).float() * 0.1 + 1.0
    for w in (h, g):
        w.alloc_combine_io()
        w.cast_back(factor)
        w.combined.fill_(7.0)
        w.combine()
    torch.cuda.synchronize()
    assert h.world.get_option("last_combine_launches") <= 2          # a rank-table upload and the reduce kernel
    rows = oracle.cast_back(ref["recv_x"], ref["scales"] if cfg.use_fp8 else None, ref["recv_count"], factor)
    want = oracle.combine(rows, data["topk_idx"], data["topk_weights"], ref["src_info"], ref["layout_range"],
                          h.num_tokens, cfg.max_tokens, cfg.num_experts)
    for r, n in enumerate(h.num_tokens):
        assert torch.equal(h.combined[r, :n].cpu().view(torch.int16), want[r, :n].view(torch.int16)), f"rank {r}"
        assert bool((h.combined[r, n:] == 7.0).all())
    assert torch.equal(h.combined.view(torch.int16), g.combined.view(torch.int16))


@pytest.mark.parametrize("arith", [0, 1], ids=["torch_arith", "kernel_arith"])
def test_one_launch_fp8_arithmetic_options(gpu_device, oracle, arith):
    cfg = EPConfig("arith", 4, 24, 2560, 16, 3, True, outlier_fraction=0.1)
    announce(f"one-launch dispatch fp8_arith={arith}")
    data = generate(cfg, seed=42)
    h = run_dispatch(cfg, data, poison=True, options={"fp8_arith": arith})
    assert launches(h) == 1
    oracle.set_fp8_arith(arith)
    try:
        ref = oracle.dispatch(data["x"], data["topk_idx"], h.num_tokens, cfg.max_tokens, cfg.num_experts, True)
    finally:
        oracle.set_fp8_arith(0)
    compare_dispatch(h, ref, check_poison=True)


def test_one_launch_with_a_silent_rank_and_a_rank_that_receives_nothing(gpu_device, oracle):
    cfg = EPConfig("silent_small", 4, 16, 1024, 16, 4, True)
    announce("one-launch dispatch with a silent rank")
    data = generate(cfg, seed=43)
    present = [1, 0, 1, 1]
    h = run_dispatch(cfg, data, poison=True, present=present)
    assert launches(h) == 1
    ref = oracle.dispatch(data["x"], data["topk_idx"], h.num_tokens, cfg.max_tokens, cfg.num_experts, True,
                          src_present=present)
    assert bool((h.recv_count[1] == -7).all()) and bool((h.src_info[1] == -7).all())   # never written
    assert bool((h.layout_range[1] == -7).all())
    for k in ("recv_count", "layout_range", "src_info"):
        ref[k][1] = -7
    h.recv_count[1] = 0
    ref["recv_count"][1] = 0
    compare_dispatch(h, ref, check_poison=False)


def test_one_launch_with_repeated_and_stray_experts(gpu_device, oracle):
    cfg = EPConfig("dups_small", 2, 16, 1024, 4, 4, True)
    announce("one-launch dispatch with repeated experts (block overflow) and stray ids")
    data = generate(cfg, seed=44)
    idx = data["topk_idx"]
    idx[:, ::3, 1] = idx[:, ::3, 0]                       # k = 1 repeats k = 0 on every third token
    idx[0, :, :] = 1                                      # rank 0: every token names expert 1 four times
    idx[1, 1, 2] = cfg.num_experts + 3
    idx[1, 2, 0] = -5
    idx[1, 3, 3] = 2 ** 40
    h = run_dispatch(cfg, data, poison=True)
    assert launches(h) == 1
    ref = oracle.dispatch(data["x"], idx, h.num_tokens, cfg.max_tokens, cfg.num_experts, True)
    assert int(ref["recv_count"].max()) == cfg.num_ranks * cfg.max_tokens   # the overflow case is exercised
    compare_dispatch(h, ref, check_poison=True)


def test_shapes_the_one_launch_dispatch_leaves_alone(gpu_device, oracle):
    announce("one-launch dispatch: thresholds and fallbacks")
    # one selection too many for the default threshold, and a ninth rank
    for cfg in (EPConfig("too_many", 8, 65, 256, 64, 8, False), EPConfig("nine_ranks", 9, 8, 256, 18, 2, False)):
        data = generate(cfg, seed=45)
        h = run_dispatch(cfg, data, poison=True)
        assert launches(h) >= 2, cfg.name
        ref = oracle.dispatch(data["x"], data["topk_idx"], h.num_tokens, cfg.max_tokens, cfg.num_experts, False)
        compare_dispatch(h, ref, check_poison=True)
    # ... which the threshold option moves
    cfg = EPConfig("too_many", 8, 65, 256, 64, 8, False)
    data = generate(cfg, seed=45)
    h = run_dispatch(cfg, data, poison=True, options={"fused_small_max": 8 * 65 * 8})
    assert launches(h) == 1
    ref = oracle.dispatch(data["x"], data["topk_idx"], h.num_tokens, cfg.max_tokens, cfg.num_experts, False)
    compare_dispatch(h, ref, check_poison=True)


def test_index_lists_that_start_inside_a_16_byte_unit(gpu_device, oracle):
    announce("one-launch dispatch: index lists 8 bytes past a 16-byte boundary")
    cfg = EPConfig("unaligned", 2, 31, 256, 8, 1, False)
    data = generate(cfg, seed=46)
    h = WorldHarness(cfg)
    h.load(data)
    backing = torch.full((cfg.num_ranks, cfg.tokens_per_rank + 1, 1), -1, dtype=torch.int64, device=h.device)
    backing[:, 1:] = h.topk_idx
    h.topk_idx = backing[:, 1:]                           # rank r's list starts 8 bytes past a 16-byte boundary
    assert h.topk_idx[0].data_ptr() % 16 == 8
    h.alloc_dispatch_outputs(poison=True)
    h.dispatch()
    torch.cuda.synchronize()
    assert launches(h) == 1
    ref = oracle.dispatch(data["x"], data["topk_idx"], h.num_tokens, cfg.max_tokens, cfg.num_experts, False)
    compare_dispatch(h, ref, check_poison=True)


def test_one_launch_dispatch_twice_on_one_world(gpu_device, oracle):
    """Two different small worlds' worth of data through one world, each followed by the combine of its own
    handle: the second dispatch's selrow replaces the first's."""
    cfg = EPConfig("again", 4, 24, 1024, 16, 4, False)
    announce("one-launch dispatch, two data sets on one world")
    a = run_dispatch(cfg, generate(cfg, seed=47), poison=False)
    b = WorldHarness(cfg, world=a.world)
    b.load(generate(cfg, seed=48))
    b.alloc_dispatch_outputs()
    b.dispatch()
    assert launches(b) == 1
    for h, seed in ((b, 48), (a, 47)):                    # b's handle is the last dispatch's, a's an older one
        data = generate(cfg, seed=seed)
        h.alloc_combine_io()
        h.cast_back(None)
        h.combine()
        torch.cuda.synchronize()
        want = oracle.combine(h.expert_out.cpu(), data["topk_idx"], data["topk_weights"], h.src_info.cpu(),
                              h.layout_range.cpu(), h.num_tokens, cfg.max_tokens, cfg.num_experts)
        assert torch.equal(h.combined.cpu().view(torch.int16), want.view(torch.int16))
