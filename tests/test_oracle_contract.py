"""Pins the oracle's layout, dispatch and combine (CPU only).

Each check is an independent statement of the contract (tests/ref_checks.py),
a closed form from the reference's own tests, or an invariant - chosen so that
a wrong index, a swapped half of layout_range, a dropped k or a wrong
accumulation order fails at least one of them.
"""
import pytest
import torch

from tests import ref_checks as rc


def gen_world(R, T, H, E, K, seed, masked=0.0, ragged=False):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(R, T, H, generator=g).to(torch.bfloat16)
    idx = torch.stack([torch.topk(torch.randn(T, E, generator=g), K, dim=-1)[1] for _ in range(R)]).to(torch.int64)
    w = torch.softmax(torch.randn(R, T, K, generator=g), dim=-1)
    if masked:
        idx[torch.rand(R, T, K, generator=g) < masked] = -1
    nt = [T - (r * 3) % max(1, T // 2) for r in range(R)] if ragged else [T] * R
    return x, idx, w, nt


@pytest.mark.parametrize("R,T,E,K,masked,ragged", [
    (2, 4, 4, 2, 0.0, False), (4, 9, 8, 3, 0.2, True), (3, 16, 12, 4, 0.1, True), (1, 5, 3, 2, 0.0, False),
    (8, 7, 8, 1, 0.3, True),
])
def test_layout_against_brute_force(oracle, R, T, E, K, masked, ragged):
    for seed in range(3):
        _, idx, _, nt = gen_world(R, T, 128, E, K, seed, masked, ragged)
        got = oracle.layout(idx, nt, T, E)
        ref = rc.brute_force_layout(idx, nt, T, E)
        L = E // R
        assert got["recv_count"].tolist() == ref["recv_count"]
        assert got["layout_range"].tolist() == ref["layout_range"]
        for q in range(R):
            for le in range(L):
                n = ref["recv_count"][q][le]
                assert got["src_info"][q, le, :n].tolist() == ref["src_info"][q][le]
                # rows at and beyond recv_count are never written
                assert bool((got["src_info"][q, le, n:] == -7).all())
        # slot_map is the inverse: row slot of expert e holds (r, t)
        sm = got["slot_map"]
        for r in range(R):
            for t in range(nt[r]):
                for k in range(K):
                    e = int(idx[r, t, k])
                    if e < 0:
                        assert int(sm[r, t, k]) == -1
                        continue
                    q, le = divmod(e, L)
                    s = int(sm[r, t, k])
                    assert ref["src_info"][q][le][s] == t and ref["src_rank"][q][le][s] == r


def test_layout_range_packing_known_answer(oracle):
    # R=2, E=2 (one local expert each), hand-computed: expert 0 gets r0:{t0,t2}, r1:{t1}; expert 1 gets r0:{t1}, r1:{}
    idx = torch.tensor([[[0], [1], [0]], [[-1], [0], [-1]]], dtype=torch.int64)
    got = oracle.layout(idx, [3, 3], 3, 2)
    assert got["recv_count"].tolist() == [[3], [1]]
    assert got["layout_range"].tolist() == [[[(0 << 32) | 2, (2 << 32) | 1]], [[(0 << 32) | 1, 0]]]
    assert got["src_info"][0, 0, :3].tolist() == [0, 2, 1]
    assert got["src_info"][1, 0, :1].tolist() == [1]
    assert got["slot_map"].tolist() == [[[0], [0], [1]], [[-1], [2], [-1]]]


def test_silent_source_rank_sends_nothing(oracle):
    _, idx, _, nt = gen_world(4, 8, 128, 8, 2, 0)
    got = oracle.layout(idx, nt, 8, 8, src_present=[1, 0, 1, 1])
    ref = rc.brute_force_layout(idx, nt, 8, 8, src_present=[1, 0, 1, 1])
    assert got["recv_count"].tolist() == ref["recv_count"]
    assert got["layout_range"].tolist() == ref["layout_range"]
    assert bool((got["layout_range"][:, :, 1] == 0).all())


def test_duplicate_expert_gets_a_row_per_occurrence(oracle):
    # out of contract (every workload picks distinct experts); pinned to the kernel's behaviour:
    # one send per k (mooncake_ep_kernel.cu:230,273)
    idx = torch.tensor([[[1, 1], [0, 1]]], dtype=torch.int64)
    got = oracle.layout(idx, [2], 4, 2)
    assert got["recv_count"].tolist() == [[1, 3]]
    assert got["slot_map"].tolist() == [[[0, 1], [0, 2]]]
    assert got["src_info"][0, 1, :3].tolist() == [0, 0, 1]
    # more duplicate rows than the block can hold: the excess is dropped, counts saturate at capacity
    got = oracle.layout(idx, [2], 2, 2)
    assert got["recv_count"].tolist() == [[1, 2]]
    assert got["slot_map"].tolist() == [[[0, 1], [0, -1]]]


@pytest.mark.parametrize("use_fp8", [False, True])
def test_dispatch_against_torch_statement(oracle, use_fp8):
    R, T, H, E, K = 4, 24, 512, 16, 4
    x, idx, _, nt = gen_world(R, T, H, E, K, 5, masked=0.1, ragged=True)
    got = oracle.dispatch(x, idx, nt, T, E, use_fp8)
    L = E // R
    for q in range(R):
        ref = rc.torch_rank_dispatch(q, x, idx, nt, T, E)
        for le in range(L):
            n = ref[le]["count"]
            assert int(got["recv_count"][q, le]) == n
            assert torch.equal(got["layout_range"][q, le], ref[le]["layout_range"])
            assert torch.equal(got["src_info"][q, le, :n], ref[le]["src_info"])
            if use_fp8:
                p_ref, s_ref = rc.reference_fp8_cast(ref[le]["rows"])
                assert torch.equal(got["recv_x"][q, le, :n].view(torch.uint8), p_ref.view(torch.uint8))
                assert torch.equal(got["scales"][q, le, :n].contiguous().view(torch.int32), s_ref.view(torch.int32))
                # unwritten rows keep their poison
                assert bool((got["recv_x"][q, le, n:].view(torch.uint8) == 0xA5).all())
                assert bool(torch.isnan(got["scales"][q, le, n:]).all())
            else:
                assert torch.equal(got["recv_x"][q, le, :n].view(torch.int16), ref[le]["rows"].view(torch.int16))
                assert bool((got["recv_x"][q, le, n:].view(torch.int16) == 0xA5A5 - 65536).all())


@pytest.mark.parametrize("use_fp8", [False, True])
def test_dispatch_structured_data_invariants(oracle, use_fp8):
    # the reference's own smoke test, mooncake-wheel/tests/test_mooncake_ep.py:18-75
    R, T, H, E, K = 4, 32, 512, 16, 4
    g = torch.Generator().manual_seed(1)
    x = rc.structured_x(R, T, H)
    idx = torch.stack([torch.topk(torch.randn(T, E, generator=g).abs() + 1, K, dim=-1)[1] for _ in range(R)])
    for _ in range(10):
        idx[torch.randint(0, R, (1,), generator=g), torch.randint(0, T, (1,), generator=g),
            torch.randint(0, K, (1,), generator=g)] = -1
    got = oracle.dispatch(x, idx, [T] * R, T, E, use_fp8)
    if use_fp8:
        RM = R * T
        rows = rc.reference_cast_back(got["recv_x"].reshape(-1, H), got["scales"].reshape(-1, H // 128).contiguous())
        rows = rows.view(R, E // R, RM, H)
    else:
        rows = got["recv_x"]
    rc.check_structured_dispatch(rows, got["recv_count"], got["src_info"], got["layout_range"], idx, T)


def run_pipeline(oracle, R, T, H, E, K, seed, use_fp8, masked=0.0, ragged=False, factor=False):
    x, idx, w, nt = gen_world(R, T, H, E, K, seed, masked, ragged)
    d = oracle.dispatch(x, idx, nt, T, E, use_fp8)
    L, RM = E // R, R * T
    if use_fp8:
        rows = rc.reference_cast_back(d["recv_x"].reshape(-1, H), d["scales"].reshape(-1, H // 128).contiguous())
        rows = rows.view(R, L, RM, H)
    else:
        rows = d["recv_x"].clone()
    rows = torch.nan_to_num(rows.float(), nan=0.0, posinf=0.0, neginf=0.0)     # poison rows are never read
    if factor:
        f = (torch.arange(E).float() * 0.1 + 1.0).view(R, L, 1, 1)               # test_ep_grid.py:86-87
        rows = rows * f
    return x, idx, w, nt, d, rows.to(torch.bfloat16)


def test_combine_closed_form_identity_expert(oracle):
    # test_mooncake_ep.py:92: expert_out = dispatched x  =>  out = x * sum of unmasked weights
    x, idx, w, nt, d, eo = run_pipeline(oracle, 4, 32, 512, 16, 4, 2, use_fp8=False, masked=0.1)
    out = oracle.combine(eo, idx, w, d["src_info"], d["layout_range"], nt, 32, 16)
    expect = x.float() * w.masked_fill(idx == -1, 0).sum(dim=2, keepdim=True)
    assert rc.calc_diff(expect, out.float()) < 1e-5
    assert not bool(torch.isnan(out.float()).any())


@pytest.mark.parametrize("use_fp8", [False, True])
def test_combine_closed_form_mock_expert(oracle, use_fp8):
    # test_ep_grid.py:100-108, :204-210
    R, T, H, E, K = 4, 32, 512, 16, 4
    x, idx, w, nt, d, eo = run_pipeline(oracle, R, T, H, E, K, 3, use_fp8, factor=True)
    out = oracle.combine(eo, idx, w, d["src_info"], d["layout_range"], nt, T, E)
    expect = (x.float() * ((idx.float() * 0.1 + 1.0) * w).sum(dim=2, keepdim=True)).to(torch.bfloat16)
    torch.testing.assert_close(out, expect, rtol=0.15 if use_fp8 else 5e-2, atol=5e-3 if use_fp8 else 1e-3)


def test_combine_against_fp64_and_accumulation_order(oracle):
    R, T, H, E, K = 4, 32, 512, 16, 4
    x, idx, w, nt, d, eo = run_pipeline(oracle, R, T, H, E, K, 4, use_fp8=False, masked=0.15, ragged=True, factor=True)
    ref = rc.combine_fp64(eo, idx, w, d["slot_map"], nt, T, E)
    out_fma = oracle.combine(eo, idx, w, d["src_info"], d["layout_range"], nt, T, E, use_fma=True)
    out_mul = oracle.combine(eo, idx, w, d["src_info"], d["layout_range"], nt, T, E, use_fma=False)
    assert bool(rc.within_one_ulp_of(out_fma, ref).all())
    assert bool(rc.within_one_ulp_of(out_mul, ref).all())
    assert bool((rc.bf16_ulp_distance(out_fma, out_mul) <= 1).all())
    # an independent fp32 restatement of the fused chain in k order, bit for bit
    acc = torch.zeros(R, T, H, dtype=torch.float64)
    flat = eo.reshape(E, -1, H)
    for k in range(K):
        e = idx[:, :, k]
        ok = (e >= 0)
        for r in range(R):
            ok[r, nt[r]:] = False
        rows = flat[e.clamp(min=0), d["slot_map"][:, :, k].clamp(min=0).long()].double()
        # fma(a, b, c) in fp32 == round_f32(a*b + c) computed exactly; float64 holds a*b (8+24 bits) + c exactly enough
        nxt = (rows * w[:, :, k].double().unsqueeze(-1) + acc).float().double()
        acc = torch.where(ok.unsqueeze(-1), nxt, acc)
    expect = acc.float().to(torch.bfloat16)
    for r in range(R):
        assert torch.equal(out_fma[r, :nt[r]].view(torch.int16), expect[r, :nt[r]].view(torch.int16))
        assert bool((out_fma[r, nt[r]:] == 0).all())


def test_combine_linearity_and_masks(oracle):
    R, T, H, E, K = 2, 16, 256, 8, 2
    x, idx, w, nt, d, eo = run_pipeline(oracle, R, T, H, E, K, 6, use_fp8=False)
    idx2 = idx.clone()
    idx2[0, 3] = -1                                     # a fully masked token combines to zeros
    d2 = oracle.dispatch(x, idx2, nt, T, E, False)
    eo2 = torch.nan_to_num(d2["recv_x"].float()).to(torch.bfloat16)
    out = oracle.combine(eo2, idx2, w, d2["src_info"], d2["layout_range"], nt, T, E)
    assert bool((out[0, 3] == 0).all())
    # scaling the weights by 2 (exact in fp32) doubles the output exactly
    out1 = oracle.combine(eo, idx, w, d["src_info"], d["layout_range"], nt, T, E)
    out2 = oracle.combine(eo, idx, w * 2, d["src_info"], d["layout_range"], nt, T, E)
    assert torch.equal((out1.float() * 2).to(torch.bfloat16).view(torch.int16), out2.view(torch.int16))


def test_combine_skips_inactive_ranks(oracle):
    # test_ep_grid.py:92-99: experts owned by a failed rank drop out of the sum
    R, T, H, E, K = 4, 16, 256, 16, 4
    x, idx, w, nt, d, eo = run_pipeline(oracle, R, T, H, E, K, 8, use_fp8=False, factor=True)
    fail = 2
    active = torch.ones(R, R, dtype=torch.int32)
    active[:, fail] = 0
    out = oracle.combine(eo, idx, w, d["src_info"], d["layout_range"], nt, T, E, active=active)
    L = E // R
    fac = (idx.float() * 0.1 + 1.0) * (idx // L != fail).float()
    expect = (x.float() * (fac * w).sum(dim=2, keepdim=True)).to(torch.bfloat16)
    torch.testing.assert_close(out, expect, rtol=5e-2, atol=1e-3)


def test_buffer_size_hint_known_answers(oracle):
    # BufferPair (mooncake_ep_buffer.h:29-63): 4 signalling areas of E ints + 4 data areas of E*max*(32 + 2H) bytes
    assert oracle.buffer_size_hint(128, 7168, 32, 256) == 4 * 256 * 4 + 4 * 256 * 128 * (32 + 2 * 7168)
    assert oracle.buffer_size_hint(128, 7168, 32, 256) == 1883246592
    assert oracle.buffer_size_hint(256, 2048, 8, 288) == 4 * 288 * 4 + 4 * 288 * 256 * (32 + 4096)
