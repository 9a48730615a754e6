"""Independent statements of the dispatch/combine contract used to pin the
oracle and (on the GPU) the HIP path.  Nothing here calls the oracle.

* brute_force_layout: the definition, as nested Python loops (tiny inputs).
* torch_rank_dispatch: the reference's PyTorch statement for one destination
  rank (mooncake-wheel/mooncake/mooncake_ep_buffer.py:787-869), written with
  torch ops (`any`, `nonzero`, index gather).
* combine_fp64: per-token weighted sum in float64.
* the structured-data invariants of mooncake-wheel/tests/test_mooncake_ep.py:28-29,61-75
  and the closed forms of :92 and mooncake-ep/tests/test_ep_grid.py:86-108.
"""
from typing import Dict, List, Optional, Sequence

import torch


def brute_force_layout(topk_idx: torch.Tensor, num_tokens: Sequence[int], max_tokens: int, num_experts: int,
                       src_present: Optional[Sequence[int]] = None) -> Dict[str, list]:
    R, Tmax, K = topk_idx.shape
    L = num_experts // R
    idx = topk_idx.tolist()
    per_expert: List[List[tuple]] = [[] for _ in range(num_experts)]
    for r in range(R):
        if src_present is not None and not src_present[r]:
            continue
        for t in range(num_tokens[r]):
            for e in idx[r][t]:                # one row per (token, k) occurrence, in k order
                if e >= 0:
                    per_expert[e].append((r, t))
    out = {"recv_count": [[0] * L for _ in range(R)],
           "layout_range": [[[0] * R for _ in range(L)] for _ in range(R)],
           "src_info": [[[] for _ in range(L)] for _ in range(R)],
           "src_rank": [[[] for _ in range(L)] for _ in range(R)]}
    for e, lst in enumerate(per_expert):
        q, le = divmod(e, L)
        lst = sorted(lst)                      # source rank ascending, then token ascending
        out["recv_count"][q][le] = len(lst)
        out["src_info"][q][le] = [t for (_, t) in lst]
        out["src_rank"][q][le] = [r for (r, _) in lst]
        for r in range(R):
            pos = [i for i, (rr, _) in enumerate(lst) if rr == r]
            if pos:
                assert pos == list(range(pos[0], pos[0] + len(pos)))
                out["layout_range"][q][le][r] = (pos[0] << 32) | len(pos)
    return out


def torch_rank_dispatch(q: int, x: torch.Tensor, topk_idx: torch.Tensor, num_tokens: Sequence[int],
                        max_tokens: int, num_experts: int):
    """Destination rank q's packed outputs (bf16 payload), valid rows only."""
    R = x.size(0)
    L = num_experts // R
    res = []
    for le in range(L):
        e = q * L + le
        rows, srcs, ranges, begin = [], [], [], 0
        for r in range(R):
            sel = (topk_idx[r, :num_tokens[r]] == e).any(dim=1).nonzero(as_tuple=False).view(-1)
            c = sel.numel()
            ranges.append(((begin << 32) | c) if c else 0)
            begin += c
            rows.append(x[r, sel])
            srcs.append(sel.to(torch.int32))
        res.append({"rows": torch.cat(rows), "src_info": torch.cat(srcs),
                    "layout_range": torch.tensor(ranges, dtype=torch.int64), "count": begin})
    return res


def reference_fp8_cast(x: torch.Tensor):
    """ep_test_utils.py:42-47, executed by torch."""
    m, n = x.shape
    x_view = x.view(m, -1, 128)
    x_amax = x_view.abs().float().amax(dim=2).view(m, -1).clamp(1e-4)
    return (x_view * (448.0 / x_amax.unsqueeze(2))).to(torch.float8_e4m3fn).view(m, n), (x_amax / 448.0).view(m, -1)


def reference_cast_back(x_fp8: torch.Tensor, x_scales: torch.Tensor) -> torch.Tensor:
    """ep_test_utils.py:50-53."""
    x_fp32 = x_fp8.to(torch.float32).view(x_fp8.size(0), -1, 128)
    return (x_fp32 * x_scales.view(x_fp8.size(0), -1, 1)).view(x_fp8.shape).to(torch.bfloat16)


def calc_diff(x: torch.Tensor, y: torch.Tensor) -> float:
    """ep_test_utils.py:35-39."""
    x, y = x.double() + 1, y.double() + 1
    return (1 - 2 * (x * y).sum() / (x * x + y * y).sum()).item()


def combine_fp64(expert_out: torch.Tensor, topk_idx: torch.Tensor, topk_weights: torch.Tensor,
                 slot_map: torch.Tensor, num_tokens: Sequence[int], max_tokens: int, num_experts: int,
                 active: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[r,t] = sum_k w * expert_out[e, slot] in float64 (no rounding of note)."""
    R, Tmax, K = topk_idx.shape
    H = expert_out.size(-1)
    L = num_experts // R
    flat = expert_out.reshape(num_experts, -1, H)
    out = torch.zeros((R, Tmax, H), dtype=torch.float64)
    for r in range(R):
        T = num_tokens[r]
        for k in range(K):
            e = topk_idx[r, :T, k]
            ok = (e >= 0) & (slot_map[r, :T, k] >= 0)
            if active is not None:
                ok &= active[r, e.clamp(min=0) // L] != 0
            rows = flat[e.clamp(min=0), slot_map[r, :T, k].clamp(min=0).long()].double()
            out[r, :T] += torch.where(ok.view(-1, 1), rows * topk_weights[r, :T, k].double().view(-1, 1),
                                      torch.zeros((), dtype=torch.float64))
    return out


def bf16_ulp_distance(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Distance in units of bf16 representable values (sign-magnitude aware)."""
    def key(t):
        i = t.contiguous().view(torch.int16).to(torch.int32) & 0xFFFF
        return torch.where(i >= 0x8000, 0x8000 - i, i)
    return (key(a) - key(b)).abs()


def within_one_ulp_of(out_bf16: torch.Tensor, ref64: torch.Tensor) -> torch.Tensor:
    """True where out is one of the two bf16 neighbours of the exact value
    (or the value itself), i.e. at most one bf16 ulp away from correct rounding."""
    r = ref64.to(torch.float32).to(torch.bfloat16)          # a nearest bf16 (double rounding is harmless here)
    return bf16_ulp_distance(out_bf16, r) <= 1


def structured_x(R: int, T: int, H: int) -> torch.Tensor:
    """test_mooncake_ep.py:28-29: rank r's rows are constant (r - 128), the last
    128 columns hold the token index."""
    x = torch.ones((R, T, H), dtype=torch.bfloat16)
    for r in range(R):
        x[r] = x[r] * (r - 128)
        x[r, :, -128:] = torch.arange(T).to(torch.bfloat16).view(-1, 1)
    return x


def check_structured_dispatch(recv_rows: torch.Tensor, recv_count: torch.Tensor, src_info: torch.Tensor,
                              layout_range: torch.Tensor, all_topk_idx: torch.Tensor, T: int) -> None:
    """test_mooncake_ep.py:59-75 for every (rank, local expert); recv_rows is
    bf16 [R, L, RM, H] (already cast back when fp8)."""
    R, L = recv_count.shape
    mask32 = (1 << 32) - 1
    for q in range(R):
        for le in range(L):
            e = q * L + le
            n = int(recv_count[q, le])
            lr = layout_range[q, le]
            assert n == int((lr & mask32).sum())
            assert n == int((all_topk_idx == e).sum())
            rows = recv_rows[q, le, :n].float()
            si = src_info[q, le, :n]
            amin = rows[:, :-128].amin(dim=-1)
            assert torch.equal(amin, rows[:, :-128].amax(dim=-1))
            assert float((rows[:, -128:] - (si.view(-1, 1) % T).float()).abs().sum()) == 0
            for j in range(R):
                begin, count = int(lr[j] >> 32), int(lr[j] & mask32)
                assert int((amin == j - 128).sum()) == int((all_topk_idx[j] == e).sum())
                assert float((rows[begin:begin + count, :-128] - (j - 128)).abs().sum()) == 0
