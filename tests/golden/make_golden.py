"""Writes the golden fixtures under tests/golden/ (run from the repo root:
`python tests/golden/make_golden.py`).

The vectors are produced by the CPU oracle after it has been pinned
(tests/test_oracle_fp8.py, tests/test_oracle_contract.py); they are data only:
seeded inputs and the expected outputs of dispatch and combine, kept small.
The reference holds no stored vectors for this path (its tests synthesise
their data), so these fixtures freeze the pinned behaviour against regressions
in the oracle and in the HIP path alike.
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

CASES = [
    # name, R, T, H, E, K, use_fp8, masked fraction, ragged
    ("tiny_bf16", 2, 4, 128, 4, 2, False, 0.0, False),
    ("tiny_fp8", 2, 4, 128, 4, 2, True, 0.0, False),
    ("ragged_masked_fp8", 4, 12, 256, 8, 3, True, 0.2, True),
    ("ragged_masked_bf16", 4, 12, 256, 8, 3, False, 0.2, True),
]


def bits16(t):
    return t.contiguous().view(torch.int16).numpy().copy()


def make(name, R, T, H, E, K, use_fp8, masked, ragged, seed=0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(R, T, H, generator=g)
    x[0, 0, :3] = torch.tensor([0.0, -0.0, 1e-6])                 # zeros and a value under the amax floor
    if H >= 256:
        x[1, 1, 128:256] *= 100.0                                   # an outlier group
    x = x.to(torch.bfloat16)
    idx = torch.stack([torch.topk(torch.randn(T, E, generator=g), K, dim=-1)[1] for _ in range(R)]).to(torch.int64)
    if masked:
        idx[torch.rand(R, T, K, generator=g) < masked] = -1
    w = torch.softmax(torch.randn(R, T, K, generator=g), dim=-1)
    nt = [T - (2 * r) % T for r in range(R)] if ragged else [T] * R
    d = oracle.dispatch(x, idx, nt, T, E, use_fp8)
    L, RM = E // R, R * T
    if use_fp8:
        rows = (d["recv_x"].float().view(R, L, RM, H // 128, 128) * d["scales"].unsqueeze(-1)).view(R, L, RM, H)
    else:
        rows = d["recv_x"].float()
    valid = torch.arange(RM).view(1, 1, RM) < d["recv_count"].unsqueeze(-1)
    factor = (torch.arange(E).float() * 0.1 + 1.0).view(R, L, 1, 1)
    expert_out = torch.where(valid.unsqueeze(-1), rows * factor, torch.zeros(())).to(torch.bfloat16)
    out = oracle.combine(expert_out, idx, w, d["src_info"], d["layout_range"], nt, T, E)
    arrays = dict(
        dims=np.array([R, T, H, E, K, int(use_fp8)], dtype=np.int64), num_tokens=np.array(nt, dtype=np.int32),
        x=bits16(x), topk_idx=idx.numpy(), topk_weights=w.numpy(),
        recv_count=d["recv_count"].numpy(), layout_range=d["layout_range"].numpy(),
        src_info=torch.where(valid, d["src_info"], torch.full((), -1, dtype=torch.int32)).numpy(),
        recv_x=(torch.where(valid.unsqueeze(-1), d["recv_x"].view(torch.uint8), torch.zeros((), dtype=torch.uint8)).numpy()
                if use_fp8 else bits16(torch.where(valid.unsqueeze(-1), d["recv_x"], torch.zeros((), dtype=torch.bfloat16)))),
        expert_out=bits16(expert_out), combined=bits16(out),
    )
    if use_fp8:
        arrays["scales"] = torch.where(valid.unsqueeze(-1), d["scales"], torch.zeros(())).contiguous().numpy()
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **arrays)
    print(name, {k: v.shape for k, v in arrays.items()})


if __name__ == "__main__":
    for case in CASES:
        make(*case)
