"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py):
the oracle must reproduce them on the CPU, the HIP path on the GPU."""
import glob
import os

import numpy as np
import pytest
import torch

# (routing_vectors.npz belongs to the benchmark's routing generators: tests/test_ep_benchmark.py)
GOLDEN = sorted(p for p in glob.glob(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "*.npz"))
                if os.path.basename(p) != "routing_vectors.npz")


def load(path):
    z = np.load(path, allow_pickle=False)
    R, T, H, E, K, fp8 = [int(v) for v in z["dims"]]
    t = {k: torch.from_numpy(z[k]) for k in z.files}
    t["x"] = t["x"].view(torch.bfloat16)
    t["expert_out"] = t["expert_out"].view(torch.bfloat16)
    return (R, T, H, E, K, bool(fp8)), [int(v) for v in z["num_tokens"]], t


def check_dispatch(dims, got, gold):
    R, T, H, E, K, fp8 = dims
    RM = R * T
    cnt = got["recv_count"]
    assert torch.equal(cnt, gold["recv_count"])
    assert torch.equal(got["layout_range"], gold["layout_range"])
    valid = torch.arange(RM).view(1, 1, RM) < cnt.unsqueeze(-1)
    assert torch.equal(got["src_info"][valid], gold["src_info"][valid])
    gx = got["recv_x"].view(torch.uint8) if fp8 else got["recv_x"].view(torch.int16)
    assert torch.equal(gx[valid], gold["recv_x"][valid])
    if fp8:
        assert torch.equal(got["scales"][valid].view(torch.int32), gold["scales"][valid].view(torch.int32))


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_oracle_reproduces_golden(oracle, path):
    dims, nt, g = load(path)
    R, T, H, E, K, fp8 = dims
    d = oracle.dispatch(g["x"], g["topk_idx"], nt, T, E, fp8)
    check_dispatch(dims, d, g)
    out = oracle.combine(g["expert_out"], g["topk_idx"], g["topk_weights"], d["src_info"], d["layout_range"], nt, T, E)
    assert torch.equal(out.view(torch.int16), g["combined"])


@pytest.mark.gpu
@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_hip_reproduces_golden(gpu_device, path):
    from mooncake_amd.harness import WorldHarness
    from mooncake_amd.workloads import EPConfig
    dims, nt, g = load(path)
    R, T, H, E, K, fp8 = dims
    print(f"[gpu-case] golden {os.path.basename(path)}", flush=True)
    h = WorldHarness(EPConfig("golden", R, T, H, E, K, fp8), num_tokens=nt)
    h.load({"x": g["x"], "topk_idx": g["topk_idx"], "topk_weights": g["topk_weights"]})
    h.alloc_dispatch_outputs(poison=True)
    h.dispatch()
    h.alloc_combine_io()
    h.expert_out.copy_(g["expert_out"].to(gpu_device))
    h.combined.zero_()
    h.combine()
    torch.cuda.synchronize()
    got = {"recv_count": h.recv_count.cpu(), "layout_range": h.layout_range.cpu(), "src_info": h.src_info.cpu(),
           "recv_x": h.recv_x.cpu(), "scales": None if not fp8 else h.recv_scales().cpu()}
    check_dispatch(dims, got, g)
    assert torch.equal(h.combined.cpu().view(torch.int16), g["combined"])
