"""The consumer kernel (packed rows -> bf16, optional per-expert factor)
against the oracle, bit for bit, through the C ABI."""
import pytest
import torch

from mooncake_amd.harness import WorldHarness
from mooncake_amd.workloads import CONFIGS, EPConfig, generate
from tests.gpu_util import announce

pytestmark = pytest.mark.gpu

FILL = 0x5A5A


def _check(h: WorldHarness, oracle, factor, present=None):
    cfg = h.cfg
    R = cfg.num_ranks
    scales = None if not cfg.use_fp8 else h.recv_scales().cpu()
    recv = h.recv_x.cpu().view(torch.uint8 if cfg.use_fp8 else torch.bfloat16)
    want = oracle.cast_back(recv, scales, h.recv_count.cpu(), factor, fill=FILL)
    got = h.expert_out.cpu()
    for r in range(R):
        if present is not None and not present[r]:
            assert bool((got[r].view(torch.int16) == FILL).all()), f"rank {r} takes no part but was written"
            continue
        nan = torch.isnan(want[r])
        assert bool(torch.isnan(got[r])[nan].all())
        assert torch.equal(got[r].view(torch.int16)[~nan], want[r].view(torch.int16)[~nan]), f"rank {r}"


@pytest.mark.parametrize("use_fp8", [True, False])
@pytest.mark.parametrize("with_factor", [False, True])
@pytest.mark.parametrize("shape", [(4, 40, 1024, 16, 4), (2, 64, 1152, 8, 3), (8, 16, 7168, 32, 8)])
def test_cast_back_after_dispatch(gpu_device, oracle, use_fp8, with_factor, shape):
    R, T, H, E, K = shape
    cfg = EPConfig("cast_back", R, T, H, E, K, use_fp8)
    announce(f"cast_back {cfg} factor={with_factor}")
    h = WorldHarness(cfg)
    h.load(generate(cfg, seed=31))
    h.alloc_dispatch_outputs(poison=True)
    h.alloc_combine_io()
    h.expert_out.view(torch.int16).fill_(FILL)
    h.dispatch()
    factor = (torch.arange(E, dtype=torch.float32) * 0.1 + 1.0) if with_factor else None
    h.cast_back(factor)
    torch.cuda.synchronize()
    _check(h, oracle, factor)


def test_cast_back_every_byte_ragged_counts_and_absent_rank(gpu_device, oracle):
    cfg = EPConfig("cast_back_bytes", 3, 44, 256, 6, 6, True)      # RM = 132: row chunks end ragged; top-6 bounds the rows
    announce(f"cast_back bytes {cfg}")
    R, L, RM, H = 3, 2, 132, 256
    h = WorldHarness(cfg)
    h.alloc_dispatch_outputs(poison=False)
    h.alloc_combine_io()
    gen = torch.Generator().manual_seed(1)
    rows = torch.stack([torch.randperm(256, generator=gen) for _ in range(R * L * RM)]).to(torch.uint8)
    h.recv_x.copy_(rows.view(R, L, RM, H))
    scales = torch.empty(R, L, H // 128, RM)
    scales[:, :, 0] = torch.logspace(-40, 36, R * L * RM, base=10.0).view(R, L, RM)
    scales[:, :, 1] = torch.rand(R, L, RM, generator=gen) + 0.01
    h.recv_scales_phys.copy_(scales)
    h.recv_count.copy_(torch.tensor([[132, 0], [1, 64], [65, 131]], dtype=torch.int32))
    factor = torch.tensor([1.0, 1.5, 0.3, 2.0, 1.1, 7.0])
    for present in (None, [1, 0, 1]):
        h.expert_out.view(torch.int16).fill_(FILL)
        h.cast_back(factor, present=present)
        torch.cuda.synchronize()
        _check(h, oracle, factor, present)


def test_cast_back_in_place_on_bf16_rows(gpu_device, oracle):
    cfg = EPConfig("cast_back_inplace", 4, 32, 512, 8, 2, False)
    announce(f"cast_back in place {cfg}")
    h = WorldHarness(cfg)
    h.load(generate(cfg, seed=2))
    h.alloc_dispatch_outputs(poison=True)
    h.dispatch()
    torch.cuda.synchronize()
    factor = torch.arange(8, dtype=torch.float32) * 0.25 + 0.5
    want = oracle.cast_back(h.recv_x.cpu().view(torch.bfloat16), None, h.recv_count.cpu(), factor,
                            fill=0xA5A5 - 65536)
    h.expert_out = h.recv_x.view(torch.bfloat16)        # out aliases the payload
    h.cast_back(factor)
    torch.cuda.synchronize()
    assert torch.equal(h.recv_x.cpu(), want.view(torch.int16))


def test_cast_back_then_combine_full_size(gpu_device):
    """DeepSeek-V3 decode shape: dispatch fp8 -> cast back with the mock expert's factor -> combine gives the
    grid test's closed form x * sum_k factor(e_k) * w_k (test_ep_grid.py:100-108, its fp8 tolerance)."""
    cfg = CONFIGS["dsv3_decode"]
    announce(f"cast_back full size {cfg}")
    data = generate(cfg, seed=0)
    h = WorldHarness(cfg)
    h.load(data)
    h.alloc_dispatch_outputs(poison=False)
    h.alloc_combine_io()
    factor = torch.arange(cfg.num_experts, dtype=torch.float32) * 0.1 + 1.0
    h.dispatch()
    h.cast_back(factor)
    h.combine()
    torch.cuda.synchronize()
    f = factor.to(gpu_device)[h.topk_idx]
    want = h.x.float() * (f * h.topk_weights).sum(-1, keepdim=True)
    torch.testing.assert_close(h.combined.float(), want, rtol=0.15, atol=5e-3)
    # and against torch's own dequantisation of one rank's valid rows, bit for bit
    r = 5
    cnt = h.recv_count[r]
    v = h.recv_x[r].view(torch.float8_e4m3fn).float().view(cfg.num_local_experts, -1, cfg.hidden // 128, 128)
    v = (v * h.recv_scales_phys[r].transpose(1, 2).unsqueeze(-1)).view(cfg.num_local_experts, -1, cfg.hidden)
    v = v.to(torch.bfloat16)
    for le in range(cfg.num_local_experts):
        c = int(cnt[le])
        w = (v[le, :c].float() * float(factor[r * cfg.num_local_experts + le])).to(torch.bfloat16)
        assert torch.equal(h.expert_out[r, le, :c].view(torch.int16), w.view(torch.int16))
