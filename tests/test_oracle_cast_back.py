"""The oracle's consumer of the packed layout against the PyTorch statements it
restates: per_token_cast_back (mooncake-wheel/tests/ep_test_utils.py:50-53) and
the grid test's mock expert (mooncake-ep/tests/test_ep_grid.py:168-173), written
out with torch ops here."""
import torch

from tests import ref_checks as rc


def _torch_cast_back(x_fp8, scales, factor):
    R, L, RM, H = x_fp8.shape
    v = (x_fp8.float().view(R, L, RM, H // 128, 128) * scales.unsqueeze(-1)).view(R, L, RM, H).to(torch.bfloat16)
    if factor is not None:
        # a bf16 tensor times a python scalar: fp32 product, rounded once
        for r in range(R):
            for le in range(L):
                v[r, le] = v[r, le] * float(factor[r * L + le])
    return v


def _same_bits_or_nan(got, want):
    nan = torch.isnan(want)
    assert bool(torch.isnan(got)[nan].all())
    assert torch.equal(got.view(torch.int16)[~nan], want.view(torch.int16)[~nan])


def test_cast_back_every_fp8_byte_and_scale_range(oracle):
    R, L, RM, H = 1, 3, 16, 256
    # every byte value appears in every row; scales from subnormal products to overflow
    x = torch.arange(256, dtype=torch.uint8).repeat(R, L, RM, 1).contiguous()
    x[..., 1::2, :] = x[..., 1::2, :].flip(-1)
    gen = torch.Generator().manual_seed(3)
    scales = torch.empty(R, L, RM, H // 128)
    scales[..., 0] = torch.logspace(-40, 36, R * L * RM, base=10.0).view(R, L, RM)
    scales[..., 1] = torch.rand(R, L, RM, generator=gen) * 3 + 1e-3
    count = torch.tensor([[16, 9, 0]], dtype=torch.int32)
    factor = torch.tensor([1.0, 1.7, 3.3])
    for f in (None, factor):
        got = oracle.cast_back(x, scales, count, f, fill=-7)
        want = _torch_cast_back(x.view(torch.float8_e4m3fn), scales, f)
        for le in range(L):
            c = int(count[0, le])
            _same_bits_or_nan(got[0, le, :c], want[0, le, :c])
            assert bool((got[0, le, c:].view(torch.int16) == -7).all())
    # factor 1.0 changes nothing: the second rounding of a bf16 value is exact
    a = oracle.cast_back(x, scales, count, None)
    b = oracle.cast_back(x, scales, count, torch.ones(3))
    _same_bits_or_nan(a, b)


def test_cast_back_matches_reference_helper_on_quantised_rows(oracle):
    # quantise real rows with the reference's own cast (per_token_cast_to_fp8), then cast back
    gen = torch.Generator().manual_seed(5)
    x = (torch.randn(24, 512, generator=gen) * 3).to(torch.bfloat16)
    q, s = rc.reference_fp8_cast(x)
    want = rc.reference_cast_back(q, s)
    got = oracle.cast_back(q.view(1, 1, 24, 512), s.view(1, 1, 24, 4), torch.tensor([[24]], dtype=torch.int32))
    assert torch.equal(got.view(24, 512).view(torch.int16), want.view(torch.int16))


def test_cast_back_bf16_payload_applies_only_the_factor(oracle):
    gen = torch.Generator().manual_seed(7)
    x = torch.randn(2, 2, 8, 128, generator=gen).to(torch.bfloat16)
    count = torch.tensor([[8, 3], [0, 5]], dtype=torch.int32)
    factor = torch.tensor([1.0, 1.1, 1.2, 1.3])
    got = oracle.cast_back(x, None, count, factor, fill=-7)
    for r in range(2):
        for le in range(2):
            c = int(count[r, le])
            want = x[r, le, :c] * float(factor[r * 2 + le])
            assert torch.equal(got[r, le, :c].view(torch.int16), want.view(torch.int16))
            assert bool((got[r, le, c:].view(torch.int16) == -7).all())
    same = oracle.cast_back(x, None, count, None, fill=-7)
    assert torch.equal(same[0, 0].view(torch.int16), x[0, 0].view(torch.int16))
