"""Pins the oracle's scalar conversions and per-128 quantisation.

* the integer e4m3fn encoder against torch's own cast (an independent
  implementation) on every bf16 value times several scales, on random fp32 bit
  patterns and on hand-picked boundaries (ties, subnormals, overflow);
* decode(encode(v)) against the format's definition;
* the row quantiser against the reference's PyTorch formula
  (mooncake-wheel/tests/ep_test_utils.py:42-47), executed by torch;
* the round-trip bound of per_token_cast_back (ep_test_utils.py:50-53).
"""
import math

import numpy as np
import torch


def torch_e4m3_bits(v: torch.Tensor) -> torch.Tensor:
    return v.to(torch.float8_e4m3fn).view(torch.uint8)


def all_bf16_as_f32() -> torch.Tensor:
    bits = torch.arange(0, 65536, dtype=torch.int32)
    return (bits << 16).view(torch.float32)


def eq_or_both_nan(a: torch.Tensor, b: torch.Tensor) -> bool:
    """byte equality; NaN encodings (0x7F / 0xFF) must agree including sign."""
    return bool(torch.equal(a, b))


def test_encoder_matches_torch_on_all_bf16_times_scales(oracle):
    base = all_bf16_as_f32()
    finite = base[torch.isfinite(base)]
    for scale in [1.0, 448.0, 0.5, 3.0, 1.0 / 3.0, 448.0 / 3.14159, 1e-3, 37.77, 2.0 ** -9, 2.0 ** -10, 1e4]:
        v = finite * scale
        assert eq_or_both_nan(oracle.f32_to_e4m3fn(v), torch_e4m3_bits(v)), scale


def test_encoder_matches_torch_on_random_f32_bits(oracle):
    g = torch.Generator().manual_seed(1234)
    bits = torch.randint(-2 ** 31, 2 ** 31 - 1, (4_000_000,), dtype=torch.int64, generator=g).to(torch.int32)
    v = bits.view(torch.float32)
    assert eq_or_both_nan(oracle.f32_to_e4m3fn(v), torch_e4m3_bits(v))
    # dense sampling of the representable range, where rounding decisions happen
    u = (torch.rand(4_000_000, generator=g) * 2 - 1) * 500.0
    assert eq_or_both_nan(oracle.f32_to_e4m3fn(u), torch_e4m3_bits(u))
    small = (torch.rand(2_000_000, generator=g) * 2 - 1) * 2.0 ** -5
    assert eq_or_both_nan(oracle.f32_to_e4m3fn(small), torch_e4m3_bits(small))


def test_encoder_known_answers(oracle):
    # values fixed by the OCP e4m3fn definition (bias 7, 3 mantissa bits, max 448, 0x7F NaN)
    cases = [
        (0.0, 0x00), (-0.0, 0x80), (1.0, 0x38), (-1.0, 0xB8), (448.0, 0x7E), (-448.0, 0xFE),
        (2.0 ** -6, 0x08), (2.0 ** -9, 0x01), (2.0 ** -10, 0x00),     # min normal, min subnormal, tie to even -> 0
        (1.5 * 2.0 ** -9, 0x02),                                      # tie between 1 and 2 quanta -> even (2)
        (2.5 * 2.0 ** -9, 0x02), (3.5 * 2.0 ** -9, 0x04),
        (1.0625, 0x38), (1.1875, 0x3A),                               # ties at 1 + 1/16, 1 + 3/16 -> even mantissa
        (464.0, 0x7E), (448.00003, 0x7E), (465.0, 0x7F), (1e9, 0x7F),  # tie at the top -> 448; beyond -> NaN
        (float("inf"), 0x7F), (float("-inf"), 0xFF), (240.0, 0x77), (0.001953125 * 7, 0x07),
    ]
    v = torch.tensor([c[0] for c in cases], dtype=torch.float32)
    got = oracle.f32_to_e4m3fn(v).tolist()
    assert got == [c[1] for c in cases]
    nan = oracle.f32_to_e4m3fn(torch.tensor([float("nan")])).item()
    assert nan & 0x7F == 0x7F


def test_decode_is_the_format_definition(oracle):
    codes = torch.arange(0, 256, dtype=torch.int32).to(torch.uint8)
    dec = oracle.e4m3fn_to_f32(codes)
    ref = codes.view(torch.float8_e4m3fn).float()
    both_nan = torch.isnan(dec) & torch.isnan(ref)
    assert bool(((dec == ref) | both_nan).all())
    # encode(decode(c)) == c for every non-NaN code
    ok = ~torch.isnan(dec)
    assert torch.equal(oracle.f32_to_e4m3fn(dec[ok]), codes[ok])


def test_bf16_rounding_matches_torch(oracle):
    g = torch.Generator().manual_seed(7)
    v = torch.randn(1_000_000, generator=g) * 100
    ties = (torch.arange(0, 65536, dtype=torch.int32) << 16 | 0x8000).view(torch.float32)
    ties = ties[torch.isfinite(ties)]
    for t in (v, ties, ties * 1.0000001):
        assert torch.equal(oracle.f32_to_bf16_bits(t), t.to(torch.bfloat16).view(torch.int16))


def reference_formula(x: torch.Tensor):
    """ep_test_utils.py:42-47 / mooncake_ep_buffer.py:694-703, executed by torch."""
    m, n = x.shape
    x_view = x.view(m, -1, 128)
    x_amax = x_view.abs().float().amax(dim=2).view(m, -1).clamp(1e-4)
    q = (x_view * (448.0 / x_amax.unsqueeze(2))).to(torch.float8_e4m3fn).view(m, n)
    return q, (x_amax / 448.0).view(m, -1)


def test_row_quantiser_matches_reference_formula(oracle):
    g = torch.Generator().manual_seed(3)
    rows = [
        torch.randn(64, 1024, generator=g),
        torch.randn(16, 1024, generator=g) * 100.0,           # outlier rows
        torch.randn(16, 1024, generator=g) * 1e-6,            # below the 1e-4 amax floor
        torch.zeros(4, 1024),
        torch.randn(16, 1024, generator=g) * 3e38,            # near bf16 max
    ]
    x = torch.cat(rows).to(torch.bfloat16)
    x[5, 100] = float("inf")
    x[6, 300] = float("-inf")
    q, s = oracle.quantise_rows(x)
    q_ref, s_ref = reference_formula(x)
    assert torch.equal(q, q_ref.view(torch.uint8))
    assert torch.equal(s.view(torch.int32), s_ref.view(torch.int32))


def test_row_quantiser_all_bf16_values(oracle):
    # every finite bf16 bit pattern appears, grouped so that groups mix magnitudes
    vals = all_bf16_as_f32()
    vals = vals[torch.isfinite(vals)]
    g = torch.Generator().manual_seed(11)
    perm = torch.randperm(vals.numel(), generator=g)
    pad = (-vals.numel()) % 1024
    v = torch.cat([vals[perm], torch.zeros(pad)]).view(-1, 1024).to(torch.bfloat16)
    # also magnitude-sorted groups (small amax groups exercise subnormal payloads)
    v2 = torch.cat([vals.sort().values, torch.zeros(pad)]).view(-1, 1024).to(torch.bfloat16)
    for x in (v, v2):
        q, s = oracle.quantise_rows(x)
        q_ref, s_ref = reference_formula(x)
        assert torch.equal(q, q_ref.view(torch.uint8))
        assert torch.equal(s.view(torch.int32), s_ref.view(torch.int32))


def kernel_formula(x: torch.Tensor):
    """The reference kernel's own arithmetic (mooncake_ep_kernel.cu:184, :247-260): one IEEE division
    448 / amax for the payload scale, amax * (1/448) with the float constant for the stored scale,
    executed by numpy in float32; the cast itself by torch."""
    import numpy as np
    m, n = x.shape
    xv = x.float().view(m, -1, 128)
    amax = xv.abs().amax(dim=2).clamp(1e-4).numpy().astype(np.float32)
    scale = (np.float32(448.0) / amax).astype(np.float32)
    scale_inv = (amax * (np.float32(1.0) / np.float32(448.0))).astype(np.float32)
    q = (xv * torch.from_numpy(scale).unsqueeze(2)).to(torch.float8_e4m3fn).view(m, n)
    return q, torch.from_numpy(scale_inv)


def test_row_quantiser_in_the_kernels_own_arithmetic(oracle):
    vals = all_bf16_as_f32()
    vals = vals[torch.isfinite(vals)]
    g = torch.Generator().manual_seed(12)
    pad = (-vals.numel()) % 1024
    shuffled = torch.cat([vals[torch.randperm(vals.numel(), generator=g)], torch.zeros(pad)]).view(-1, 1024)
    ordered = torch.cat([vals.sort().values, torch.zeros(pad)]).view(-1, 1024)
    x = torch.cat([shuffled, ordered, torch.randn(64, 1024, generator=g), torch.randn(16, 1024, generator=g) * 100.0])
    x = x.to(torch.bfloat16)
    q_py, s_py = oracle.quantise_rows(x)
    oracle.set_fp8_arith(1)
    try:
        q, s = oracle.quantise_rows(x)
    finally:
        oracle.set_fp8_arith(0)
    q_ref, s_ref = kernel_formula(x)
    assert torch.equal(q, q_ref.view(torch.uint8))
    assert torch.equal(s.view(torch.int32), s_ref.view(torch.int32))
    # the two statements of the reference really are different functions: the stored scale differs in its
    # last bit for a good part of the groups, and some payload bytes follow the payload scale
    differ = (s.view(torch.int32) != s_py.view(torch.int32)).float().mean().item()
    assert 0.05 < differ < 0.6
    assert (s.view(torch.int32) - s_py.view(torch.int32)).abs().max().item() == 1
    assert 0 < (q != q_py).float().mean().item() < 0.01
    # A known answer, worked in exact rational arithmetic: amax = 3.  float32(1/448) = 0x3B124925, and
    # 3 * that rounds to 0x3BDB6DB8 - the kernel's stored scale - while 3/448 itself rounds to 0x3BDB6DB7,
    # the PyTorch statement's.  Both give 448/3 -> 0x43155555 or a neighbour, and 3 * scale -> code 0x7E (448).
    one = torch.zeros(1, 128, dtype=torch.bfloat16)
    one[0, 0] = 3.0
    q0, s0 = oracle.quantise_rows(one)
    oracle.set_fp8_arith(1)
    try:
        q1, s1 = oracle.quantise_rows(one)
    finally:
        oracle.set_fp8_arith(0)
    assert s1.view(torch.int32)[0, 0].item() == 0x3BDB6DB8
    assert s0.view(torch.int32)[0, 0].item() == 0x3BDB6DB7
    assert q1[0, 0].item() == 0x7E and q0[0, 0].item() == 0x7E


def test_nan_elements_do_not_poison_their_group(oracle):
    # the kernel's fmaxf drops NaN from amax (mooncake_ep_kernel.cu:247); the NaN element itself stays NaN
    x = torch.ones(1, 128, dtype=torch.bfloat16) * 2.0
    x[0, 5] = float("nan")
    q, s = oracle.quantise_rows(x)
    assert s[0, 0].item() == 2.0 / 448.0 or math.isclose(s[0, 0].item(), 2.0 / 448.0, rel_tol=1e-7)
    assert q[0, 5].item() & 0x7F == 0x7F
    assert q[0, 0].item() == 0x7E


def test_cast_back_round_trip_bound(oracle):
    g = torch.Generator().manual_seed(5)
    x = torch.randn(32, 2048, generator=g).to(torch.bfloat16)
    q, s = oracle.quantise_rows(x)
    back = (q.view(torch.float8_e4m3fn).float().view(32, -1, 128) * s.view(32, -1, 1)).view(32, -1)
    amax = x.float().view(32, -1, 128).abs().amax(dim=2, keepdim=True).clamp(1e-4).expand(-1, -1, 128).reshape(32, -1)
    # e4m3 has 3 mantissa bits: relative error <= 2^-4 of the value, absolute floor of half a subnormal quantum
    err = (back - x.float()).abs()
    bound = torch.maximum(x.float().abs() * 2.0 ** -4, amax / 448.0 * 2.0 ** -10) * 1.001
    assert bool((err <= bound).all())
