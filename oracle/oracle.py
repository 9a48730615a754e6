"""ctypes front end of the CPU oracle (oracle/mc_ep_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and
by bench.py's cpu_baseline leg, never by the shipped package.  All tensors are
CPU torch tensors in the whole-world layout documented at the top of the C
file (rank-major, contiguous).
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Dict, Optional, Sequence

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libmc_ep_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (oracle/Makefile)."""
    if force or not os.path.exists(_SO):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True, capture_output=True)
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.oracle_buffer_size_hint.restype = ctypes.c_uint64
    return _lib


def _p(t: Optional[torch.Tensor]):
    if t is None:
        return ctypes.c_void_p(0)
    assert t.device.type == "cpu" and t.is_contiguous()
    return ctypes.c_void_p(t.data_ptr())


def _i32(v: Sequence[int]) -> torch.Tensor:
    return torch.tensor(list(v), dtype=torch.int32)


def f32_to_e4m3fn(v: torch.Tensor) -> torch.Tensor:
    v = v.contiguous().float()
    out = torch.empty(v.shape, dtype=torch.uint8)
    lib().oracle_f32_to_e4m3fn(_p(v), _p(out), ctypes.c_int64(v.numel()))
    return out


def e4m3fn_to_f32(v: torch.Tensor) -> torch.Tensor:
    v = v.contiguous().view(torch.uint8)
    out = torch.empty(v.shape, dtype=torch.float32)
    lib().oracle_e4m3fn_to_f32(_p(v), _p(out), ctypes.c_int64(v.numel()))
    return out


def f32_to_bf16_bits(v: torch.Tensor) -> torch.Tensor:
    v = v.contiguous().float()
    out = torch.empty(v.shape, dtype=torch.int16)
    lib().oracle_f32_to_bf16(_p(v), _p(out), ctypes.c_int64(v.numel()))
    return out


def set_fp8_arith(mode: int) -> None:
    """0: the scale arithmetic of the reference's PyTorch statement (default); 1: the CUDA kernel's own."""
    lib().oracle_set_fp8_arith(int(mode))


def quantise_rows(x: torch.Tensor):
    """x [rows, H] bf16 -> (payload uint8 [rows, H], scales f32 [rows, H/128])."""
    assert x.dtype == torch.bfloat16 and x.dim() == 2 and x.size(1) % 128 == 0
    x = x.contiguous()
    rows, H = x.shape
    q = torch.empty((rows, H), dtype=torch.uint8)
    s = torch.empty((rows, H // 128), dtype=torch.float32)
    lib().oracle_quantise_rows(_p(x), ctypes.c_int64(rows), ctypes.c_int(H), _p(q), _p(s))
    return q, s


def layout(topk_idx: torch.Tensor, num_tokens: Sequence[int], max_tokens: int, num_experts: int,
           src_present: Optional[Sequence[int]] = None, poison: int = -7) -> Dict[str, torch.Tensor]:
    """topk_idx int64 [R, Tmax, K] -> recv_count [R,L], layout_range [R,L,R],
    src_info [R,L,RM] (unwritten rows keep `poison`), slot_map [R,Tmax,K]."""
    assert topk_idx.dtype == torch.int64 and topk_idx.dim() == 3
    topk_idx = topk_idx.contiguous()
    R, Tmax, K = topk_idx.shape
    E = num_experts
    L = E // R
    RM = R * max_tokens
    out = {
        "recv_count": torch.full((R, L), poison, dtype=torch.int32),
        "layout_range": torch.full((R, L, R), poison, dtype=torch.int64),
        "src_info": torch.full((R, L, RM), poison, dtype=torch.int32),
        "slot_map": torch.full((R, Tmax, K), poison, dtype=torch.int32),
    }
    nt = _i32(num_tokens)
    sp = None if src_present is None else _i32(src_present)
    lib().oracle_layout(R, E, K, Tmax, max_tokens, _p(nt), _p(topk_idx), _p(sp), _p(out["recv_count"]),
                        _p(out["layout_range"]), _p(out["src_info"]), _p(out["slot_map"]))
    return out


def dispatch(x: torch.Tensor, topk_idx: torch.Tensor, num_tokens: Sequence[int], max_tokens: int,
             num_experts: int, use_fp8: bool, src_present: Optional[Sequence[int]] = None,
             poison: Optional[int] = -7) -> Dict[str, torch.Tensor]:
    """Whole-world dispatch.  x bf16 [R, Tmax, H], topk_idx int64 [R, Tmax, K].

    Returns recv_x ([R,L,RM,H] float8_e4m3fn or bf16; unwritten rows keep the
    byte pattern 0xA5, or are uninitialised - and never touched, so that large
    worlds cost only their valid rows - when poison is None), scales (logical [R,L,RM,H/128] view of a physical
    [R,L,H/128,RM] tensor, or None), recv_count, src_info, layout_range, slot_map.
    """
    assert x.dtype == torch.bfloat16 and x.dim() == 3
    x = x.contiguous()
    topk_idx = topk_idx.contiguous()
    R, Tmax, H = x.shape
    K = topk_idx.size(2)
    E = num_experts
    L = E // R
    RM = R * max_tokens
    G = H // 128
    def _new(shape, dtype, fill):
        return torch.empty(shape, dtype=dtype) if poison is None else torch.full(shape, fill, dtype=dtype)

    if use_fp8:
        recv_x = _new((R, L, RM, H), torch.uint8, 0xA5)
        scales_phys = _new((R, L, G, RM), torch.float32, float("nan"))
    else:
        recv_x = _new((R, L, RM, H), torch.int16, 0xA5A5 - 65536)
        scales_phys = None
    out = {
        "recv_count": _new((R, L), torch.int32, poison),
        "layout_range": _new((R, L, R), torch.int64, poison),
        "src_info": _new((R, L, RM), torch.int32, poison),
        "slot_map": _new((R, Tmax, K), torch.int32, poison),
    }
    nt = _i32(num_tokens)
    sp = None if src_present is None else _i32(src_present)
    lib().oracle_dispatch(R, E, K, Tmax, max_tokens, H, int(bool(use_fp8)), _p(nt), _p(x), _p(topk_idx), _p(sp),
                          _p(recv_x), _p(scales_phys), _p(out["recv_count"]), _p(out["layout_range"]),
                          _p(out["src_info"]), _p(out["slot_map"]))
    out["recv_x"] = recv_x.view(torch.float8_e4m3fn) if use_fp8 else recv_x.view(torch.bfloat16)
    out["scales"] = None if scales_phys is None else scales_phys.transpose(2, 3)
    return out


def combine(expert_out: torch.Tensor, topk_idx: torch.Tensor, topk_weights: torch.Tensor,
            src_info: torch.Tensor, layout_range: torch.Tensor, num_tokens: Sequence[int], max_tokens: int,
            num_experts: int, active: Optional[torch.Tensor] = None, use_fma: bool = True) -> torch.Tensor:
    """Whole-world combine.  expert_out bf16 [R, L, RM, H]; returns bf16
    [R, Tmax, H] with rows >= num_tokens[r] zeroed."""
    assert expert_out.dtype == torch.bfloat16 and expert_out.dim() == 4
    expert_out = expert_out.contiguous()
    topk_idx = topk_idx.contiguous()
    topk_weights = topk_weights.contiguous().float()
    R, Tmax, K = topk_idx.shape
    H = expert_out.size(3)
    out = torch.zeros((R, Tmax, H), dtype=torch.bfloat16)
    nt = _i32(num_tokens)
    act = None if active is None else active.contiguous().to(torch.int32)
    if act is not None:
        assert act.shape == (R, R)
    lib().oracle_combine(R, num_experts, K, Tmax, max_tokens, H, int(bool(use_fma)), _p(nt), _p(expert_out),
                         _p(topk_idx), _p(topk_weights), _p(src_info.contiguous()), _p(layout_range.contiguous()),
                         _p(act), _p(out))
    return out


def cast_back(recv_x: torch.Tensor, scales: Optional[torch.Tensor], recv_count: torch.Tensor,
              factor: Optional[torch.Tensor] = None, fill: int = 0) -> torch.Tensor:
    """Valid packed rows -> bf16.  recv_x [R, L, RM, H] float8_e4m3fn / uint8 (with scales: the logical
    [R, L, RM, H/128] view dispatch returns, or any tensor of that shape) or bf16 (scales None);
    factor f32 [E] or None.  Rows at and beyond recv_count keep the 16-bit pattern `fill`."""
    R, L, RM, H = recv_x.shape
    phys = None
    if scales is not None:
        phys = scales.transpose(2, 3).contiguous().float()          # [R, L, H/128, RM]
        raw = recv_x.contiguous().view(torch.uint8)
    else:
        assert recv_x.dtype == torch.bfloat16
        raw = recv_x.contiguous()
    out = torch.full((R, L, RM, H), fill, dtype=torch.int16)
    cnt = recv_count.contiguous().to(torch.int32)
    f = None if factor is None else factor.contiguous().float()
    lib().oracle_cast_back(R * L, RM, H, _p(raw), _p(phys), _p(cnt), _p(f), _p(out))
    return out.view(torch.bfloat16)


def buffer_size_hint(max_tokens: int, hidden: int, num_ranks: int, num_experts: int) -> int:
    return int(lib().oracle_buffer_size_hint(max_tokens, hidden, num_ranks, num_experts))


def set_threads(n: int) -> None:
    """OpenMP thread count for the payload loops (cpu_baseline reports it)."""
    gomp = ctypes.CDLL("libgomp.so.1")
    gomp.omp_set_num_threads(int(n))
