"""Whole-world driver for tests and benchmarks: keeps every logical rank's
tensors of one `EPConfig` on the device and calls the library's whole-world
entry points (one launch sequence for all ranks).

Per-rank tensors are slices of rank-major allocations, so rank r's
`packed_recv_x` is `recv_x[r]` with the reference's per-rank shape
`[num_local_experts, num_ranks * max_tokens, hidden]`.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from . import _lib, ep
from .workloads import EPConfig


class WorldHarness:
    def __init__(self, cfg: EPConfig, device: str = "cuda", world: Optional[ep.World] = None,
                 num_tokens: Optional[Sequence[int]] = None):
        self.cfg = cfg
        self.device = torch.device(device)
        self.world = world if world is not None else ep.World(cfg.num_ranks)
        R, T = cfg.num_ranks, cfg.tokens_per_rank
        self.num_tokens: List[int] = list(num_tokens) if num_tokens is not None else [T] * R
        assert len(self.num_tokens) == R and all(0 <= t <= cfg.max_tokens for t in self.num_tokens)
        self.x = self.topk_idx = self.topk_weights = None
        self.recv_x = self.recv_scales_phys = self.recv_count = self.src_info = self.layout_range = None
        self.expert_out = self.combined = None
        self.active_ranks = torch.ones((R, R), dtype=torch.int32, device=self.device)
        self._prepared = {}     # marshalled whole-world calls, keyed by (kind, present)

    # ------------------------------------------------------------------
    def load(self, data: Dict[str, torch.Tensor]) -> None:
        self.x = data["x"].to(self.device).contiguous()
        self.topk_idx = data["topk_idx"].to(self.device).contiguous()
        self.topk_weights = data["topk_weights"].to(self.device).contiguous()

    def alloc_dispatch_outputs(self, poison: bool = False) -> None:
        c = self.cfg
        R, L, RM, H = c.num_ranks, c.num_local_experts, c.num_ranks * c.max_tokens, c.hidden
        dev = self.device
        if c.use_fp8:
            self.recv_x = torch.empty((R, L, RM, H), dtype=torch.uint8, device=dev)
            self.recv_scales_phys = torch.empty((R, L, H // 128, RM), dtype=torch.float32, device=dev)
        else:
            self.recv_x = torch.empty((R, L, RM, H), dtype=torch.int16, device=dev)
            self.recv_scales_phys = None
        self.recv_count = torch.empty((R, L), dtype=torch.int32, device=dev)
        self.src_info = torch.empty((R, L, RM), dtype=torch.int32, device=dev)
        self.layout_range = torch.empty((R, L, R), dtype=torch.int64, device=dev)
        if poison:
            self.recv_x.fill_(0xA5 if c.use_fp8 else 0xA5A5 - 65536)
            if self.recv_scales_phys is not None:
                self.recv_scales_phys.fill_(float("nan"))
            self.recv_count.fill_(-7)
            self.src_info.fill_(-7)
            self.layout_range.fill_(-7)

    def alloc_combine_io(self) -> None:
        c = self.cfg
        R, L, RM, H = c.num_ranks, c.num_local_experts, c.num_ranks * c.max_tokens, c.hidden
        if self.expert_out is None:
            self.expert_out = torch.empty((R, L, RM, H), dtype=torch.bfloat16, device=self.device)
        self.combined = torch.empty((R, c.tokens_per_rank, H), dtype=torch.bfloat16, device=self.device)

    # ------------------------------------------------------------------
    @staticmethod
    def _ptrs(t: Optional[torch.Tensor], R: int, present: Optional[Sequence[int]] = None) -> List[int]:
        if t is None:
            return [0] * R
        return [t[r].data_ptr() if (present is None or present[r]) else 0 for r in range(R)]

    def _stream(self, stream: Optional[torch.cuda.Stream]) -> int:
        s = stream if stream is not None else torch.cuda.current_stream(self.device)
        return int(s.cuda_stream)

    def dispatch(self, phases: int = _lib.PHASE_ALL, stream: Optional[torch.cuda.Stream] = None,
                 present: Optional[Sequence[int]] = None, noalloc: bool = False) -> None:
        """present[r] == 0 makes rank r silent: it neither sends nor receives.  noalloc: through the
        allocation-free entry point (all phases)."""
        c = self.cfg
        R = c.num_ranks
        if noalloc:
            nt = [n if (present is None or present[r]) else 0 for r, n in enumerate(self.num_tokens)]
            self.world.dispatch_noalloc(
                self._ptrs(self.x, R), self._ptrs(self.topk_idx, R), nt, c.hidden, c.num_topk, c.max_tokens,
                c.num_experts, c.use_fp8, self._ptrs(self.recv_x, R, present),
                self._ptrs(self.recv_scales_phys, R, present) if c.use_fp8 else None,
                self._ptrs(self.recv_count, R, present), self._ptrs(self.src_info, R, present),
                self._ptrs(self.layout_range, R, present), self._stream(stream))
            return
        key = ("dispatch", None if present is None else tuple(present), self.x.data_ptr(), self.recv_x.data_ptr())
        call = self._prepared.get(key)
        if call is None:
            nt = [n if (present is None or present[r]) else 0 for r, n in enumerate(self.num_tokens)]
            call = self.world.prepare_dispatch(
                self._ptrs(self.x, R), self._ptrs(self.topk_idx, R), nt, c.hidden, c.num_topk, c.max_tokens,
                c.num_experts, c.use_fp8, self._ptrs(self.recv_x, R, present),
                self._ptrs(self.recv_scales_phys, R, present) if c.use_fp8 else None,
                self._ptrs(self.recv_count, R, present), self._ptrs(self.src_info, R, present),
                self._ptrs(self.layout_range, R, present))
            self._prepared[key] = call
        call(self._stream(stream), phases)

    def combine(self, phases: int = _lib.PHASE_ALL, stream: Optional[torch.cuda.Stream] = None,
                present: Optional[Sequence[int]] = None) -> None:
        c = self.cfg
        R = c.num_ranks
        key = ("combine", None if present is None else tuple(present), self.expert_out.data_ptr(),
               self.combined.data_ptr(), self.src_info.data_ptr())
        call = self._prepared.get(key)
        if call is None:
            nt = [n if (present is None or present[r]) else 0 for r, n in enumerate(self.num_tokens)]
            call = self.world.prepare_combine(
                self._ptrs(self.expert_out, R, present), self._ptrs(self.topk_idx, R),
                self._ptrs(self.topk_weights, R), self._ptrs(self.src_info, R), self._ptrs(self.layout_range, R),
                self._ptrs(self.active_ranks, R), nt, c.hidden, c.num_topk, c.max_tokens, c.num_experts,
                self._ptrs(self.combined, R))
            self._prepared[key] = call
        call(self._stream(stream), phases)

    def combine_packed(self, factor_per_expert: Optional[torch.Tensor] = None, phases: int = _lib.PHASE_ALL,
                       stream: Optional[torch.cuda.Stream] = None, present: Optional[Sequence[int]] = None) -> None:
        """combined = combine(cast_back(recv_x, factor)) in one kernel, reading dispatch's packed output."""
        c = self.cfg
        R = c.num_ranks
        self._factor = None if factor_per_expert is None else \
            factor_per_expert.to(device=self.device, dtype=torch.float32).contiguous()
        fptr = 0 if self._factor is None else self._factor.data_ptr()
        key = ("combine_packed", None if present is None else tuple(present), self.recv_x.data_ptr(),
               self.combined.data_ptr(), self.src_info.data_ptr(), fptr)
        call = self._prepared.get(key)
        if call is None:
            nt = [n if (present is None or present[r]) else 0 for r, n in enumerate(self.num_tokens)]
            call = self.world.prepare_combine_packed(
                self._ptrs(self.recv_x, R, present),
                self._ptrs(self.recv_scales_phys, R, present) if c.use_fp8 else None, fptr,
                self._ptrs(self.topk_idx, R), self._ptrs(self.topk_weights, R), self._ptrs(self.src_info, R),
                self._ptrs(self.layout_range, R), self._ptrs(self.active_ranks, R), nt, c.hidden, c.num_topk,
                c.max_tokens, c.num_experts, self._ptrs(self.combined, R))
            self._prepared[key] = call
        call(self._stream(stream), phases)

    # ------------------------------------------------------------------
    def recv_x_typed(self) -> torch.Tensor:
        return self.recv_x.view(torch.float8_e4m3fn) if self.cfg.use_fp8 else self.recv_x.view(torch.bfloat16)

    def recv_scales(self) -> Optional[torch.Tensor]:
        """Logical [R, L, R*max, H/128] view of the column-major scales."""
        return None if self.recv_scales_phys is None else self.recv_scales_phys.transpose(2, 3)

    def cast_back(self, factor_per_expert: Optional[torch.Tensor] = None,
                  stream: Optional[torch.cuda.Stream] = None, present: Optional[Sequence[int]] = None) -> None:
        """expert_out = the dispatched rows as bf16 (times a per-expert factor), valid rows only, by the
        library's consumer kernel."""
        c = self.cfg
        R = c.num_ranks
        if self.expert_out is None:
            self.alloc_combine_io()
        self._factor = None if factor_per_expert is None else \
            factor_per_expert.to(device=self.device, dtype=torch.float32).contiguous()
        self.world.cast_back(self._ptrs(self.recv_x, R, present),
                             self._ptrs(self.recv_scales_phys, R, present) if c.use_fp8 else None,
                             self._ptrs(self.recv_count, R), 0 if self._factor is None else self._factor.data_ptr(),
                             self._ptrs(self.expert_out, R), c.hidden, c.num_topk, c.max_tokens, c.num_experts,
                             self._stream(stream))

    def fill_expert_out_from_recv(self, factor_per_expert: Optional[torch.Tensor] = None) -> None:
        """Mock expert: expert_out = dequantised dispatched rows (times a per-expert
        factor), rank by rank to bound temporaries."""
        c = self.cfg
        if self.expert_out is None:
            self.alloc_combine_io()
        R, L = c.num_ranks, c.num_local_experts
        for r in range(R):
            if c.use_fp8:
                v = self.recv_x[r].view(torch.float8_e4m3fn).float()
                s = self.recv_scales_phys[r].transpose(1, 2)            # [L, RM, G]
                v = (v.view(L, -1, c.hidden // 128, 128) * s.unsqueeze(-1)).view(L, -1, c.hidden)
            else:
                v = self.recv_x[r].view(torch.bfloat16).float()
            if factor_per_expert is not None:
                v = v * factor_per_expert[r * L:(r + 1) * L].view(L, 1, 1).to(v.device)
            self.expert_out[r] = v.to(torch.bfloat16)


def valid_rows(t: torch.Tensor, recv_count: torch.Tensor) -> torch.Tensor:
    """Rows [0, recv_count) of every (rank, local expert) block of a
    [R, L, RM, ...] tensor, concatenated in (rank, expert, row) order."""
    R, L, RM = t.shape[:3]
    counts = recv_count.reshape(-1).to(torch.int64)
    ar = torch.arange(RM, device=t.device).unsqueeze(0)
    mask = ar < counts.to(t.device).unsqueeze(1)            # [R*L, RM]
    flat = t.reshape(R * L, RM, *t.shape[3:])
    return flat[mask]
