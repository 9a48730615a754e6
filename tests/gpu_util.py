"""Helpers shared by the GPU parity tests: run the HIP path through the C ABI
for a whole logical world and compare it with the CPU oracle on the same
seeded inputs."""
import sys
from typing import Dict, Optional, Sequence

import torch

from mooncake_amd.harness import WorldHarness, valid_rows
from mooncake_amd.workloads import EPConfig


def announce(msg: str) -> None:
    print(f"[gpu-case] {msg}", flush=True)
    sys.stdout.flush()


# library options every world made by run_dispatch gets before the test's own (set by the `fused_small`
# fixture of conftest.py, which runs a test once per dispatch path)
DEFAULT_OPTIONS: Dict[str, int] = {}


def run_dispatch(cfg: EPConfig, data: Dict[str, torch.Tensor], num_tokens: Optional[Sequence[int]] = None,
                 poison: bool = True, present: Optional[Sequence[int]] = None, options: Optional[dict] = None):
    h = WorldHarness(cfg, num_tokens=num_tokens)
    for k, v in {**DEFAULT_OPTIONS, **(options or {})}.items():
        h.world.set_option(k, v)
    h.load(data)
    h.alloc_dispatch_outputs(poison=poison)
    h.dispatch(present=present)
    torch.cuda.synchronize()
    return h


def compare_dispatch(h: WorldHarness, ref: Dict[str, torch.Tensor], check_poison: bool) -> None:
    """Bit-exact: counts, ranges, src_info / payload / scales on valid rows;
    rows at and beyond recv_count untouched when the outputs were poisoned."""
    cfg = h.cfg
    cnt = h.recv_count.cpu()
    assert torch.equal(cnt, ref["recv_count"]), "recv_count"
    assert torch.equal(h.layout_range.cpu(), ref["layout_range"]), "layout_range"
    assert torch.equal(valid_rows(h.src_info, h.recv_count).cpu(), valid_rows(ref["src_info"], cnt)), "src_info"
    got_rows = valid_rows(h.recv_x, h.recv_count).cpu()
    ref_x = ref["recv_x"].view(torch.uint8) if cfg.use_fp8 else ref["recv_x"].view(torch.int16)
    assert torch.equal(got_rows, valid_rows(ref_x, cnt)), "payload rows"
    if cfg.use_fp8:
        got_s = valid_rows(h.recv_scales().contiguous(), h.recv_count).cpu().view(torch.int32)
        ref_s = valid_rows(ref["scales"].contiguous(), cnt).view(torch.int32)
        assert torch.equal(got_s, ref_s), "scales"
    if check_poison:
        RM = cfg.num_ranks * cfg.max_tokens
        ar = torch.arange(RM, device=h.recv_x.device).view(1, 1, RM)
        pad = ar >= h.recv_count.unsqueeze(-1).to(torch.int64)
        assert bool((h.src_info[pad] == -7).all()), "src_info padding written"
        fill = 0xA5 if cfg.use_fp8 else 0xA5A5 - 65536
        assert bool((h.recv_x[pad] == fill).all()), "payload padding written"
        if cfg.use_fp8:
            assert bool(torch.isnan(h.recv_scales()[pad]).all()), "scale padding written"
