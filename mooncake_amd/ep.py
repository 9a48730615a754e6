"""Replacement for the reference's native module `mooncake._ep`
(mooncake-ep/src/ep_py.cpp:14-46, loaded through mooncake/ep.py:10-17):
`Buffer`, `EventHandle`, `get_ep_buffer_size_hint`, `MAX_QP_COUNT`, with the
bound names and argument order of the reference, on top of the C ABI.

Two bindings of the same C ABI exist.  The compiled one, `mooncake_amd._ep`
(pybind11, csrc/ep_py.cpp - what the reference's own module is), is the one
used; `MOONCAKE_AMD_EP_BINDING=ctypes` selects the ctypes binding in this file
instead (a build without a host compiler).  `BINDING` names the one in use.
Either way every call ends in libmooncake_ep_hip.so: there is no other
implementation behind this module.

One GPU holds the whole expert-parallel world: Buffers created with the same
`World` (or, by default, with the same `num_ranks` in this process) are the
logical ranks of one world.
"""
from __future__ import annotations

import collections
import ctypes
import os
from ctypes import c_void_p
from typing import Callable, Dict, List, Optional, Sequence, Tuple

# PyTorch first, as in the reference's ep.py (mooncake-wheel/mooncake/ep.py:4): a ROCm build of PyTorch ships
# its own HIP runtime, and the library must bind to that one - the runtime that owns the tensors it is handed -
# rather than bring a second one into the process by being loaded before it.
import torch  # noqa: F401

from . import _lib

MAX_QP_COUNT = 256   # mooncake_ep_configs.cuh:5
PendingError = _lib.PendingError   # raised by either binding for MC_EP_ERR_PENDING

_native = None
if os.environ.get("MOONCAKE_AMD_EP_BINDING", "pybind11") != "ctypes":
    try:
        from . import _ep as _native
    except ImportError as exc:
        raise ImportError(
            "mooncake_amd._ep (the compiled Python module) is not built; run "
            f"`make -C {os.path.join(os.path.dirname(os.path.abspath(__file__)), 'csrc')}` "
            "or set MOONCAKE_AMD_EP_BINDING=ctypes") from exc
    assert _native.MAX_QP_COUNT == MAX_QP_COUNT
BINDING = "pybind11" if _native is not None else "ctypes"


def get_ep_buffer_size_hint(num_max_dispatch_tokens_per_rank: int, hidden: int, num_ranks: int,
                            num_experts: int) -> int:
    return int(_lib.lib().mc_ep_get_buffer_size_hint(num_max_dispatch_tokens_per_rank, hidden, num_ranks,
                                                     num_experts))


class World:
    """R logical EP ranks resident in the current device's HBM."""

    def __init__(self, num_ranks: int):
        _lib.lib()                       # the HIP library itself must load, whichever binding is used
        if _native is not None:
            # the compiled module owns the world (its Buffers, events and hooks keep it alive)
            self._native = _native.World(int(num_ranks))
            self._h = c_void_p(self._native.handle)
        else:
            self._native = None
            handle = c_void_p()
            _lib.check(_lib.lib().mc_ep_world_create(int(num_ranks), ctypes.byref(handle)))
            self._h = handle
        self.num_ranks = int(num_ranks)

    def close(self) -> None:
        if self._native is not None:
            self._native = None          # destroyed when the last Buffer / event / hook of the world goes
            self._h = None
        elif self._h:
            _lib.lib().mc_ep_world_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_rank_silent(self, rank: int, silent: bool = True) -> None:
        """The rank stops calling dispatch/combine (a failed process)."""
        _lib.check(_lib.lib().mc_ep_world_set_rank_silent(self._h, int(rank), int(bool(silent))))

    def set_option(self, name: str, value: int) -> None:
        _lib.check(_lib.lib().mc_ep_world_set_option(self._h, name.encode(), int(value)))

    def get_option(self, name: str) -> int:
        out = ctypes.c_int()
        _lib.check(_lib.lib().mc_ep_world_get_option(self._h, name.encode(), ctypes.byref(out)))
        return out.value

    # whole-world calls: every rank's tensors in one launch sequence.  The
    # prepare_* forms marshal the per-rank pointer arrays once and return a
    # callable (stream_ptr, phases) for callers that repeat the same call.
    def prepare_dispatch(self, x_ptrs, topk_idx_ptrs, num_tokens, hidden, num_topk,
                         num_max_dispatch_tokens_per_rank, num_experts, use_fp8, recv_x_ptrs, recv_scales_ptrs,
                         recv_count_ptrs, src_info_ptrs, layout_range_ptrs):
        if self._native is not None:
            return self._native.prepare_dispatch(
                [int(v) for v in x_ptrs], [int(v) for v in topk_idx_ptrs], [int(v) for v in num_tokens], hidden,
                num_topk, num_max_dispatch_tokens_per_rank, num_experts, bool(use_fp8),
                [int(v) for v in recv_x_ptrs],
                [int(v) for v in recv_scales_ptrs] if (use_fp8 and recv_scales_ptrs is not None) else None,
                [int(v) for v in recv_count_ptrs], [int(v) for v in src_info_ptrs],
                [int(v) for v in layout_range_ptrs])
        u = _lib.u64_array
        fn = _lib.lib().mc_ep_world_dispatch
        args = (self._h, u(x_ptrs), u(topk_idx_ptrs), _lib.i32_array(num_tokens), hidden, num_topk,
                num_max_dispatch_tokens_per_rank, num_experts, int(bool(use_fp8)), u(recv_x_ptrs),
                u(recv_scales_ptrs) if recv_scales_ptrs is not None else None, u(recv_count_ptrs),
                u(src_info_ptrs), u(layout_range_ptrs))

        def call(stream_ptr: int, phases: int = _lib.PHASE_ALL) -> None:
            rc = fn(*args, phases, stream_ptr)
            if rc:
                _lib.check(rc)
        return call

    def dispatch_noalloc(self, x_ptrs, topk_idx_ptrs, num_tokens, hidden, num_topk, num_max_dispatch_tokens_per_rank,
                         num_experts, use_fp8, recv_x_ptrs, recv_scales_ptrs, recv_count_ptrs, src_info_ptrs,
                         layout_range_ptrs, stream_ptr: int) -> None:
        """`dispatch` without any device allocation: its scratch is the library's static device array
        (16 MiB per GPU, shared by every call on that GPU); larger shapes raise."""
        u = _lib.u64_array
        _lib.check(_lib.lib().mc_ep_world_dispatch_noalloc(
            self._h, u(x_ptrs), u(topk_idx_ptrs), _lib.i32_array(num_tokens), hidden, num_topk,
            num_max_dispatch_tokens_per_rank, num_experts, int(bool(use_fp8)), u(recv_x_ptrs),
            u(recv_scales_ptrs) if recv_scales_ptrs is not None else None, u(recv_count_ptrs), u(src_info_ptrs),
            u(layout_range_ptrs), stream_ptr))

    def prepare_combine(self, x_ptrs, topk_idx_ptrs, topk_weights_ptrs, src_info_ptrs, layout_range_ptrs,
                        active_ranks_ptrs, num_combined_tokens, hidden, num_topk, num_max_dispatch_tokens_per_rank,
                        num_experts, combined_x_ptrs):
        if self._native is not None:
            ints = lambda vs: [int(v) for v in vs]
            return self._native.prepare_combine(
                ints(x_ptrs), None, 0, False, ints(topk_idx_ptrs), ints(topk_weights_ptrs), ints(src_info_ptrs),
                ints(layout_range_ptrs), ints(active_ranks_ptrs), ints(num_combined_tokens), hidden, num_topk,
                num_max_dispatch_tokens_per_rank, num_experts, ints(combined_x_ptrs))
        u = _lib.u64_array
        fn = _lib.lib().mc_ep_world_combine
        args = (self._h, u(x_ptrs), u(topk_idx_ptrs), u(topk_weights_ptrs), u(src_info_ptrs), u(layout_range_ptrs),
                u(active_ranks_ptrs), _lib.i32_array(num_combined_tokens), hidden, num_topk,
                num_max_dispatch_tokens_per_rank, num_experts, u(combined_x_ptrs))

        def call(stream_ptr: int, phases: int = _lib.PHASE_ALL) -> None:
            rc = fn(*args, phases, stream_ptr)
            if rc:
                _lib.check(rc)
        return call

    def prepare_combine_packed(self, recv_x_ptrs, recv_scales_ptrs, expert_factor_ptr, topk_idx_ptrs,
                               topk_weights_ptrs, src_info_ptrs, layout_range_ptrs, active_ranks_ptrs,
                               num_combined_tokens, hidden, num_topk, num_max_dispatch_tokens_per_rank, num_experts,
                               combined_x_ptrs):
        """Combine straight from dispatch's packed output (fp8 payload with scales, or bf16 when
        recv_scales_ptrs is None) times expert_factor[expert] (0: none): cast_back + combine in one."""
        if self._native is not None:
            ints = lambda vs: [int(v) for v in vs]
            return self._native.prepare_combine(
                ints(recv_x_ptrs), ints(recv_scales_ptrs) if recv_scales_ptrs is not None else None,
                int(expert_factor_ptr), True, ints(topk_idx_ptrs), ints(topk_weights_ptrs), ints(src_info_ptrs),
                ints(layout_range_ptrs), ints(active_ranks_ptrs), ints(num_combined_tokens), hidden, num_topk,
                num_max_dispatch_tokens_per_rank, num_experts, ints(combined_x_ptrs))
        u = _lib.u64_array
        fn = _lib.lib().mc_ep_world_combine_packed
        args = (self._h, u(recv_x_ptrs), u(recv_scales_ptrs) if recv_scales_ptrs is not None else None,
                int(expert_factor_ptr), u(topk_idx_ptrs), u(topk_weights_ptrs), u(src_info_ptrs),
                u(layout_range_ptrs), u(active_ranks_ptrs), _lib.i32_array(num_combined_tokens), hidden, num_topk,
                num_max_dispatch_tokens_per_rank, num_experts, u(combined_x_ptrs))

        def call(stream_ptr: int, phases: int = _lib.PHASE_ALL) -> None:
            rc = fn(*args, phases, stream_ptr)
            if rc:
                _lib.check(rc)
        return call

    def dispatch(self, x_ptrs, topk_idx_ptrs, num_tokens, hidden, num_topk, num_max_dispatch_tokens_per_rank,
                 num_experts, use_fp8, recv_x_ptrs, recv_scales_ptrs, recv_count_ptrs, src_info_ptrs,
                 layout_range_ptrs, stream_ptr: int, phases: int = _lib.PHASE_ALL) -> None:
        self.prepare_dispatch(x_ptrs, topk_idx_ptrs, num_tokens, hidden, num_topk, num_max_dispatch_tokens_per_rank,
                              num_experts, use_fp8, recv_x_ptrs, recv_scales_ptrs, recv_count_ptrs, src_info_ptrs,
                              layout_range_ptrs)(stream_ptr, phases)

    def combine(self, x_ptrs, topk_idx_ptrs, topk_weights_ptrs, src_info_ptrs, layout_range_ptrs,
                active_ranks_ptrs, num_combined_tokens, hidden, num_topk, num_max_dispatch_tokens_per_rank,
                num_experts, combined_x_ptrs, stream_ptr: int, phases: int = _lib.PHASE_ALL) -> None:
        self.prepare_combine(x_ptrs, topk_idx_ptrs, topk_weights_ptrs, src_info_ptrs, layout_range_ptrs,
                             active_ranks_ptrs, num_combined_tokens, hidden, num_topk,
                             num_max_dispatch_tokens_per_rank, num_experts, combined_x_ptrs)(stream_ptr, phases)


    def cast_back(self, recv_x_ptrs, recv_scales_ptrs, recv_count_ptrs, expert_factor_ptr: int, out_ptrs,
                  hidden: int, num_topk: int, num_max_dispatch_tokens_per_rank: int, num_experts: int,
                  stream_ptr: int) -> None:
        """Valid packed rows -> bf16 rows (fp8 payload times its scales; bf16 payload when
        recv_scales_ptrs is None), times expert_factor[expert] when a factor array is given."""
        u = _lib.u64_array
        _lib.check(_lib.lib().mc_ep_world_cast_back(
            self._h, u(recv_x_ptrs), u(recv_scales_ptrs) if recv_scales_ptrs is not None else None,
            u(recv_count_ptrs), int(expert_factor_ptr), u(out_ptrs), hidden, num_topk,
            num_max_dispatch_tokens_per_rank, num_experts, stream_ptr))

    def legacy_buffer_perf(self, tensors: Dict[str, Sequence[int]], num_tokens: int, hidden: int, num_topk: int,
                           num_local_experts: int, num_max_dispatch_tokens_per_rank: int, num_experts: int,
                           warmups: int = 20, iterations: int = 30, timeout_us: int = -1,
                           compute_stream_ptr: int = 0) -> Tuple[float, float, float]:
        """The native loop `mooncake._ep._benchmark_legacy_buffer` runs
        (mooncake-ep/benchmarks/legacy_buffer_perf.cpp:84-146), over the whole
        world: returns (average_us, min_us, max_us) of recv_count clear + bf16
        dispatch + combine.  `tensors` maps the field names of
        LegacyBufferPerfTensors (x_ptr -> "x", ...) to per-rank addresses."""
        if self._native is not None:
            # the compiled module's binding of the loop, as the reference's script calls it
            # (mooncake-ep/benchmarks/legacy_buffer_perf.py:84-107)
            nt, nc = _native._LegacyBufferPerfTensors(), _native._LegacyBufferPerfConfig()
            for field, _ in _lib.LegacyPerfTensors._fields_:
                values = tensors.get(field[:-len("_ptrs")])
                setattr(nt, field[:-1], [int(v) for v in values] if values is not None else [])
            nc.num_tokens, nc.hidden, nc.num_topk, nc.num_local_experts = num_tokens, hidden, num_topk, num_local_experts
            nc.num_max_dispatch_tokens_per_rank, nc.num_experts = num_max_dispatch_tokens_per_rank, num_experts
            nc.timeout_us, nc.warmups, nc.iterations = timeout_us, warmups, iterations
            nc.compute_stream_ptr = int(compute_stream_ptr)
            res = _native._benchmark_legacy_buffer(self._native, nt, nc)
            return res.average_us, res.min_us, res.max_us
        t = _lib.LegacyPerfTensors()
        keep = []
        for field, _ in _lib.LegacyPerfTensors._fields_:
            values = tensors.get(field[:-len("_ptrs")])
            arr = _lib.u64_array(values) if values is not None else None
            keep.append(arr)
            setattr(t, field, arr)
        c = _lib.LegacyPerfConfig(num_tokens, hidden, num_topk, num_local_experts, num_max_dispatch_tokens_per_rank,
                                  num_experts, timeout_us, warmups, iterations, compute_stream_ptr)
        r = _lib.LegacyPerfResult()
        _lib.check(_lib.lib().mc_ep_world_legacy_buffer_perf(self._h, ctypes.byref(t), ctypes.byref(c),
                                                             ctypes.byref(r)))
        return r.average_us, r.min_us, r.max_us


_default_worlds: Dict[int, World] = {}


def default_world(num_ranks: int) -> World:
    """The process-wide world that Buffers of `num_ranks` ranks join unless told otherwise."""
    w = _default_worlds.get(num_ranks)
    if w is None or w._h is None:
        w = World(num_ranks)
        _default_worlds[num_ranks] = w
    return w


class _CtypesEventHandle:
    """mooncake_ep_event.h:9-42 (ctypes binding)."""

    def __init__(self, stream_ptr: int = 0, _handle: Optional[c_void_p] = None):
        if _handle is not None:
            self._h = _handle
        else:
            handle = c_void_p()
            _lib.check(_lib.lib().mc_ep_event_create(int(stream_ptr), ctypes.byref(handle)))
            self._h = handle

    def current_stream_wait(self, stream_ptr: int) -> None:
        _lib.check(_lib.lib().mc_ep_event_current_stream_wait(self._h, int(stream_ptr)))

    def synchronize(self) -> None:
        _lib.check(_lib.lib().mc_ep_event_synchronize(self._h))

    def __del__(self):
        try:
            if self._h:
                _lib.lib().mc_ep_event_destroy(self._h)
                self._h = None
        except Exception:
            pass


class _RecvHook:
    def __init__(self, handle: c_void_p, world: "World"):
        self._h = handle
        self._world = world          # the hook enqueues work of its world: keep it alive

    def __call__(self) -> None:
        _lib.check(_lib.lib().mc_ep_hook_call(self._h))

    def __del__(self):
        try:
            if self._h:
                _lib.lib().mc_ep_hook_destroy(self._h)
                self._h = None
        except Exception:
            pass


class _CtypesBuffer:
    """One logical rank's MooncakeEpBuffer (ep_py.cpp:26-46), ctypes binding."""

    def __init__(self, rank: int, num_ranks: int, num_ep_buffer_bytes: int, disable_p2p: bool = False,
                 world: Optional[World] = None):
        self.world = world if world is not None else default_world(num_ranks)
        if self.world.num_ranks != num_ranks:
            raise RuntimeError(f"world has {self.world.num_ranks} ranks, Buffer asked for {num_ranks}")
        handle = c_void_p()
        _lib.check(_lib.lib().mc_ep_buffer_create(self.world._h, int(rank), int(num_ep_buffer_bytes),
                                                  int(bool(disable_p2p)), ctypes.byref(handle)))
        self._h = handle
        self.rank = int(rank)
        self.num_ranks = int(num_ranks)
        self._kept = (collections.deque(), collections.deque())   # keep_alive objects: dispatch, combine

    def _retain(self, kind: int, rc: int, keep_alive) -> None:
        """Holds a call's `keep_alive` until the call's round has been enqueued (also for a call that gave up
        waiting for its peers and stays posted), as the compiled module's Buffer does."""
        if keep_alive is None or rc not in (_lib.OK, _lib.ERR_PENDING):
            return
        kept = self._kept[kind]
        kept.append(keep_alive)
        pending = self.pending_calls()[kind]
        while len(kept) > pending:
            kept.popleft()

    def retained(self) -> Tuple[int, int]:
        return len(self._kept[0]), len(self._kept[1])

    def __del__(self):
        try:
            if self._h:
                _lib.lib().mc_ep_buffer_destroy(self._h)
                self._h = None
        except Exception:
            pass

    def pending_calls(self) -> Tuple[int, int]:
        """(dispatch, combine) calls of this rank whose kernels are not all enqueued yet."""
        d, c = ctypes.c_int(), ctypes.c_int()
        _lib.check(_lib.lib().mc_ep_buffer_pending_calls(self._h, ctypes.byref(d), ctypes.byref(c)))
        return d.value, c.value

    # --- transport introspection: one address space, no NIC ---------------
    def ibgda_disabled(self) -> bool:
        return bool(_lib.lib().mc_ep_buffer_ibgda_disabled(self._h))

    def p2p_enabled(self) -> bool:
        return bool(_lib.lib().mc_ep_buffer_p2p_enabled(self._h))

    def use_fast_path(self) -> bool:
        return bool(_lib.lib().mc_ep_buffer_use_fast_path(self._h))

    def is_roce(self) -> bool:
        return bool(_lib.lib().mc_ep_buffer_is_roce(self._h))

    def update_local_qpns(self) -> None:
        return None

    def sync_ibgda_peers(self, remote_addrs, remote_keys, peer_qpns, peer_lids, subnet_prefixes, interface_ids,
                         active_ranks_mask) -> None:
        return None

    def get_mr_info(self) -> Tuple[int, int]:
        return (0, 0)

    def get_gid(self) -> Tuple[int, int]:
        return (0, 0)

    def get_local_qpns(self) -> List[int]:
        return []

    def get_local_lids(self) -> List[int]:
        return []

    def get_ipc_handle(self) -> List[int]:
        return []

    def sync_nvlink_ipc_handles(self, remote_handles, active_ranks_mask) -> None:
        return None

    # --- the two hot calls ------------------------------------------------
    def dispatch(self, x_ptr: int, topk_idx_ptr: int, active_ranks_ptr: int, num_tokens: int, hidden: int,
                 num_topk: int, num_max_dispatch_tokens_per_rank: int, num_experts: int, timeout_us: int,
                 use_fp8: bool, packed_recv_x_ptr: int, packed_recv_x_scales_ptr: int, packed_recv_count_ptr: int,
                 packed_recv_src_info_ptr: int, packed_recv_layout_range_ptr: int, async_: bool,
                 return_recv_hook: bool, compute_stream_ptr: int, keep_alive=None
                 ) -> Tuple[Optional[object], Optional[Callable[[], None]]]:
        ev, hook = c_void_p(), c_void_p()
        rc = (_lib.lib().mc_ep_buffer_dispatch(
            self._h, x_ptr, topk_idx_ptr, active_ranks_ptr, num_tokens, hidden, num_topk,
            num_max_dispatch_tokens_per_rank, num_experts, timeout_us, int(bool(use_fp8)), packed_recv_x_ptr,
            packed_recv_x_scales_ptr, packed_recv_count_ptr, packed_recv_src_info_ptr,
            packed_recv_layout_range_ptr, int(bool(async_)), int(bool(return_recv_hook)), compute_stream_ptr,
            ctypes.byref(ev), ctypes.byref(hook)))
        self._retain(0, rc, keep_alive)
        _lib.check(rc)
        return (_CtypesEventHandle(_handle=ev) if ev else None, _RecvHook(hook, self.world) if hook else None)

    def combine(self, x_ptr: int, topk_idx_ptr: int, topk_weights_ptr: int, src_info_ptr: int,
                layout_range_ptr: int, active_ranks_ptr: int, num_local_experts: int, num_combined_tokens: int,
                hidden: int, num_topk: int, num_max_dispatch_tokens_per_rank: int, num_experts: int,
                timeout_us: int, zero_copy: bool, combined_x_ptr: int, async_: bool, return_recv_hook: bool,
                compute_stream_ptr: int, keep_alive=None) -> Tuple[Optional[object], Optional[Callable[[], None]]]:
        ev, hook = c_void_p(), c_void_p()
        rc = (_lib.lib().mc_ep_buffer_combine(
            self._h, x_ptr, topk_idx_ptr, topk_weights_ptr, src_info_ptr, layout_range_ptr, active_ranks_ptr,
            num_local_experts, num_combined_tokens, hidden, num_topk, num_max_dispatch_tokens_per_rank,
            num_experts, timeout_us, int(bool(zero_copy)), combined_x_ptr, int(bool(async_)),
            int(bool(return_recv_hook)), compute_stream_ptr, ctypes.byref(ev), ctypes.byref(hook)))
        self._retain(1, rc, keep_alive)
        _lib.check(rc)
        return (_CtypesEventHandle(_handle=ev) if ev else None, _RecvHook(hook, self.world) if hook else None)


if _native is not None:
    EventHandle = _native.EventHandle

    class Buffer(_native.Buffer):
        """One logical rank's MooncakeEpBuffer (ep_py.cpp:26-46): the compiled module's class, which takes
        the world it belongs to as this package's `World`."""

        def __init__(self, rank: int, num_ranks: int, num_ep_buffer_bytes: int, disable_p2p: bool = False,
                     world: Optional[World] = None):
            w = world if world is not None else default_world(num_ranks)
            if w.num_ranks != num_ranks:
                raise RuntimeError(f"world has {w.num_ranks} ranks, Buffer asked for {num_ranks}")
            _native.Buffer.__init__(self, int(rank), int(num_ranks), int(num_ep_buffer_bytes), bool(disable_p2p),
                                    w._native)
            self._world = w

    _benchmark_legacy_buffer = _native._benchmark_legacy_buffer
    _LegacyBufferPerfTensors = _native._LegacyBufferPerfTensors
    _LegacyBufferPerfConfig = _native._LegacyBufferPerfConfig
    _LegacyBufferPerfResult = _native._LegacyBufferPerfResult
else:
    EventHandle = _CtypesEventHandle
    Buffer = _CtypesBuffer
