"""Python `Buffer` for the low-latency dispatch/combine path with the
signature, checks and return shapes of the reference wrapper
(mooncake-wheel/mooncake/mooncake_ep_buffer.py:92-119, :360-535, :538-681),
running on the HIP library for one MI355X.

The expert-parallel world is a set of logical ranks in one process: a
`LogicalGroup` stands in for the torch process group (`rank()`, `size()`),
and dispatch/combine are collectives over the group's ranks - the kernels for
all ranks are launched by the call that completes the round, so outputs are
valid (in stream order) once every live rank has made its call.
"""
from __future__ import annotations

import sys
from typing import Any, Callable, Optional, Tuple, Union

import torch

from . import ep

_ZERO_COPY_COMBINE_UNSUPPORTED = (
    "Mooncake EP zero-copy combine is not supported; pass the expert output "
    "tensor to combine() with zero_copy=False"
)


# torch.cuda.current_stream() builds a Stream object behind several Python-level device look-ups (about 4 us
# a call, twice per dispatch or combine); torch's own raw-stream query gives the same address directly
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


_FAST_STREAM = _raw_stream is not None and _raw_device is not None


def _native_current_stream_ptr() -> int:
    if _FAST_STREAM:
        return int(_raw_stream(_raw_device()))
    return int(torch.cuda.current_stream().cuda_stream)


_storage_use_count = getattr(torch._C, "_storage_Use_Count", None)
_getrefcount = sys.getrefcount
_BF16, _I64, _I32, _F32, _FP8 = torch.bfloat16, torch.int64, torch.int32, torch.float32, torch.float8_e4m3fn


class _OutputPool:
    """Dispatch allocates five output tensors per call (reference :446-487).  A caller that has let go of an
    earlier call's outputs - no name, tuple, handle, view or keep-alive list refers to them any more - cannot
    tell a recycled tensor from a fresh one, and five `torch.empty` cost more host time than the rest of the
    call.  So the outputs of earlier calls are offered again, under exactly that condition: every tensor of the
    set is referenced by nothing but this pool (Python reference count) and its storage by nothing but that
    tensor (storage use count, which views and dtype reinterpretations raise).  Otherwise the call gets fresh
    tensors, as in the reference.  Sets are kept per shape, dtype, device and current stream - the caching
    allocator, too, reuses a freed block only for the stream it was allocated on - and at most `limit` of them,
    so memory held by the pool stays bounded (a caller that keeps every output alive pools nothing)."""

    limit = 4

    def __init__(self) -> None:
        self._sets: dict = {}

    @staticmethod
    def _count(t: torch.Tensor) -> int:
        return _storage_use_count(t.untyped_storage()._cdata)

    def find(self, key: tuple) -> Optional[list]:
        """A set of earlier outputs for `key` that nothing refers to any more, or None."""
        sets = self._sets.get(key)
        if sets is None or _storage_use_count is None:     # no way to see views of a storage: never recycle
            return None
        refs, uses = _getrefcount, _storage_use_count
        for tensors, baseline in sets:
            for i in range(len(tensors)):
                # tensors[i] inside the call: one reference from the list, one from the argument
                if refs(tensors[i]) != 2 or uses(tensors[i].untyped_storage()._cdata) != baseline[i]:
                    break
            else:
                return list(tensors)                       # the caller's own references
        return None

    def add(self, key: tuple, tensors: list) -> list:
        """Fresh outputs join the pool while it has room; returns the caller's own list of them."""
        if _storage_use_count is not None:
            sets = self._sets.setdefault(key, [])
            if len(sets) < self.limit:
                sets.append((tensors, [self._count(t) for t in tensors]))
                return list(tensors)
        return tensors

    def take(self, key: tuple, make: Callable[[], list]) -> list:
        found = self.find(key)
        return found if found is not None else self.add(key, make())


class LogicalGroup:
    """Stands in for `dist.ProcessGroup`: one logical rank of an `ep.World`."""

    def __init__(self, world: ep.World, rank: int):
        assert 0 <= rank < world.num_ranks
        self.world = world
        self._rank = int(rank)

    def rank(self) -> int:
        return self._rank

    def size(self) -> int:
        return self.world.num_ranks

    @staticmethod
    def make_world(num_ranks: int):
        """A fresh world and its R groups."""
        world = ep.World(num_ranks)
        return world, [LogicalGroup(world, r) for r in range(num_ranks)]


def spawn_ranks(fn: Callable, num_ranks: int, args: tuple = (), join_timeout: Optional[float] = None,
                block_timeout_ms: Optional[int] = None) -> list:
    """Runs `fn(rank, group, *args)` on one thread per logical rank of a fresh world and returns the ranks'
    results: the counterpart, for logical ranks, of the `torch.multiprocessing.spawn(worker, nprocs=world_size)`
    that the reference's tests start their per-rank code with (mooncake-ep/tests/test_ep_grid.py:412-430).
    `group` stands in for the process group (`Buffer(group, ...)`).  The world's per-rank calls block until their
    collective has been enqueued (option "blocking"), so `fn` may use a call's results as soon as the call
    returns, as a process of the reference does.  The first exception of any rank is raised again here."""
    import threading
    world, groups = LogicalGroup.make_world(num_ranks)
    world.set_option("blocking", 1)
    if block_timeout_ms is not None:
        world.set_option("block_timeout_ms", int(block_timeout_ms))
    device = torch.cuda.current_device() if torch.cuda.is_available() else None
    results: list = [None] * num_ranks
    errors: list = [None] * num_ranks

    def run(rank: int) -> None:
        try:
            if device is not None:
                torch.cuda.set_device(device)       # the current device is per thread
            results[rank] = fn(rank, groups[rank], *args)
        except BaseException as exc:                # noqa: BLE001 - handed to the caller below
            errors[rank] = exc
            # a rank that stops calling would leave its peers waiting for the time limit: take it out of their rounds
            try:
                world.set_rank_silent(rank)
            except Exception:                       # noqa: BLE001
                pass

    threads = [threading.Thread(target=run, args=(r,), name=f"ep-rank-{r}") for r in range(num_ranks)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(join_timeout)
    alive = [t.name for t in threads if t.is_alive()]
    for rank, exc in enumerate(errors):
        if exc is not None:
            raise RuntimeError(f"logical rank {rank} failed: {exc!r}") from exc
    if alive:
        raise TimeoutError(f"ranks still running after {join_timeout} s: {alive}")
    return results


class EventOverlap:
    """Event wrapper with the `with` protocol (reference :34-89)."""

    def __init__(self, event: Optional[ep.EventHandle] = None,
                 extra_tensors: Optional[Tuple[torch.Tensor, ...]] = None) -> None:
        self.event = event
        # keeps inputs/outputs alive until the event has been waited on
        self.extra_tensors = extra_tensors

    def current_stream_wait(self) -> None:
        assert self.event is not None
        self.event.current_stream_wait(_raw_stream(_raw_device()) if _FAST_STREAM else _native_current_stream_ptr())

    def __enter__(self) -> Any:
        return self

    def __exit__(self, exc_type: Any, exc_val: Any, exc_tb: Any) -> None:
        if self.event is not None:
            self.event.current_stream_wait(_native_current_stream_ptr())


class Buffer:
    def __init__(self, group, num_ep_buffer_bytes: int = 0, disable_p2p: bool = False):
        self.rank = group.rank()
        self.group_size = group.size()
        self.group = group
        self.num_ep_buffer_bytes = num_ep_buffer_bytes
        self.backend = self.group
        world = getattr(group, "world", None)
        self.runtime = ep.Buffer(self.rank, self.group_size, num_ep_buffer_bytes, disable_p2p, world=world)
        # there is no slow path here: the HIP kernels are the only implementation
        self._use_fallback = False
        # A round's kernels are enqueued by the call of its last rank, from the raw addresses every rank
        # posted: each call hands its tensors to the runtime (`keep_alive`), which holds them until it
        # has enqueued the call's round, however far ahead of its peers this rank runs.
        self._outputs = _OutputPool()
        self.connect()

    @staticmethod
    def _hook_keeping(hook: Optional[Callable], tensors: tuple) -> Optional[Callable]:
        """The receive hook, holding the call's tensors until it has run: in hook mode nothing else
        orders the caller's later work on those tensors after the round's kernels."""
        if hook is None:
            return None
        kept = [tensors]

        def call() -> None:
            hook()
            kept.clear()
        return call

    def connect(self, is_update: bool = False) -> None:
        """Peer exchange of the reference (:185-304; is_update re-runs it for a changed membership, :306-307)
        has nothing to do when every rank lives in the same address space."""
        if not self.runtime.use_fast_path():
            raise RuntimeError("mooncake_amd has no fallback path")

    def update_ep_member(self) -> None:
        self.connect(is_update=True)

    @staticmethod
    def get_ep_buffer_size_hint(num_max_dispatch_tokens_per_rank: int, hidden: int, num_ranks: int,
                                num_experts: int) -> int:
        return ep.get_ep_buffer_size_hint(num_max_dispatch_tokens_per_rank, hidden, num_ranks, num_experts)

    def _default_active_ranks(self, device: torch.device) -> torch.Tensor:
        return torch.ones((self.group_size,), dtype=torch.int32, device=device)

    # noinspection PyTypeChecker
    def dispatch(self, x: torch.Tensor, topk_idx: torch.Tensor, active_ranks: Optional[torch.Tensor],
                 num_max_dispatch_tokens_per_rank: int, num_experts: int, timeout_us: int,
                 use_fp8: Optional[bool] = None, async_finish: bool = False, return_recv_hook: bool = False,
                 ) -> Tuple[Union[Tuple[torch.Tensor, torch.Tensor], torch.Tensor], torch.Tensor, Tuple,
                            EventOverlap, Callable]:
        # the reference's checks (:378-393), on each tensor's shape tuple: this wrapper is all host time
        xs, ts, group_size = x.shape, topk_idx.shape, self.group_size
        assert len(xs) == 2 and x.is_contiguous()
        assert x.dtype == _BF16
        assert len(ts) == 2 and topk_idx.is_contiguous()
        assert topk_idx.dtype == _I64
        num_tokens, hidden = xs
        assert num_tokens == ts[0]
        assert num_tokens <= num_max_dispatch_tokens_per_rank
        assert hidden % 16 == 0 and hidden % 128 == 0
        assert num_experts % group_size == 0
        if active_ranks is None:
            active_ranks = self._default_active_ranks(x.device)
        else:
            assert active_ranks.dim() == 1 and active_ranks.is_contiguous()
            assert active_ranks.dtype == _I32
            if active_ranks.numel() != group_size:
                active_ranks = self._default_active_ranks(x.device)
        if use_fp8 is None:
            use_fp8 = True

        num_local_experts = num_experts // group_size
        rm = group_size * num_max_dispatch_tokens_per_rank
        if use_fp8:
            assert rm % 4 == 0
        device = x.device
        stream_ptr = _native_current_stream_ptr()
        key = (num_local_experts, rm, hidden, bool(use_fp8), device, stream_ptr)
        outs = self._outputs.find(key)
        if outs is None:
            # outputs are not cleared: rows at and beyond packed_recv_count stay unwritten
            outs = [torch.empty((num_local_experts, rm, hidden), dtype=_FP8 if use_fp8 else _BF16, device=device),
                    torch.empty((num_local_experts,), dtype=_I32, device=device),
                    torch.empty((num_local_experts, rm), dtype=_I32, device=device),
                    torch.empty((num_local_experts, group_size), dtype=_I64, device=device)]
            if use_fp8:
                # column-major per expert: [L, H/128, R*max] storage viewed as [L, R*max, H/128]
                outs.append(torch.empty((num_local_experts, hidden // 128, rm), dtype=_F32,
                                        device=device).transpose(1, 2))
            outs = self._outputs.add(key, outs)
        if use_fp8:
            packed_recv_x, packed_recv_count, packed_recv_src_info, packed_recv_layout_range, packed_recv_x_scales = outs
            scales_ptr = packed_recv_x_scales.data_ptr()
        else:
            packed_recv_x, packed_recv_count, packed_recv_src_info, packed_recv_layout_range = outs
            packed_recv_x_scales, scales_ptr = None, 0
        del outs
        tensors_to_record = (x, topk_idx, active_ranks, packed_recv_x, packed_recv_x_scales, packed_recv_count,
                             packed_recv_src_info, packed_recv_layout_range)
        event, hook = self.runtime.dispatch(
            x.data_ptr(), topk_idx.data_ptr(), active_ranks.data_ptr(), num_tokens, hidden, ts[1],
            num_max_dispatch_tokens_per_rank, num_experts, timeout_us, use_fp8, packed_recv_x.data_ptr(),
            scales_ptr, packed_recv_count.data_ptr(), packed_recv_src_info.data_ptr(),
            packed_recv_layout_range.data_ptr(), async_finish, return_recv_hook, stream_ptr, tensors_to_record)
        handle = (packed_recv_src_info, packed_recv_layout_range, num_max_dispatch_tokens_per_rank, hidden,
                  num_experts)
        return ((packed_recv_x, packed_recv_x_scales) if use_fp8 else packed_recv_x, packed_recv_count, handle,
                EventOverlap(event, tensors_to_record if async_finish else None),
                None if hook is None else self._hook_keeping(hook, tensors_to_record))

    # noinspection PyTypeChecker
    def combine(self, x: torch.Tensor, topk_idx: torch.Tensor, topk_weights: torch.Tensor,
                active_ranks: Optional[torch.Tensor], timeout_us: int, handle: tuple, zero_copy: bool = False,
                async_finish: bool = False, return_recv_hook: bool = False, out: Optional[torch.Tensor] = None,
                ) -> Tuple[torch.Tensor, EventOverlap, Callable]:
        if zero_copy:
            raise NotImplementedError(_ZERO_COPY_COMBINE_UNSUPPORTED)
        # the reference's checks (:554-567, :616-640), on each tensor's shape tuple
        xs, ts, ws, group_size = x.shape, topk_idx.shape, topk_weights.shape, self.group_size
        assert len(xs) == 3 and x.is_contiguous()
        assert x.dtype == _BF16
        assert len(ts) == 2 and topk_idx.is_contiguous()
        assert topk_idx.dtype == _I64
        assert len(ws) == 2 and topk_weights.is_contiguous()
        assert topk_weights.dtype == _F32
        if active_ranks is None:
            active_ranks = self._default_active_ranks(x.device)
        else:
            assert active_ranks.dim() == 1 and active_ranks.is_contiguous()
            assert active_ranks.dtype == _I32
            if active_ranks.numel() != group_size:
                active_ranks = self._default_active_ranks(x.device)
        src_info, layout_range, num_max_dispatch_tokens_per_rank, hidden, num_experts = handle
        num_local_experts = num_experts // group_size
        ss, ls = src_info.shape, layout_range.shape
        assert xs[0] == num_local_experts
        assert xs[1] == group_size * num_max_dispatch_tokens_per_rank
        assert xs[2] == hidden
        assert hidden % 16 == 0 and hidden % 128 == 0
        assert ts == ws
        num_combined_tokens = ws[0]
        assert num_combined_tokens <= num_max_dispatch_tokens_per_rank
        assert len(ss) == 2 and src_info.is_contiguous()
        assert src_info.dtype == _I32
        assert ss[0] == xs[0]
        assert len(ls) == 2 and layout_range.is_contiguous()
        assert layout_range.dtype == _I64
        assert ls[0] == num_local_experts
        assert ls[1] == group_size
        if out is not None:
            os_ = out.shape
            assert len(os_) == 2 and out.is_contiguous()
            assert os_[0] == num_combined_tokens
            assert os_[1] == hidden
            assert out.dtype == _BF16
            combined_x = out
        else:
            combined_x = torch.empty((num_combined_tokens, hidden), dtype=_BF16, device=x.device)
        tensors_to_record = (x, topk_idx, topk_weights, active_ranks, src_info, layout_range, combined_x)
        event, hook = self.runtime.combine(
            x.data_ptr(), topk_idx.data_ptr(), topk_weights.data_ptr(), src_info.data_ptr(),
            layout_range.data_ptr(), active_ranks.data_ptr(), num_local_experts, num_combined_tokens, hidden,
            ws[1], num_max_dispatch_tokens_per_rank, num_experts, timeout_us, zero_copy,
            combined_x.data_ptr(), async_finish, return_recv_hook, _native_current_stream_ptr(), tensors_to_record)
        return (combined_x, EventOverlap(event, tensors_to_record if async_finish else None),
                None if hook is None else self._hook_keeping(hook, tensors_to_record))

    def get_next_combine_buffer(self, handle: object):
        raise NotImplementedError(_ZERO_COPY_COMBINE_UNSUPPORTED)
