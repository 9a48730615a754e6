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

import collections
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


def _native_current_stream_ptr() -> int:
    if _raw_stream is not None and _raw_device is not None:
        return int(_raw_stream(_raw_device()))
    return int(torch.cuda.current_stream().cuda_stream)


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
        self.event.current_stream_wait(_native_current_stream_ptr())

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
        # A round's kernels are enqueued by the call of its last rank, with the raw addresses every
        # rank posted: the tensors of a call stay referenced here until the runtime reports that the
        # call's round has been enqueued (however far ahead of its peers this rank runs).
        self._posted_dispatch = collections.deque()
        self._posted_combine = collections.deque()
        self.connect()

    def _retain(self, posted: collections.deque, tensors: tuple, kind: int) -> None:
        posted.append(tensors)
        pending = self.runtime.pending_calls()[kind]
        while len(posted) > pending:
            posted.popleft()

    def _retain_if_posted(self, exc: RuntimeError, posted: collections.deque, tensors: tuple, kind: int) -> None:
        """A blocking call that gave up waiting for its peers (option "blocking": the one way a dispatch or
        combine call fails with MC_EP_ERR_PENDING) has recorded its arguments all the same: the round is enqueued
        when the peers arrive, so the tensors stay referenced as for any call."""
        if isinstance(exc, ep.PendingError):
            self._retain(posted, tensors, kind)

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
        assert x.dim() == 2 and x.is_contiguous()
        assert x.dtype == torch.bfloat16
        assert topk_idx.dim() == 2 and topk_idx.is_contiguous()
        assert topk_idx.dtype == torch.int64
        assert x.size(0) == topk_idx.size(0)
        assert x.size(0) <= num_max_dispatch_tokens_per_rank
        assert x.size(1) % 16 == 0 and x.size(1) % 128 == 0
        assert num_experts % self.group_size == 0
        if active_ranks is None:
            active_ranks = self._default_active_ranks(x.device)
        else:
            assert active_ranks.dim() == 1 and active_ranks.is_contiguous()
            assert active_ranks.dtype == torch.int32
            if active_ranks.numel() != self.group_size:
                active_ranks = self._default_active_ranks(x.device)
        if use_fp8 is None:
            use_fp8 = True

        num_local_experts = num_experts // self.group_size
        rm = self.group_size * num_max_dispatch_tokens_per_rank
        hidden = x.size(1)
        # outputs are not cleared: rows at and beyond packed_recv_count stay unwritten
        packed_recv_x = torch.empty((num_local_experts, rm, hidden),
                                    dtype=torch.float8_e4m3fn if use_fp8 else torch.bfloat16, device=x.device)
        packed_recv_count = torch.empty((num_local_experts,), dtype=torch.int32, device=x.device)
        packed_recv_src_info = torch.empty((num_local_experts, rm), dtype=torch.int32, device=x.device)
        packed_recv_layout_range = torch.empty((num_local_experts, self.group_size), dtype=torch.int64,
                                               device=x.device)
        packed_recv_x_scales = None
        if use_fp8:
            assert rm % 4 == 0
            # column-major per expert: [L, H/128, R*max] storage viewed as [L, R*max, H/128]
            packed_recv_x_scales = torch.empty((num_local_experts, hidden // 128, rm), dtype=torch.float32,
                                               device=x.device).transpose(1, 2)
        tensors_to_record = (x, topk_idx, active_ranks, packed_recv_x, packed_recv_x_scales, packed_recv_count,
                             packed_recv_src_info, packed_recv_layout_range)
        try:
            event, hook = self.runtime.dispatch(
                x.data_ptr(), topk_idx.data_ptr(), active_ranks.data_ptr(), x.size(0), hidden, topk_idx.size(1),
                num_max_dispatch_tokens_per_rank, num_experts, timeout_us, use_fp8, packed_recv_x.data_ptr(),
                0 if packed_recv_x_scales is None else packed_recv_x_scales.data_ptr(), packed_recv_count.data_ptr(),
                packed_recv_src_info.data_ptr(), packed_recv_layout_range.data_ptr(), async_finish, return_recv_hook,
                _native_current_stream_ptr())
        except RuntimeError as exc:
            self._retain_if_posted(exc, self._posted_dispatch, tensors_to_record, 0)
            raise
        handle = (packed_recv_src_info, packed_recv_layout_range, num_max_dispatch_tokens_per_rank, hidden,
                  num_experts)
        self._retain(self._posted_dispatch, tensors_to_record, 0)
        return ((packed_recv_x, packed_recv_x_scales) if use_fp8 else packed_recv_x, packed_recv_count, handle,
                EventOverlap(event, tensors_to_record if async_finish else None),
                self._hook_keeping(hook, tensors_to_record))

    # noinspection PyTypeChecker
    def combine(self, x: torch.Tensor, topk_idx: torch.Tensor, topk_weights: torch.Tensor,
                active_ranks: Optional[torch.Tensor], timeout_us: int, handle: tuple, zero_copy: bool = False,
                async_finish: bool = False, return_recv_hook: bool = False, out: Optional[torch.Tensor] = None,
                ) -> Tuple[torch.Tensor, EventOverlap, Callable]:
        if zero_copy:
            raise NotImplementedError(_ZERO_COPY_COMBINE_UNSUPPORTED)
        assert x.dim() == 3 and x.is_contiguous()
        assert x.dtype == torch.bfloat16
        assert topk_idx.dim() == 2 and topk_idx.is_contiguous()
        assert topk_idx.dtype == torch.int64
        assert topk_weights.dim() == 2 and topk_weights.is_contiguous()
        assert topk_weights.dtype == torch.float32
        if active_ranks is None:
            active_ranks = self._default_active_ranks(x.device)
        else:
            assert active_ranks.dim() == 1 and active_ranks.is_contiguous()
            assert active_ranks.dtype == torch.int32
            if active_ranks.numel() != self.group_size:
                active_ranks = self._default_active_ranks(x.device)
        src_info, layout_range, num_max_dispatch_tokens_per_rank, hidden, num_experts = handle
        assert x.size(0) == num_experts // self.group_size
        assert x.size(1) == self.group_size * num_max_dispatch_tokens_per_rank
        assert x.size(2) == hidden
        assert x.size(2) % 16 == 0 and x.size(2) % 128 == 0
        assert topk_idx.size() == topk_weights.size()
        assert topk_weights.size(0) <= num_max_dispatch_tokens_per_rank
        assert src_info.dim() == 2 and src_info.is_contiguous()
        assert src_info.dtype == torch.int32
        assert src_info.size(0) == x.size(0)
        assert layout_range.dim() == 2 and layout_range.is_contiguous()
        assert layout_range.dtype == torch.int64
        assert layout_range.size(0) == num_experts // self.group_size
        assert layout_range.size(1) == self.group_size
        if out is not None:
            assert out.dim() == 2 and out.is_contiguous()
            assert out.size(0) == topk_weights.size(0)
            assert out.size(1) == hidden
            assert out.dtype == x.dtype
            combined_x = out
        else:
            combined_x = torch.empty((topk_weights.size(0), hidden), dtype=x.dtype, device=x.device)
        tensors_to_record = (x, topk_idx, topk_weights, active_ranks, src_info, layout_range, combined_x)
        try:
            event, hook = self.runtime.combine(
                x.data_ptr(), topk_idx.data_ptr(), topk_weights.data_ptr(), src_info.data_ptr(),
                layout_range.data_ptr(), active_ranks.data_ptr(), x.size(0), topk_weights.size(0), hidden,
                topk_weights.size(1), num_max_dispatch_tokens_per_rank, num_experts, timeout_us, zero_copy,
                combined_x.data_ptr(), async_finish, return_recv_hook, _native_current_stream_ptr())
        except RuntimeError as exc:
            self._retain_if_posted(exc, self._posted_combine, tensors_to_record, 1)
            raise
        self._retain(self._posted_combine, tensors_to_record, 1)
        return (combined_x, EventOverlap(event, tensors_to_record if async_finish else None),
                self._hook_keeping(hook, tensors_to_record))

    def get_next_combine_buffer(self, handle: object):
        raise NotImplementedError(_ZERO_COPY_COMBINE_UNSUPPORTED)
