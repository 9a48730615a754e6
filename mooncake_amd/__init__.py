"""mooncake-ep low-latency MoE dispatch / combine for one AMD MI355X (gfx950).

`mooncake_amd.mooncake_ep_buffer.Buffer` mirrors the reference's Python
`Buffer`; `mooncake_amd.ep` mirrors its native module; both run on
`libmooncake_ep_hip.so` and fail loudly without it.
"""
from . import ep  # noqa: F401
from .mooncake_ep_buffer import Buffer, EventOverlap, LogicalGroup, spawn_ranks  # noqa: F401

__all__ = ["ep", "Buffer", "EventOverlap", "LogicalGroup", "spawn_ranks"]
