"""ctypes loader for libmooncake_ep_hip.so (C ABI: include/mooncake_ep_hip.h).

There is no CPU or PyTorch fallback behind this module: if the HIP library is
missing, loading raises and every entry point of the package fails with it.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_double, c_int, c_int32, c_int64, c_uint64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmooncake_ep_hip.so")

OK, ERR_ASSERT, ERR_HIP, ERR_PENDING, ERR_UNSUPPORTED, ERR_INVALID = 0, 1, 2, 3, 4, 5
PHASE_LAYOUT, PHASE_DATA, PHASE_FINISH, PHASE_ALL = 1, 2, 4, 7

_lib = None

_U64P = POINTER(c_uint64)
_I32P = POINTER(c_int32)
_VPP = POINTER(c_void_p)



class LegacyPerfTensors(Structure):
    """mc_ep_legacy_perf_tensors_t: one array of per-rank device addresses per tensor."""
    _fields_ = [(name, _U64P) for name in (
        "x_ptrs", "topk_idx_ptrs", "topk_weights_ptrs", "active_ranks_ptrs", "expert_x_ptrs", "packed_recv_x_ptrs",
        "packed_recv_count_ptrs", "packed_recv_src_info_ptrs", "packed_recv_layout_range_ptrs", "combined_x_ptrs")]


class LegacyPerfConfig(Structure):
    """mc_ep_legacy_perf_config_t"""
    _fields_ = [(name, c_int) for name in (
        "num_tokens", "hidden", "num_topk", "num_local_experts", "num_max_dispatch_tokens_per_rank", "num_experts",
        "timeout_us", "warmups", "iterations")] + [("compute_stream_ptr", c_uint64)]


class LegacyPerfResult(Structure):
    """mc_ep_legacy_perf_result_t"""
    _fields_ = [("average_us", c_double), ("min_us", c_double), ("max_us", c_double)]


# name -> (restype, argtypes); one entry per declaration in include/mooncake_ep_hip.h
SIGNATURES = {
    "mc_ep_last_error": (c_char_p, []),
    "mc_ep_get_buffer_size_hint": (c_uint64, [c_int, c_int, c_int, c_int]),
    "mc_ep_world_create": (c_int, [c_int, _VPP]),
    "mc_ep_world_destroy": (c_int, [c_void_p]),
    "mc_ep_world_num_ranks": (c_int, [c_void_p]),
    "mc_ep_world_set_rank_silent": (c_int, [c_void_p, c_int, c_int]),
    "mc_ep_world_set_option": (c_int, [c_void_p, c_char_p, c_int]),
    "mc_ep_world_get_option": (c_int, [c_void_p, c_char_p, POINTER(c_int)]),
    "mc_ep_world_dispatch": (c_int, [c_void_p, _U64P, _U64P, _I32P, c_int, c_int, c_int, c_int, c_int,
                                     _U64P, _U64P, _U64P, _U64P, _U64P, c_int, c_uint64]),
    "mc_ep_world_dispatch_noalloc": (c_int, [c_void_p, _U64P, _U64P, _I32P, c_int, c_int, c_int, c_int, c_int,
                                             _U64P, _U64P, _U64P, _U64P, _U64P, c_uint64]),
    "mc_ep_world_combine": (c_int, [c_void_p, _U64P, _U64P, _U64P, _U64P, _U64P, _U64P, _I32P, c_int, c_int,
                                    c_int, c_int, _U64P, c_int, c_uint64]),
    "mc_ep_world_combine_packed": (c_int, [c_void_p, _U64P, _U64P, c_uint64, _U64P, _U64P, _U64P, _U64P, _U64P, _I32P,
                                           c_int, c_int, c_int, c_int, _U64P, c_int, c_uint64]),
    "mc_ep_world_cast_back": (c_int, [c_void_p, _U64P, _U64P, _U64P, c_uint64, _U64P, c_int, c_int, c_int, c_int,
                                      c_uint64]),
    "mc_ep_world_legacy_buffer_perf": (c_int, [c_void_p, POINTER(LegacyPerfTensors), POINTER(LegacyPerfConfig),
                                               POINTER(LegacyPerfResult)]),
    "mc_ep_buffer_create": (c_int, [c_void_p, c_int, c_int64, c_int, _VPP]),
    "mc_ep_buffer_destroy": (c_int, [c_void_p]),
    "mc_ep_buffer_pending_calls": (c_int, [c_void_p, POINTER(c_int), POINTER(c_int)]),
    "mc_ep_buffer_ibgda_disabled": (c_int, [c_void_p]),
    "mc_ep_buffer_p2p_enabled": (c_int, [c_void_p]),
    "mc_ep_buffer_use_fast_path": (c_int, [c_void_p]),
    "mc_ep_buffer_is_roce": (c_int, [c_void_p]),
    "mc_ep_buffer_dispatch": (c_int, [c_void_p, c_uint64, c_uint64, c_uint64, c_int, c_int, c_int, c_int, c_int,
                                      c_int, c_int, c_uint64, c_uint64, c_uint64, c_uint64, c_uint64, c_int, c_int,
                                      c_uint64, _VPP, _VPP]),
    "mc_ep_buffer_combine": (c_int, [c_void_p, c_uint64, c_uint64, c_uint64, c_uint64, c_uint64, c_uint64, c_int,
                                     c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_uint64, c_int, c_int,
                                     c_uint64, _VPP, _VPP]),
    "mc_ep_event_create": (c_int, [c_uint64, _VPP]),
    "mc_ep_event_current_stream_wait": (c_int, [c_void_p, c_uint64]),
    "mc_ep_event_synchronize": (c_int, [c_void_p]),
    "mc_ep_event_destroy": (c_int, [c_void_p]),
    "mc_ep_hook_call": (c_int, [c_void_p]),
    "mc_ep_hook_destroy": (c_int, [c_void_p]),
}

# measurement helpers the library exports beside its public ABI (csrc/ep_debug.h)
DEBUG_SIGNATURES = {
    "mc_ep_debug_copy": (c_int, [c_uint64, c_uint64, c_uint64, c_uint64]),
    "mc_ep_debug_stream": (c_int, [c_int, c_uint64, c_uint64, c_uint64, c_uint64]),
    "mc_ep_debug_set_stream_occupancy": (c_int, [c_int]),
    "mc_ep_debug_gather_rows": (c_int, [c_uint64, c_uint64, c_int, c_int64, c_int, c_int64, c_int, c_uint64]),
    "mc_ep_debug_scatter_rows": (c_int, [c_uint64, c_uint64, c_int, c_int64, c_int, c_int64, c_int, c_uint64]),
}


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is not built; run `make -C {os.path.join(_HERE, 'csrc')}` "
                "(the dispatch/combine path has no fallback without it)")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in list(SIGNATURES.items()) + list(DEBUG_SIGNATURES.items()):
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


class PendingError(RuntimeError):
    """MC_EP_ERR_PENDING: a collective was waited on before every live rank had called it - an event or hook of
    an incomplete round, or a blocking per-rank call that waited `block_timeout_ms` for its peers.  Such a call
    stays posted: its round is enqueued when the peers arrive, so its tensors must stay alive."""


def last_error() -> str:
    msg = lib().mc_ep_last_error()
    return msg.decode("utf-8", "replace") if msg else ""


def check(rc: int) -> None:
    """Map an MC_EP_ERR_* code to the exception the reference raises: host
    assertions and HIP failures become RuntimeError (EPException through
    pybind11), unsupported features NotImplementedError, what the reference
    rejects with std::invalid_argument ValueError."""
    if rc == OK:
        return
    msg = last_error()
    if rc == ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    if rc == ERR_INVALID:
        raise ValueError(msg)          # std::invalid_argument through pybind11
    if rc == ERR_PENDING:
        raise PendingError(msg)
    raise RuntimeError(msg)


def u64_array(values) -> ctypes.Array:
    return (c_uint64 * len(values))(*[int(v) for v in values])


def i32_array(values) -> ctypes.Array:
    return (c_int32 * len(values))(*[int(v) for v in values])
