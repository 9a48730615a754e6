"""The C-ABI library loads and exports every symbol include/mooncake_ep_hip.h
declares; the host-only entry points behave (no kernel is launched here)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mooncake_ep_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mc_ep_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from mooncake_amd import _lib
    assert os.path.exists(_lib.LIB_PATH), "build the HIP library first (python -c 'import __graft_entry__ as g; g.build()')"
    handle = ctypes.CDLL(_lib.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 25
    for n in names:
        assert hasattr(handle, n), f"{n} is declared in the header but not exported"
    # and the ctypes signature table covers exactly the header
    assert sorted(_lib.SIGNATURES) == names


def test_size_hint_and_constants(oracle):
    from mooncake_amd import ep
    assert ep.MAX_QP_COUNT == 256
    for args in [(128, 7168, 32, 256), (256, 2048, 8, 288), (1, 128, 1, 1)]:
        assert ep.get_ep_buffer_size_hint(*args) == oracle.buffer_size_hint(*args)
    assert ep.get_ep_buffer_size_hint(128, 7168, 32, 256) == 1883246592


def test_missing_library_fails_loudly(monkeypatch):
    from mooncake_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libmooncake_ep_hip.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.lib()


def test_header_is_plain_c_and_structs_match_ctypes(tmp_path):
    """The boundary is a C ABI: the header compiles as C99 on its own (no HIP, torch or C++ in it), and the
    struct layouts the Python binding assumes are the ones a C compiler gives."""
    import subprocess
    from mooncake_amd import _lib
    src = tmp_path / "abi.c"
    src.write_text(
        '#include <stdio.h>\n#include <stddef.h>\n#include "mooncake_ep_hip.h"\n'
        "int main(void) {\n"
        '  printf("%zu %zu %zu %zu %zu\\n", sizeof(mc_ep_legacy_perf_tensors_t), sizeof(mc_ep_legacy_perf_config_t),\n'
        "         offsetof(mc_ep_legacy_perf_config_t, compute_stream_ptr), sizeof(mc_ep_legacy_perf_result_t),\n"
        "         offsetof(mc_ep_legacy_perf_tensors_t, combined_x_ptrs));\n"
        "  return (MC_EP_PHASE_ALL == (MC_EP_PHASE_LAYOUT | MC_EP_PHASE_DATA | MC_EP_PHASE_FINISH)) ? 0 : 1;\n"
        "}\n")
    exe = tmp_path / "abi"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"),
                    str(src), "-o", str(exe)], check=True, capture_output=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    sizes = [int(v) for v in out]
    assert sizes == [ctypes.sizeof(_lib.LegacyPerfTensors), ctypes.sizeof(_lib.LegacyPerfConfig),
                     _lib.LegacyPerfConfig.compute_stream_ptr.offset, ctypes.sizeof(_lib.LegacyPerfResult),
                     _lib.LegacyPerfTensors.combined_x_ptrs.offset]


def test_compiled_module_binds_what_the_reference_module_binds():
    """mooncake_amd._ep is the compiled counterpart of mooncake._ep (mooncake-ep/src/ep_py.cpp:14-46): the same
    module-level names, the same methods on Buffer and EventHandle, the legacy benchmark's three structs with the
    reference's field names (legacy_buffer_perf.cpp:151-199).  Importing it needs no GPU."""
    from mooncake_amd import _ep, ep
    assert ep.BINDING == "pybind11" and ep.Buffer.__mro__[1] is _ep.Buffer and ep.EventHandle is _ep.EventHandle
    for name in ("get_ep_buffer_size_hint", "EventHandle", "MAX_QP_COUNT", "Buffer", "_benchmark_legacy_buffer",
                 "_LegacyBufferPerfTensors", "_LegacyBufferPerfConfig", "_LegacyBufferPerfResult"):
        assert hasattr(_ep, name), name
    for method in ("ibgda_disabled", "p2p_enabled", "use_fast_path", "update_local_qpns", "is_roce", "sync_ibgda_peers",
                   "get_mr_info", "get_gid", "get_local_qpns", "get_local_lids", "get_ipc_handle",
                   "sync_nvlink_ipc_handles", "dispatch", "combine"):
        assert callable(getattr(_ep.Buffer, method)), method
    for method in ("current_stream_wait", "synchronize"):
        assert callable(getattr(_ep.EventHandle, method)), method
    t, c = _ep._LegacyBufferPerfTensors(), _ep._LegacyBufferPerfConfig()
    for field in ("x_ptr", "topk_idx_ptr", "topk_weights_ptr", "active_ranks_ptr", "expert_x_ptr", "packed_recv_x_ptr",
                  "packed_recv_count_ptr", "packed_recv_src_info_ptr", "packed_recv_layout_range_ptr", "combined_x_ptr"):
        assert getattr(t, field) == []
    assert (c.timeout_us, c.warmups, c.iterations, c.compute_stream_ptr) == (-1, 20, 30, 0)
    assert _ep.MAX_QP_COUNT == 256 and _ep.get_ep_buffer_size_hint(128, 7168, 32, 256) == 1883246592
    # the constructor's signature: (rank, num_ranks, num_ep_buffer_bytes, disable_p2p=False[, world])
    import re
    sig = _ep.Buffer.__init__.__doc__
    assert re.findall(r"(\w+): ", sig) == ["self", "rank", "num_ranks", "num_ep_buffer_bytes", "disable_p2p", "world"]
    assert "disable_p2p: bool = False" in sig
