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
