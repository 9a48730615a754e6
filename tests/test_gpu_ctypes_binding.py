"""The ctypes binding of the per-rank calls (`MOONCAKE_AMD_EP_BINDING=ctypes`: `Buffer`, `EventHandle` and the
receive hook of mooncake_amd/ep.py over the same C ABI, for a build without a host compiler) is chosen when the
package is imported, so it is exercised in a child process: the per-rank API tests - the reference's grid of
completion modes, its structured-data invariants, the pending-round errors, the host assertions - run there
against that binding."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = r"""
import sys
import pytest
from mooncake_amd import ep
assert ep.BINDING == "ctypes", ep.BINDING
assert ep.Buffer is ep._CtypesBuffer and ep.EventHandle is ep._CtypesEventHandle
sys.exit(pytest.main(["-x", "-q", "-m", "gpu", "--timeout", "120", "--timeout-method", "thread", "-p", "no:cacheprovider",
                      "tests/test_gpu_buffer_api.py", "tests/test_gpu_thread_per_rank.py"]))
"""


def test_per_rank_api_through_the_ctypes_binding(gpu_device):
    print("[gpu-case] per-rank Buffer API tests in a child process with MOONCAKE_AMD_EP_BINDING=ctypes", flush=True)
    env = dict(os.environ, MOONCAKE_AMD_EP_BINDING="ctypes")
    proc = subprocess.run([sys.executable, "-u", "-c", CHILD], cwd=ROOT, env=env, stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True, timeout=900)
    tail = proc.stdout[-3000:]
    assert proc.returncode == 0, tail
    assert " passed" in tail and "failed" not in tail, tail
