import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as orc
    orc.lib()
    return orc


@pytest.fixture(scope="session")
def gpu_device():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")


@pytest.fixture(params=[1, 0], ids=["one_launch", "three_launch"])
def fused_small(request):
    """Runs a test once per dispatch path: worlds small enough for the one-launch dispatch take it (1), or
    take the count / pack / scale-transpose launches like any other world (0)."""
    from tests import gpu_util
    gpu_util.DEFAULT_OPTIONS["fused_small"] = request.param
    # (whatever the size rule of the default would say about a shape: the tests are about results)
    gpu_util.DEFAULT_OPTIONS["fused_small_rounds"] = 1 << 20
    yield request.param
    gpu_util.DEFAULT_OPTIONS.pop("fused_small", None)
    gpu_util.DEFAULT_OPTIONS.pop("fused_small_rounds", None)
