import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (MI355X); run with -m gpu")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no HIP device")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(params=["fused", "two_step"])
def core_mode(request):
    """Runs a model test with both attention cores: the fused one (one histogram per (atom, head); untruncated
    angle basis and, in its default mode, a +-5 sigma distance window: the reference's pure-PyTorch formulation
    with full Gaussian bases) and the reference's sequence of operators (9- and 33-bin windows of its CUDA kernels).
    Yields the ``windows`` argument that makes the CPU oracle compute what the path is held to."""
    import crystalframer_amd as cf
    from crystalframer_amd import attention, _lib
    saved = attention.FUSED_CORE, cf.KernelManager.CORE_WINDOW_MODE
    attention.FUSED_CORE = request.param == "fused"
    cf.KernelManager.CORE_WINDOW_MODE = _lib.CFH_WINDOW_WIDE
    yield "full" if attention.FUSED_CORE else "reference"
    attention.FUSED_CORE, cf.KernelManager.CORE_WINDOW_MODE = saved
