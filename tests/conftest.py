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
    """Runs a model test with both attention cores: the fused one (one histogram per (atom, head); its angle
    encoding is the untruncated Gaussian basis) and the reference's sequence of operators (33-bin angle windows).
    Yields the ``windows`` argument that makes the CPU oracle compute the same thing."""
    from crystalframer_amd import attention
    saved = attention.FUSED_CORE
    attention.FUSED_CORE = request.param == "fused"
    yield (9, None) if attention.FUSED_CORE else "reference"
    attention.FUSED_CORE = saved
