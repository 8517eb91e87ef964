import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("markers", "default_scale_division: runs with the package's own default scale-division mode")


def _gpu_present():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _gpu_present():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _pinned_scale_division(request):
    """The oracle's default arithmetic is the CPU's (true division by Qmax), and most parity tests quantise
    GPU-resident weights and compare with it: they run in mode "ieee".  The package's own default ("auto": follow
    the tensor's device) is the subject of the tests marked `default_scale_division`, which run untouched."""
    if "default_scale_division" in request.keywords:
        yield
        return
    import bitween_amd
    previous = bitween_amd.set_scale_division("ieee")
    try:
        yield
    finally:
        bitween_amd.set_scale_division(previous)
