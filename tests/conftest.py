import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("filterwarnings", "ignore:.*torch.jit.script.*is deprecated.*:DeprecationWarning")


def _backends():
    return ["emul", pytest.param("hip", marks=pytest.mark.gpu)]


@pytest.fixture(params=_backends())
def backend(request):
    """'emul': the lowered bytecode runs in the CPU emulator (host logic only);
    'hip': the region runs through the C ABI on cuda:0."""
    if request.param == "hip":
        import torch
        if not torch.cuda.is_available():
            pytest.fail("a gpu-marked test was selected but no GPU is visible")
    return request.param
