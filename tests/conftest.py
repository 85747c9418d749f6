import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950) device")


@pytest.fixture(scope="session")
def hip():
    """The HIP path: the C-ABI library must be built and a GPU present; there is no fallback."""
    import torch
    from frisk_amd import runtime

    runtime.lib()  # raises ImportError when libfrisk_hip.so is missing
    assert torch.cuda.is_available(), "GPU tests need a visible MI355X"
    return runtime
