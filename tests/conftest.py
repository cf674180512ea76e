import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def gpu_device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from streamdiffusionv2_amd import _capi, build_ext

    build_ext.ensure_built()   # a GPU box normally gets the library with the tree; build only when it did not
    _capi.lib()                # fail loudly when the HIP extension is missing
    return torch.device("cuda:0")
