import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
if os.path.join(ROOT, "python") not in sys.path:   # avelang_kernels, the reference's import path
    sys.path.insert(1, os.path.join(ROOT, "python"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from avelang_amd import _lib

    _lib.load()  # the HIP library must be present on a GPU box: no fallback
    return torch.device("cuda:0")
