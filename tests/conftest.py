import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu():
    """The HIP device; GPU tests fail loudly (not skip) when the extension is missing."""
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from loongforge_amd import _lib

    _lib.load()  # raises if the in-tree HIP library is absent
    return torch.device("cuda:0")
