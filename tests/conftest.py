import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU checker.  Built on demand; tests are the only place it is loaded."""
    from oracle import oracle as o

    o.build()
    return o


@pytest.fixture(scope="session")
def gpu():
    """torch device of the GPU under test; GPU tests fail (not skip) when the HIP library is missing."""
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU in this process")
    return torch.device("cuda:0")
