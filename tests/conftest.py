import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")


@pytest.fixture
def progress(capsys):
    """print(...) that reaches the terminal while output capture is on: long CPU legs (the oracle on a full-size
    graph) show that the run is alive."""

    def say(*args):
        with capsys.disabled():
            print(*args, flush=True)

    return say
