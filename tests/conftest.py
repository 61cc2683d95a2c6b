import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionstart(session):
    """The tests load the library that is built; only when none is there do they build it."""
    from flextrain_amd._lib import LIB_PATH

    if not os.path.exists(LIB_PATH):
        import __graft_entry__

        __graft_entry__.build()


def pytest_runtest_setup(item):
    """Name every GPU test on the real stderr, flushed, before it touches the card: a run that ends with
    the machine (a fault takes the box and its files along) still shows which test it was in."""
    if item.get_closest_marker("gpu") is not None:
        sys.__stderr__.write(f"[gpu test] {item.nodeid}\n")
        sys.__stderr__.flush()


@pytest.fixture(scope="session")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU in this process")
    return torch.device("cuda:0")
