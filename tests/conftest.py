import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


from hostsim import mode as hostsim_mode  # noqa: E402  (tests/ is on the path when pytest collects from it)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    if hostsim_mode.ACTIVE:       # FLEXTRAIN_HOSTSIM=1: the GPU tests run against the host simulation
        hostsim_mode.activate()


def pytest_sessionstart(session):
    """The tests load the library that is built; only when none is there do they build it."""
    from flextrain_amd._lib import LIB_PATH

    if not os.path.exists(LIB_PATH):
        import __graft_entry__

        __graft_entry__.build()


def pytest_collection_modifyitems(config, items):
    """FLEXTRAIN_HOSTSIM=1: tests that have no meaning in the simulation or are too large for it are skipped."""
    if not hostsim_mode.ACTIVE:
        return
    listed = [line.strip() for line in open(os.path.join(ROOT, "tests", "hostsim", "skip_in_simulation.txt"))
              if line.strip() and not line.startswith("#")]
    for item in items:
        if any(item.nodeid.startswith(prefix) for prefix in listed):
            item.add_marker(pytest.mark.skip(reason="listed in tests/hostsim/skip_in_simulation.txt"))


def pytest_runtest_setup(item):
    """Name every GPU test on the real stderr, flushed, before it touches the card: a run that ends with
    the machine (a fault takes the box and its files along) still shows which test it was in."""
    if item.get_closest_marker("gpu") is not None:
        sys.__stderr__.write(f"[gpu test] {item.nodeid}\n")
        sys.__stderr__.flush()


@pytest.fixture(scope="session")
def dev():
    if hostsim_mode.ACTIVE:
        return torch.device("cpu")
    if not torch.cuda.is_available():
        pytest.skip("no GPU in this process")
    return torch.device("cuda:0")
