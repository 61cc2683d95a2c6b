"""The GPU parity tests of this directory, run against the host simulation (tests/hostsim): the package's
Python layer and the kernels' own source on the CPU, checked against the oracle by the very tests that
check the GPU.  Tests that take two seconds or more there are left to the run by hand
(``FLEXTRAIN_HOSTSIM=1 python -m pytest tests -m gpu -n 6``: every GPU test except the 18 listed in
tests/hostsim/skip_in_simulation.txt, 20 minutes).  Here the lanes of a workgroup are scheduled in descending
order between barriers (the tests of the simulation itself use the ascending order): a value that one wave
leaves in LDS for another with no barrier in between is read before it is written in one of the two."""
from __future__ import annotations

import os
import re
import subprocess
import sys

from tests.hostsim.build import needs_host_clang

pytestmark = needs_host_clang

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_gpu_parity_tests_pass_against_the_host_simulation():
    from tests.hostsim import build

    build.build()                         # once, before the workers start
    slow = [line.strip() for line in open(os.path.join(ROOT, "tests", "hostsim", "slow_in_simulation.txt"))
            if line.strip() and not line.startswith("#")]
    cmd = [sys.executable, "-m", "pytest", "tests", "-m", "gpu", "-q", "-p", "no:cacheprovider", "-n", "4", "--timeout", "300"]
    for nodeid in slow:
        cmd += ["--deselect", nodeid]
    run = subprocess.run(cmd, cwd=ROOT, env=dict(os.environ, FLEXTRAIN_HOSTSIM="1", HOSTSIM_LANE_ORDER="descending"),
                         capture_output=True, text=True, timeout=3000)
    tail = run.stdout[-3000:]
    assert run.returncode == 0, tail + run.stderr[-2000:]
    m = re.search(r"(\d+) passed", tail)
    assert m and int(m.group(1)) >= 250 and "failed" not in tail and "error" not in tail.lower(), tail
