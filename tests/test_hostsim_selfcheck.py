"""The host simulation's own promise, checked: a kernel that reads or writes one pack past a guarded
buffer kills the process (so a test that passes has seen no such access)."""
from __future__ import annotations

import signal
import subprocess
import sys
import textwrap

import os

from tests.hostsim.build import needs_host_clang

pytestmark = needs_host_clang

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _child(code):
    return subprocess.run([sys.executable, "-c", textwrap.dedent(code)], cwd=ROOT, capture_output=True, text=True, timeout=600)


def test_an_overrun_of_one_pack_dies_on_the_guard_page():
    ok = _child("""
        import torch
        from tests.hostsim import sim
        n = 4096
        a, b, o = (sim.guard(torch.zeros(n, dtype=torch.bfloat16)) for _ in range(3))
        assert sim.lib().fx_glu_fwd(sim.p(a), sim.p(b), sim.p(o), n, 2, 2, 0, None) == 0
        print("fine")
    """)
    assert ok.returncode == 0 and "fine" in ok.stdout, ok.stderr[-2000:]
    for victim in ("a", "o"):          # an input read, then an output written, 8 elements too far
        bad = _child(f"""
            import torch
            from tests.hostsim import sim
            n = 4096
            a, b, o = (sim.guard(torch.zeros(n + (0 if name == "{victim}" else 8), dtype=torch.bfloat16)) for name in "abo")
            sim.lib().fx_glu_fwd(sim.p(a), sim.p(b), sim.p(o), n + 8, 2, 2, 0, None)
            print("survived")
        """)
        assert bad.returncode == -signal.SIGSEGV and "survived" not in bad.stdout, (victim, bad.returncode, bad.stderr[-500:])
