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


def test_tensors_of_the_simulated_gpu_suite_end_at_a_guard_page():
    """With FLEXTRAIN_HOSTSIM=1 every tensor created, cloned or moved "to the device" is guarded: the same
    overrun through the package's own ops dies there as well, and the tensor releases its pages when it dies."""
    prologue = """
        import os, sys
        os.environ["FLEXTRAIN_HOSTSIM"] = "1"
        sys.path.insert(0, "tests")
        import torch
        from hostsim import mode
        mode.ACTIVE = True
        mode.activate()
        from flextrain_amd._lib import lib
        n = 4096
        dev = torch.device("cpu")               # what the tests' device fixture hands out in this mode
    """
    ok = _child(prologue + """
        for _ in range(200):                    # 200 x 3 x 4 MB = 2.4 GB if the mappings were kept
            a = torch.zeros(1 << 21, dtype=torch.bfloat16, device=dev)
            b, c = a.clone(), torch.ones(1 << 21, dtype=torch.bfloat16).to(dev)
        resident = int(open("/proc/self/statm").read().split()[1]) * os.sysconf("SC_PAGE_SIZE")
        assert resident < (1 << 30), "guarded tensors are not released"
        a, b, o = (torch.zeros(n, dtype=torch.bfloat16, device=dev) for _ in range(3))
        assert lib().fx_glu_fwd(a.data_ptr(), b.data_ptr(), o.data_ptr(), n, 2, 2, 0, None) == 0
        print("fine")
    """)
    assert ok.returncode == 0 and "fine" in ok.stdout, ok.stderr[-2000:]
    for make in ('torch.zeros(n, dtype=torch.bfloat16, device=dev)', 'torch.zeros(n, dtype=torch.bfloat16).to(dev)',
                 'torch.zeros(n, dtype=torch.bfloat16).clone()', 'torch.empty_like(torch.zeros(n, dtype=torch.bfloat16))'):
        bad = _child(prologue + f"""
        a, b = (torch.zeros(n + 8, dtype=torch.bfloat16, device=dev) for _ in range(2))
        o = {make}
        lib().fx_glu_fwd(a.data_ptr(), b.data_ptr(), o.data_ptr(), n + 8, 2, 2, 0, None)
        print("survived")
        """)
        assert bad.returncode == -signal.SIGSEGV and "survived" not in bad.stdout, (make, bad.returncode, bad.stderr[-500:])


def test_a_removed_wait_in_the_streamed_optimizer_step_is_reported():
    """The happens-before check of the simulated run: the pipelined optimizer step over the layer rings passes
    with many cross-stream pairs examined, and taking away any one class of its waits (the compute stream's
    wait for a layer's fetches, the outbound stream's wait for the update, the inbound stream's wait before a
    slot is refilled) raises StreamOrderError at the enqueue that is no longer ordered."""
    prologue = """
        import os, sys
        os.environ["FLEXTRAIN_HOSTSIM"] = "1"
        sys.path.insert(0, "tests")
        import torch
        from hostsim import mode, order
        mode.ACTIVE = True
        mode.activate()
        import test_gpu_layer_ring as t
        from flextrain_amd.layer_ring import ring_optimizer_step
        from flextrain_amd.streams import EventBook, StreamBundle
        dev = torch.device("cpu")
        def run():
            specs, buf = t._make(dev, 5, 2, 2, 7)
            streams = StreamBundle.create(dev)
            return streams, ring_optimizer_step(buf, streams, EventBook(), n_gpu_opt_layers=2, step_num=4, **t.HP)
    """
    ok = _child(prologue + """
        assert run()[1] == 0
        assert order.CLOCKS.checked > 50, order.CLOCKS.checked
        print("fine", order.CLOCKS.checked)
    """)
    assert ok.returncode == 0 and "fine" in ok.stdout, ok.stderr[-2000:]
    for role in ("compute", "outbound", "inbound"):
        bad = _child(prologue + f"""
        streams = StreamBundle.create(dev)
        deaf = streams.{role}.cuda_stream
        plain = order.CLOCKS.wait
        order.CLOCKS.wait = lambda sid, clock: None if sid == deaf else plain(sid, clock)   # this stream waits for nothing
        StreamBundle.create = classmethod(lambda cls, *a, **k: streams)
        try:
            run()
            print("unnoticed")
        except order.StreamOrderError as exc:
            print("reported:", exc)
        """)
        assert bad.returncode == 0 and "reported:" in bad.stdout and "unnoticed" not in bad.stdout, (role, bad.stdout[-500:], bad.stderr[-1500:])
