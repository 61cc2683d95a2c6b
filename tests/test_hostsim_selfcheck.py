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
    """The happens-before check of the simulated run: the pipelined optimizer step over the layer rings and the
    library's own streamed chunk pass with many cross-stream pairs examined, and with the waits of any one of
    the three streams taken away the enqueue that is no longer ordered fails and says why."""
    prologue = """
        import os, sys
        os.environ["FLEXTRAIN_HOSTSIM"] = "1"
        sys.path.insert(0, "tests")
        import torch
        from hostsim import mode
        mode.ACTIVE = True
        mode.activate()
        import test_gpu_layer_ring as t
        from flextrain_amd.layer_ring import ring_optimizer_step
        from flextrain_amd.optim import flextrain_adamw_step_streamed
        from flextrain_amd.streams import EventBook, StreamBundle
        dev = torch.device("cpu")
        streams = StreamBundle.create(dev)
        def rings():
            specs, buf = t._make(dev, 5, 2, 2, 7)
            return ring_optimizer_step(buf, streams, EventBook(), n_gpu_opt_layers=2, step_num=4, **t.HP)
        def chunk():
            from flextrain_amd.host_memory import LocalPinnedHostBackend
            n, be = 40000, LocalPinnedHostBackend()
            p, m, v = (be.allocate_tensor((n,), torch.float32) for _ in range(3))
            g = be.allocate_tensor((n,), torch.bfloat16)
            return flextrain_adamw_step_streamed(p, g, m, v, streams=streams, sub_elems=4096, n_slots=2, step=1, **t.HP)
        def deafen(role):
            mode.CLOCKS.deafen(getattr(streams, role).cuda_stream)
    """
    ok = _child(prologue + """
        assert rings() == 0 and chunk() == 0
        assert mode.CLOCKS.checked > 50 and mode.CLOCKS.last_violation == "", (mode.CLOCKS.checked, mode.CLOCKS.last_violation)
        print("fine", mode.CLOCKS.checked)
    """)
    assert ok.returncode == 0 and "fine" in ok.stdout, ok.stderr[-2000:]
    for role in ("compute", "outbound", "inbound"):
        bad = _child(prologue + f"""
        deafen("{role}")
        for schedule in (rings, chunk):
            try:
                print(schedule.__name__, "returned", schedule())
            except RuntimeError as exc:
                print(schedule.__name__, "raised", exc)
            print("violation:", mode.CLOCKS.last_violation)
        """)
        out = bad.stdout
        assert bad.returncode == 0 and out.count("is not ordered after") == 2 and "returned 0" not in out, (role, out[-900:], bad.stderr[-1500:])
