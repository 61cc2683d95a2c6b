"""``FLEXTRAIN_HOSTSIM=1``: run the GPU parity tests of this directory against the host simulation.

The package's Python layer is unchanged; what changes is what it stands on: ``flextrain_amd._lib.lib()``
returns the simulated library, tensors stay in host memory and claim to be on the GPU and pinned, and the
``torch.cuda`` stream / event calls the package and the tests make become no-ops (the simulated library
completes every launch and copy at the call).  Nothing here is active unless the variable is set, and
nothing in the package knows about it."""
from __future__ import annotations

import contextlib
import os

import torch

ACTIVE = os.environ.get("FLEXTRAIN_HOSTSIM") == "1"


class _Event:
    def __init__(self, *a, **k):
        pass

    def record(self, *a, **k):
        pass

    def wait(self, *a, **k):
        pass

    def synchronize(self):
        pass

    def query(self):
        return True

    def elapsed_time(self, other):
        return 0.0


class _Stream:
    device = torch.device("cpu")
    _handles = 0

    def __init__(self, *a, **k):
        _Stream._handles += 1
        self.cuda_stream = 0x1000 * _Stream._handles       # a distinct non-null handle per stream object

    def synchronize(self):
        pass

    def wait_stream(self, other):
        pass

    def wait_event(self, event):
        pass

    def record_event(self, event=None):
        return event or _Event()

    def query(self):
        return True


def _host_only(fn):
    def wrapped(*args, **kwargs):
        kwargs.pop("pin_memory", None)
        dev = kwargs.get("device")
        if dev is not None and torch.device(dev).type == "cuda":
            kwargs["device"] = "cpu"
        return fn(*args, **kwargs)
    return wrapped


def activate():
    from flextrain_amd import _lib

    from . import sim

    _lib._lib = sim.lib()
    default = _Stream()
    default.cuda_stream = 0
    current = [default]

    @contextlib.contextmanager
    def stream_context(s):
        if s is None:
            yield
            return
        current.append(s)
        try:
            yield
        finally:
            current.pop()

    torch.cuda.current_stream = lambda device=None: current[-1]
    torch.cuda.default_stream = lambda device=None: default
    torch.cuda.stream = stream_context
    torch.cuda.synchronize = lambda device=None: None
    torch.cuda.Stream = _Stream
    torch.cuda.Event = _Event
    torch.cuda.memory_allocated = lambda device=None: 0
    torch.cuda.set_device = lambda device: None
    torch.cuda.init = lambda: None
    # a tensor "moved to the GPU" is a copy there, and the tests rely on it (in-place kernels must not touch
    # the host original that the oracle is given afterwards); on one device Tensor.to returns the tensor itself
    plain_to = torch.Tensor.to

    def to(self, *args, **kwargs):
        out = plain_to(self, *args, **kwargs)
        moved = "device" in kwargs or any(isinstance(a, (torch.device, str)) for a in args)
        return out.clone() if (out is self and moved) else out

    torch.Tensor.to = to
    # every tensor is "on the GPU" except those the package's pinned-host allocator made
    from flextrain_amd import host_memory

    def in_pinned_host_memory(t):
        p = t.data_ptr()
        return any(base <= p < base + nbytes for base, (_, nbytes) in host_memory._PROCESS_PINNED.items())

    torch.Tensor.is_cuda = property(lambda self: not in_pinned_host_memory(self))
    torch.Tensor.cpu = lambda self, *a, **k: self.clone()      # a device-to-host copy is a copy
    torch.Tensor.is_pinned = lambda self, device=None: True
    torch.Tensor.pin_memory = lambda self, device=None: self
    torch.Tensor.record_stream = lambda self, stream: None
    for name in ("empty", "zeros", "ones", "full", "tensor", "randn", "rand", "arange"):
        setattr(torch, name, _host_only(getattr(torch, name)))
