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

from . import order

ACTIVE = os.environ.get("FLEXTRAIN_HOSTSIM") == "1"
CLOCKS = None        # order.Clocks of the simulated library, set by activate()


def _current():
    return torch.cuda.current_stream()


class _Event:
    """Completes at once (the simulated library finishes every launch and copy at the call); what it keeps is
    the vector clock of its stream at ``record``, for the happens-before check of ``order.py``."""

    def __init__(self, *a, **k):
        self.clock = None

    def record(self, stream=None):
        self.clock = CLOCKS.snapshot((stream or _current()).cuda_stream)

    def wait(self, stream=None):
        if self.clock is not None:
            CLOCKS.wait((stream or _current()).cuda_stream, self.clock)

    def synchronize(self):
        if self.clock is not None:
            CLOCKS.host_sync(self.clock)

    def query(self):
        self.synchronize()          # "complete", and the host has now seen it
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
        CLOCKS.stream_sync(self.cuda_stream)

    def wait_stream(self, other):
        CLOCKS.wait_stream(self.cuda_stream, other.cuda_stream)

    def wait_event(self, event):
        event.wait(self)

    def record_event(self, event=None):
        event = event or _Event()
        event.record(self)
        return event

    def query(self):
        self.synchronize()
        return True


def _behind_a_guard_page(t):
    """A fresh, dense tensor moves to storage that ends at an inaccessible page (released with the tensor):
    a kernel that reads or writes past the end of an operand, an output or a workspace then ends the test
    with a segmentation fault instead of passing unnoticed.  Anything else is returned as it is."""
    from . import sim

    if (not isinstance(t, torch.Tensor) or type(t) is not torch.Tensor or t.requires_grad or t.grad_fn is not None
            or t.layout != torch.strided or t.device.type != "cpu" or t.numel() == 0 or not t.is_contiguous()
            or t.dtype in (torch.bool, torch.complex64, torch.complex128)):
        return t
    return sim.guard(t, align=16, keep=False)       # 16-byte aligned starts, as every device allocation has


def _host_only(fn, poison=False):
    """``poison``: memory that the caller did not initialise (torch.empty) reads as NaN / -1 (all bits set)
    instead of the zeros a fresh mapping holds, so a kernel that consumes scratch memory or an output it
    never wrote cannot pass by luck."""
    def wrapped(*args, **kwargs):
        kwargs.pop("pin_memory", None)
        dev = kwargs.get("device")
        if dev is not None and torch.device(dev).type == "cuda":
            kwargs["device"] = "cpu"
        if kwargs.get("out") is not None:
            return fn(*args, **kwargs)
        out = _behind_a_guard_page(fn(*args, **kwargs))
        if poison and isinstance(out, torch.Tensor) and out.numel() and out.is_contiguous() and out.dtype != torch.bool:
            out.view(-1).view(torch.uint8).fill_(0xFF)
        return out
    return wrapped


def activate():
    from flextrain_amd import _lib

    from . import sim

    global CLOCKS
    _lib._lib = sim.lib()
    CLOCKS = order.Clocks(sim.lib())
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
    torch.cuda.synchronize = lambda device=None: CLOCKS.host_sync()
    torch.cuda.Stream = _Stream
    torch.cuda.Event = _Event
    torch.cuda.memory_allocated = lambda device=None: 0
    torch.cuda.set_device = lambda device: None
    torch.cuda.set_stream = lambda s: current.__setitem__(len(current) - 1, s)
    torch.cuda.empty_cache = lambda: None
    torch.cuda.init = lambda: None
    # a tensor "moved to the GPU" is a copy there, and the tests rely on it (in-place kernels must not touch
    # the host original that the oracle is given afterwards); on one device Tensor.to returns the tensor itself
    plain_to = torch.Tensor.to

    plain_clone = torch.Tensor.clone

    def simulated(d):
        """A CUDA device named by the caller is the simulated one: host memory."""
        if isinstance(d, (torch.device, str)) and not isinstance(d, torch.dtype) and torch.device(d).type == "cuda":
            return torch.device("cpu")
        return d

    def to(self, *args, **kwargs):
        moved = "device" in kwargs or any(isinstance(a, (torch.device, str)) for a in args)
        args = tuple(simulated(a) for a in args)
        if "device" in kwargs:
            kwargs["device"] = simulated(kwargs["device"])
        out = plain_to(self, *args, **kwargs)
        if not moved:
            return out
        return _behind_a_guard_page(plain_clone(out) if out is self else out)

    def clone(self, *args, **kwargs):
        return _behind_a_guard_page(plain_clone(self, *args, **kwargs))

    torch.Tensor.clone = clone

    torch.Tensor.to = to
    # every tensor is "on the GPU" except those the package's pinned-host allocator made
    from flextrain_amd import host_memory

    def in_pinned_host_memory(t):
        p = t.data_ptr()
        return any(base <= p < base + nbytes for base, (_, nbytes) in host_memory._PROCESS_PINNED.items())

    torch.Tensor.is_cuda = property(lambda self: not in_pinned_host_memory(self))
    torch.Tensor.cpu = lambda self, *a, **k: plain_clone(self)      # a device-to-host copy is a copy
    torch.Tensor.is_pinned = lambda self, device=None: True
    torch.Tensor.pin_memory = lambda self, device=None: self
    torch.Tensor.record_stream = lambda self, stream: None
    for name in ("empty", "zeros", "ones", "full", "tensor", "randn", "rand", "arange", "randint", "empty_like", "zeros_like",
                 "ones_like", "full_like", "randn_like", "rand_like"):
        setattr(torch, name, _host_only(getattr(torch, name), poison=name in ("empty", "empty_like")))
