"""Python side of the host simulation: the simulated library bound with the package's own ctypes
signatures, and tensors whose storage ends at an inaccessible page."""
from __future__ import annotations

import ctypes
import mmap
import os

import torch

from . import build as _build

_PAGE = mmap.PAGESIZE
_libc = ctypes.CDLL(None, use_errno=True)
_libc.mprotect.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
_keep = []          # mappings of guard(..., keep=True): they live as long as the process
_lib = None


def lib():
    """The simulated libflexhip, every entry point it exports bound with the signature the package binds
    the real library with (``flextrain_amd._lib._SIGNATURES``)."""
    global _lib
    if _lib is None:
        from flextrain_amd._lib import _SIGNATURES

        handle = ctypes.CDLL(_build.build())
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(handle, name, None)
            if fn is not None:
                fn.restype, fn.argtypes = restype, argtypes
        handle.hostsim_set_reverse_schedule(int(os.environ.get("HOSTSIM_LANE_ORDER", "ascending") == "descending"))
        _lib = handle
    return _lib


def guard(t: torch.Tensor, align: int = 16, keep: bool = True) -> torch.Tensor:
    """A copy of ``t`` (contiguous) whose last byte is followed, within ``align`` bytes, by a page that
    may be neither read nor written; the page before the mapping's first is protected too.  With ``keep``
    the mapping lives as long as the process, so that a test may pass ``p(guard(x))`` of a temporary;
    without it the tensor alone holds the mapping (``torch.frombuffer`` keeps its buffer) and releases it
    when it dies."""
    t = t.detach().contiguous()
    nbytes = t.numel() * t.element_size()
    if nbytes == 0:
        return torch.empty_like(t)
    body = (nbytes + _PAGE - 1) // _PAGE * _PAGE
    mm = mmap.mmap(-1, body + 2 * _PAGE)
    probe = ctypes.c_char.from_buffer(mm)
    base = ctypes.addressof(probe)
    del probe
    if _libc.mprotect(base, _PAGE, 0) != 0 or _libc.mprotect(base + _PAGE + body, _PAGE, 0) != 0:
        raise OSError(ctypes.get_errno(), "mprotect")
    # HOSTSIM_GUARD_SIDE=front puts the tensor right after the protected first page instead: the check for
    # accesses BEFORE a buffer (a negative index, an offset subtracted twice)
    start = _PAGE if os.environ.get("HOSTSIM_GUARD_SIDE") == "front" else (_PAGE + body - nbytes) // align * align
    if keep:
        _keep.append(mm)
    out = torch.frombuffer(mm, dtype=t.dtype, count=t.numel(), offset=start).view(t.shape)
    out.copy_(t)
    return out


def p(t):
    return None if t is None else t.data_ptr()


DT = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def pi64(t):
    """An int64 tensor as the POINTER(c_int64) the stride arguments are declared with."""
    return None if t is None else ctypes.cast(t.data_ptr(), ctypes.POINTER(ctypes.c_int64))
