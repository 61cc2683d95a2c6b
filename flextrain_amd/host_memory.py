"""Pinned host memory for the engine's master weights, gradients and optimizer state,
with the interface of flextrain/engine/host_memory.py:109-225
(``HostMemoryBackend``, ``LocalPinnedHostBackend``) and of
flextrain/ops/_kernels/_mem_register.py:4-20 (``pin_tensor``, ``destory_tensor``,
re-exported by the reference as ``destroy_pinned_tensor``).

The reference allocates ordinary host tensors and registers them with the driver
afterwards, to avoid the power-of-two rounding of torch's pinned caching allocator.
Here the same goal — exact-size pinned memory — is met by allocating the memory pinned
in the first place (``fx_host_alloc`` = hipHostMalloc): registering memory that already
exists is refused on some systems, and a failed registration leaves an error behind
that a later, unrelated GPU call would report.
"""
from __future__ import annotations

import ctypes
from typing import Protocol, runtime_checkable

import torch

from ._lib import lib

# data_ptr -> (ctypes buffer object, nbytes) of every live allocation made here
_PROCESS_PINNED: dict[int, tuple[object, int]] = {}


def _alloc_pinned_bytes(nbytes: int) -> torch.Tensor:
    """A uint8 tensor over ``nbytes`` freshly allocated pinned bytes (zero-filled)."""
    torch.cuda.init()   # torch reports memory as pinned only once its own GPU context exists
    out = ctypes.c_void_p()
    if lib().fx_host_alloc(nbytes, ctypes.byref(out)) != 0 or not out.value:
        raise RuntimeError(f"pinned host allocation of {nbytes} bytes failed")
    buf = (ctypes.c_uint8 * nbytes).from_address(out.value)
    t = torch.frombuffer(buf, dtype=torch.uint8)
    t.zero_()
    _PROCESS_PINNED[out.value] = (buf, nbytes)
    return t


def _free_pinned(ptr: int) -> bool:
    if _PROCESS_PINNED.pop(ptr, None) is None:
        return False
    lib().fx_host_free(ptr)
    return True


@runtime_checkable
class HostMemoryBackend(Protocol):
    """flextrain/engine/host_memory.py:109-155."""

    name: str

    def allocate_tensor(self, shape, dtype) -> torch.Tensor: ...

    def release(self, tensor: torch.Tensor) -> None: ...


class LocalPinnedHostBackend:
    """Zero-initialised, exactly-sized pinned tensors in local host RAM
    (flextrain/engine/host_memory.py:161-212).  ``release`` is idempotent; the tensor
    must not be used afterwards."""

    name = "local_pinned"

    def __init__(self) -> None:
        self._owned: set[int] = set()

    def allocate_tensor(self, shape, dtype) -> torch.Tensor:
        shape = tuple(int(s) for s in shape)
        numel = 1
        for s in shape:
            numel *= s
        if numel == 0:
            return torch.zeros(shape, dtype=dtype)
        raw = _alloc_pinned_bytes(numel * torch.empty((), dtype=dtype).element_size())
        self._owned.add(raw.data_ptr())
        return raw.view(dtype).view(shape)

    def release(self, tensor: torch.Tensor) -> None:
        ptr = tensor.data_ptr()
        if ptr in self._owned:
            self._owned.discard(ptr)
            _free_pinned(ptr)

    def available_bytes(self) -> int:
        import os
        return os.sysconf("SC_AVPHYS_PAGES") * os.sysconf("SC_PAGE_SIZE")


def unregister_all_process_pinned_memory() -> None:
    """Free every pinned allocation this process still holds
    (flextrain/engine/host_memory.py:215-225)."""
    for ptr in list(_PROCESS_PINNED):
        _free_pinned(ptr)


def pin_tensor(tensor: torch.Tensor) -> torch.Tensor:
    """Make a CPU tensor usable for asynchronous GPU copies and return it
    (flextrain/ops/_kernels/_mem_register.py:4-9).  The tensor object is kept; its
    storage is replaced by pinned memory holding the same values, so other views of the
    OLD storage no longer alias it (the reference pins the existing pages in place)."""
    if tensor.device.type != "cpu" or tensor.numel() == 0 or tensor.is_pinned():
        return tensor
    if not tensor.is_contiguous():
        raise ValueError("pin_tensor needs a contiguous tensor")
    raw = _alloc_pinned_bytes(tensor.numel() * tensor.element_size())
    pinned = raw.view(tensor.dtype).view(tensor.shape)
    pinned.copy_(tensor)
    tensor.set_(pinned)
    return tensor


def destory_tensor(tensor: torch.Tensor, is_pinned: bool = True) -> None:
    """Release the pinned memory behind ``tensor`` (the reference's spelling,
    flextrain/ops/_kernels/_mem_register.py:11-20)."""
    if tensor.device.type == "cpu" and is_pinned:
        if not _free_pinned(tensor.data_ptr()):
            print(f"Failed to unregsiter cpu tensor at addr: {tensor.data_ptr()} of size "
                  f"{tensor.numel() * tensor.element_size()}")


destroy_pinned_tensor = destory_tensor

__all__ = ["HostMemoryBackend", "LocalPinnedHostBackend", "pin_tensor", "destory_tensor", "destroy_pinned_tensor",
           "unregister_all_process_pinned_memory"]
