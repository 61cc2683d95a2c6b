"""Happens-before check of multi-stream schedules, for the simulated run of the GPU tests: the Python side.

The clocks live in the simulated library (tests/hostsim/order.cpp): one clock space for what the library
enqueues itself (the copies and optimizer launches of the streamed AdamW chunk, the batched field copies)
and for what the Python layer's streams and events do.  On the GPU a missing wait between two streams shows
only when the timing is unlucky, and the tests of the streamed schedules compare values; here an access that
overlaps an earlier one on another stream (at least one of the two a write) with no chain of events or a
synchronisation from the earlier to the later makes the enqueuing call fail -- deterministically."""
from __future__ import annotations

import ctypes


class StreamOrderError(AssertionError):
    pass


class Clocks:
    def __init__(self, handle):
        u64 = ctypes.c_uint64
        for name, restype, argtypes in (("hostsim_order_snapshot", u64, [u64]), ("hostsim_order_wait", None, [u64, u64]),
                                        ("hostsim_order_wait_stream", None, [u64, u64]), ("hostsim_order_host_sync", None, [u64]),
                                        ("hostsim_order_stream_sync", None, [u64]), ("hostsim_order_checked", u64, []),
                                        ("hostsim_order_deafen", None, [u64]),
                                        ("hostsim_order_last_violation", ctypes.c_char_p, [])):
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = restype, argtypes
        self._h = handle

    def snapshot(self, stream):
        return self._h.hostsim_order_snapshot(stream)

    def wait(self, stream, snapshot):
        self._h.hostsim_order_wait(stream, snapshot)

    def wait_stream(self, stream, other):
        self._h.hostsim_order_wait_stream(stream, other)

    def host_sync(self, snapshot=0):
        """The host has seen the snapshot complete (0: every stream)."""
        self._h.hostsim_order_host_sync(snapshot)

    def stream_sync(self, stream):
        self._h.hostsim_order_stream_sync(stream)

    def deafen(self, stream):
        """For the check's own test: the stream's waits are ignored from now on, as if never made."""
        self._h.hostsim_order_deafen(stream)

    @property
    def checked(self):
        """Cross-stream pairs of overlapping accesses examined so far."""
        return int(self._h.hostsim_order_checked())

    @property
    def last_violation(self):
        return self._h.hostsim_order_last_violation().decode()
