"""Happens-before check of multi-stream schedules, for the simulated run of the GPU tests.

On the GPU a missing wait between two streams shows only when the timing is unlucky; the tests of the
streamed optimizer step and of the activation streamer compare values and can pass by luck.  Here every
stream carries a vector clock: an enqueued operation ticks its stream, ``Event.record`` takes a snapshot,
``wait_event`` / ``wait_stream`` merge one in, a host-side synchronisation makes everything enqueued so far
precede everything enqueued later.  The copies and optimizer launches that the schedules enqueue
(``fx_copy_fields``, ``fx_adamw_step``) declare the byte ranges they read and write, and an access that
overlaps an earlier one on another stream (at least one of the two a write) without a chain of events from
the earlier to the later raises ``StreamOrderError`` at the enqueue -- deterministically, whatever the
timing would have been."""
from __future__ import annotations

import ctypes


class StreamOrderError(AssertionError):
    pass


_ELEM = {0: 4, 1: 2, 2: 2}          # dtype enum of the C ABI -> bytes per element


class Clocks:
    """All streams of a process, their clocks and the accesses not yet ordered before the host."""

    def __init__(self):
        self.host = {}                  # stream id -> tick known to be complete by the host
        self.ticks = {}                 # stream id -> ticks issued
        self.seen = {}                  # stream id -> clock (dict) of the stream: what its next operation follows
        self.names = {}
        self.history = []               # (lo, hi, is_write, stream id, tick, what)
        self.checked = 0

    # ---- clocks
    def _clock(self, sid):
        return self.seen.setdefault(sid, {})

    @staticmethod
    def _merge(into, other):
        for k, v in other.items():
            if into.get(k, 0) < v:
                into[k] = v

    def snapshot(self, sid):
        """What an event recorded on the stream now stands for."""
        c = dict(self._clock(sid))
        self._merge(c, self.host)
        c[sid] = self.ticks.get(sid, 0)
        return c

    def wait(self, sid, clock):
        self._merge(self._clock(sid), clock)

    def host_sync(self, clock=None):
        """The host has seen ``clock`` complete (all streams when None)."""
        if clock is None:
            clock = {}
            for sid in set(self.ticks) | set(self.seen):
                self._merge(clock, self.snapshot(sid))
        self._merge(self.host, clock)
        self.history = [h for h in self.history if self.host.get(h[3], 0) < h[4]]

    # ---- accesses
    def enqueue(self, sid, what, reads=(), writes=()):
        tick = self.ticks[sid] = self.ticks.get(sid, 0) + 1
        after = dict(self._clock(sid))
        self._merge(after, self.host)
        mine = [(lo, lo + n, False) for lo, n in reads if lo and n > 0] + [(lo, lo + n, True) for lo, n in writes if lo and n > 0]
        for lo, hi, is_write in mine:
            for plo, phi, pwrite, psid, ptick, pwhat in self.history:
                if psid == sid or not (is_write or pwrite) or phi <= lo or hi <= plo:
                    continue
                self.checked += 1
                if after.get(psid, 0) < ptick:
                    kind = ("write" if pwrite else "read") + " then " + ("write" if is_write else "read")
                    raise StreamOrderError(
                        f"{what} on stream {self.names.get(sid, sid)} is not ordered after {pwhat} on stream "
                        f"{self.names.get(psid, psid)} ({kind} of overlapping bytes [{max(lo, plo):#x}, {min(hi, phi):#x})): "
                        f"no event or synchronisation leads from the earlier to the later")
        for lo, hi, is_write in mine:
            self.history.append((lo, hi, is_write, sid, tick, what))


CLOCKS = Clocks()


def _i64s(pointer, n):
    return ctypes.cast(pointer, ctypes.POINTER(ctypes.c_int64))[:n] if pointer else [0] * n


def _ptrs(pointer, n):
    return [int(v or 0) for v in ctypes.cast(pointer, ctypes.POINTER(ctypes.c_void_p))[:n]]


def _stream_id(stream):
    return int(getattr(stream, "value", stream) or 0)


def _address(p):
    return int(getattr(p, "value", p) or 0)


class OrderedLibrary:
    """The simulated library with the enqueues of the multi-stream schedules declared to ``CLOCKS``."""

    def __init__(self, handle):
        self._handle = handle

    def __getattr__(self, name):
        return getattr(self._handle, name)

    def fx_copy_fields(self, n, dst, src, rows, row_bytes, dst_pitch, src_pitch, direction, stream):
        d, s = _ptrs(dst, n), _ptrs(src, n)
        r, rb, dp, sp = (_i64s(a, n) for a in (rows, row_bytes, dst_pitch, src_pitch))
        span = lambda i, pitch: (r[i] - 1) * pitch[i] + rb[i] if r[i] > 0 else 0
        CLOCKS.enqueue(_stream_id(stream), f"copy of {n} field(s), direction {direction}",
                       reads=[(s[i], span(i, sp)) for i in range(n)], writes=[(d[i], span(i, dp)) for i in range(n)])
        return self._handle.fx_copy_fields(n, dst, src, rows, row_bytes, dst_pitch, src_pitch, direction, stream)

    def fx_adamw_step(self, p, g, m, v, p_bf16_out, n, p_dt, g_dt, state_dt, *rest):
        stream = rest[-1]
        pb, gb, sb = n * _ELEM[p_dt], n * _ELEM[g_dt], n * _ELEM[state_dt]
        p, g, m, v, out = (_address(a) for a in (p, g, m, v, p_bf16_out))
        CLOCKS.enqueue(_stream_id(stream), f"AdamW step over {n} elements", reads=[(g, gb)],
                       writes=[(p, pb), (m, sb), (v, sb), (out, 2 * n)])
        return self._handle.fx_adamw_step(p or None, g or None, m or None, v or None, out or None, n, p_dt, g_dt, state_dt, *rest)
