"""Save-level transmission scheduler oracle (CPU, NumPy).  Test infrastructure — see
oracle/__init__.py.

Restates helpers/transmission_scheduler/transmission_scheduler/transmission_scheduler.c:
tick conversion (:35-59), the per-task dynamic programme with its tie-breaks (:77-187,
strict ``>`` keeps the first writer; options ascending; the idle-link predecessor before
busy predecessors in ascending finish time), the final earliest-maximum pick and the
traceback (:189-207); ``compute_buf_size`` (:463-533); and the Python wrapper's value
shift (helpers/transmission_scheduler/transmission_scheduler/__init__.py:88-141).

The dynamic programme is written over one dense array of absolute ticks.  The
reference keeps a sliding window of ``buf_size`` ticks instead and DROPS states that
fall outside it (:133, :151); its origin moves to the band's lower edge once a task's
arrival is at least half a window past it (:90-103).  Passing ``buf_size`` reproduces
that rule — needed for identical answers, because the width ``compute_buf_size``
returns does not always prevent drops (golden case "tradeoff_64x4": the windowed
answer is 35200, the unwindowed optimum 35700); ``buf_size=None`` is the plain
optimum that exhaustive enumeration checks.

Pinned by tests/test_scheduler.py: the README known answer
(orig/transmission_scheduler_pkg/README.md:47-59), golden vectors written by the
compiled reference (tests/golden/scheduler_cases.json, both its AVX2 and scalar
builds), and exhaustive enumeration of all k^T option vectors for small T
(``brute_force`` below), which fixes the optimum and feasibility independently of any
dynamic programme.
"""
from __future__ import annotations

import itertools

import numpy as np

UNREACHED = -1.0e18


def to_ticks(compute, durations, deadline, time_scale, N):
    """-> (arrival[T], limit[T], dur[T,k]) as Python ints / int arrays (C truncation)."""
    compute = np.asarray(compute, dtype=np.float64)
    durations = np.asarray(durations, dtype=np.float64)
    T = compute.shape[0]
    clock = 0.0
    arrival = np.empty(T, dtype=np.int64)
    for i in range(T):                       # sequential sum, as the C loop
        clock += float(compute[i])
        arrival[i] = int(clock * time_scale)
    final_tick = int(deadline * time_scale)
    limit = np.full(T, final_tick, dtype=np.int64)
    for i in range(T):
        j = i + N - 1
        if 0 <= j < T and arrival[j] < limit[i]:
            limit[i] = arrival[j]
    dur = np.maximum(1, np.trunc(durations * time_scale).astype(np.int64))
    return arrival, limit, dur


def solve_scheduler(compute, durations, sizes, deadline, time_scale, N, buf_size=None):
    """-> (best total, choices int32[T]) or (0.0, None) when infeasible."""
    durations = np.asarray(durations, dtype=np.float64)
    sizes = np.asarray(sizes, dtype=np.float64)
    T, k = durations.shape
    arrival, limit, dur = to_ticks(compute, durations, deadline, time_scale, N)
    horizon = int(max(limit.max(), arrival.max())) + int(dur.max()) + 2
    cur = np.full(horizon, UNREACHED)
    cur[0] = 0.0
    lo = hi = 0
    opt_trace = np.zeros((T, horizon), dtype=np.int8)
    src_trace = np.zeros((T, horizon), dtype=np.int64)
    origin = 0
    for i in range(T):
        a, lim = int(arrival[i]), int(limit[i])
        if buf_size is not None:
            if a - origin >= buf_size // 2 and lo > origin:
                origin = lo
            lim = min(lim, origin + buf_size - 1)      # finish - origin < buf_size
        nxt = np.full(horizon, UNREACHED)
        idle_best, idle_from = UNREACHED, 0
        if lo <= min(hi, a):
            seg = cur[lo:min(hi, a) + 1]
            j = int(np.argmax(seg))          # first maximum
            if seg[j] > UNREACHED:
                idle_best, idle_from = float(seg[j]), lo + j
        busy_first = max(a + 1, lo)
        for o in range(k):
            d, s = int(dur[i, o]), float(sizes[i, o])
            if idle_best > UNREACHED:
                f = a + d
                if f <= lim and idle_best + s > nxt[f]:
                    nxt[f] = idle_best + s
                    opt_trace[i, f], src_trace[i, f] = o, idle_from
            if busy_first <= hi:
                src = np.arange(busy_first, hi + 1)
                v = cur[src]
                dest = src + d
                ok = (v > UNREACHED) & (dest <= lim)
                src, dest, cand = src[ok], dest[ok], v[ok] + s
                win = cand > nxt[dest]
                nxt[dest[win]] = cand[win]
                opt_trace[i, dest[win]] = o
                src_trace[i, dest[win]] = src[win]
        reached = np.nonzero(nxt > UNREACHED)[0]
        if reached.size == 0:
            return 0.0, None
        lo, hi = int(reached[0]), int(reached[-1])
        cur = nxt
    seg = cur[lo:hi + 1]
    at = lo + int(np.argmax(seg))
    best = float(cur[at])
    choices = np.zeros(T, dtype=np.int32)
    for i in range(T - 1, -1, -1):
        choices[i] = opt_trace[i, at]
        at = int(src_trace[i, at])
    return best, choices


def compute_buf_size(compute, durations, deadline, time_scale, N):
    durations = np.asarray(durations, dtype=np.float64)
    T, k = durations.shape
    arrival, _, dur = to_ticks(compute, durations, deadline, time_scale, 1)
    final_tick = int(deadline * time_scale)
    longest, shortest = int(max(1, dur.max())), int(dur.min())
    band_lo = band_hi = widest = 0
    for i in range(T):
        a = int(arrival[i])
        lim = int(arrival[i + N - 1]) if 0 <= i + N - 1 < T else final_tick
        widest = max(widest, a - band_lo + longest, band_hi - band_lo + longest)
        band_hi = min(max(band_hi, a) + longest, lim)
        band_lo = a + shortest
    size = 1
    while size < widest + 256:
        size <<= 1
    return max(size, 2048)


def wrapper_solve(compute, durations, sizes, N, time_scale=10):
    """``TransmissionScheduler.solve``: -> (value, choices) or (None, None)."""
    compute = np.asarray(compute, dtype=np.float64)
    durations = np.asarray(durations, dtype=np.float64)
    sizes = np.asarray(sizes, dtype=np.float64)
    T = durations.shape[0]
    deadline = float(np.sum(compute) + np.sum(np.max(durations, axis=1)) + 1000.0)
    lowest = float(np.min(sizes))
    offset = abs(lowest) + 1.0 if lowest <= 0 else 0.0
    buf = compute_buf_size(compute, durations, deadline, time_scale, N)
    raw, choices = solve_scheduler(compute, durations, sizes + offset, deadline, time_scale, N, buf_size=buf)
    if raw == 0.0:
        return None, None
    return raw - T * offset, choices


def simulate(choices, compute, durations, sizes, deadline, time_scale, N):
    """Total value of one option vector, or None when a transfer misses its limit."""
    arrival, limit, dur = to_ticks(compute, durations, deadline, time_scale, N)
    sizes = np.asarray(sizes, dtype=np.float64)
    t, total = 0, 0.0
    for i, o in enumerate(choices):
        t = max(t, int(arrival[i])) + int(dur[i, o])
        if t > limit[i]:
            return None
        total += float(sizes[i, o])
    return total


def brute_force(compute, durations, sizes, deadline, time_scale, N):
    """Best total over all k^T option vectors (None when none is feasible)."""
    T, k = np.asarray(durations).shape
    best = None
    for choice in itertools.product(range(k), repeat=T):
        v = simulate(choice, compute, durations, sizes, deadline, time_scale, N)
        if v is not None and (best is None or v > best):
            best = v
    return best
