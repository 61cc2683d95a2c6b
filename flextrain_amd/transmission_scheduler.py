"""``TransmissionScheduler`` with the interface of the reference helper package
(helpers/transmission_scheduler/transmission_scheduler/__init__.py:7-141), on top of
``solve_scheduler`` / ``compute_buf_size`` of libflexhip.so.  CPU only: nothing here
touches the GPU."""
from __future__ import annotations

import numpy as np

from ._lib import lib

TIME_SCALE = 10          # ticks per millisecond (0.1 ms resolution), as the reference wrapper


class TransmissionScheduler:
    def __init__(self):
        self.lib = lib()

    def solve(self, compute, durations, sizes, N):
        """``(best_val, choices)`` or ``(None, None)`` when no schedule keeps every
        transfer inside its buffer window.

        compute ``(T,)``: time between task arrivals (ms); durations, sizes ``(T, k)``:
        transfer time (ms) and value of each option; ``N``: buffer depth — task ``i`` must
        finish before task ``i + N - 1`` arrives.  Non-positive sizes are shifted to be
        >= 1 for the solver and the returned value is corrected
        (helpers/transmission_scheduler/transmission_scheduler/__init__.py:88-141)."""
        compute = np.ascontiguousarray(compute, dtype=np.float64)
        durations = np.ascontiguousarray(durations, dtype=np.float64)
        sizes = np.ascontiguousarray(sizes, dtype=np.float64)
        T, k = durations.shape
        safe_deadline = float(np.sum(compute) + np.sum(np.max(durations, axis=1)) + 1000.0)
        flat_durs = np.ascontiguousarray(durations.reshape(-1))
        buf_size = self.lib.compute_buf_size(T, N, k, compute.ctypes.data, flat_durs.ctypes.data, safe_deadline,
                                             TIME_SCALE)
        min_val = float(np.min(sizes))
        offset = abs(min_val) + 1.0 if min_val <= 0 else 0.0
        flat_sizes = np.ascontiguousarray((sizes + offset).reshape(-1)) if offset > 0 else np.ascontiguousarray(
            sizes.reshape(-1))
        choices = np.zeros(T, dtype=np.int32)
        raw_val = self.lib.solve_scheduler(T, N, k, compute.ctypes.data, flat_durs.ctypes.data,
                                           flat_sizes.ctypes.data, safe_deadline, TIME_SCALE, buf_size,
                                           choices.ctypes.data)
        if raw_val == 0.0:
            return None, None
        return raw_val - T * offset, choices
