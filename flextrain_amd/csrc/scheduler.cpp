// Save-level transmission scheduler: choose, for each of T tasks that arrive one after
// another, one of k transfer options (duration, value) so that every transfer finishes
// before the buffer it occupies is needed again, maximising the total value.
//
// Host code (the problem is a few hundred tasks, solved once per planning round).
// Exports the two entry points of the reference helper with identical names, argument
// order and return conventions
// (helpers/transmission_scheduler/transmission_scheduler/transmission_scheduler.h:23-36)
// and follows its tick rules and tie-breaks
// (helpers/transmission_scheduler/transmission_scheduler/transmission_scheduler.c:35-59,
// :120-171, :184-207) so that the chosen option vector is the same one:
//   arrival[i]  = trunc(sum_{j<=i} compute[j] * time_scale)      (running sum in double)
//   deadline[i] = min(trunc(deadline * time_scale), arrival[i+N-1])   when i+N-1 < T
//   dur         = max(1, trunc(duration * time_scale))
//   a transfer starts at max(arrival, finish of the previous transfer)
//   among equal totals the earliest writer wins: options ascending; within an option the
//   "link was idle at arrival" predecessor (the best-valued idle state, earliest first)
//   before busy predecessors in ascending finish time; the final state is the earliest
//   finish time with the maximal total.
//
// The dynamic programme is kept over absolute ticks on a band [lo, hi] of reachable finish
// times.  buf_size keeps its meaning as the width of the reference's sliding window: a
// state further than buf_size ticks from the window origin is dropped, and the origin
// moves to the band's lower edge once the arrival is past half the window.
#include <cstdint>
#include <cstdlib>
#include <limits>
#include <vector>

#include <hip/hip_runtime_api.h>  // hipStream_t for the shared header

#include "flexhip.h"

namespace {

constexpr double kUnreached = -1.0e18;

struct Step {           // how the best state with a given finish time was reached
    int8_t option;
    int32_t from;       // absolute finish time of the predecessor state
};

struct Ticks {
    std::vector<int> arrival, limit, dur;  // dur is T*k
};

Ticks to_ticks(int T, int N, int k, const double* compute, const double* durations, double deadline,
               int time_scale) {
    Ticks tk;
    tk.arrival.resize(T);
    tk.limit.resize(T);
    tk.dur.resize((size_t)T * k);
    double clock = 0.0;
    for (int i = 0; i < T; ++i) {
        clock += compute[i];
        tk.arrival[i] = (int)(clock * time_scale);
    }
    const int final_tick = (int)(deadline * time_scale);
    for (int i = 0; i < T; ++i) {
        int lim = final_tick;
        const int j = i + N - 1;
        if (j >= 0 && j < T && tk.arrival[j] < lim) lim = tk.arrival[j];
        tk.limit[i] = lim;
    }
    for (size_t i = 0; i < (size_t)T * k; ++i) {
        const int d = (int)(durations[i] * time_scale);
        tk.dur[i] = d < 1 ? 1 : d;
    }
    return tk;
}

}  // namespace

extern "C" double solve_scheduler(int T, int N, int k, const double* compute, const double* durations,
                                  const double* sizes, double deadline, int time_scale, int buf_size,
                                  int* out_choices) {
    if (T <= 0 || k <= 0 || k > 127 || buf_size <= 0 || !compute || !durations || !sizes || !out_choices) return 0.0;
    const Ticks tk = to_ticks(T, N, k, compute, durations, deadline, time_scale);

    // band of the current states: value[t - lo] for finish times lo..hi
    std::vector<double> cur(1, 0.0), nxt;
    int lo = 0, hi = 0;
    int origin = 0;  // absolute tick of the reference window's index 0
    std::vector<std::vector<Step>> trace(T);
    std::vector<int> trace_lo(T);

    for (int i = 0; i < T; ++i) {
        const int a = tk.arrival[i];
        const int lim = tk.limit[i];
        const int* dur = &tk.dur[(size_t)i * k];
        const double* val = &sizes[(size_t)i * k];
        if (a - origin >= buf_size / 2 && lo > origin) origin = lo;

        int longest = 0;
        for (int o = 0; o < k; ++o) longest = dur[o] > longest ? dur[o] : longest;

        // best predecessor that leaves the link idle at the arrival (finish <= a)
        double idle_best = kUnreached;
        int idle_from = 0;
        for (int t = lo; t <= hi && t <= a; ++t) {
            if (cur[t - lo] > idle_best) { idle_best = cur[t - lo]; idle_from = t; }
        }

        const int busy_first = a + 1 > lo ? a + 1 : lo;           // predecessors still transmitting at a
        const int out_lo = (a < lo ? a : lo) + 1;                 // earliest conceivable finish
        const int out_hi = (a > hi ? a : hi) + longest;
        nxt.assign((size_t)(out_hi - out_lo + 1), kUnreached);
        std::vector<Step>& steps = trace[i];
        steps.assign(nxt.size(), Step{0, 0});
        trace_lo[i] = out_lo;
        int new_lo = std::numeric_limits<int>::max(), new_hi = -1;

        auto offer = [&](int finish, double total, int option, int from) {
            const int rel = finish - origin;
            if (finish > lim || rel < 0 || rel >= buf_size) return;
            double& slot = nxt[finish - out_lo];
            if (total > slot) {
                slot = total;
                steps[finish - out_lo] = Step{(int8_t)option, from};
                if (finish < new_lo) new_lo = finish;
                if (finish > new_hi) new_hi = finish;
            }
        };

        for (int o = 0; o < k; ++o) {
            if (idle_best > kUnreached) offer(a + dur[o], idle_best + val[o], o, idle_from);
            for (int t = busy_first; t <= hi; ++t) {
                const double v = cur[t - lo];
                if (v > kUnreached) offer(t + dur[o], v + val[o], o, t);
            }
        }
        if (new_hi < 0) return 0.0;  // no option of this task meets its deadline

        // keep the reached part of the band
        cur.assign(nxt.begin() + (new_lo - out_lo), nxt.begin() + (new_hi - out_lo + 1));
        lo = new_lo;
        hi = new_hi;
    }

    double best = kUnreached;
    int at = -1;
    for (int t = lo; t <= hi; ++t) {
        if (cur[t - lo] > best) { best = cur[t - lo]; at = t; }
    }
    if (at < 0) return 0.0;
    for (int i = T - 1; i >= 0; --i) {
        const Step s = trace[i][at - trace_lo[i]];
        out_choices[i] = s.option;
        at = s.from;
    }
    return best;
}

// Window width for solve_scheduler: a power of two, at least 2048, that covers the widest
// span the band can take (simulated from the earliest / latest possible finish times)
// plus 256 ticks.  helpers/transmission_scheduler/transmission_scheduler/transmission_scheduler.c:463-533.
extern "C" int compute_buf_size(int T, int N, int k, const double* compute, const double* durations,
                                double deadline, int time_scale) {
    if (T <= 0 || k <= 0 || !compute || !durations) return 2048;
    const Ticks tk = to_ticks(T, 1, k, compute, durations, deadline, time_scale);  // limits recomputed below
    const int final_tick = (int)(deadline * time_scale);
    int longest = 1, shortest = std::numeric_limits<int>::max();
    for (int d : tk.dur) {
        longest = d > longest ? d : longest;
        shortest = d < shortest ? d : shortest;
    }
    int band_lo = 0, band_hi = 0, widest = 0;
    for (int i = 0; i < T; ++i) {
        const int a = tk.arrival[i];
        const int j = i + N - 1;
        const int lim = (j >= 0 && j < T) ? tk.arrival[j] : final_tick;   // as the reference: no min()
        const int from_idle = a - band_lo + longest;
        const int from_busy = band_hi - band_lo + longest;
        const int reach = from_idle > from_busy ? from_idle : from_busy;
        widest = reach > widest ? reach : widest;
        int next_hi = (band_hi > a ? band_hi : a) + longest;
        if (next_hi > lim) next_hi = lim;
        band_lo = a + shortest;
        band_hi = next_hi;
    }
    const int needed = widest + 256;
    int size = 1;
    while (size < needed) size <<= 1;
    return size < 2048 ? 2048 : size;
}
