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

// The two inner loops are built once per vector width and picked by the CPU the library runs on; every
// build gives the same results (no reassociation, compares and selects only).  Defining the macro empty
// builds the single baseline form, e.g. to compare the forms with each other.
#ifndef FX_VECTOR_BUILDS
#define FX_VECTOR_BUILDS __attribute__((target_clones("avx512f", "avx2", "default")))
#endif

// One option of one task over the part of the band that was still transmitting at the arrival: a state
// with finish time t becomes finish time t + dur with the option's value added.  cur and nxt are already
// shifted so that element j of both is the same new finish time.  Strictly greater only: an earlier
// writer (a lower option) keeps a tie.  The pick is kept as wide as the values so that the loop is one
// compare and two blends per vector.
FX_VECTOR_BUILDS
void relax(const double* __restrict__ cur, double* __restrict__ nxt, int64_t* __restrict__ pick, int n, double value,
           int64_t option) {
    for (int j = 0; j < n; ++j) {
        const double cand = cur[j] + value;
        const bool better = cand > nxt[j];
        nxt[j] = better ? cand : nxt[j];
        pick[j] = better ? option : pick[j];
    }
}

FX_VECTOR_BUILDS
void narrow(const int64_t* __restrict__ pick, uint8_t* __restrict__ out, int n) {
    for (int j = 0; j < n; ++j) out[j] = (uint8_t)pick[j];
}

constexpr int64_t kFromIdle = 0x80;   // the state was reached from the link-idle predecessor of its task

}  // namespace

static double solve(int T, int N, int k, const double* compute, const double* durations, const double* sizes,
                    double deadline, int time_scale, int buf_size, int* out_choices) {
    if (T <= 0 || k <= 0 || k > 127 || buf_size <= 0 || !compute || !durations || !sizes || !out_choices) return 0.0;
    const Ticks tk = to_ticks(T, N, k, compute, durations, deadline, time_scale);
    constexpr double kNone = -std::numeric_limits<double>::infinity();   // stays "unreached" under any addition

    // Band of the current states: cur[t - lo] for finish times lo..hi.  Two buffers alternate; the one
    // that is written next holds nothing live and grows to the width the task can reach (at most
    // buf_size: every kept finish time lies within buf_size ticks of the window origin).
    std::vector<double> store[2];
    std::vector<int64_t> pick;
    int cur_in = 0;                  // which buffer holds the current band
    store[0].assign(1, 0.0);
    const double* cur = store[0].data();
    int lo = 0, hi = 0;
    int origin = 0;  // absolute tick of the reference window's index 0
    // How each state was reached, one byte per state and task: the option, and whether the predecessor
    // was the idle one (kept per task) or the busy one (its finish time is this one minus the duration).
    std::vector<uint8_t> trace;
    std::vector<size_t> trace_at(T);
    std::vector<int> trace_lo(T), idle_from(T);

    for (int i = 0; i < T; ++i) {
        const int a = tk.arrival[i];
        const int* dur = &tk.dur[(size_t)i * k];
        const double* val = &sizes[(size_t)i * k];
        if (a - origin >= buf_size / 2 && lo > origin) origin = lo;

        int longest = 0;
        for (int o = 0; o < k; ++o) longest = dur[o] > longest ? dur[o] : longest;

        // best predecessor that leaves the link idle at the arrival (finish <= a), earliest first
        double idle_best = kNone;
        for (int t = lo; t <= hi && t <= a; ++t) {
            if (cur[t - lo] > idle_best) { idle_best = cur[t - lo]; idle_from[i] = t; }
        }

        const int busy_first = a + 1 > lo ? a + 1 : lo;           // predecessors still transmitting at a
        // finish times this task can reach and may keep: before its deadline, inside the window
        int out_lo = (a < lo ? a : lo) + 1;
        int out_hi = (a > hi ? a : hi) + longest;
        if (out_lo < origin) out_lo = origin;
        if (out_hi > tk.limit[i]) out_hi = tk.limit[i];
        if ((int64_t)out_hi > (int64_t)origin + buf_size - 1) out_hi = (int)((int64_t)origin + buf_size - 1);
        if (out_hi < out_lo) return 0.0;
        const int width = out_hi - out_lo + 1;
        store[cur_in ^ 1].assign((size_t)width, kNone);
        pick.assign((size_t)width, 0);
        double* nxt = store[cur_in ^ 1].data();

        for (int o = 0; o < k; ++o) {
            const int d = dur[o];
            const int f_idle = a + d;
            if (idle_best > kNone && f_idle >= out_lo && f_idle <= out_hi && idle_best + val[o] > nxt[f_idle - out_lo]) {
                nxt[f_idle - out_lo] = idle_best + val[o];
                pick[f_idle - out_lo] = o | kFromIdle;
            }
            const int f0 = busy_first + d > out_lo ? busy_first + d : out_lo;
            const int f1 = hi + d < out_hi ? hi + d : out_hi;
            if (f1 >= f0) relax(cur + (f0 - d - lo), nxt + (f0 - out_lo), pick.data() + (f0 - out_lo), f1 - f0 + 1, val[o], o);
        }

        int first = 0, last = width - 1;
        while (first < width && !(nxt[first] > kNone)) ++first;
        if (first == width) return 0.0;  // no option of this task meets its deadline
        while (!(nxt[last] > kNone)) --last;

        trace_at[i] = trace.size();
        trace_lo[i] = out_lo + first;
        trace.resize(trace.size() + (size_t)(last - first + 1));
        narrow(pick.data() + first, trace.data() + trace_at[i], last - first + 1);

        // the reached part of the band becomes the current one; the other buffer is written next
        cur_in ^= 1;
        cur = nxt + first;
        lo = out_lo + first;
        hi = out_lo + last;
    }

    double best = kNone;
    int at = -1;
    for (int t = lo; t <= hi; ++t) {
        if (cur[t - lo] > best) { best = cur[t - lo]; at = t; }
    }
    if (at < 0) return 0.0;
    for (int i = T - 1; i >= 0; --i) {
        const uint8_t how = trace[trace_at[i] + (size_t)(at - trace_lo[i])];
        const int option = how & 0x7f;
        out_choices[i] = option;
        at = (how & kFromIdle) ? idle_from[i] : at - tk.dur[(size_t)i * k + option];
    }
    return best;
}

extern "C" double solve_scheduler(int T, int N, int k, const double* compute, const double* durations,
                                  const double* sizes, double deadline, int time_scale, int buf_size,
                                  int* out_choices) {
    try {
        return solve(T, N, k, compute, durations, sizes, deadline, time_scale, buf_size, out_choices);
    } catch (...) {      // out of memory: "no schedule", as every other failure; nothing is thrown across the C ABI
        return 0.0;
    }
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
