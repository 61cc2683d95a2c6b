// Happens-before check of multi-stream schedules in the host simulation.
//
// Every stream carries a vector clock.  An enqueued operation ticks its stream; an event record takes a
// snapshot of the stream's clock; a wait merges a snapshot into the waiting stream's clock; a host-side
// synchronisation makes what it covers precede everything enqueued later.  Operations declare the byte
// ranges they read and write, and an access that overlaps an earlier one on another stream (at least one
// of the two a write) with no chain of events from the earlier to the later is a violation -- found at
// the enqueue, whatever the timing on a GPU would have been.  One clock space serves the operations the
// library enqueues itself (copies of the streamed optimizer chunk) and those the Python layer enqueues.
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <set>
#include <string>
#include <vector>

namespace {

typedef std::map<uint64_t, uint64_t> Clock;        // stream -> tick

struct Access {
    uint64_t lo, hi;
    bool write;
    uint64_t stream, tick;
    std::string what;
};

Clock g_host;                                       // per stream: the tick the host has seen complete
std::map<uint64_t, uint64_t> g_ticks;               // per stream: ticks issued
std::map<uint64_t, Clock> g_seen;                   // per stream: what its next operation follows
std::vector<Clock> g_snapshots(1);                  // handle -> clock (handle 0: nothing)
std::vector<Access> g_history;
uint64_t g_checked = 0;
std::string g_violation;
std::set<uint64_t> g_deaf;                          // streams whose waits are ignored (the check's own test)

void merge(Clock& into, const Clock& other) {
    for (const auto& kv : other)
        if (into[kv.first] < kv.second) into[kv.first] = kv.second;
}

Clock snapshot_of(uint64_t stream) {
    Clock c = g_seen[stream];
    merge(c, g_host);
    c[stream] = g_ticks[stream];
    return c;
}

}  // namespace

extern "C" {

// What an event recorded on the stream now stands for; the handle stays valid for the process.
uint64_t hostsim_order_snapshot(uint64_t stream) {
    g_snapshots.push_back(snapshot_of(stream));
    return g_snapshots.size() - 1;
}

void hostsim_order_wait(uint64_t stream, uint64_t handle) {
    if (g_deaf.count(stream)) return;
    if (handle && handle < g_snapshots.size()) merge(g_seen[stream], g_snapshots[handle]);
}

void hostsim_order_wait_stream(uint64_t stream, uint64_t other) {
    if (!g_deaf.count(stream)) merge(g_seen[stream], snapshot_of(other));
}

// For the check's own test: from now on the stream's waits are ignored, as if the code never made them.
void hostsim_order_deafen(uint64_t stream) { g_deaf.insert(stream); }

// The host has seen the snapshot complete (handle 0: every stream, as a device synchronisation).
void hostsim_order_host_sync(uint64_t handle) {
    if (handle && handle < g_snapshots.size()) {
        merge(g_host, g_snapshots[handle]);
    } else {
        for (const auto& kv : g_ticks) merge(g_host, snapshot_of(kv.first));
    }
    size_t kept = 0;
    for (size_t i = 0; i < g_history.size(); ++i)
        if (g_host[g_history[i].stream] < g_history[i].tick) g_history[kept++] = g_history[i];
    g_history.resize(kept);
}

void hostsim_order_stream_sync(uint64_t stream) {
    g_snapshots.push_back(snapshot_of(stream));
    hostsim_order_host_sync(g_snapshots.size() - 1);
}

// One operation on `stream` with n byte ranges (lo[i], bytes[i], is_write[i]).  Returns 0, or 1 when one
// of them is not ordered after an earlier overlapping access (text: hostsim_order_last_violation()).
int hostsim_order_enqueue(uint64_t stream, const char* what, int n, const uint64_t* lo, const uint64_t* bytes, const int* is_write) {
    const uint64_t tick = ++g_ticks[stream];
    Clock after = g_seen[stream];
    merge(after, g_host);
    int bad = 0;
    for (int i = 0; i < n && !bad; ++i) {
        if (!lo[i] || !bytes[i]) continue;
        const uint64_t a = lo[i], b = lo[i] + bytes[i];
        for (const Access& p : g_history) {
            if (p.stream == stream || !(is_write[i] || p.write) || p.hi <= a || b <= p.lo) continue;
            ++g_checked;
            if (after[p.stream] < p.tick) {
                char text[600];
                snprintf(text, sizeof text,
                         "%s on stream %#llx is not ordered after %s on stream %#llx (%s then %s of overlapping bytes "
                         "[%#llx, %#llx)): no event or synchronisation leads from the earlier to the later",
                         what, (unsigned long long)stream, p.what.c_str(), (unsigned long long)p.stream, p.write ? "write" : "read",
                         is_write[i] ? "write" : "read", (unsigned long long)(a > p.lo ? a : p.lo), (unsigned long long)(b < p.hi ? b : p.hi));
                g_violation = text;
                fprintf(stderr, "hostsim: %s\n", text);
                bad = 1;
                break;
            }
        }
    }
    for (int i = 0; i < n; ++i)
        if (lo[i] && bytes[i]) g_history.push_back(Access{lo[i], lo[i] + bytes[i], is_write[i] != 0, stream, tick, what});
    return bad;
}

const char* hostsim_order_last_violation() { return g_violation.c_str(); }
uint64_t hostsim_order_checked() { return g_checked; }

}  // extern "C"
