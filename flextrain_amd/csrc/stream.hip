// Host <-> HBM streaming of one offloaded optimizer chunk, and pinned host memory.
//
// The reference engine keeps master weights, gradients and Adam moments of a layer in
// pinned host memory and, for the optimizer step, copies a whole layer in on an
// "inbound" stream, runs one kernel per tensor on the "compute" stream and copies the
// layer back on an "outbound" stream, rotating layers through ring slots
// (flextrain/engine/active_model.py:486-655, flextrain/engine/buffers.py:1088-1291,
// streams of flextrain/engine/streams.py:85-128).  fx_adamw_stream_chunk does the same
// for ONE flat chunk at a finer grain: the chunk is cut into sub-chunks that rotate
// through n_slots device staging slots, so the copy-in of sub-chunk i+1, the kernel of
// sub-chunk i and the copy-out of sub-chunk i-1 overlap and both PCIe directions stay
// busy.  Everything is enqueued without blocking the host; ordering is by events:
//     copy-in(i)  waits for copy-out(i - n_slots)     (the slot is free again)
//     kernel(i)   waits for copy-in(i)
//     copy-out(i) waits for kernel(i)
// The events belong to an FxStreamRing that the owner of the staging workspace keeps, so
// the same ordering holds from one call to the next on that workspace (a call without a
// ring orders its first copy-ins after everything enqueued so far on compute and outbound).
// Pinned host memory comes from hipHostMalloc (exact size, no power-of-two rounding:
// the reason the reference registers plain allocations instead of using the caching
// pinned allocator, flextrain/engine/host_memory.py:161-176).
#include "common.h"
#include "flexhip.h"

using namespace fx;

namespace {

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

struct SlotLayout {
    size_t p, g, m, v, pc, stride;  // byte offsets inside a slot, slot stride
};

SlotLayout slot_layout(int64_t sub, int p_dt, int g_dt, int s_dt, bool staged_copy) {
    SlotLayout L;
    size_t o = 0;
    L.p = o;  o = align_up(o + (size_t)sub * elem_size(p_dt), 256);
    L.g = o;  o = align_up(o + (size_t)sub * elem_size(g_dt), 256);
    L.m = o;  o = align_up(o + (size_t)sub * elem_size(s_dt), 256);
    L.v = o;  o = align_up(o + (size_t)sub * elem_size(s_dt), 256);
    L.pc = o; if (staged_copy) o = align_up(o + (size_t)sub * 2, 256);
    L.stride = o;
    return L;
}

#define FX_HIP_OK(expr, what)                                                          \
    do {                                                                               \
        hipError_t e__ = (expr);                                                       \
        if (e__ != hipSuccess) {                                                       \
            fprintf(stderr, "flexhip: %s: %s\n", what, hipGetErrorString(e__));        \
            rc = -1;                                                                   \
            goto done;                                                                 \
        }                                                                              \
    } while (0)

}  // namespace

extern "C" size_t fx_adamw_stream_ws_bytes(int64_t sub_elems, int n_slots, int p_dt, int g_dt, int state_dt,
                                           int stage_bf16_copy) {
    if (sub_elems <= 0 || n_slots <= 0) return 0;
    return slot_layout(sub_elems, p_dt, g_dt, state_dt, stage_bf16_copy != 0).stride * (size_t)n_slots;
}

// Persistent per-slot events of one staging workspace.  A call of fx_adamw_stream_chunk only
// enqueues work, so the NEXT call on the same workspace starts while the previous one's last
// kernels and copy-outs are still in flight: the events that say "slot s is free again" must
// outlive the call that recorded them.
struct FxStreamRing {
    int n_slots = 0;
    size_t stride = 0;          // slot stride of the layout the slots were last used with (0: never used)
    int64_t next = 0;           // running sub-chunk number: slot rotation continues across calls
    bool busy[16] = {};         // out_done[s] has been recorded at least once
    hipEvent_t in_done[16] = {}, k_done[16] = {}, out_done[16] = {}, fence[2] = {};
};

extern "C" int fx_stream_ring_destroy(FxStreamRing* ring) {
    if (!ring) return 0;
    // Destroying an event that is still pending is allowed: its resources are released when it completes.
    for (int s = 0; s < 16; ++s) {
        if (ring->in_done[s]) (void)hipEventDestroy(ring->in_done[s]);
        if (ring->k_done[s]) (void)hipEventDestroy(ring->k_done[s]);
        if (ring->out_done[s]) (void)hipEventDestroy(ring->out_done[s]);
    }
    for (int s = 0; s < 2; ++s)
        if (ring->fence[s]) (void)hipEventDestroy(ring->fence[s]);
    delete ring;
    return 0;
}

extern "C" int fx_stream_ring_create(int n_slots, FxStreamRing** out) {
    if (!out) FX_FAIL("fx_stream_ring_create: null output pointer");
    *out = nullptr;
    if (n_slots < 1 || n_slots > 16) FX_FAIL("fx_stream_ring_create: 1 <= n_slots <= 16");
    FxStreamRing* r = new FxStreamRing();
    r->n_slots = n_slots;
    bool ok = true;
    for (int s = 0; s < n_slots && ok; ++s)
        ok = hipEventCreateWithFlags(&r->in_done[s], hipEventDisableTiming) == hipSuccess &&
             hipEventCreateWithFlags(&r->k_done[s], hipEventDisableTiming) == hipSuccess &&
             hipEventCreateWithFlags(&r->out_done[s], hipEventDisableTiming) == hipSuccess;
    for (int s = 0; s < 2 && ok; ++s) ok = hipEventCreateWithFlags(&r->fence[s], hipEventDisableTiming) == hipSuccess;
    if (!ok) {
        (void)hipGetLastError();
        fx_stream_ring_destroy(r);
        FX_FAIL("fx_stream_ring_create: event creation failed");
    }
    *out = r;
    return 0;
}

extern "C" int fx_adamw_stream_chunk(void* p_host, const void* g_host, void* m_host, void* v_host,
                                     void* p_bf16_out, int p_bf16_out_on_device, int64_t n, int p_dt, int g_dt,
                                     int state_dt, float lr, float beta1, float beta2, float eps, float weight_decay,
                                     float bias_correction1, float bias_correction2, void* ws, size_t ws_bytes,
                                     int64_t sub_elems, int n_slots, hipStream_t inbound, hipStream_t compute,
                                     hipStream_t outbound, FxStreamRing* ring) {
    if (n < 0) FX_FAIL("fx_adamw_stream_chunk: negative element count");
    if (n == 0) return 0;
    if (!p_host || !g_host || !m_host || !v_host || !ws) FX_FAIL("fx_adamw_stream_chunk: null pointer");
    if (sub_elems <= 0 || (sub_elems & 7) || n_slots < 1 || n_slots > 16)
        FX_FAIL("fx_adamw_stream_chunk: sub_elems must be a positive multiple of 8 and 1 <= n_slots <= 16");
    if (!inbound || !compute || !outbound) FX_FAIL("fx_adamw_stream_chunk: the three streams must be explicit (non-null)");
    if (!aligned16(ws) || !aligned16(p_host) || !aligned16(g_host) || !aligned16(m_host) || !aligned16(v_host) ||
        (p_bf16_out && !aligned16(p_bf16_out)))
        FX_FAIL("fx_adamw_stream_chunk: buffers must be 16-byte aligned");
    if (ring && ring->n_slots != n_slots)
        FX_FAIL("fx_adamw_stream_chunk: the ring was created for %d slots, the call uses %d", ring->n_slots, n_slots);
    const bool stage_copy = p_bf16_out && !p_bf16_out_on_device;
    const SlotLayout L = slot_layout(sub_elems, p_dt, g_dt, state_dt, stage_copy);
    if (ws_bytes < L.stride * (size_t)n_slots)
        FX_FAIL("fx_adamw_stream_chunk: workspace too small (%zu < %zu bytes)", ws_bytes, L.stride * (size_t)n_slots);

    const size_t psz = elem_size(p_dt), gsz = elem_size(g_dt), ssz = elem_size(state_dt);
    int rc = 0;
    FxStreamRing* r = ring;
    if (!r && fx_stream_ring_create(n_slots, &r) != 0) return -1;
    {
        // Without a ring of its own the workspace's earlier users are unknown; with one whose slots were
        // last cut differently a slot overlaps several old ones.  Both cases: order the copy-ins after
        // everything enqueued so far on the two streams that read or write staging memory.
        if (!ring || (r->stride != 0 && r->stride != L.stride)) {
            FX_HIP_OK(hipEventRecord(r->fence[0], compute), "record fence");
            FX_HIP_OK(hipEventRecord(r->fence[1], outbound), "record fence");
            FX_HIP_OK(hipStreamWaitEvent(inbound, r->fence[0], 0), "wait for the workspace's earlier kernels");
            FX_HIP_OK(hipStreamWaitEvent(inbound, r->fence[1], 0), "wait for the workspace's earlier copies");
            for (int s = 0; s < n_slots; ++s) r->busy[s] = false;
        }
        r->stride = L.stride;
        char* base = reinterpret_cast<char*>(ws);
        char* ph = reinterpret_cast<char*>(p_host);
        const char* gh = reinterpret_cast<const char*>(g_host);
        char* mh = reinterpret_cast<char*>(m_host);
        char* vh = reinterpret_cast<char*>(v_host);
        char* ch = reinterpret_cast<char*>(p_bf16_out);
        for (int64_t off = 0; off < n; off += sub_elems) {
            const int64_t cnt = (n - off < sub_elems) ? (n - off) : sub_elems;
            const int s = (int)(r->next++ % n_slots);
            char* slot = base + (size_t)s * L.stride;
            if (r->busy[s]) FX_HIP_OK(hipStreamWaitEvent(inbound, r->out_done[s], 0), "wait for a free slot");
            FX_HIP_OK(hipMemcpyAsync(slot + L.p, ph + off * psz, cnt * psz, hipMemcpyHostToDevice, inbound), "copy-in p");
            FX_HIP_OK(hipMemcpyAsync(slot + L.g, gh + off * gsz, cnt * gsz, hipMemcpyHostToDevice, inbound), "copy-in g");
            FX_HIP_OK(hipMemcpyAsync(slot + L.m, mh + off * ssz, cnt * ssz, hipMemcpyHostToDevice, inbound), "copy-in m");
            FX_HIP_OK(hipMemcpyAsync(slot + L.v, vh + off * ssz, cnt * ssz, hipMemcpyHostToDevice, inbound), "copy-in v");
            FX_HIP_OK(hipEventRecord(r->in_done[s], inbound), "record copy-in");

            FX_HIP_OK(hipStreamWaitEvent(compute, r->in_done[s], 0), "wait for copy-in");
            void* copy_dst = nullptr;
            if (p_bf16_out) copy_dst = stage_copy ? (void*)(slot + L.pc) : (void*)(ch + off * 2);
            if (fx_adamw_step(slot + L.p, slot + L.g, slot + L.m, slot + L.v, copy_dst, cnt, p_dt, g_dt, state_dt, lr,
                              beta1, beta2, eps, weight_decay, bias_correction1, bias_correction2, compute) != 0) {
                rc = -1;
                goto done;
            }
            FX_HIP_OK(hipEventRecord(r->k_done[s], compute), "record kernel");

            FX_HIP_OK(hipStreamWaitEvent(outbound, r->k_done[s], 0), "wait for the kernel");
            FX_HIP_OK(hipMemcpyAsync(ph + off * psz, slot + L.p, cnt * psz, hipMemcpyDeviceToHost, outbound), "copy-out p");
            FX_HIP_OK(hipMemcpyAsync(mh + off * ssz, slot + L.m, cnt * ssz, hipMemcpyDeviceToHost, outbound), "copy-out m");
            FX_HIP_OK(hipMemcpyAsync(vh + off * ssz, slot + L.v, cnt * ssz, hipMemcpyDeviceToHost, outbound), "copy-out v");
            if (stage_copy)
                FX_HIP_OK(hipMemcpyAsync(ch + off * 2, slot + L.pc, cnt * 2, hipMemcpyDeviceToHost, outbound), "copy-out bf16 p");
            FX_HIP_OK(hipEventRecord(r->out_done[s], outbound), "record copy-out");
            r->busy[s] = true;
        }
    }
done:
    if (!ring) fx_stream_ring_destroy(r);
    return rc;
}

extern "C" int fx_host_alloc(size_t bytes, void** out) {
    if (!out) FX_FAIL("fx_host_alloc: null output pointer");
    *out = nullptr;
    if (bytes == 0) return 0;
    hipError_t e = hipHostMalloc(out, bytes, hipHostMallocDefault);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        FX_FAIL("fx_host_alloc: hipHostMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
    }
    return 0;
}

extern "C" int fx_host_free(void* ptr) {
    if (!ptr) return 0;
    hipError_t e = hipHostFree(ptr);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        FX_FAIL("fx_host_free: %s", hipGetErrorString(e));
    }
    return 0;
}

// Every field of one activation slot moved in ONE call: field i is rows[i] rows of row_bytes[i]
// bytes, source and destination rows src_pitch[i] / dst_pitch[i] bytes apart (a pitch equal to
// row_bytes means contiguous, and the whole field goes as one linear copy; a wider pitch is the
// narrowed view of a tensor sized for more tokens and goes as a 2-D copy).  The reference issues
// one torch copy_ per field (flextrain/core/activation_schema.py:483-519); batching them keeps the
// host cost of an offload at one library call per (chunk, layer) slot.
extern "C" int fx_copy_fields(int n, void* const* dst, const void* const* src, const int64_t* rows,
                              const int64_t* row_bytes, const int64_t* dst_pitch, const int64_t* src_pitch,
                              int direction, hipStream_t stream) {
    if (n < 0) FX_FAIL("fx_copy_fields: negative field count");
    if (n == 0) return 0;
    if (!dst || !src || !rows || !row_bytes || !dst_pitch || !src_pitch) FX_FAIL("fx_copy_fields: null array");
    hipMemcpyKind kind;
    switch (direction) {
        case 0: kind = hipMemcpyDeviceToHost; break;
        case 1: kind = hipMemcpyHostToDevice; break;
        case 2: kind = hipMemcpyDeviceToDevice; break;
        default: FX_FAIL("fx_copy_fields: direction must be 0 (device to host), 1 (host to device) or 2 (device to device)");
    }
    for (int i = 0; i < n; ++i) {
        if (rows[i] < 0 || row_bytes[i] < 0) FX_FAIL("fx_copy_fields: field %d has a negative extent", i);
        if (rows[i] == 0 || row_bytes[i] == 0) continue;
        if (!dst[i] || !src[i]) FX_FAIL("fx_copy_fields: field %d has a null pointer", i);
        if (dst_pitch[i] < row_bytes[i] || src_pitch[i] < row_bytes[i])
            FX_FAIL("fx_copy_fields: field %d has a pitch smaller than its row", i);
        hipError_t e;
        if (rows[i] == 1 || (dst_pitch[i] == row_bytes[i] && src_pitch[i] == row_bytes[i]))
            e = hipMemcpyAsync(dst[i], src[i], (size_t)(rows[i] * row_bytes[i]), kind, stream);
        else
            e = hipMemcpy2DAsync(dst[i], (size_t)dst_pitch[i], src[i], (size_t)src_pitch[i], (size_t)row_bytes[i],
                                 (size_t)rows[i], kind, stream);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            FX_FAIL("fx_copy_fields: copy of field %d failed: %s", i, hipGetErrorString(e));
        }
    }
    return 0;
}
