// ns_hip.cpp: devices, memory, copies, tickets and stamps of the C ABI (ns.h) over HIP.
#include "ns_internal.hpp"

#include <cstdio>
#include <cstring>

namespace {
thread_local std::string g_err;
constexpr size_t EV_RING = 1 << 16;
constexpr size_t OWN_SCRATCH_FLOATS = (size_t) 256 << 20;   // 1 GiB of the card's 288

// the event of a ticket the ring still holds, or null: tickets are 0 .. next_ev - 1, the ring keeps the last EV_RING
hipEvent_t ticket_event(ns_gpu* g, int64_t t) {
    if (t < 0 || t >= g->next_ev || g->next_ev - t > (int64_t) EV_RING) return nullptr;
    return g->ev[(size_t) t % EV_RING];
}

int bad_index(int index, int n) { return ns_fail("no GPU " + std::to_string(index) + " (" + std::to_string(n) + " found)"); }

// the event of ticket slot t, created on first use
hipEvent_t* slot(ns_gpu* g, int64_t t) {
    hipEvent_t* e = &g->ev[(size_t) t % EV_RING];
    if (!*e && hipEventCreate(e) != hipSuccess) return nullptr;
    return e;
}
}  // namespace

int ns_fail(const std::string& what) {
    g_err = what;
    return -1;
}

int ns_hip_check(hipError_t e, const char* what) {
    if (e == hipSuccess) return 0;
    return ns_fail(std::string("hip: ") + what + ": " + hipGetErrorString(e));
}

int ns_profile_mark(ns_gpu* g, int i) {
    if (!g->profile) return 0;
    if (!g->pev[i]) NS_HIP(hipEventCreate(&g->pev[i]));
    NS_HIP(hipEventRecord(g->pev[i], g->q));
    if (i + 1 > g->pev_used) g->pev_used = i + 1;
    return 0;
}

extern "C" {

int ns_attn_profile(ns_gpu* g, int on) {
    if (on != 0 && on != 1) return ns_fail("ns_attn_profile: 0 (off) or 1 (events around the kernels of every attention call)");
    g->profile = on == 1;
    g->pev_used = 0;
    return 0;
}

int ns_attn_profile_last(ns_gpu* g, double* main_ns, double* merge_ns) {
    NS_TRY
    *main_ns = *merge_ns = 0.0;
    if (g->recording) return ns_fail("ns_attn_profile_last: the compute stream is recording a graph (ns_q35_graph_end first)");
    if (g->pev_used < 2) return ns_fail("ns_attn_profile_last: no profiled attention call yet");
    NS_HIP(hipSetDevice(g->dev));
    NS_HIP(hipEventSynchronize(g->pev[g->pev_used - 1]));
    float ms = 0.0f;
    NS_HIP(hipEventElapsedTime(&ms, g->pev[0], g->pev[1]));
    *main_ns = (double) ms * 1.0e6;
    if (g->pev_used > 2) {
        NS_HIP(hipEventElapsedTime(&ms, g->pev[1], g->pev[2]));
        *merge_ns = (double) ms * 1.0e6;
    }
    return 0;
    NS_CATCH
}

const char* ns_last_error(void) { return g_err.c_str(); }
const char* ns_version(void) { return "nextsycl-amd 0.1 (hip, gfx950)"; }

int ns_gpu_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

int ns_gpu_name(int index, char* buf, size_t len) {
    NS_TRY
    const int n = ns_gpu_count();
    if (index < 0 || index >= n) return bad_index(index, n);
    hipDeviceProp_t p;
    NS_HIP(hipGetDeviceProperties(&p, index));
    std::snprintf(buf, len, "%s", p.name[0] ? p.name : p.gcnArchName);
    return 0;
    NS_CATCH
}

int ns_gpu_pci(int index, char* buf, size_t len) {
    NS_TRY
    const int n = ns_gpu_count();
    if (index < 0 || index >= n) return bad_index(index, n);
    hipDeviceProp_t p;
    NS_HIP(hipGetDeviceProperties(&p, index));
    std::snprintf(buf, len, "%04x:%02x:%02x.0", p.pciDomainID, p.pciBusID, p.pciDeviceID);
    return 0;
    NS_CATCH
}

int ns_gpu_units(int index, int* units, int* mhz) {
    NS_TRY
    const int n = ns_gpu_count();
    if (index < 0 || index >= n) return bad_index(index, n);
    hipDeviceProp_t p;
    NS_HIP(hipGetDeviceProperties(&p, index));
    *units = p.multiProcessorCount;
    *mhz = p.clockRate / 1000;
    return 0;
    NS_CATCH
}

int ns_gpu_open(int index, ns_gpu** out) {
    NS_TRY
    const int n = ns_gpu_count();
    if (index < 0 || index >= n) return bad_index(index, n);
    NS_HIP(hipSetDevice(index));
    ns_gpu* g = new ns_gpu;
    g->dev = index;
    g->ev.assign(EV_RING, nullptr);
    // default priority on all three: streams of unequal priority are not used anywhere in this library
    if (ns_hip_check(hipStreamCreateWithFlags(&g->q, hipStreamNonBlocking), "compute stream") ||
        ns_hip_check(hipStreamCreateWithFlags(&g->cq, hipStreamNonBlocking), "copy stream 0") ||
        ns_hip_check(hipStreamCreateWithFlags(&g->cq2, hipStreamNonBlocking), "copy stream 1") ||
        ns_hip_check(hipMalloc((void**) &g->own_scratch, OWN_SCRATCH_FLOATS * sizeof(float)), "library scratch") ||
        ns_attn_static_scratch_init(index)) {
        ns_gpu_close(g);
        return -1;
    }
    g->own_scratch_floats = OWN_SCRATCH_FLOATS;
    *out = g;
    return 0;
    NS_CATCH
}

void ns_gpu_close(ns_gpu* g) {
    if (!g) return;
    (void) hipSetDevice(g->dev);
    if (g->recording) ns_graph_drop(g->recording);                // (a recording still open ends here; its handle stays the caller's to free)
    if (g->q) (void) hipStreamSynchronize(g->q);
    if (g->cq) (void) hipStreamSynchronize(g->cq);
    if (g->cq2) (void) hipStreamSynchronize(g->cq2);
    for (hipEvent_t e : g->ev)
        if (e) (void) hipEventDestroy(e);
    for (hipEvent_t e : g->pev)
        if (e) (void) hipEventDestroy(e);
    if (g->own_scratch) (void) hipFree(g->own_scratch);
    if (g->q) (void) hipStreamDestroy(g->q);
    if (g->cq) (void) hipStreamDestroy(g->cq);
    if (g->cq2) (void) hipStreamDestroy(g->cq2);
    delete g;
}

void* ns_gpu_queue(ns_gpu* g) { return &g->q; }

// ---- a stretch of a pass as one submission: what is queued on the handle's compute stream between begin and end is
// recorded into a HIP graph instead of run (stream capture: kernel launches only - no entry point of this library
// records a memset or allocates), instantiated at end, replayed by launch (kernels/llm/qwen35/q35.cpp:505-549: the same
// four calls over a SYCL command graph)
namespace {
struct NsGraph {
    int dev = 0;
    hipStream_t q = nullptr;          // the stream that records; null once recording has ended
    ns_gpu* owner = nullptr;          // the handle that records (null once recording has ended, or the handle has been closed)
    hipGraphExec_t exec = nullptr;
};
// ends a recording that is still open and drops what it recorded
void drop_recording(NsGraph* gr) {
    if (!gr->q) return;
    hipGraph_t graph = nullptr;
    (void) hipSetDevice(gr->dev);
    if (hipStreamEndCapture(gr->q, &graph) == hipSuccess && graph) (void) hipGraphDestroy(graph);
    gr->q = nullptr;
    if (gr->owner) gr->owner->recording = nullptr;
    gr->owner = nullptr;
}
}  // namespace

void ns_graph_drop(void* h) { drop_recording(static_cast<NsGraph*>(h)); }

int ns_q35_graph_begin(ns_gpu* g, void** out) {
    NS_TRY
    if (!g || !out) return ns_fail("ns_q35_graph_begin: a null argument");
    if (g->recording) return ns_fail("ns_q35_graph_begin: this GPU is recording a graph already");
    NS_HIP(hipSetDevice(g->dev));
    NsGraph* gr = new NsGraph;        // (before the capture begins: a failure here leaves the stream as it was)
    gr->dev = g->dev;
    gr->q = g->q;
    gr->owner = g;
    // (relaxed: other threads of the engine may be allocating or copying on their own streams meanwhile)
    if (ns_hip_check(hipStreamBeginCapture(g->q, hipStreamCaptureModeRelaxed), "hipStreamBeginCapture") != 0) {
        delete gr;
        return -1;
    }
    g->recording = gr;
    *out = gr;
    return 0;
    NS_CATCH
}

int ns_q35_graph_end(ns_gpu* g, void* h) {
    NS_TRY
    NsGraph* gr = static_cast<NsGraph*>(h);
    if (!g || !gr) return ns_fail("ns_q35_graph_end: a null argument");
    if (!gr->q || gr->q != g->q) return ns_fail("ns_q35_graph_end: not the graph this GPU is recording");
    NS_HIP(hipSetDevice(g->dev));
    gr->q = nullptr;
    gr->owner = nullptr;
    g->recording = nullptr;
    hipGraph_t graph = nullptr;
    NS_HIP(hipStreamEndCapture(g->q, &graph));
    if (!graph) return ns_fail("ns_q35_graph_end: the recording was dropped (a call that cannot be recorded was made on the stream)");
    const hipError_t e = hipGraphInstantiate(&gr->exec, graph, nullptr, nullptr, 0);
    (void) hipGraphDestroy(graph);
    NS_HIP(e);
    return 0;
    NS_CATCH
}

int ns_q35_graph_launch(ns_gpu* g, void* h) {
    NS_TRY
    NsGraph* gr = static_cast<NsGraph*>(h);
    if (!g || !gr) return ns_fail("ns_q35_graph_launch: a null argument");
    if (!gr->exec) return ns_fail("ns_q35_graph_launch: a graph not finished");
    if (gr->dev != g->dev) return ns_fail("ns_q35_graph_launch: a graph of another GPU");
    NS_HIP(hipSetDevice(g->dev));
    NS_HIP(hipGraphLaunch(gr->exec, g->q));
    return 0;
    NS_CATCH
}

void ns_q35_graph_free(void* h) {
    NsGraph* gr = static_cast<NsGraph*>(h);
    if (!gr) return;
    drop_recording(gr);               // (freed while still recording: the recording ends here, and is dropped)
    if (gr->exec) {
        (void) hipSetDevice(gr->dev);
        (void) hipGraphExecDestroy(gr->exec);
    }
    delete gr;
}

int ns_gpu_memory(ns_gpu* g, uint64_t* total, int64_t* free_bytes) {
    NS_TRY
    NS_HIP(hipSetDevice(g->dev));
    size_t f = 0, t = 0;
    NS_HIP(hipMemGetInfo(&f, &t));
    *total = t;
    *free_bytes = (int64_t) f;
    return 0;
    NS_CATCH
}

int ns_alloc(ns_gpu* g, size_t bytes, void** out) {
    NS_TRY
    NS_HIP(hipSetDevice(g->dev));
    *out = nullptr;
    if (hipMalloc(out, bytes ? bytes : 1) != hipSuccess || !*out) {
        (void) hipGetLastError();
        return ns_fail("device allocation of " + std::to_string(bytes) + " bytes failed");
    }
    return 0;
    NS_CATCH
}

int ns_free(ns_gpu* g, void* p) {
    NS_TRY
    NS_HIP(hipSetDevice(g->dev));
    NS_HIP(hipFree(p));
    return 0;
    NS_CATCH
}

int ns_alloc_host(ns_gpu* g, size_t bytes, void** out) {
    NS_TRY
    NS_HIP(hipSetDevice(g->dev));
    *out = nullptr;
    if (hipHostMalloc(out, bytes ? bytes : 1, hipHostMallocDefault) != hipSuccess || !*out) {
        (void) hipGetLastError();
        return ns_fail("pinned host allocation of " + std::to_string(bytes) + " bytes failed");
    }
    return 0;
    NS_CATCH
}

int ns_free_host(ns_gpu* g, void* p) {
    NS_TRY
    NS_HIP(hipSetDevice(g->dev));
    NS_HIP(hipHostFree(p));
    return 0;
    NS_CATCH
}

int ns_copy_to(ns_gpu* g, void* dst, const void* src, size_t bytes) {
    NS_TRY
    if (!bytes) return 0;
    NS_HIP(hipSetDevice(g->dev));
    NS_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, g->q));
    return 0;
    NS_CATCH
}

int ns_copy_from(ns_gpu* g, void* dst, const void* src, size_t bytes) {
    NS_TRY
    if (!bytes) return 0;
    NS_HIP(hipSetDevice(g->dev));
    NS_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, g->q));
    return 0;
    NS_CATCH
}

int ns_copy_dev(ns_gpu* g, void* dst, const void* src, size_t bytes) {
    NS_TRY
    if (!bytes) return 0;
    NS_HIP(hipSetDevice(g->dev));
    NS_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, g->q));
    return 0;
    NS_CATCH
}

int ns_copy_2d(ns_gpu* g, void* dst, size_t dst_pitch, const void* src, size_t src_pitch, size_t width, size_t height) {
    NS_TRY
    if (width == 0 || height == 0) return 0;
    NS_HIP(hipSetDevice(g->dev));
    NS_HIP(hipMemcpy2DAsync(dst, dst_pitch, src, src_pitch, width, height, hipMemcpyDeviceToDevice, g->q));
    return 0;
    NS_CATCH
}

int ns_mark(ns_gpu* g, int64_t* ticket) {
    NS_TRY
    NS_HIP(hipSetDevice(g->dev));
    const int64_t t = g->next_ev++;
    hipEvent_t* e = slot(g, t);
    if (!e) return ns_fail("ns_mark: no event");
    NS_HIP(hipEventRecord(*e, g->q));
    *ticket = t;
    return 0;
    NS_CATCH
}

int ns_stream_copy(ns_gpu* g, void* dst, const void* src, size_t bytes, const int64_t* after, int ndeps, int lane, int64_t* ticket) {
    NS_TRY
    NS_HIP(hipSetDevice(g->dev));
    hipStream_t s = lane ? g->cq2 : g->cq;
    for (int i = 0; i < ndeps; ++i) {
        if (!after) return ns_fail("ns_stream_copy: tickets to wait for, but no list");
        hipEvent_t e = ticket_event(g, after[i]);
        if (!e) return ns_fail("ns_stream_copy: ticket " + std::to_string(after[i]) + " was never issued");
        NS_HIP(hipStreamWaitEvent(s, e, 0));
    }
    if (bytes) NS_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDefault, s));
    const int64_t t = g->next_ev++;
    hipEvent_t* e = slot(g, t);
    if (!e) return ns_fail("ns_stream_copy: no event");
    NS_HIP(hipEventRecord(*e, s));
    *ticket = t;
    return 0;
    NS_CATCH
}

int ns_await(ns_gpu* g, int64_t t) {
    NS_TRY
    NS_HIP(hipSetDevice(g->dev));
    hipEvent_t e = ticket_event(g, t);
    if (!e) return ns_fail("ns_await: ticket " + std::to_string(t) + " was never issued");
    NS_HIP(hipStreamWaitEvent(g->q, e, 0));
    return 0;
    NS_CATCH
}

int ns_stamp(ns_gpu* g, int64_t* ticket) { return ns_mark(g, ticket); }

int ns_elapsed(ns_gpu* g, int64_t t0, int64_t t1, double* ns) {
    NS_TRY
    if (g->recording) return ns_fail("ns_elapsed: the compute stream is recording a graph (ns_q35_graph_end first)");
    NS_HIP(hipSetDevice(g->dev));
    hipEvent_t a = ticket_event(g, t0), b = ticket_event(g, t1);
    if (!a || !b) return ns_fail("ns_elapsed: a ticket that was never issued");
    NS_HIP(hipEventSynchronize(a));
    NS_HIP(hipEventSynchronize(b));
    float ms = 0.0f;
    NS_HIP(hipEventElapsedTime(&ms, a, b));
    *ns = (double) ms * 1.0e6;
    return 0;
    NS_CATCH
}

int ns_sync(ns_gpu* g) {
    NS_TRY
    if (g->recording) return ns_fail("ns_sync: the compute stream is recording a graph (ns_q35_graph_end first)");
    NS_HIP(hipSetDevice(g->dev));
    NS_HIP(hipStreamSynchronize(g->q));
    return 0;
    NS_CATCH
}

int ns_copy_peer(ns_gpu* to, void* dst, ns_gpu* from, const void* src, size_t bytes, void* staging) {
    NS_TRY
    if (!bytes) return 0;
    NS_HIP(hipSetDevice(from->dev));
    NS_HIP(hipMemcpyAsync(staging, src, bytes, hipMemcpyDeviceToHost, from->q));
    NS_HIP(hipStreamSynchronize(from->q));
    NS_HIP(hipSetDevice(to->dev));
    NS_HIP(hipMemcpyAsync(dst, staging, bytes, hipMemcpyHostToDevice, to->q));
    NS_HIP(hipStreamSynchronize(to->q));
    return 0;
    NS_CATCH
}

}  // extern "C"
