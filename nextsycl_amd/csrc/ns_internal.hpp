// ns_internal.hpp: what the library's translation units share; not part of the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>
#include <string>
#include <vector>

#include "ns.h"

// One opened device: the in-order compute stream every kernel and queued copy goes to, two copy streams for copies
// that overlap it, and a ring of events - the "tickets" of ns_mark / ns_stream_copy / ns_stamp.
struct ns_gpu {
    int dev = 0;
    hipStream_t q = nullptr;     // compute, in order
    hipStream_t cq = nullptr;    // copy lane 0
    hipStream_t cq2 = nullptr;   // copy lane 1
    std::vector<hipEvent_t> ev;  // created on first use of a slot, re-recorded when the ring wraps
    int64_t next_ev = 0;
    // scratch the library keeps for entry points whose reference signature has no scratch argument
    // (ns_llm_minimaxm3_attend); allocated once at ns_gpu_open, never inside a kernel call
    float* own_scratch = nullptr;
    size_t own_scratch_floats = 0;
    // ns_attn_profile: events around the kernels of the last attention call (measurement only; off by default)
    bool profile = false;
    hipEvent_t pev[3] = {nullptr, nullptr, nullptr};
    int pev_used = 0;
    // the graph this handle's compute stream is recording into (ns_q35_graph_begin .. _end), or null: while it is set, calls
    // that wait for the stream (ns_sync, ns_elapsed, ns_attn_profile_last) are refused, and ns_gpu_close drops the recording
    void* recording = nullptr;
};

// records profile event i on the compute stream when profiling is on (creates it on first use); 0 or -1
int ns_profile_mark(ns_gpu* g, int i);

// attn_decode.hip: looks up, once a device and with that device current, the address of the device-resident scratch
// array that ns_attn_decode_static uses (called by ns_gpu_open); 0 or -1
int ns_attn_static_scratch_init(int dev);

// ns_hip.cpp: ends the recording of a graph handle (ns_q35_graph_begin) that is still open and drops what it recorded
extern "C" void ns_graph_drop(void* h);

// sets the calling thread's error text (ns_last_error) and returns -1
int ns_fail(const std::string& what);
// -1 with "hip: <what>: <error string>" when e is an error, else 0
int ns_hip_check(hipError_t e, const char* what);

#define NS_HIP(call)                                        \
    do {                                                    \
        if (ns_hip_check((call), #call) != 0) return -1;    \
    } while (0)

// every entry point runs with its device current (a caller's thread may have switched) and turns C++ exceptions into -1
#define NS_TRY try {
#define NS_CATCH                                                      \
    }                                                                 \
    catch (const std::exception& e) { return ns_fail(e.what()); }     \
    catch (...) { return ns_fail("unknown C++ exception"); }

// after a kernel launch: launch errors (bad configuration) surface here, not at the next sync
#define NS_LAUNCHED(name) NS_HIP(hipGetLastError())
