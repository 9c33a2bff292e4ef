// kv_rows.hip: byte work on device buffers - a queued fill (ns_fill), and the rows of a span of positions moved between
// caches of different geometry: a ring (slot = position % cap) into position order for a checkpoint, a checkpoint back
// into a ring, one session's rings into another's. The
// reference's engines do this on the host as runs of copies, one or two a head and cache
// (llm/museglimmer/src/engine.rs:1334-1346, 1475-1528; llm/qwen35/src/engine.rs:2977-3011); here it is one launch a
// cache, every head at once, so a checkpoint is a handful of launches and ONE copy across PCIe.
//
// Byte work, HBM-bound: a thread moves one unit (16, 8, 4 or 2 bytes - the widest that divides the row and the
// addresses), consecutive threads consecutive units of a row and then the next position's row, so a wave reads and
// writes whole lines except where the ring wraps. Bytes a launch: 2 x heads x positions x row bytes.
#include <algorithm>

#include "ns_internal.hpp"
#include "ns_attn.h"

namespace {

struct RowsCopy {
    const void* src;
    void* dst;
    uint32_t upr;        // units a row
    uint32_t n;          // positions
    uint32_t scap, s0;   // source: slots a head, the first position's slot
    uint32_t dcap, d0;   // destination: the same
};

template <typename U>
__global__ void kv_rows_copy_kernel(RowsCopy p) {
    const uint64_t i = (uint64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (uint64_t) p.n * p.upr) return;
    const uint32_t r = (uint32_t) (i / p.upr), u = (uint32_t) (i - (uint64_t) r * p.upr), h = blockIdx.y;
    uint32_t ss = p.s0 + r, ds = p.d0 + r;      // r < n <= both capacities: one wrap at most
    if (ss >= p.scap) ss -= p.scap;
    if (ds >= p.dcap) ds -= p.dcap;
    const U* s = reinterpret_cast<const U*>(p.src) + ((uint64_t) h * p.scap + ss) * p.upr + u;
    U* d = reinterpret_cast<U*>(p.dst) + ((uint64_t) h * p.dcap + ds) * p.upr + u;
    *d = *s;
}

template <typename U>
void launch_rows(ns_gpu* g, RowsCopy p, int64_t heads, int64_t row_bytes) {
    p.upr = (uint32_t) (row_bytes / (int64_t) sizeof(U));
    const uint64_t units = (uint64_t) p.n * p.upr;
    kv_rows_copy_kernel<U><<<dim3((unsigned) ((units + 255) / 256), (unsigned) heads), 256, 0, g->q>>>(p);
}

// bytes set to one value: 16-byte stores over the aligned body, byte stores over the ends
__global__ void fill_kernel(uint8_t* dst, uint32_t word, uint32_t head, uint64_t units, uint32_t tail) {
    const uint64_t i = (uint64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (i < units) reinterpret_cast<uint4*>(dst + head)[i] = make_uint4(word, word, word, word);
    if (i < head) dst[i] = (uint8_t) word;
    if (i < tail) dst[head + units * 16 + i] = (uint8_t) word;
}

}  // namespace

extern "C" {

// A queued fill (kernels/ns/ns.h's ns_fill). A kernel of this library's own rather than a memset node: a caller may
// capture the queue into a graph, and memset nodes have replayed wrongly on this platform.
int ns_fill(ns_gpu* g, void* dst, uint8_t value, size_t bytes) {
    NS_TRY
    if (!bytes) return 0;
    if (!dst) return ns_fail("ns_fill: no buffer");
    NS_HIP(hipSetDevice(g->dev));
    uint8_t* d = (uint8_t*) dst;
    const size_t head = std::min<size_t>(bytes, (16 - (uintptr_t) d % 16) % 16), units = (bytes - head) / 16, tail = bytes - head - units * 16;
    const size_t threads = std::max<size_t>(units, 16), blocks = (threads + 255) / 256;
    if (blocks >= (size_t) 1 << 31) return ns_fail("ns_fill: more than 2^39 bytes");
    const uint32_t word = value * 0x01010101u;
    fill_kernel<<<(unsigned) blocks, 256, 0, g->q>>>(d, word, (uint32_t) head, (uint64_t) units, (uint32_t) tail);
    NS_LAUNCHED("ns_fill");
    return 0;
    NS_CATCH
}

int ns_attn_kv_rows_copy(ns_gpu* g, const void* src, int64_t scap, int64_t sbase, void* dst, int64_t dcap, int64_t dbase, int64_t heads,
                         int64_t row_bytes, int64_t from, int64_t to) {
    NS_TRY
    if (to <= from) return 0;
    if (heads <= 0 || heads > 65535 || row_bytes <= 0 || row_bytes % 2) return ns_fail("ns_attn_kv_rows_copy: 1..65535 heads, rows of an even number of bytes");
    if (scap <= 0 || dcap <= 0 || sbase < 0 || dbase < 0 || from < sbase || from < dbase)
        return ns_fail("ns_attn_kv_rows_copy: capacities above 0, positions at or past each cache's first");
    const int64_t n = to - from;
    if (n > scap || n > dcap) return ns_fail("ns_attn_kv_rows_copy: more positions than a cache has slots");
    if (scap >= (int64_t) 1 << 31 || dcap >= (int64_t) 1 << 31 || n * (row_bytes / 2) >= (int64_t) 1 << 38)
        return ns_fail("ns_attn_kv_rows_copy: caches of fewer than 2^31 slots, under 2^39 bytes a head");
    if (!src || !dst) return ns_fail("ns_attn_kv_rows_copy: no cache");
    RowsCopy p;
    p.src = src;
    p.dst = dst;
    p.n = (uint32_t) n;
    p.scap = (uint32_t) scap;
    p.s0 = (uint32_t) ((from - sbase) % scap);
    p.dcap = (uint32_t) dcap;
    p.d0 = (uint32_t) ((from - dbase) % dcap);
    NS_HIP(hipSetDevice(g->dev));
    const uintptr_t a = (uintptr_t) src | (uintptr_t) dst | (uintptr_t) row_bytes;
    if (a % 16 == 0) launch_rows<uint4>(g, p, heads, row_bytes);
    else if (a % 8 == 0) launch_rows<uint2>(g, p, heads, row_bytes);
    else if (a % 4 == 0) launch_rows<uint32_t>(g, p, heads, row_bytes);
    else if (a % 2 == 0) launch_rows<uint16_t>(g, p, heads, row_bytes);
    else return ns_fail("ns_attn_kv_rows_copy: caches 2-byte aligned");
    NS_LAUNCHED("kv_rows_copy");
    return 0;
    NS_CATCH
}

}  // extern "C"
