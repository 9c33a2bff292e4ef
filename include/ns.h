/* ns.h - the device layer of libnextsycl-llm.so on one AMD MI355X (gfx950), over HIP.
 *
 * These are the 26 entry points the reference runtime binds with dlsym when it opens a kind's kernel library
 * (reference: kernels/ns/ns.h:18-56, bound in crates/sys/src/lib.rs:204-235). Names, argument order and meaning are
 * the reference's, so the Rust `Api` table loads this library unchanged; what stands behind them is HIP:
 *
 *   ns_gpu            one device + one in-order compute stream + two copy streams + a ring of events ("tickets")
 *   device memory     hipMalloc / hipFree          pinned host memory   hipHostMalloc / hipHostFree
 *   queued copies     hipMemcpyAsync on the compute stream (ordered with the kernels)
 *   tickets           hipEventRecord into the ring; waits are device-side (hipStreamWaitEvent), never host waits
 *   stamps            hipEventRecord with timing; ns_elapsed = hipEventElapsedTime
 *
 * Every call returns 0, or -1 with the reason kept per thread (ns_last_error). Nothing is synchronous except ns_sync,
 * ns_elapsed and ns_copy_peer. All kernels of ns_attn.h are queued on the same compute stream.
 */
#ifndef NS_H
#define NS_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ns_gpu ns_gpu;

/* reference: kernels/ns/ns.h:20-21 */
const char* ns_last_error(void);
const char* ns_version(void);

/* the HIP devices in hipGetDevice order - reference: kernels/ns/ns.h:23-27 (there: the Level Zero GPUs) */
int ns_gpu_count(void);
int ns_gpu_name(int index, char* buf, size_t len);
int ns_gpu_pci(int index, char* buf, size_t len);            /* "0000:03:00.0" */
int ns_gpu_units(int index, int* units, int* mhz);           /* compute units, their clock */
/* reference: kernels/ns/ns.h:28-35 */
int ns_gpu_open(int index, ns_gpu** out);
void ns_gpu_close(ns_gpu* g);
void* ns_gpu_queue(ns_gpu* g);                               /* hipStream_t* of the compute stream */
int ns_gpu_memory(ns_gpu* g, uint64_t* total, int64_t* free_bytes);

/* reference: kernels/ns/ns.h:37-41 */
int ns_alloc(ns_gpu* g, size_t bytes, void** out);
int ns_free(ns_gpu* g, void* p);
int ns_alloc_host(ns_gpu* g, size_t bytes, void** out);
int ns_free_host(ns_gpu* g, void* p);
/* queued in order on the compute stream; a pageable host source must stay valid until ns_sync - reference:
 * kernels/ns/ns.h:42-47 */
int ns_copy_to(ns_gpu* g, void* dst, const void* src_host, size_t bytes);
int ns_copy_from(ns_gpu* g, void* dst_host, const void* src, size_t bytes);
int ns_copy_dev(ns_gpu* g, void* dst, const void* src, size_t bytes);
int ns_copy_2d(ns_gpu* g, void* dst, size_t dst_pitch, const void* src, size_t src_pitch, size_t width, size_t height);
/* tickets - reference: kernels/ns/ns.h:48-52. ns_mark: everything queued so far; ns_stream_copy: a copy on copy lane 0
 * or 1 after the tickets `after`; ns_await: the compute stream waits (on the device) for a ticket; ns_stamp /
 * ns_elapsed: device time between two stamps, in nanoseconds (waits for them) */
int ns_mark(ns_gpu* g, int64_t* ticket);
int ns_stream_copy(ns_gpu* g, void* dst, const void* src, size_t bytes, const int64_t* after, int ndeps, int lane, int64_t* ticket);
int ns_await(ns_gpu* g, int64_t ticket);
int ns_stamp(ns_gpu* g, int64_t* ticket);
int ns_elapsed(ns_gpu* g, int64_t t0, int64_t t1, double* ns);
/* reference: kernels/ns/ns.h:53-54 */
int ns_fill(ns_gpu* g, void* dst, uint8_t value, size_t bytes);
int ns_sync(ns_gpu* g);
/* one device's memory to another's through `staging` host memory; waits - reference: kernels/ns/ns.h:55-57 */
int ns_copy_peer(ns_gpu* to, void* dst, ns_gpu* from, const void* src, size_t bytes, void* staging);

#ifdef __cplusplus
}
#endif
#endif
