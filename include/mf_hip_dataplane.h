/*
 * Native entry points of libmf_hip_dataplane.so beyond the drop-in surface of
 * mf_xcopy_api.h: raw batch enqueues (host arrays, a table in device memory,
 * strided rectangles), the local MoE dispatch / combine, and the runtime
 * services a host program needs to own GPU memory and streams without
 * touching HIP itself.  This is the stable native ABI.  Test views, replay
 * loops for benchmarks and tuning switches are exported too but declared in
 * mf_hip_dataplane_internal.h, without a stability promise.
 * Plain C types only; a stream or event is an opaque void*.  Functions
 * returning int32_t give 0 or a negative BM_* code unless stated; the mfrt_*
 * services return 0 or a positive HIP error number.
 *
 * None of these has a counterpart in the reference's public headers; where
 * one stands in for reference-internal code the comment says which.
 */
#ifndef MF_HIP_DATAPLANE_H
#define MF_HIP_DATAPLANE_H

#include <stdint.h>

#include "mf_xcopy_types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* A flag of this build for the `flags` argument of smem_bm_copy[_batch] / hybm_data_[batch_]copy, beside the
 * reference's ASYNC_COPY_FLAG and COPY_EXTEND_FLAG (no counterpart in the reference; a bit far from theirs).
 * Together with ASYNC_COPY_FLAG it declares that the copy is independent of everything the caller has
 * submitted on the same stream and not yet waited for: it may run while earlier copies still run and
 * later unordered copies may run beside it.  A copy WITHOUT the flag submitted afterwards still waits for
 * it, and so do smem_bm_wait / hybm_wait and a stream synchronisation.  KV blocks of different requests
 * are such copies.  What it buys: consecutive batches of up to 128 segments from one thread overlap their
 * start-up and drain on the GPU (a 9 MB batch: 5.3 instead of 5.9 us per batch on one stream).  Copies the
 * flag cannot help (more than 128 segments, pageable memory, blocking calls) ignore it. */
#define MF_COPY_UNORDERED_FLAG (1UL << 16)

/* Who launches unordered copies.  0 or 1 (the default): the calling thread, on its own stream, without a barrier.
 * 2 to 8: batches of up to 128 segments and 64 MiB between device addresses, submitted with MF_COPY_UNORDERED_FLAG and
 * no stream of the caller's, are planned by the caller and handed in turn to that many submit threads of the
 * library's, each with a stream of its own on a hardware queue of its own as far as there are queues (four here; hybm_init
 * asks the GPU which of its streams share one): one calling thread then gets the overlap several submitting threads get
 * (the reference gives every thread one stream, src/hybm/csrc/ts_engine/hybm_stream_manager.cpp:73-90): 9 MB batches take
 * 4.3 / 3.8 / 3.6 / 3.8 / 3.6-4.0 us each with 2 / 3 / 4 / 6 / 8 submit threads against 4.5 us without, and 1.2 us of the calling
 * thread's time instead of 3.5.  Four is the number to use where the runtime has four hardware queues.  One
 * thread that launches on several streams itself does not: the launches then cost it more than on one stream.
 * The next copy WITHOUT the flag, smem_bm_wait / hybm_wait and every other call that uses the thread's stream first
 * make that stream wait for them.  What changes for the caller: a synchronisation of mf_xcopy_thread_stream() that it
 * issues itself covers the unordered copies only if it fetched the stream after the last of them (the fetch is
 * such a call); a launch that fails is reported by that next call instead of the one that submitted it; the submit
 * threads poll for some tens of microseconds after their last batch before they sleep, and live until hybm_uninit.
 * Returns BM_INVALID_PARAM beyond 8. */
int32_t mf_xcopy_unordered_streams(uint32_t count);

/* ---- which memory a copy touches (selects the kernel's cache policy) ---- */
#define MF_ROUTE_HBM 0
#define MF_ROUTE_TO_HOST 1
#define MF_ROUTE_FROM_HOST 2

/* Enqueue `n` independent copies dst[i][0..len[i]) = src[i][0..len[i]) as one
 * fused launch on `stream` (NULL: the calling thread's stream).  This is the
 * body of HostDataOpSDMA::BatchCopyG2G
 * (src/hybm/csrc/data_operation/host/hybm_data_op_sdma.cpp:545-595) without
 * the pool range checks of the entry layer: every address must be
 * device-accessible.  Does not wait. */
int32_t mf_xcopy_batch(const uint64_t *src, const uint64_t *dst, const uint64_t *len, uint32_t n, int32_t route,
                       void *stream);

/* An enqueue of mf_xcopy_batch for a {src,dst,len} triple table that already lives in device memory. */
int32_t mf_xcopy_device_table(const void *triples, uint32_t n, int32_t route, void *stream);

/* No counterpart in the reference.  mf_xcopy_device_table for callers that cannot allocate: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  What the planner
 * leaves for the copy launch (header, chunk prefix, group map) lives in a statically allocated device
 * array (257 KiB per GPU, held until the process ends) instead of memory the library allocates on
 * demand, and the call creates no stream, event or staging either: `stream` is used as given (NULL is
 * the null stream).
 * Limits: n <= MF_XCOPY_STATIC_TABLE_MAX segments (BM_INVALID_PARAM beyond); every call on one GPU
 * uses the same array.  Calls on one stream are ordered by the stream; a call on another stream than
 * the call before is made to wait for that one (by an event created at hybm_init).  Outside that
 * protection: calls under stream capture (replays of two graphs that hold such a call, or a replay
 * and a plain call, must not run at the same time) and a graph replayed on several streams at once.
 * Before a call is captured, one plain call must have run in the process (a kernel's first launch makes
 * the runtime load its code, which is not capturable).  hybm_init must have run (it looks the array's
 * address up).  Same results as mf_xcopy_device_table. */
#define MF_XCOPY_STATIC_TABLE_MAX 32768u
int32_t mf_xcopy_device_table_static(const void *triples, uint32_t n, int32_t route, void *stream);

/* The stream copies of the calling thread run on when the caller passes none
 * (the per-thread stream of the reference's HybmStreamManager,
 * src/hybm/csrc/ts_engine/hybm_stream_manager.cpp:73-90).  NULL before init. */
void *mf_xcopy_thread_stream(void);

/* Batched strided 2-D copy: for each descriptor, `height` rows of `width` bytes,
 * consecutive rows `spitch` / `dpitch` bytes apart (cudaMemcpy2D-style geometry;
 * the reference loads aclrtMemcpy2d at src/hybm/csrc/under_api/dl_acl_api.cpp:87-88
 * but never calls it).  Rectangles of one call must not overlap each other's
 * destinations.  Enqueues on `stream` (NULL: thread stream), does not wait. */
typedef struct {
    uint64_t src;
    uint64_t dst;
    uint64_t width;
    uint64_t height;
    uint64_t spitch;
    uint64_t dpitch;
} mf_copy2d_desc;
int32_t mf_xcopy_2d_batch(const mf_copy2d_desc *descs, uint32_t n, int32_t route, void *stream);

/* ---- local MoE dispatch / combine over pooled memory ------------------------
 * No reference implementation exists; the specification is the stable counting
 * sort / fixed-order fp32 FMA chain stated in oracle/mf_oracle.c.  All buffers
 * are device memory; x, out, rows, y hold 16-bit (bf16) elements, 16-byte
 * aligned, hidden a multiple of 8; topK <= 16, experts <= 512.
 *
 * dispatch: x[tokens][hidden], topk[tokens][topK] expert ids ->
 *   counts[experts], offsets[experts] (exclusive scan of counts),
 *   rowOf[tokens*topK] (destination row of entry t*topK+k, -1 for an id outside
 *   [0, experts)), srcOf[tokens*topK] (inverse, may be NULL),
 *   out[tokens*topK][hidden] expert-contiguous (x and out may both be NULL to
 *   compute the permutation only).
 * workspace: mf_moe_workspace_bytes() bytes of device memory (status, the
 *   [expert][block] histogram and 8 bytes per entry for the order in which the
 *   rows are written), no initialisation needed; after the stream has drained its first uint32 is 1 if any expert id
 *   was out of range.  Enqueues on `stream` (NULL: thread stream), does not wait. */
uint64_t mf_moe_workspace_bytes(uint32_t tokens, uint32_t topK, uint32_t experts);
int32_t mf_moe_dispatch(const void *x, const int32_t *topk, uint32_t tokens, uint32_t hidden, uint32_t topK,
                        uint32_t experts, void *out, int32_t *counts, int32_t *offsets, int32_t *rowOf, int32_t *srcOf,
                        void *workspace, uint64_t workspaceBytes, void *stream);
/* combine: y[t][h] = bf16(sum_k weights[t][k] * rows[rowOf[t*topK+k]][h]), fp32
 * fused multiply-add in slot order k = 0..topK-1 starting from 0, one final
 * round-to-nearest-even; entries with rowOf < 0 contribute nothing. */
int32_t mf_moe_combine(const void *rows, const int32_t *rowOf, const float *weights, uint32_t tokens, uint32_t hidden,
                       uint32_t topK, void *y, void *stream);
/* ---- optional: where the submitting thread runs ------------------------------
 * The only two functions of this header that touch anything outside the library: they CHANGE THE CALLING
 * THREAD'S CPU AFFINITY (mf_host_launch_costs restores it, mf_pin_thread_near_gpu keeps the narrowed set, and
 * threads created afterwards inherit it).  Nothing in the library calls them on its own.
 * What one launch costs the submitting thread depends on the CPU it runs on (3.1 against
 * 4.3 us per smem_bm_copy_batch call on the hosts this was built on, half of the CPUs each, with nothing in the
 * operating system's topology to tell them apart), and a thread the scheduler moves between the two kinds changes
 * pace mid-run.  mf_host_launch_costs measures it: it pins the calling thread to each CPU of its affinity set in
 * turn, times 256 launches of an empty kernel with a full argument block from there, restores the set, and
 * returns how many (cpu, microseconds per launch) pairs it wrote (at most `capacity`).  mf_pin_thread_near_gpu
 * leaves the set alone where the dearest CPU is within 25 % of the cheapest (hosts with one kind of CPU measure
 * 2.5 to 3.0 us) and otherwise narrows the calling thread's affinity set to the CPUs within 15 % of the cheapest;
 * it returns the size of the resulting set, and threads created afterwards inherit it.  Both take some 20 ms and wait for the thread's stream.  No
 * counterpart in the reference (a deployment would use numactl where the topology is visible). */
int32_t mf_host_launch_costs(uint32_t *cpus, float *micros, uint32_t capacity);
int32_t mf_pin_thread_near_gpu(void);

/* ---- runtime services (thin layer over HIP) ------------------------------ */
int mfrt_init(int device);
void mfrt_shutdown(void);
int mfrt_is_initialised(void);
int mfrt_device_id(void);
int mfrt_current_device(void);
int mfrt_bind_thread(void);
uint32_t mfrt_cu_count(void);
const char *mfrt_error_string(int err);
void *mfrt_alloc_device(uint64_t bytes);
int mfrt_free_device(void *p);
void *mfrt_alloc_host(uint64_t bytes);
int mfrt_free_host(void *p);
int mfrt_pointer_kind(const void *p);
void *mfrt_stream_create(void);
int mfrt_stream_destroy(void *stream);
int mfrt_stream_sync(void *stream);
int mfrt_device_sync(void);
void *mfrt_event_create(void);
int mfrt_event_destroy(void *event);
int mfrt_event_record(void *event, void *stream);
int mfrt_event_sync(void *event);
int mfrt_stream_wait_event(void *stream, void *event);
/* Whether two idle streams share a hardware queue: 1 (launches on them run one after the other however independent
 * they are), 0 (they run side by side), -1 (not known).  The runtime spreads the streams of a process over a few hardware
 * queues, not evenly; the library's own streams are handed out one per queue, a caller that brings
 * streams of its own can ask here.  Takes about 50 us (a lane waits 40 us by the clock on `a`, an empty kernel on `b`). */
int mfrt_streams_share_queue(void *a, void *b);
int mfrt_event_done(void *event);
float mfrt_event_elapsed_ms(void *start, void *stop);
int mfrt_memcpy(void *dst, const void *src, uint64_t bytes);
int mfrt_memset(void *dst, int value, uint64_t bytes);
int mfrt_memcpy_async(void *dst, const void *src, uint64_t bytes, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* MF_HIP_DATAPLANE_H */
