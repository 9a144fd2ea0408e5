/*
 * Native entry points of libmf_hip_dataplane.so beyond the drop-in surface of
 * mf_xcopy_api.h: the raw batch enqueue the benchmark times, runtime services
 * a host program needs to own GPU memory and streams without touching HIP
 * itself, and read-only views of the host logic (planner, address registry,
 * direction algebra) for tests.  Plain C types only; a stream or event is an
 * opaque void*.  Functions returning int32_t give 0 or a negative BM_* code
 * unless stated; the mfrt_* services return 0 or a positive HIP error number.
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

/* `steps` calls of smem_bm_copy_batch(handle, batches[i % count], t, flags), i = 0 .. steps-1,
 * issued from C: what the loop of a C or C++ caller does (the reference's benchmark,
 * example/bm/BmBenchmark/band_width_calculator.cpp:530-590, is such a loop), for callers
 * written in an interpreted language whose per-call overhead would otherwise set the pace.
 * Stops at the first call that fails and returns its code. */
int32_t mf_bm_copy_batch_replay(smem_bm_t handle, smem_batch_copy_params *const *batches, uint32_t count,
                                uint32_t steps, smem_bm_copy_type t, uint32_t flags);

/* The same for the transfer front-end: `steps` calls of smem_trans_batch_write_submit(handle, sources, remoteUniqueId,
 * destinations, dataSizes, batchSize, stream, 0) with the arrays of batches[i % count] (sources = local addresses,
 * destinations = addresses in the peer's registered memory). */
int32_t mf_trans_batch_write_replay(smem_trans_t handle, smem_batch_copy_params *const *batches, uint32_t count, uint32_t steps,
                                    const char *remoteUniqueId, void *stream);

/* The same `steps` calls shared out over `threads` host threads (call i goes to thread
 * i % threads), each thread on its own stream as the reference gives every calling thread its
 * own (src/hybm/csrc/ts_engine/hybm_stream_manager.cpp:73-90), all asynchronous with one
 * smem_bm_wait per thread at the end.  *seconds receives the wall-clock time from the moment
 * all threads (already warmed up) are released until the last one has returned from its wait.
 * The threads share `batches`: the library rewrites the address arrays in place with the same
 * values, which is harmless.  Returns the first failing call's code. */
int32_t mf_bm_copy_batch_replay_threads(smem_bm_t handle, smem_batch_copy_params *const *batches, uint32_t count,
                                        uint32_t steps, smem_bm_copy_type t, uint32_t threads, double *seconds);

/* An enqueue of mf_xcopy_batch for a {src,dst,len} triple table that already lives in device memory. */
int32_t mf_xcopy_device_table(const void *triples, uint32_t n, int32_t route, void *stream);

/* No counterpart in the reference.  mf_xcopy_device_table for callers that cannot allocate: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  The chunk prefix
 * the kernels need lives in a statically allocated device array (132 KiB per GPU, held until the
 * process ends) instead of memory the library allocates on demand, and the call creates no stream,
 * event or staging either: `stream` is used as given (NULL is the null stream).
 * Limits: n <= MF_XCOPY_STATIC_TABLE_MAX segments (BM_INVALID_PARAM beyond); every call on one GPU
 * uses the same array, so two calls whose kernels may run at the same time (different streams,
 * different threads) race: keep them on one stream or order them yourself.  hybm_init must have
 * run (it looks the array's address up).  Same results as mf_xcopy_device_table. */
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

/* Host-only views of the 2-D kernel's index arithmetic, for tests.  mf_copy2d_describe: rows one
 * workgroup takes and the division constant for rows of `width` bytes.  mf_copy2d_rowcol_mismatches:
 * how many of the units 0 .. unitsInChunk-1 of a chunk the kernel's (row, column) formula places
 * differently from u / widthUnits, u % widthUnits (0 for every plan the library builds). */
void mf_copy2d_describe(uint64_t width, uint32_t *rowsPerChunk, uint32_t *magic);
uint32_t mf_copy2d_rowcol_mismatches(uint32_t widthUnits, uint32_t rowsPerChunk, uint32_t magic, uint32_t unitsInChunk);

/* Launch-shape knobs.  units: 16-byte units per workgroup chunk (0 = choose
 * per batch); wgPerCu: grid cap in workgroups per CU on HBM routes (0 = the
 * default: one workgroup per chunk, no cap); wgPerCuLink: workgroups per CU
 * on host-link routes (0 = the default, 1). */
int32_t mf_xcopy_tune(uint32_t units, uint32_t wgPerCu, uint32_t wgPerCuLink);
/* Stores held back.  A batch of 960 to 6144 chunks of 4 KiB between HBM addresses (4 to 25 MB in up
 * to 128 segments) is copied 7 to 20 % faster when every wave waits with its stores until the loads of
 * the whole launch are out, so that HBM sees a burst of reads and then a burst of writes instead of both
 * mixed.  nanos: -1 = the library's rule for how long a wave waits after its start (the default),
 * 0 = never wait, otherwise that many ns for every launch the rule would pick.  Other launches, and
 * batches submitted with MF_COPY_UNORDERED_FLAG, never wait. */
int32_t mf_xcopy_hold_stores(int32_t nanos);
/* Read and write windows.  A batch of up to 128 segments and 512 MiB or more between HBM addresses is copied
 * by 4096 waves that alternate, all together and by the GPU's constant-rate clock, between a read half and a
 * write half of a period, so that HBM sees long bursts of one direction: 6.65-6.75 TB/s instead of 6.1-6.35 on
 * aligned copies of 512 MiB to 2 GiB, 6.05-6.3 instead of 5.75-5.85 when sources sit at odd addresses.  The
 * period is cut for a rate of HBM traffic (read + written) in MB/s, 6 800 000 by default; at 7 000 000 the waves
 * of a 2 GiB copy now and then no longer keep up, the windows dissolve and the copy runs at about the rate it
 * has without them; at 7 200 000 and above most launches do.  0 switches the form off.  While several threads
 * submit on streams of their own it is not used. */
int32_t mf_xcopy_windows(uint32_t megabytesPerSecond);
uint32_t mf_xcopy_choose_units(uint64_t totalBytes, uint32_t cuCount, int32_t route);
uint64_t mf_xcopy_launch_count(void);

/* Host-only view of the work decomposition: writes, for every chunk of the
 * normalised batch, up to three byte ranges {srcAddr, dstAddr, bytes, chunk}
 * (head, 16-byte body, tail) into out[4*i..].  Returns the number of ranges,
 * or -(needed) when capacity (in ranges) is too small.  inlineForm receives 1
 * when the batch fits the kernel-argument form. */
int64_t mf_xcopy_describe_plan(const uint64_t *src, const uint64_t *dst, const uint64_t *len, uint32_t n,
                               uint32_t units, uint64_t *out, uint64_t capacity, int32_t *inlineForm);

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
/* A combine of topK == 8 or 6 with rows of 2048 elements and more, on enough tokens to give every wave of the chip six
 * slices of 128 x 8 elements (about 3500 tokens of 7168 elements on 256 CUs), runs as waves that stay for the whole
 * launch and alternate, chip-wide and by the clock, between reading rows and writing results.  readMBps / writeMBps
 * (MB/s of HBM traffic, 1 000 000 ... 16 000 000) set the pace of the two parts; the defaults are 6 800 000 and
 * 6 200 000, both 0 turns the form off (one workgroup per slice, as for smaller inputs, and as long as a second
 * thread holds a stream of the library).  Results do not depend on it.  No counterpart in the reference.  Returns BM_INVALID_PARAM for other values. */
int32_t mf_moe_combine_windows(uint32_t readMBps, uint32_t writeMBps);
/* 1 if hybm_init found that the GPU deals consecutive workgroups to its eight XCDs in turn (an MI355X in its default
 * partition does): the dispatch of rows of whole cache lines then writes its output in runs of consecutive rows, one stream of runs
 * per XCD; 0: it keeps to the token-ordered permute.  No counterpart in the reference. */
int32_t mf_moe_xcd_streams(void);

/* Host side of a launch.  What one launch costs the submitting thread depends on the CPU it runs on (3.1 against
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
int mfrt_event_done(void *event);
float mfrt_event_elapsed_ms(void *start, void *stop);
int mfrt_memcpy(void *dst, const void *src, uint64_t bytes);
int mfrt_memset(void *dst, int value, uint64_t bytes);
int mfrt_memcpy_async(void *dst, const void *src, uint64_t bytes, void *stream);

/* ---- address registry view (HybmVaManager counterpart,
 *      src/hybm/csrc/mm/hybm_va_manager.h:175-264) -------------------------- */
void mf_va_clear(void);
int32_t mf_va_add(uint64_t gva, uint64_t size, int32_t memType, uint64_t lva, uint32_t localRank);
int32_t mf_va_add_external(uint64_t gva, uint64_t size, int32_t memType, uint64_t lva, uint32_t localRank,
                           uint32_t importedRank);
void mf_va_remove(uint64_t va);
uint64_t mf_va_gva_of_lva(uint64_t lva);
uint64_t mf_va_lva_of_gva(uint64_t gva);
int32_t mf_va_is_gva(uint64_t va);
int32_t mf_va_is_known(uint64_t va);
int32_t mf_va_mem_type(uint64_t va);
int64_t mf_va_rank(uint64_t gva);                    /* -1 when not found */
int32_t mf_va_infer_direction(uint64_t srcVa, uint64_t dstVa);
uint64_t mf_va_reserve(uint32_t localRank, uint64_t size, int32_t memType);
void mf_va_unreserve(uint64_t start);
uint64_t mf_va_range_count(void);
uint64_t mf_va_reserved_count(void);

/* ---- direction algebra and window arithmetic views ------------------------ */
int32_t mf_dir_compose(int32_t srcPool, int32_t srcDevice, int32_t dstPool, int32_t dstDevice);
int32_t mf_dir_translate_smem(int32_t copyType, int32_t srcPoolType, int32_t dstPoolType);
int32_t mf_dir_checks(int32_t direction);            /* bit 0: source checked, bit 1: destination checked */
int32_t mf_gva_contains(uint64_t base, uint64_t stride, uint64_t rankCount, uint64_t addr, uint64_t size);
uint32_t mf_gva_rank(uint64_t base, uint64_t stride, uint64_t rankCount, uint64_t rankSpace, uint64_t addr);
uint64_t mf_gva_mask48(uint64_t addr);

/* ---- transfer front-end arithmetic views ----------------------------------
 * mf_trans_combine: union of n (start, size) pairs (pairs[2*n]) into sorted, disjoint runs
 * written to out[2*k..] (room for n pairs); returns k.  mf_trans_translate: look one peer range
 * up in n runs {start, size, mapped} (slices[3*n]); the mapped address or 0 when the range is not
 * inside one run.  mf_trans_parse_name: 1 when the name is a valid "ip:port" / "[ipv6]:port" and,
 * then, its 20-byte binary form in key. */
uint32_t mf_trans_combine(const uint64_t *pairs, uint32_t n, uint64_t *out);
uint64_t mf_trans_translate(const uint64_t *slices, uint32_t n, uint64_t remote, uint64_t size);
int32_t mf_trans_parse_name(const char *name, uint8_t *key);

#ifdef __cplusplus
}
#endif

#endif /* MF_HIP_DATAPLANE_H */
