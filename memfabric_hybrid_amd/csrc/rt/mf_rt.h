// Thin C layer over HIP.  Host C++ above this line never sees a HIP type:
// streams, events and device pointers travel as void*, sizes as integers.
// mfrt_* = runtime services, mfk_* = kernel launchers (enqueue only).
// Every int return is 0 on success or the hipError_t value.
#ifndef MF_RT_H
#define MF_RT_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* The plugin library keeps the runtime layer private so that it can share a
 * process with the data-plane library. */
#ifndef MF_RT_HIDDEN
#pragma GCC visibility push(default)
#endif

#define MFRT_ROUTE_HBM 0        /* source and destination in HBM            */
#define MFRT_ROUTE_TO_HOST 1    /* destination in pinned, mapped host DRAM  */
#define MFRT_ROUTE_FROM_HOST 2  /* source in pinned, mapped host DRAM       */

#define MFRT_PTR_PAGEABLE 0     /* ordinary host memory the GPU cannot address */
#define MFRT_PTR_DEVICE 1
#define MFRT_PTR_PINNED_HOST 2

/* ---- runtime ------------------------------------------------------------ */
int mfrt_init(int device);
int mfrt_current_device(void);          /* device current on the calling thread, -1 on error */
int mfrt_bind_thread(void);             /* make the initialised device current on this thread */
void mfrt_shutdown(void);
int mfrt_is_initialised(void);
int mfrt_device_id(void);
uint32_t mfrt_cu_count(void);
const char *mfrt_error_string(int err);

void *mfrt_alloc_device(uint64_t bytes);
int mfrt_free_device(void *p);
void *mfrt_alloc_host(uint64_t bytes);  /* pinned + device-mapped + portable */
int mfrt_free_host(void *p);
int mfrt_pointer_kind(const void *p);

/* Address windows: reserve virtual addresses first, back pieces of them with HBM later
 * (hipMemAddressReserve / hipMemCreate / hipMemMap).  Sizes and offsets are multiples of
 * mfrt_window_granularity().  A mapping is named by the handle mfrt_window_map returns;
 * [accessBase, +accessBytes) is the contiguous mapped run that ends with the new piece. */
uint64_t mfrt_window_granularity(void);
void *mfrt_window_reserve(uint64_t bytes);
int mfrt_window_release(void *base, uint64_t bytes);
void *mfrt_window_map(void *addr, uint64_t bytes, void *accessBase, uint64_t accessBytes);  /* handle, NULL on failure */
int mfrt_window_unmap(void *addr, uint64_t bytes, void *handle);
int mfrt_window_last_error(void);                       /* failed step (1 create, 2 map, 3 access) * 10000 + hipError_t */

void *mfrt_stream_create(void);
int mfrt_stream_destroy(void *stream);
int mfrt_stream_sync(void *stream);
int mfrt_device_sync(void);

void *mfrt_event_create(void);
int mfrt_event_destroy(void *event);
int mfrt_event_record(void *event, void *stream);
int mfrt_event_sync(void *event);
int mfrt_stream_wait_event(void *stream, void *event);
/* 1: launches on the two (idle) streams run one after the other because the streams share a hardware queue; 0: they
 * run side by side; -1: not known.  About 50 us. */
int mfrt_streams_share_queue(void *a, void *b);   /* work queued on `stream` afterwards waits for the event */
int mfrt_event_done(void *event);       /* 1 finished, 0 pending, <0 error */
float mfrt_event_elapsed_ms(void *start, void *stop);

int mfrt_memcpy(void *dst, const void *src, uint64_t bytes);  /* blocking hipMemcpy, direction inferred */
int mfrt_memset(void *dst, int value, uint64_t bytes);
int mfrt_memcpy_async(void *dst, const void *src, uint64_t bytes, void *stream);  /* the runtime's own DMA path */

/* ---- xcopy launchers (kernels/xcopy.hip) --------------------------------- */
/* anyOrder != 0: the launch does not wait for launches queued before it on `stream` (it carries no barrier);
 * launches queued after it without that option still wait for it. */
/* holdNanos != 0: every wave keeps its loaded data until that long after its own start (see HoldNanosFor in
 * kernels/xcopy_plan.h); honoured only by a launch of one chunk per workgroup, the chunk being 4 KiB or
 * mfk_xcopy_window_units() units (16 KiB, copied by single waves with sixteen loads per lane in flight). */
int mfk_xcopy_inline(const void *inlinePlan, int route, uint32_t grid, void *mask, uint32_t maskValue, void *stream,
                     int anyOrder, uint32_t holdNanos);
/* HBM to HBM copies of hundreds of MiB: the plan's chunks are mfk_xcopy_window_units() units (16 KiB), copied by up to
 * mfk_xcopy_window_waves() single-wave workgroups that alternate, chip-wide and by the clock, between a read half and a
 * write half of a period cut for `windowMBps` MB/s of HBM traffic (see XcopyWindowKernel). */
int mfk_xcopy_windows_available(void);   /* 1 when the current device's constant-rate clock is known, which the period is cut by */
uint32_t mfk_xcopy_window_units(void);
uint32_t mfk_xcopy_window_waves(void);
int mfk_xcopy_windowed(const void *inlinePlan, uint32_t windowMBps, void *mask, uint32_t maskValue, void *stream);
/* tablePlan: a mf::TablePlan (kernels/xcopy_plan.h).  Under a pattern its triples may live in pinned host
 * memory and neither prefix nor group map is read; with a header (left by mfk_xcopy_plan on the same stream)
 * chunk count, group shift and pattern are read from device memory and `grid` workgroups walk the chunks.
 * holdNanos: as for mfk_xcopy_inline, for a launch of one chunk per workgroup between HBM addresses. */
int mfk_xcopy_table(const void *tablePlan, int route, uint32_t grid, void *mask, uint32_t maskValue, void *stream,
                    uint32_t holdNanos);
/* Launches every copy kernel once on empty plans (a kernel's first launch is not capturable into a HIP graph). */
int mfk_xcopy_prelaunch(void *stream);
/* Times the calibration workloads on `stream` with HIP events, in 1 GiB of device memory it allocates and frees:
 * out[0 .. 3] = us per 2196-chunk batch without a hold and held for holdNanos[0 .. 2]; out[4 .. 7] = us per 512 MiB
 * copy without windows and in windows cut for windowMBps[0 .. 2].  0, or a HIP error number. */
int mfk_xcopy_calibrate(void *stream, const uint32_t *holdNanos, const uint32_t *windowMBps, float *out);
/* One lane stores `value` (as a 64-bit word, released at system scope) into `word` once everything queued on
 * `stream` before it has finished. */
int mfk_xcopy_signal(void *word, uint32_t value, void *stream);
/* Device-side planner for a triple table in device memory: one launch (two beyond 8192 segments) that leaves
 * header, chunk prefix and group map in `scratch` (mfk_xcopy_plan_scratch_words(nseg, groupCapacity) 32-bit words of
 * device memory; groupCapacity: entries of room for the group map, the more the finer) and fills *tablePlan
 * (a mf::TablePlan) for the mfk_xcopy_table call behind it on the same stream. */
uint64_t mfk_xcopy_plan_scratch_words(uint32_t nseg, uint32_t groupCapacity);
int mfk_xcopy_plan(const void *triples, uint32_t nseg, uint32_t units, void *scratch, uint32_t groupCapacity, void *tablePlan,
                   void *stream);
/* The table form with the planner's scratch in a statically allocated device array instead of memory the
 * engine allocates: no allocation anywhere, at most MFK_STATIC_TABLE_SEGMENTS segments, one call at a
 * time per GPU.  mfk_xcopy_static_setup looks the array's address up for the current device (once per
 * device, at start-up); mfk_xcopy_table_static returns -2 when that has not happened. */
#define MFK_STATIC_TABLE_SEGMENTS 32768u
int mfk_xcopy_static_setup(void);
int mfk_xcopy_table_static(const void *triples, uint32_t nseg, uint32_t units, int route, uint32_t grid, void *stream);

/* ---- MoE launchers (kernels/moe.hip) ---------------------------------------- */
uint64_t mfk_moe_workspace_bytes(uint32_t tokens, uint32_t topK, uint32_t experts);
int mfk_moe_dispatch(const void *x, const void *topk, uint32_t tokens, uint32_t hidden, uint32_t topK, uint32_t experts,
                     void *out, void *counts, void *offsets, void *rowOf, void *srcOf, void *workspace, void *stream);
/* paced != 0: the form whose waves stay and alternate between reading and writing may be used (see mfk_moe_combine_windows) */
int mfk_moe_combine(const void *rows, const void *rowOf, const void *weights, uint32_t tokens, uint32_t hidden,
                    uint32_t topK, void *y, void *stream, int paced);
/* once after the GPU is bound: finds out whether consecutive workgroups go to the eight XCDs in turn (the tile permute
 * of the dispatch needs it); mfk_moe_xcd_streams() is 1 if they do */
int mfk_moe_setup(void);
int mfk_moe_xcd_streams(void);
/* pace of the combine that keeps reads and writes apart in time, MB/s for its read and write parts; 0 = never */
void mfk_moe_combine_windows(uint32_t readMBps, uint32_t writeMBps);

/* ---- 2-D copy launcher (kernels/copy2d.hip) ----------------------------------- */
int mfk_copy2d(const void *rectPlan, uint32_t grid, void *stream);
/* The same rectangles in read and write windows cut for windowMBps; plan.first counts chunks of RectWindowChunks(). */
int mfk_copy2d_windowed(const void *rectPlan, uint32_t windowMBps, void *stream);
/* Both rectangle kernels once on an empty plan. */
int mfk_copy2d_prelaunch(void *stream);

#ifndef MF_RT_HIDDEN
#pragma GCC visibility pop
#endif

#ifdef __cplusplus
}
#endif

#endif /* MF_RT_H */
