/*
 * Exported by libmf_hip_dataplane.so WITHOUT a stability promise: read-only views of the host logic
 * (planner, address registry, direction algebra, transfer arithmetic) for tests, loops that replay
 * API calls from C for benchmarks, and switches over measured defaults (chunk size, grids, held
 * stores, read and write windows).  An integrator needs none of them; the defaults are what was
 * measured fastest.  The stable native surface is mf_hip_dataplane.h.
 */
#ifndef MF_HIP_DATAPLANE_INTERNAL_H
#define MF_HIP_DATAPLANE_INTERNAL_H

#include "mf_hip_dataplane.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- replay loops (benchmarks) --------------------------------------------- */
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

/* ---- switches over measured defaults ---------------------------------------- */
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
 * has without them; at 7 200 000 and above most launches do.  That holds for segments that start between
 * cache lines.  Segments whose sources and destinations all start on 128-byte lines are paced for
 * 7 100 000 (32 x 16 MiB back to back: 6.95 instead of 6.65 TB/s), those of 64 MiB and
 * more on average for 7 400 000, and a batch of 1 GiB and more of such long segments is cut into launches of
 * about 512 MiB, which hold their schedule more often than longer ones (1 GiB: 7.1-7.2 instead of 6.7 TB/s).
 * Segments whose source and destination differ modulo 16 take no windows.  The call sets all three rates; 0
 * switches the form off, MF_XCOPY_WINDOWS_OWN_CHOICE brings back the rates the library chose itself (what
 * hybm_init measured, else the defaults above).  While several threads submit on streams of their own the
 * form is not used. */
#define MF_XCOPY_WINDOWS_OWN_CHOICE 1u
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

/* What hybm_init measured on its GPU and chose (about 15 ms, 1 GiB of HBM for that long; the environment variable
 * MF_HIP_CALIBRATE=0 skips it and keeps the fitted defaults).  A batch of 2196 chunks is timed with its stores not held
 * and held for the rule's wait and 200 ns either side: the best of the three becomes the process's offset to every wait
 * (holdDeltaNanos), and holding is switched off where it does not beat the plain launch by 3 % (holdEnabled 0).  A copy
 * of 512 MiB is timed without windows, at the default rate, at 94 % of it and at the highest rate, the one long segments on
 * cache lines take: windowMBps receives the rate in force (0: windows did not beat the plain kernel and are off),
 * windowAlignedMBps and windowLongMBps the ones for segments on cache lines and for long ones among them (the higher
 * rates where the highest was 2 % faster here, else the same as windowMBps).  micros (8 floats,
 * may be NULL): the eight times in that order, us per batch / per copy.  Returns 1 if the calibration ran, 0 if not.
 * mf_xcopy_hold_stores / mf_xcopy_windows still override what it chose (a rate set by hand holds for both). */
int32_t mf_xcopy_calibration(int32_t *holdEnabled, int32_t *holdDeltaNanos, uint32_t *windowMBps, uint32_t *windowAlignedMBps,
                             uint32_t *windowLongMBps, float *micros);
/* The streams hybm_init makes for calling threads and submit threads, in the order they are handed out (the calling
 * thread of hybm_init holds the first): queues[i] is the hardware queue stream i sits on, numbered in order of
 * appearance.  The library asks the GPU which of its streams share a queue (launches on such streams run one
 * after the other) and hands out one stream of every queue before the second of any.  Returns the number of streams
 * (at most `capacity` are written); all entries differ where the GPU gave no answer. */
uint32_t mf_xcopy_stream_queues(uint32_t *queues, uint32_t capacity);
/* Table launches.  stageUnordered: 1 (default) launches the upload of a ragged table's descriptors without a
 * barrier, so that it runs while the caller's earlier copies still do; 0 orders it behind them.
 * deviceTableWgPerCu: workgroups per CU of the launch that copies a table in device memory, whose chunk
 * count only the GPU knows (0 = the default: eight workgroups per segment, between 32 and 4096 per CU); each walks
 * the chunks with the grid as its stride. */
int32_t mf_xcopy_tune_table(uint32_t stageUnordered, uint32_t deviceTableWgPerCu);
/* Held stores beyond the kernel-argument form.  deepHold: 1 (default) lets batches of 24 to 64 MiB whose segments
 * average 32 KiB and more be copied in 16 KiB chunks, one single wave each with sixteen loads per lane in flight,
 * stores held like those of the smaller batches; 0 keeps them on 4 KiB chunks that store at once.
 * pinnedExtraNanos: added to the wait of launches of more than 128 segments, whose descriptors come out of pinned
 * host memory rather than out of the kernel arguments (default 1600: a wave's loads start a link round trip later;
 * launches on 16 KiB chunks wait 800 ns more than that).
 * holdOnSideStreams: 1 lets batches launched by the submit threads (mf_xcopy_unordered_streams) hold their stores too;
 * 0 (default): they overlap one another on purpose and store at once. */
int32_t mf_xcopy_tune_hold(uint32_t deepHold, int32_t pinnedExtraNanos, uint32_t holdOnSideStreams);

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

/* ---- views of the 2-D kernel's arithmetic ------------------------------------- */
/* Host-only views of the 2-D kernel's index arithmetic, for tests.  mf_copy2d_describe: rows one
 * workgroup takes and the division constant for rows of `width` bytes.  mf_copy2d_rowcol_mismatches:
 * how many of the units 0 .. unitsInChunk-1 of a chunk the kernel's (row, column) formula places
 * differently from u / widthUnits, u % widthUnits (0 for every plan the library builds). */
void mf_copy2d_describe(uint64_t width, uint32_t *rowsPerChunk, uint32_t *magic);
uint32_t mf_copy2d_rowcol_mismatches(uint32_t widthUnits, uint32_t rowsPerChunk, uint32_t magic, uint32_t unitsInChunk);

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

#endif /* MF_HIP_DATAPLANE_INTERNAL_H */
