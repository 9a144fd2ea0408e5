/*
 * The two-symbol copy-kernel plugin, exported by libmf_hybm_copy_extend.so.
 *
 * This is the file the reference's loader dlopen()s from the directory named
 * by MEMFABRIC_HYBRID_EXTEND_LIB_PATH and resolves by name
 * (src/hybm/csrc/under_api/dl_hybm_copy_extend.cpp:20,32,50,57-58; function
 * pointer types at src/hybm/csrc/under_api/dl_hybm_copy_extend.h:21-22).
 * Both symbols must be present or the loader unloads the library again.
 *
 * Neither function has an error channel (they return void in the reference,
 * src/hybm/csrc/copy_extend/hybm_copy_kernel.cpp:80-83,121-124).  A launch
 * that fails is reported through the logger, counted (mf_copy_extend_failures)
 * and leaves the stream and the completion word untouched: a caller that
 * waits for the word of a failed launch waits for ever, as it would behind a
 * failed launch of the reference's kernel.
 */
#ifndef MF_HIP_COPY_EXTEND_H
#define MF_HIP_COPY_EXTEND_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Replaces hybm_copy_extend (src/hybm/csrc/copy_extend/hybm_copy_kernel.cpp:80-83).
 * Enqueue dst[0..len) = src[0..len) on `stream` (a hipStream_t; NULL = the
 * null stream).  src/dst: any device-accessible addresses (HBM or pinned,
 * mapped host memory), any alignment.  `dim` is the caller's concurrency
 * hint (the reference passes 32 AI-vector cores); the grid here is sized
 * from len instead and dim is ignored.  Returns without waiting. */
void hybm_copy_extend(void *src, void *dst, uint64_t len, uint32_t dim, void *stream);

/* Replaces hybm_batch_copy_extend (src/hybm/csrc/copy_extend/hybm_copy_kernel.cpp:121-124).
 * param: device-accessible address of uint64_t[3*count] laid out
 *        {src_i, dst_i, len_i} (src/hybm/csrc/data_operation/host/hybm_data_op_sdma.cpp:520-528);
 *        count <= 16384 per call in the reference, any count here.
 * mask:  device-accessible address of one uint64_t that the caller zeroed; it
 *        receives `dim` once `param` will not be read again (the reference's
 *        "slot is free again" marker, hybm_data_op_sdma.cpp:487-497 and
 *        hybm_copy_kernel.cpp:113-118; the caller learns that the copy itself
 *        has finished from the stream, :537-540).  A table the CPU can read
 *        is consumed inside this call, so a word the CPU can write is stored
 *        before the call returns; for a table or a word in device memory a
 *        one-lane launch queued behind the copy on the same stream stores it.
 *        May be NULL.
 * Enqueues on `stream` and returns without waiting. */
void hybm_batch_copy_extend(void *param, uint32_t count, void *mask, uint32_t dim, void *stream);

/* No counterpart in the reference: launches of the two functions above that
 * failed since the library was loaded (they cannot return an error). */
uint64_t mf_copy_extend_failures(void);

#ifdef __cplusplus
}
#endif

#endif /* MF_HIP_COPY_EXTEND_H */
