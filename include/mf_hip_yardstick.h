/*
 * libmf_hip_yardstick.so: streaming kernels of known traffic.  Measurement
 * tooling for the benchmark and the tests, not part of the data plane and not
 * linked into it; nothing in the reference corresponds to it.
 */
#ifndef MF_HIP_YARDSTICK_H
#define MF_HIP_YARDSTICK_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* One workgroup per 16 KiB tile, 128-bit nontemporal accesses: kind 0 copies
 * `bytes` from src to dst, kind 1 fills dst with the word 0x5A, kind 2 reads
 * src (dst: a 4-byte device sink).  They show what this GPU sustains for a
 * flat copy, a pure write and a pure read, and calibrate hardware byte
 * counters.  bytes: a non-zero multiple of 16.  Enqueues on `stream` (a
 * hipStream_t; NULL is the null stream) on the current device and returns 0,
 * -2 for bad arguments, -1 when the launch failed. */
int32_t mf_probe_hbm(int32_t kind, void *dst, const void *src, uint64_t bytes, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* MF_HIP_YARDSTICK_H */
