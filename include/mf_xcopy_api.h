/*
 * Drop-in C entry points of the xcopy data path, exported by
 * libmf_hip_dataplane.so.  Names, argument order and return conventions are
 * those of the reference's public headers, so a program written against
 * them links unchanged; each declaration cites the interface it replaces.
 *
 * Scope of this build: one process, one GPU, rank 0 of a world of 1.  The
 * control plane of the reference (config store, join/leave exchange, TLS,
 * RDMA transports) is not part of it; calls that would need it say so
 * through their return code instead of pretending.
 */
#ifndef MF_XCOPY_API_H
#define MF_XCOPY_API_H

#include "mf_xcopy_types.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ======================= hybm layer ==================================== */

/* src/hybm/include/hybm.h:28 — select the GPU, create the copy runtime.
 * deviceId is the HIP device ordinal.  Idempotent. */
int32_t hybm_init(uint16_t deviceId, uint64_t flags);
/* src/hybm/include/hybm.h:33 */
void hybm_uninit(void);
/* src/hybm/include/hybm.h:57 — static text for a BM_* code. */
const char *hybm_get_error_string(int32_t errCode);
/* src/hybm/include/hybm.h:41,49 */
void hybm_set_extern_logger(void (*logger)(int level, const char *msg));
int32_t hybm_set_log_level(int level);

/* src/hybm/include/hybm_big_mem.h:31 — id <= 510; options->rankCount must be 1
 * and rankId 0 in this build (BM_NOT_SUPPORTED otherwise -> NULL). */
hybm_entity_t hybm_create_entity(uint16_t id, const hybm_options *options, uint32_t flags);
/* src/hybm/include/hybm_big_mem.h:39 */
void hybm_destroy_entity(hybm_entity_t e, uint32_t flags);
/* src/hybm/include/hybm_big_mem.h:48,57 — reserve / release the GVA windows
 * (device window: rankCount*maxHBMSize, host window: rankCount*maxDRAMSize). */
int32_t hybm_reserve_mem_space(hybm_entity_t e, uint32_t flags);
int32_t hybm_unreserve_mem_space(hybm_entity_t e, uint32_t flags);
/* src/hybm/include/hybm_big_mem.h:65 — base of the window of one memory type. */
void *hybm_get_memory_ptr(hybm_entity_t e, hybm_mem_type mType);
/* src/hybm/include/hybm_big_mem.h:76 — back the local rank's window with HBM
 * (hipMalloc) or pinned, device-mapped DRAM (hipHostMalloc); size must be a
 * multiple of 2 MiB (src/hybm/csrc/entity/hybm_entity_default.cpp:180-183). */
hybm_mem_slice_t hybm_alloc_local_memory(hybm_entity_t e, hybm_mem_type mType, uint64_t size, uint32_t flags);
/* src/hybm/include/hybm_big_mem.h:87 */
int32_t hybm_free_local_memory(hybm_entity_t e, hybm_mem_slice_t slice, uint32_t count, uint32_t flags);
/* src/hybm/include/hybm_big_mem.h:96 */
void *hybm_get_slice_va(hybm_entity_t e, hybm_mem_slice_t slice);

/* src/hybm/include/hybm_big_mem.h:106 — make memory the caller owns (HBM from hipMalloc, or
 * pinned host memory) part of the entity, so that pool-side range checks accept it.  Ordinary
 * pageable memory is refused: it cannot be pinned after the fact on this platform. */
hybm_mem_slice_t hybm_register_local_memory(hybm_entity_t e, const void *ptr, uint64_t size, uint32_t flags);

/* src/hybm/include/hybm_data_op.h:36-37 — one contiguous copy.
 * BM_INVALID_PARAM for NULL e/params/src/dest, dataSize == 0, direction >= BUTT,
 * an AUTO direction that cannot be inferred, an unknown entity handle, or a
 * pool-side ("G") range that leaves the entity's windows
 * (src/hybm/csrc/hybm_data_op_entry.cpp:32-73).
 * stream: a hipStream_t passed as void*, or NULL for the calling thread's own
 * stream.  flags: ASYNC_COPY_FLAG | COPY_EXTEND_FLAG. */
int32_t hybm_data_copy(hybm_entity_t e, hybm_copy_params *params, hybm_data_copy_direction direction, void *stream,
                       uint32_t flags);

/* src/hybm/include/hybm_data_op.h:48-49 — batchSize independent copies,
 * result == for i: memcpy(destinations[i], sources[i], dataSizes[i]).
 * Direction AUTO is inferred from element 0 only; zero-length elements are
 * legal no-ops; NULL element pointers are BM_INVALID_PARAM
 * (src/hybm/csrc/hybm_data_op_entry.cpp:85-132).  Destination ranges of one
 * batch must not overlap each other or any source range: the copies run
 * concurrently on the GPU. */
int32_t hybm_data_batch_copy(hybm_entity_t e, hybm_batch_copy_params *params, hybm_data_copy_direction direction,
                             void *stream, uint32_t flags);

/* src/hybm/include/hybm_data_op.h:56 — drain the calling thread's stream. */
int32_t hybm_wait(hybm_entity_t e);

/* ======================= smem BM layer ================================= */

/* src/smem/include/host/smem_bm.h:28 */
int32_t smem_bm_config_init(smem_bm_config_t *config);
/* src/smem/include/host/smem_bm.h:43 — worldSize must be 1 here (SM_ERROR
 * otherwise, after the reference's own argument checks,
 * src/smem/csrc/smem_bm/smem_bm.cpp:62-68); storeURL is validated non-NULL and
 * otherwise unused. */
int32_t smem_bm_init(const char *storeURL, uint32_t worldSize, uint16_t deviceId, const smem_bm_config_t *config);
/* src/smem/include/host/smem_bm.h:50 */
void smem_bm_uninit(uint32_t flags);
/* src/smem/include/host/smem_bm.h:57 */
uint32_t smem_bm_get_rank_id(void);
/* src/smem/include/host/smem_bm.h:73-74 */
smem_bm_t smem_bm_create(uint32_t id, uint32_t memberSize, smem_bm_data_op_type dataOpType, uint64_t localDRAMSize,
                         uint64_t localHBMSize, uint32_t flags);
/* src/smem/include/host/smem_bm.h:86 */
smem_bm_t smem_bm_create2(uint32_t id, const smem_bm_create_option_t *option);
/* src/smem/include/host/smem_bm.h:93 */
void smem_bm_destroy(smem_bm_t handle);
/* src/smem/include/host/smem_bm.h:103,112 — world of one: join/leave only flip
 * the entry's joined state. */
int32_t smem_bm_join(smem_bm_t handle, uint32_t flags);
int32_t smem_bm_leave(smem_bm_t handle, uint32_t flags);
/* src/smem/include/host/smem_bm.h:121 */
uint64_t smem_bm_get_local_mem_size_by_mem_type(smem_bm_t handle, smem_bm_mem_type memType);
/* src/smem/include/host/smem_bm.h:131 — base + max{HBM,DRAM}Size * peerRankId
 * (src/smem/csrc/smem_bm/smem_bm.cpp:290-317). */
void *smem_bm_ptr_by_mem_type(smem_bm_t handle, smem_bm_mem_type memType, uint16_t peerRankId);
/* src/smem/include/host/smem_bm.h:149 */
int32_t smem_bm_copy(smem_bm_t handle, smem_copy_params *params, smem_bm_copy_type t, uint32_t flags);
/* src/smem/include/host/smem_bm.h:164 — the hot path. */
int32_t smem_bm_copy_batch(smem_bm_t handle, smem_batch_copy_params *params, smem_bm_copy_type t, uint32_t flags);
/* src/smem/include/host/smem_bm.h:171 */
int32_t smem_bm_wait(smem_bm_t handle);
/* src/smem/include/host/smem_bm.h:180,188 — pin + map caller memory so that it
 * can be used as the local side of a copy without staging. */
int32_t smem_bm_register_user_mem(smem_bm_t handle, uint64_t addr, uint64_t size);
int32_t smem_bm_unregister_user_mem(smem_bm_t handle, uint64_t addr);
/* src/smem/include/host/smem_bm.h:197 */
uint32_t smem_bm_get_rank_id_by_gva(smem_bm_t handle, void *gva);

/* src/smem/include/host/smem.h:58,66,111 (same logger sink as hybm_*) and the
 * thread-local error text of src/smem/csrc/common/smem_last_error.h. */
int32_t smem_set_extern_logger(void (*func)(int level, const char *msg));
int32_t smem_set_log_level(int level);
const char *smem_get_last_err_msg(void);

/* ---- smem transfer front-end: one-sided read / write between transfer objects by name --------
 * src/smem/include/host/smem_trans.h:24-239.  Objects of one process find each other through an
 * in-process directory (the config store and its watch threads are not part of this library):
 * a sender sees the memory receivers registered and the other way round, immediately, so
 * registration does not sleep.  Remote addresses are the peer's own virtual addresses; they are
 * translated through the slice map (src/smem/csrc/smem_trans/smem_trans_entry.cpp:307-372) and
 * handed to hybm_data_batch_copy as one fused launch.  The copy direction follows what the
 * memory really is (HBM or host) instead of assuming HBM on both sides. */
int32_t smem_trans_config_init(smem_trans_config_t *config);                        /* smem_trans.h:30 */
int32_t smem_trans_init(const smem_trans_config_t *config);                         /* :39 */
void smem_trans_uninit(uint32_t flags);                                             /* :46 */
/* uniqueId: "ip:port" or "[ipv6]:port"; storeUrl must be non-empty and is otherwise unused. */
smem_trans_t smem_trans_create(const char *storeUrl, const char *uniqueId, const smem_trans_config_t *config); /* :57 */
void smem_trans_destroy(smem_trans_t handle, uint32_t flags);                       /* :65 */
/* Pinned, device-mapped host memory that is registered on return (size rounded up to 2 MiB). */
void *smem_trans_malloc(smem_trans_t handle, size_t capacity);                      /* :74 */
int32_t smem_trans_free(smem_trans_t handle, void *address);                        /* :84 */
int32_t smem_trans_register_mem(smem_trans_t handle, void *address, size_t capacity, uint32_t flags); /* :95 */
int32_t smem_trans_batch_register_mem(smem_trans_t handle, void *addresses[], size_t capacities[], uint32_t count,
                                      uint32_t flags);                              /* :107-108 */
/* Unlike the reference (a no-op there, smem_trans.cpp:210-217) this withdraws the memory. */
int32_t smem_trans_deregister_mem(smem_trans_t handle, void *address);              /* :117 */
int32_t smem_trans_write(smem_trans_t handle, const void *localAddr, const char *remoteUniqueId, void *remoteAddr,
                         size_t dataSize, uint32_t flags);                          /* :130-131 */
int32_t smem_trans_batch_write(smem_trans_t handle, const void *localAddrs[], const char *remoteUniqueId,
                               void *remoteAddrs[], size_t dataSizes[], uint32_t batchSize, uint32_t flags); /* :145-146 */
int32_t smem_trans_read(smem_trans_t handle, void *localAddr, const char *remoteUniqueId, const void *remoteAddr,
                        size_t dataSize, uint32_t flags);                           /* :159-160 */
int32_t smem_trans_batch_read(smem_trans_t handle, void *localAddrs[], const char *remoteUniqueId,
                              const void *remoteAddrs[], size_t dataSizes[], uint32_t batchSize, uint32_t flags); /* :174-175 */
/* The *_submit forms enqueue on the caller's hipStream_t (must not be NULL) and return at once. */
int32_t smem_trans_read_submit(smem_trans_t handle, void *localAddr, const char *remoteUniqueId,
                               const void *remoteAddr, size_t dataSize, void *stream, uint32_t flags);   /* :189-190 */
int32_t smem_trans_write_submit(smem_trans_t handle, const void *localAddr, const char *remoteUniqueId,
                                void *remoteAddr, size_t dataSize, void *stream, uint32_t flags);        /* :204-205 */
int32_t smem_trans_batch_read_submit(smem_trans_t handle, void *localAddrs[], const char *remoteUniqueId,
                                     const void *remoteAddrs[], size_t dataSizes[], uint32_t batchSize, void *stream,
                                     uint32_t flags);                                                   /* :220-222 */
int32_t smem_trans_batch_write_submit(smem_trans_t handle, const void *localAddrs[], const char *remoteUniqueId,
                                      void *remoteAddrs[], size_t dataSizes[], uint32_t batchSize, void *stream,
                                      uint32_t flags);                                                  /* :237-239 */

#ifdef __cplusplus
}
#endif

#endif /* MF_XCOPY_API_H */
