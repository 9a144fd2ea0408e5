/*
 * Public value types of the xcopy data path (C, no HIP types).
 *
 * Every enumerator value, struct field order and field width below is part of
 * the binary contract with existing MemFabric callers; they restate
 *   src/hybm/include/hybm_def.h:45-62,100-154      (hybm_* enums, options, copy params)
 *   src/hybm/include/hybm_data_op.h:23-24          (copy flags)
 *   src/smem/include/host/smem_bm_def.h:34-122     (smem_bm_* enums, config, copy params)
 *   src/smem/include/host/smem.h:22-25             (flags, world-size limit)
 * of the reference tree.  The _Static_assert block at the end pins each value
 * so that an accidental edit fails the build instead of silently breaking a
 * caller compiled against the original headers.
 *
 * MF_WITH_REFERENCE_HEADERS: for a build inside the reference tree (its
 * include directories on the search path).  The reference's own headers then
 * define every type and this file only adds the pins, so code written against
 * this header and code written against theirs share one set of definitions.
 */
#ifndef MF_XCOPY_TYPES_H
#define MF_XCOPY_TYPES_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef MF_WITH_REFERENCE_HEADERS

#include "hybm_def.h"
#include "hybm_data_op.h"
#include "smem.h"
#include "smem_bm_def.h"
#include "smem_trans_def.h"
#ifdef __cplusplus
/* the return codes are C++ enumerations of the reference's namespaces */
#include "hybm_types.h"
#include "smem_types.h"
using namespace ock::mf;
using namespace ock::smem;
#endif

#else /* definitions of this build */

#ifdef __cplusplus
extern "C" {
#endif

/* ---- opaque handles -------------------------------------------------- */
typedef void *hybm_entity_t;
typedef void *hybm_mem_slice_t;
typedef void *smem_bm_t;

/* ---- flag bits accepted by every copy entry point --------------------- */
#ifndef ASYNC_COPY_FLAG
#define ASYNC_COPY_FLAG (1UL << (0))  /* enqueue only; completion via *_wait */
#endif
#ifndef COPY_EXTEND_FLAG
#define COPY_EXTEND_FLAG (1UL << (1)) /* route through the copy-kernel plugin */
#endif

#define SMEM_WORLD_SIZE_MAX 1024U
#define SMEM_INVALID_DEV_ID (-1)

#define HYBM_FLAG_EXPORT_ENTITY 1U
#define HYBM_TLS_PATH_SIZE 256
#define HYBM_FLAG_INIT_SHMEM_META (1ULL << 63)
#define HYBM_FLAG_CREATE_WITH_SHM (1U << 8)
#define HYBM_PRE_REG_SIZE_THRES (8192U * 1024)

#define SMEM_BM_TIMEOUT_MAX UINT32_MAX
#define SMEM_TLS_PATH_SIZE 256
#define SMEM_BM_FLAG_CREATE_WITH_SHM (1U << 8)

/* ---- hybm layer ------------------------------------------------------- */
typedef enum { HYBM_TYPE_AI_CORE_INITIATE = 0, HYBM_TYPE_HOST_INITIATE, HYBM_TYPE_BUTT } hybm_type;

typedef enum {
    HYBM_DOP_TYPE_DEFAULT = 0U,
    HYBM_DOP_TYPE_MTE = 1U << 0,
    HYBM_DOP_TYPE_SDMA = 1U << 1,
    HYBM_DOP_TYPE_DEVICE_RDMA = 1U << 2,
    HYBM_DOP_TYPE_HOST_RDMA = 1U << 3,
    HYBM_DOP_TYPE_HOST_TCP = 1U << 4,
    HYBM_DOP_TYPE_HOST_URMA = 1U << 5,
    HYBM_DOP_TYPE_BUTT
} hybm_data_op_type;

typedef enum { HYBM_MEM_TYPE_DEVICE = 1U << 0, HYBM_MEM_TYPE_HOST = 1U << 1, HYBM_MEM_TYPE_BUTT } hybm_mem_type;

typedef enum { HYBM_SCENE_DEFAULT = 1U << 0, HYBM_SCENE_TRANS = 1U << 1, HYBM_SCENE_SHM = 1U << 2, HYBM_SCENE_BUTT } hybm_scene;

typedef enum { HYBM_ROLE_PEER = 0, HYBM_ROLE_SENDER, HYBM_ROLE_RECEIVER, HYBM_ROLE_BUTT } hybm_role_type;

typedef struct {
    uint8_t desc[512L];
    uint32_t descLen;
} hybm_exchange_info;

typedef struct {
    bool tlsEnable;
    char caPath[HYBM_TLS_PATH_SIZE];
    char crlPath[HYBM_TLS_PATH_SIZE];
    char certPath[HYBM_TLS_PATH_SIZE];
    char keyPath[HYBM_TLS_PATH_SIZE];
    char keyPassPath[HYBM_TLS_PATH_SIZE];
    char packagePath[HYBM_TLS_PATH_SIZE];
    char decrypterLibPath[HYBM_TLS_PATH_SIZE];
} hybm_tls_config;

typedef struct {
    hybm_type bmType;
    hybm_mem_type memType;
    hybm_data_op_type bmDataOpType;
    uint16_t rankCount;
    uint16_t rankId;
    uint16_t devId;
    uint64_t maxHBMSize;     /* stride of one rank's window in the device GVA range */
    uint64_t maxDRAMSize;    /* stride of one rank's window in the host GVA range   */
    uint64_t deviceVASpace;  /* bytes of HBM this rank actually contributes         */
    uint64_t hostVASpace;    /* bytes of DRAM this rank actually contributes        */
    hybm_scene scene;
    bool globalUniqueAddress;
    hybm_role_type role;
    uint32_t flags;
    char transUrl[64];
    char tag[32];
    char tagOpInfo[256];
    hybm_tls_config tlsOption;
    int dramShmFd;
} hybm_options;

/* (source kind) x (destination kind); L = caller-private, G = inside the pool,
 * H = host DRAM, D = device HBM. */
typedef enum {
    HYBM_LOCAL_HOST_TO_GLOBAL_HOST = 0,
    HYBM_LOCAL_HOST_TO_GLOBAL_DEVICE = 1,
    HYBM_LOCAL_DEVICE_TO_GLOBAL_HOST = 2,
    HYBM_LOCAL_DEVICE_TO_GLOBAL_DEVICE = 3,
    HYBM_GLOBAL_HOST_TO_GLOBAL_HOST = 4,
    HYBM_GLOBAL_HOST_TO_GLOBAL_DEVICE = 5,
    HYBM_GLOBAL_HOST_TO_LOCAL_HOST = 6,
    HYBM_GLOBAL_HOST_TO_LOCAL_DEVICE = 7,
    HYBM_GLOBAL_DEVICE_TO_GLOBAL_HOST = 8,
    HYBM_GLOBAL_DEVICE_TO_GLOBAL_DEVICE = 9,
    HYBM_GLOBAL_DEVICE_TO_LOCAL_HOST = 10,
    HYBM_GLOBAL_DEVICE_TO_LOCAL_DEVICE = 11,
    HYBM_DATA_COPY_DIRECTION_AUTO = 12,
    HYBM_DATA_COPY_DIRECTION_BUTT
} hybm_data_copy_direction;

typedef struct {
    void *src;
    void *dest;
    uint64_t dataSize;
} hybm_copy_params;

/* Structure-of-arrays segment list.  The callee may rewrite sources[] and
 * destinations[] in place (upper 16 address bits cleared). */
typedef struct {
    void **sources;
    void **destinations;
    const uint64_t *dataSizes;
    uint32_t batchSize;
} hybm_batch_copy_params;

/* ---- smem BM layer ------------------------------------------------------ */
typedef enum {
    SMEM_MEM_TYPE_LOCAL_DEVICE = 0,
    SMEM_MEM_TYPE_LOCAL_HOST,
    SMEM_MEM_TYPE_DEVICE,
    SMEM_MEM_TYPE_HOST,
    SMEM_MEM_TYPE_BUTT
} smem_bm_mem_type;

typedef enum {
    SMEMB_DATA_OP_SDMA = 1U << 0,
    SMEMB_DATA_OP_HOST_RDMA = 1U << 1,
    SMEMB_DATA_OP_HOST_TCP = 1U << 2,
    SMEMB_DATA_OP_DEVICE_RDMA = 1U << 3,
    SMEMB_DATA_OP_HOST_URMA = 1U << 4,
    SMEMB_DATA_OP_BUTT
} smem_bm_data_op_type;

typedef enum {
    SMEMB_COPY_L2G = 0,  /* local HBM   -> pool            */
    SMEMB_COPY_G2L = 1,  /* pool        -> local HBM       */
    SMEMB_COPY_G2H = 2,  /* pool        -> local host DRAM */
    SMEMB_COPY_H2G = 3,  /* local host  -> pool            */
    SMEMB_COPY_L2GH = 4, /* local HBM   -> pool host range */
    SMEMB_COPY_GH2L = 5, /* pool host   -> local HBM       */
    SMEMB_COPY_GH2H = 6, /* pool host   -> local host      */
    SMEMB_COPY_H2GH = 7, /* local host  -> pool host range */
    SMEMB_COPY_G2G = 8,  /* pool        -> pool            */
    SMEMB_COPY_AUTO = 9,
    SMEMB_COPY_BUTT
} smem_bm_copy_type;

typedef struct {
    bool tlsEnable;
    char caPath[SMEM_TLS_PATH_SIZE];
    char crlPath[SMEM_TLS_PATH_SIZE];
    char certPath[SMEM_TLS_PATH_SIZE];
    char keyPath[SMEM_TLS_PATH_SIZE];
    char keyPassPath[SMEM_TLS_PATH_SIZE];
    char packagePath[SMEM_TLS_PATH_SIZE];
    char decrypterLibPath[SMEM_TLS_PATH_SIZE];
} smem_tls_config;

typedef struct {
    uint32_t initTimeout;
    uint32_t createTimeout;
    uint32_t controlOperationTimeout;
    bool startConfigStoreServer;
    bool startConfigStoreOnly;
    bool dynamicWorldSize;
    bool unifiedAddressSpace;
    bool autoRanking;
    uint16_t rankId;
    uint32_t flags;
    char hcomUrl[64];
    smem_tls_config hcomTlsConfig;
    smem_tls_config storeTlsConfig;
} smem_bm_config_t;

typedef struct {
    uint64_t maxDramSize;
    uint64_t maxHbmSize;
    uint64_t localDRAMSize;
    uint64_t localHBMSize;
    smem_bm_data_op_type dataOpType;
    uint32_t flags;
    char tag[32];
    char tagOpInfo[256];
    int dramShmFd;
} smem_bm_create_option_t;

typedef struct {
    const void *src;
    void *dest;
    size_t dataSize;
} smem_copy_params;

typedef struct {
    void **sources;
    void **destinations;
    const uint64_t *dataSizes;
    uint32_t batchSize;
} smem_batch_copy_params;

/* ---- return codes --------------------------------------------------------
 * hybm layer: src/hybm/csrc/common/hybm_types.h:22-35
 * smem layer: src/smem/csrc/common/smem_types.h:21-36                        */
enum {
    BM_OK = 0,
    BM_ERROR = -1,
    BM_INVALID_PARAM = -2,
    BM_MALLOC_FAILED = -3,
    BM_NEW_OBJECT_FAILED = -4,
    BM_FILE_NOT_ACCESS = -5,
    BM_DL_FUNCTION_FAILED = -6,
    BM_TIMEOUT = -7,
    BM_UNDER_API_UNLOAD = -8,
    BM_NOT_INITIALIZED = -9,
    BM_NOT_SUPPORT_FUNC = -10,
    BM_NOT_SUPPORTED = -100
};

enum {
    SM_OK = 0,
    SM_ERROR = -1,
    SM_INVALID_PARAM = -2000,
    SM_MALLOC_FAILED = -2001,
    SM_NEW_OBJECT_FAILED = -2002,
    SM_NOT_STARTED = -2003,
    SM_TIMEOUT = -2004,
    SM_REPEAT_CALL = -2005,
    SM_DUPLICATED_OBJECT = -2006,
    SM_OBJECT_NOT_EXISTS = -2007,
    SM_NOT_INITIALIZED = -2008,
    SM_RESOURCE_IN_USE = -2009,
    SM_RECONNECT = -2010,
    SM_GET_OBJIECT = -2011
};

/* ---- smem transfer front-end (src/smem/include/host/smem_trans_def.h:24-48) ---- */
typedef void *smem_trans_t;

typedef enum {
    SMEM_TRANS_NONE = 0,
    SMEM_TRANS_SENDER,
    SMEM_TRANS_RECEIVER,
    SMEM_TRANS_BOTH,
    SMEM_TRANS_BUTT
} smem_trans_role_t;

typedef struct {
    smem_trans_role_t role;          /* sender, receiver or both */
    uint32_t initTimeout;            /* seconds; 120 by default */
    uint32_t deviceId;               /* GPU ordinal */
    uint32_t flags;
    smem_bm_data_op_type dataOpType; /* engines to use; the copy kernels serve SMEMB_DATA_OP_SDMA */
    bool startConfigServer;
} smem_trans_config_t;

#ifdef __cplusplus
}
#endif

#endif /* MF_WITH_REFERENCE_HEADERS */

/* ---- contract pins ------------------------------------------------------ */
#ifdef __cplusplus
#define MF_PIN(expr) static_assert(expr, #expr)
#else
#define MF_PIN(expr) _Static_assert(expr, #expr)
#endif
MF_PIN(HYBM_DOP_TYPE_SDMA == 2 && HYBM_DOP_TYPE_HOST_URMA == 32);
MF_PIN(HYBM_MEM_TYPE_DEVICE == 1 && HYBM_MEM_TYPE_HOST == 2 && HYBM_MEM_TYPE_BUTT == 3);
MF_PIN(HYBM_LOCAL_HOST_TO_GLOBAL_HOST == 0 && HYBM_GLOBAL_HOST_TO_GLOBAL_HOST == 4);
MF_PIN(HYBM_GLOBAL_DEVICE_TO_GLOBAL_DEVICE == 9 && HYBM_GLOBAL_DEVICE_TO_LOCAL_DEVICE == 11);
MF_PIN(HYBM_DATA_COPY_DIRECTION_AUTO == 12 && HYBM_DATA_COPY_DIRECTION_BUTT == 13);
MF_PIN(SMEM_MEM_TYPE_LOCAL_DEVICE == 0 && SMEM_MEM_TYPE_HOST == 3 && SMEM_MEM_TYPE_BUTT == 4);
MF_PIN(SMEMB_DATA_OP_SDMA == 1 && SMEMB_DATA_OP_HOST_RDMA == 2 && SMEMB_DATA_OP_HOST_TCP == 4);
MF_PIN(SMEMB_DATA_OP_DEVICE_RDMA == 8 && SMEMB_DATA_OP_HOST_URMA == 16);
MF_PIN(SMEMB_COPY_L2G == 0 && SMEMB_COPY_G2G == 8 && SMEMB_COPY_AUTO == 9 && SMEMB_COPY_BUTT == 10);
MF_PIN(ASYNC_COPY_FLAG == 1 && COPY_EXTEND_FLAG == 2);
MF_PIN(sizeof(hybm_copy_params) == 24 && offsetof(hybm_copy_params, dataSize) == 16);
MF_PIN(sizeof(hybm_batch_copy_params) == 32 && offsetof(hybm_batch_copy_params, batchSize) == 24);
MF_PIN(sizeof(smem_copy_params) == 24 && sizeof(smem_batch_copy_params) == 32);
MF_PIN(sizeof(hybm_exchange_info) == 516);
MF_PIN(offsetof(hybm_options, maxHBMSize) == 24 && offsetof(hybm_options, scene) == 56);
MF_PIN(offsetof(smem_bm_create_option_t, dataOpType) == 32 && offsetof(smem_bm_create_option_t, tag) == 40);
MF_PIN(SMEM_TRANS_SENDER == 1 && SMEM_TRANS_RECEIVER == 2 && SMEM_TRANS_BOTH == 3 && SMEM_TRANS_BUTT == 4);
MF_PIN(sizeof(smem_trans_config_t) == 24 && offsetof(smem_trans_config_t, dataOpType) == 16);
#if !defined(MF_WITH_REFERENCE_HEADERS) || defined(__cplusplus)
MF_PIN(BM_NOT_INITIALIZED == -9 && BM_NOT_SUPPORTED == -100 && SM_INVALID_PARAM == -2000 && SM_NOT_INITIALIZED == -2008);
#endif
#undef MF_PIN

#endif /* MF_XCOPY_TYPES_H */
