// extern "C" surface of the hybm layer (declared in include/mf_xcopy_api.h).
// Argument validation follows src/hybm/csrc/hybm_data_op_entry.cpp:32-132 and
// src/hybm/csrc/hybm_big_mem_entry.cpp; initialisation follows
// src/hybm/csrc/hybm_entry.cpp:76-161 minus everything that loads vendor
// libraries, since the runtime here is linked, not dlopen'ed.
#include <atomic>
#include <mutex>

#include "../../../include/mf_xcopy_api.h"
#include "../rt/mf_rt.h"
#include "copy_direction.h"
#include "mem_entity.h"
#include "mf_log.h"
#include "va_manager.h"
#include "xcopy_engine.h"

using namespace mf;

#define MF_EXPORT extern "C" __attribute__((visibility("default")))

namespace {

std::mutex g_initLock;
int g_initCount = 0;

bool HipDeviceProbe(uint64_t va)
{
    return mfrt_pointer_kind(reinterpret_cast<const void *>(va)) == MFRT_PTR_DEVICE;
}

}  // namespace

MF_EXPORT int32_t hybm_init(uint16_t deviceId, uint64_t flags)
{
    (void)flags;
    std::lock_guard<std::mutex> guard(g_initLock);
    if (g_initCount > 0) {
        if (mfrt_device_id() != static_cast<int>(deviceId)) {
            MF_FAIL(BM_ERROR, "already initialised on GPU " << mfrt_device_id() << ", not " << deviceId);
        }
        ++g_initCount;
        return BM_OK;
    }
    int ret = XcopyEngine::Instance().Start(static_cast<int>(deviceId));
    if (ret != BM_OK) {
        return ret;
    }
    VaManager::Global().SetDeviceProbe(HipDeviceProbe);
    {
        // the rectangle kernels once, as the engine did with the copy kernels: a kernel's first launch is not capturable
        void *stream = XcopyEngine::Instance().ThreadStream();
        if (stream == nullptr || mfk_copy2d_prelaunch(stream) != 0 || mfrt_stream_sync(stream) != 0) {
            MF_ERROR("the rectangle kernels could not be launched once at start");
        }
    }
    if (mfk_moe_setup() != 0) {
        MF_ERROR("the MoE dispatch could not probe the XCD order and keeps to its token-ordered permute");
    }
    g_initCount = 1;
    return BM_OK;
}

MF_EXPORT void hybm_uninit(void)
{
    std::lock_guard<std::mutex> guard(g_initLock);
    if (g_initCount <= 0) {
        return;
    }
    if (--g_initCount > 0) {
        return;
    }
    EntityRegistry::Instance().Clear();
    VaManager::Global().Clear();
    VaManager::Global().SetDeviceProbe(nullptr);
    XcopyEngine::Instance().Stop();
}

MF_EXPORT const char *hybm_get_error_string(int32_t errCode)
{
    switch (errCode) {
        case BM_OK:
            return "success";
        case BM_ERROR:
            return "error";
        case BM_INVALID_PARAM:
            return "invalid parameter";
        case BM_MALLOC_FAILED:
            return "memory allocation failed";
        case BM_NEW_OBJECT_FAILED:
            return "object creation failed";
        case BM_FILE_NOT_ACCESS:
            return "file not accessible";
        case BM_DL_FUNCTION_FAILED:
            return "runtime library call failed";
        case BM_TIMEOUT:
            return "timeout";
        case BM_UNDER_API_UNLOAD:
            return "runtime library not loaded";
        case BM_NOT_INITIALIZED:
            return "not initialized";
        case BM_NOT_SUPPORT_FUNC:
            return "function not supported";
        case BM_NOT_SUPPORTED:
            return "not supported";
        default:
            return "unknown error";
    }
}

MF_EXPORT void hybm_set_extern_logger(void (*logger)(int level, const char *msg))
{
    SetLogSink(logger);
}

MF_EXPORT int32_t hybm_set_log_level(int level)
{
    return SetLogLevel(level) == 0 ? BM_OK : BM_INVALID_PARAM;
}

MF_EXPORT hybm_entity_t hybm_create_entity(uint16_t id, const hybm_options *options, uint32_t flags)
{
    (void)flags;
    if (options == nullptr || id > kEntityIdMax) {
        MF_ERROR("pool creation with null options or id " << id << " > " << kEntityIdMax);
        return nullptr;
    }
    if (!XcopyEngine::Instance().Started()) {
        MF_ERROR("pool creation before hybm_init");
        return nullptr;
    }
    if (options->rankCount != 1 || options->rankId != 0) {
        SetLastError("this build serves a world of one rank");
        MF_ERROR("pool creation for rank " << options->rankId << " of " << options->rankCount
                                           << ": only a single-rank world is supported");
        return nullptr;
    }
    if (options->maxHBMSize < options->deviceVASpace || options->maxDRAMSize < options->hostVASpace) {
        MF_ERROR("pool creation with a local size above the per-rank window");
        return nullptr;
    }
    int result = BM_OK;
    auto entity = EntityRegistry::Instance().Create(id, *options, result);
    return entity.get();
}

MF_EXPORT void hybm_destroy_entity(hybm_entity_t e, uint32_t flags)
{
    (void)flags;
    if (e != nullptr) {
        (void)EntityRegistry::Instance().Remove(e);
    }
}

MF_EXPORT int32_t hybm_reserve_mem_space(hybm_entity_t e, uint32_t flags)
{
    (void)flags;
    auto entity = EntityRegistry::Instance().FindByPtr(e);
    return entity == nullptr ? BM_INVALID_PARAM : entity->ReserveSpace();
}

MF_EXPORT int32_t hybm_unreserve_mem_space(hybm_entity_t e, uint32_t flags)
{
    (void)flags;
    auto entity = EntityRegistry::Instance().FindByPtr(e);
    return entity == nullptr ? BM_INVALID_PARAM : entity->UnreserveSpace();
}

MF_EXPORT void *hybm_get_memory_ptr(hybm_entity_t e, hybm_mem_type mType)
{
    auto entity = EntityRegistry::Instance().FindByPtr(e);
    return entity == nullptr ? nullptr : entity->WindowBase(mType);
}

MF_EXPORT hybm_mem_slice_t hybm_alloc_local_memory(hybm_entity_t e, hybm_mem_type mType, uint64_t size, uint32_t flags)
{
    (void)flags;
    auto entity = EntityRegistry::Instance().FindByPtr(e);
    return entity == nullptr ? nullptr : entity->AllocLocal(mType, size);
}

MF_EXPORT int32_t hybm_free_local_memory(hybm_entity_t e, hybm_mem_slice_t slice, uint32_t count, uint32_t flags)
{
    (void)count;
    (void)flags;
    auto entity = EntityRegistry::Instance().FindByPtr(e);
    return entity == nullptr ? BM_INVALID_PARAM : entity->FreeLocal(static_cast<LocalSlice *>(slice));
}

MF_EXPORT hybm_mem_slice_t hybm_register_local_memory(hybm_entity_t e, const void *ptr, uint64_t size, uint32_t flags)
{
    (void)flags;
    auto entity = EntityRegistry::Instance().FindByPtr(e);
    if (entity == nullptr) {
        MF_ERROR("hybm_register_local_memory: unknown pool handle");
        return nullptr;
    }
    return entity->RegisterLocal(ptr, size);
}

MF_EXPORT void *hybm_get_slice_va(hybm_entity_t e, hybm_mem_slice_t slice)
{
    auto entity = EntityRegistry::Instance().FindByPtr(e);
    if (entity == nullptr || slice == nullptr) {
        return nullptr;
    }
    return reinterpret_cast<void *>(static_cast<LocalSlice *>(slice)->va);
}

MF_EXPORT int32_t hybm_data_copy(hybm_entity_t e, hybm_copy_params *params, hybm_data_copy_direction direction,
                                 void *stream, uint32_t flags)
{
    if (e == nullptr || params == nullptr || params->src == nullptr || params->dest == nullptr ||
        params->dataSize == 0 || direction >= HYBM_DATA_COPY_DIRECTION_BUTT) {
        MF_FAIL(BM_INVALID_PARAM, "hybm_data_copy: null handle/params/address, zero size or bad direction");
    }
    if (direction == HYBM_DATA_COPY_DIRECTION_AUTO) {
        direction = VaManager::Global().InferDirection(reinterpret_cast<uint64_t>(params->src),
                                                       reinterpret_cast<uint64_t>(params->dest));
        if (direction == HYBM_DATA_COPY_DIRECTION_BUTT) {
            MF_FAIL(BM_INVALID_PARAM, "cannot infer a copy direction: neither address is inside the pool");
        }
    }
    auto entity = EntityRegistry::Instance().FindByPtr(e);
    if (entity == nullptr) {
        MF_FAIL(BM_INVALID_PARAM, "hybm_data_copy: unknown pool handle");
    }
    MemEntity::SubmitScope inFlight(*entity);   // from the range check to the enqueue: a slice being freed waits for it
    bool ok = true;
    if (MustCheckDestination(direction)) {
        ok = entity->CheckAddressInEntity(params->dest, params->dataSize);
    }
    if (MustCheckSource(direction)) {
        ok = ok && entity->CheckAddressInEntity(params->src, params->dataSize);
    }
    if (!ok) {
        MF_FAIL(BM_INVALID_PARAM, "copy range of " << params->dataSize << " bytes leaves the pool, direction " << direction);
    }
    return entity->CopyData(*params, direction, stream, flags);
}

MF_EXPORT int32_t hybm_wait(hybm_entity_t e)
{
    if (e == nullptr) {
        MF_FAIL(BM_INVALID_PARAM, "hybm_wait: null pool handle");
    }
    auto entity = EntityRegistry::Instance().FindByPtr(e);
    if (entity == nullptr) {
        MF_FAIL(BM_INVALID_PARAM, "hybm_wait: unknown pool handle");
    }
    return entity->Wait();
}

MF_EXPORT int32_t hybm_data_batch_copy(hybm_entity_t e, hybm_batch_copy_params *params,
                                       hybm_data_copy_direction direction, void *stream, uint32_t flags)
{
    if (e == nullptr || params == nullptr || params->sources == nullptr || params->destinations == nullptr ||
        params->dataSizes == nullptr || params->batchSize == 0 || direction >= HYBM_DATA_COPY_DIRECTION_BUTT) {
        MF_FAIL(BM_INVALID_PARAM, "hybm_data_batch_copy: null handle/params/array, empty batch or bad direction");
    }
    if (direction == HYBM_DATA_COPY_DIRECTION_AUTO) {
        direction = VaManager::Global().InferDirection(reinterpret_cast<uint64_t>(params->sources[0]),
                                                       reinterpret_cast<uint64_t>(params->destinations[0]));
        if (direction == HYBM_DATA_COPY_DIRECTION_BUTT) {
            MF_FAIL(BM_INVALID_PARAM, "cannot infer a copy direction from element 0");
        }
    }
    // The reference trusts the handle here; a registry lookup costs one map probe and turns a
    // stale handle into an error instead of a crash.
    auto entity = EntityRegistry::Instance().FindByPtr(e);
    if (entity == nullptr) {
        MF_FAIL(BM_INVALID_PARAM, "hybm_data_batch_copy: unknown pool handle");
    }
    MemEntity::SubmitScope inFlight(*entity);   // from the range check to the enqueue: a slice being freed waits for it
    const uint32_t n = params->batchSize;
    uint32_t bad = n;
    if (MustCheckDestination(direction)) {
        bad = entity->FirstOutside(params->destinations, params->dataSizes, n);
    }
    if (bad == n && MustCheckSource(direction)) {
        bad = entity->FirstOutside(params->sources, params->dataSizes, n);
    }
    if (bad == n && MustCheckDestination(direction) && MustCheckSource(direction)) {
        // both sides lie in the pool, and no pool address is null
    } else if (bad == n) {   // sides that are not checked against the pool must at least not be null
        for (uint32_t i = 0; i < n; ++i) {
            if (params->sources[i] == nullptr || params->destinations[i] == nullptr) {
                MF_FAIL(BM_INVALID_PARAM, "batch element " << i << " has a null address");
            }
        }
    } else if (params->sources[bad] == nullptr || params->destinations[bad] == nullptr) {
        MF_FAIL(BM_INVALID_PARAM, "batch element " << bad << " has a null address");
    } else {
        MF_FAIL(BM_INVALID_PARAM, "batch element " << bad << " (" << params->dataSizes[bad]
                                                   << " bytes) leaves the pool, direction " << direction);
    }
    return entity->BatchCopyData(*params, direction, stream, flags);
}
