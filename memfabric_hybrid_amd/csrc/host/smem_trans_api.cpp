// extern "C" surface of the transfer front-end (declared in include/mf_xcopy_api.h).
// Checks, their order and their return codes follow
// src/smem/csrc/smem_trans/smem_trans.cpp:24-375; the entry behind the handle is
// TransEntry.  Registration returns as soon as every object of the process has
// the new memory in its map, so the reference's 8-second wait for the watch
// threads of other ranks (smem_trans.cpp:124,206) has no counterpart.
#include <cstring>
#include <limits>
#include <mutex>

#include "../../../include/mf_xcopy_api.h"
#include "mf_log.h"
#include "trans_entry.h"

using namespace mf;

#define MF_EXPORT extern "C" __attribute__((visibility("default")))

namespace {

std::mutex g_transLock;
bool g_transInited = false;

#define ST_CHECK(cond, code, text)   \
    do {                             \
        if (!(cond)) {               \
            MF_FAIL((code), text);   \
        }                            \
    } while (0)

#define ST_ENTRY_OR_RETURN(handle, entry)                                    \
    auto entry = TransDirectory::Instance().FindByHandle(handle);            \
    if (entry == nullptr) {                                                  \
        MF_FAIL(SM_OBJECT_NOT_EXISTS, "no transfer object behind this handle"); \
    }

bool Inited()
{
    std::lock_guard<std::mutex> guard(g_transLock);
    return g_transInited;
}

int Transfer(smem_trans_t handle, void *localAddrs[], const char *remoteName, void *remoteAddrs[],
             const size_t dataSizes[], uint32_t batchSize, smem_bm_copy_type opcode, void *stream, bool needStream,
             uint32_t flags)
{
    ST_CHECK(Inited(), SM_INVALID_PARAM, "smem trans not initialized yet");
    ST_CHECK(handle != nullptr, SM_INVALID_PARAM, "invalid handle, which is null");
    ST_CHECK(remoteName != nullptr, SM_INVALID_PARAM, "invalid remote unique id, which is null");
    ST_CHECK(!needStream || stream != nullptr, SM_INVALID_PARAM, "invalid stream, which is null");
    ST_ENTRY_OR_RETURN(handle, entry);
    return entry->BatchTransfer(localAddrs, remoteName, remoteAddrs, dataSizes, batchSize, opcode, stream, flags);
}

}  // namespace

MF_EXPORT int32_t smem_trans_config_init(smem_trans_config_t *config)
{
    ST_CHECK(config != nullptr, SM_INVALID_PARAM, "Invalid config");
    config->initTimeout = 120;
    config->role = SMEM_TRANS_SENDER;
    config->deviceId = std::numeric_limits<uint32_t>::max();
    config->flags = 0;
    config->startConfigServer = false;
    return SM_OK;
}

MF_EXPORT int32_t smem_trans_init(const smem_trans_config_t *config)
{
    ST_CHECK(config != nullptr, SM_INVALID_PARAM, "invalid config, which is null");
    std::lock_guard<std::mutex> guard(g_transLock);
    if (g_transInited) {
        return SM_OK;
    }
    const int ret = hybm_init(static_cast<uint16_t>(config->deviceId), config->flags);
    if (ret != 0) {
        MF_FAIL(ret, "hybm core init failed: " << ret);
    }
    g_transInited = true;
    return SM_OK;
}

MF_EXPORT void smem_trans_uninit(uint32_t flags)
{
    (void)flags;
    std::lock_guard<std::mutex> guard(g_transLock);
    if (!g_transInited) {
        return;
    }
    hybm_uninit();
    g_transInited = false;
}

MF_EXPORT smem_trans_t smem_trans_create(const char *storeUrl, const char *uniqueId, const smem_trans_config_t *config)
{
    if (!Inited() || storeUrl == nullptr || uniqueId == nullptr || config == nullptr || std::strlen(storeUrl) == 0 ||
        std::strlen(uniqueId) == 0) {
        SetLastError("smem_trans_create: not initialised, or a null / empty store url, unique id or config");
        MF_ERROR("smem_trans_create: not initialised, or a null / empty store url, unique id or config");
        return nullptr;
    }
    auto entry = std::make_shared<TransEntry>(uniqueId, *config);
    if (entry->Initialize() != SM_OK) {
        return nullptr;
    }
    TransDirectory::Instance().Adopt(entry);
    return entry.get();
}

MF_EXPORT void smem_trans_destroy(smem_trans_t handle, uint32_t flags)
{
    (void)flags;
    if (handle == nullptr) {
        return;
    }
    auto entry = TransDirectory::Instance().Release(handle);
    if (entry == nullptr) {
        SetLastError("not found handle");
        return;
    }
    entry->UnInitialize();
}

MF_EXPORT void *smem_trans_malloc(smem_trans_t handle, size_t capacity)
{
    if (!Inited() || handle == nullptr || capacity == 0) {
        SetLastError("smem_trans_malloc: not initialised, null handle or capacity 0");
        return nullptr;
    }
    auto entry = TransDirectory::Instance().FindByHandle(handle);
    if (entry == nullptr) {
        SetLastError("no transfer object behind this handle");
        return nullptr;
    }
    return entry->MallocHost(capacity);
}

MF_EXPORT int32_t smem_trans_free(smem_trans_t handle, void *address)
{
    ST_CHECK(Inited(), SM_INVALID_PARAM, "smem trans not initialized yet");
    ST_CHECK(handle != nullptr, SM_INVALID_PARAM, "invalid handle, which is null");
    ST_CHECK(address != nullptr, SM_INVALID_PARAM, "invalid address, which is null");
    ST_ENTRY_OR_RETURN(handle, entry);
    return entry->FreeHost(address);
}

MF_EXPORT int32_t smem_trans_register_mem(smem_trans_t handle, void *address, size_t capacity, uint32_t flags)
{
    ST_CHECK(Inited(), SM_INVALID_PARAM, "smem trans not initialized yet");
    ST_CHECK(handle != nullptr, SM_INVALID_PARAM, "invalid handle, which is null");
    ST_CHECK(address != nullptr, SM_INVALID_PARAM, "invalid address, which is null");
    ST_CHECK(capacity != 0, SM_INVALID_PARAM, "invalid capacity, which is 0");
    ST_ENTRY_OR_RETURN(handle, entry);
    return entry->RegisterLocalMemory(address, capacity, flags);
}

MF_EXPORT int32_t smem_trans_batch_register_mem(smem_trans_t handle, void *addresses[], size_t capacities[],
                                                uint32_t count, uint32_t flags)
{
    ST_CHECK(Inited(), SM_INVALID_PARAM, "smem trans not initialized yet");
    ST_CHECK(handle != nullptr, SM_INVALID_PARAM, "invalid handle, which is null");
    ST_CHECK(addresses != nullptr, SM_INVALID_PARAM, "invalid addresses, which is null");
    ST_CHECK(capacities != nullptr, SM_INVALID_PARAM, "invalid capacities, which is null");
    ST_CHECK(count != 0, SM_INVALID_PARAM, "invalid count, which is 0");
    std::vector<std::pair<const void *, size_t>> memories;
    memories.reserve(count);
    for (uint32_t i = 0; i < count; ++i) {
        ST_CHECK(addresses[i] != nullptr, SM_INVALID_PARAM, "invalid address, which is null");
        ST_CHECK(capacities[i] != 0, SM_INVALID_PARAM, "invalid capacity, which is 0");
        memories.emplace_back(addresses[i], capacities[i]);
    }
    ST_ENTRY_OR_RETURN(handle, entry);
    return entry->RegisterLocalMemories(memories, flags);
}

MF_EXPORT int32_t smem_trans_deregister_mem(smem_trans_t handle, void *address)
{
    ST_CHECK(Inited(), SM_INVALID_PARAM, "smem trans not initialized yet");
    ST_CHECK(handle != nullptr, SM_INVALID_PARAM, "invalid handle, which is null");
    ST_CHECK(address != nullptr, SM_INVALID_PARAM, "invalid address, which is null");
    ST_ENTRY_OR_RETURN(handle, entry);
    return entry->DeregisterLocalMemory(address);
}

MF_EXPORT int32_t smem_trans_write(smem_trans_t handle, const void *localAddr, const char *remoteUniqueId,
                                   void *remoteAddr, size_t dataSize, uint32_t flags)
{
    void *local = const_cast<void *>(localAddr);
    return Transfer(handle, &local, remoteUniqueId, &remoteAddr, &dataSize, 1, SMEMB_COPY_L2G, nullptr, false, flags);
}

MF_EXPORT int32_t smem_trans_batch_write(smem_trans_t handle, const void *localAddrs[], const char *remoteUniqueId,
                                         void *remoteAddrs[], size_t dataSizes[], uint32_t batchSize, uint32_t flags)
{
    return Transfer(handle, const_cast<void **>(localAddrs), remoteUniqueId, remoteAddrs, dataSizes, batchSize,
                    SMEMB_COPY_L2G, nullptr, false, flags);
}

MF_EXPORT int32_t smem_trans_read(smem_trans_t handle, void *localAddr, const char *remoteUniqueId,
                                  const void *remoteAddr, size_t dataSize, uint32_t flags)
{
    void *remote = const_cast<void *>(remoteAddr);
    return Transfer(handle, &localAddr, remoteUniqueId, &remote, &dataSize, 1, SMEMB_COPY_G2L, nullptr, false, flags);
}

MF_EXPORT int32_t smem_trans_batch_read(smem_trans_t handle, void *localAddrs[], const char *remoteUniqueId,
                                        const void *remoteAddrs[], size_t dataSizes[], uint32_t batchSize,
                                        uint32_t flags)
{
    return Transfer(handle, localAddrs, remoteUniqueId, const_cast<void **>(remoteAddrs), dataSizes, batchSize,
                    SMEMB_COPY_G2L, nullptr, false, flags);
}

MF_EXPORT int32_t smem_trans_read_submit(smem_trans_t handle, void *localAddr, const char *remoteUniqueId,
                                         const void *remoteAddr, size_t dataSize, void *stream, uint32_t flags)
{
    void *remote = const_cast<void *>(remoteAddr);
    return Transfer(handle, &localAddr, remoteUniqueId, &remote, &dataSize, 1, SMEMB_COPY_G2L, stream, true, flags);
}

MF_EXPORT int32_t smem_trans_write_submit(smem_trans_t handle, const void *localAddr, const char *remoteUniqueId,
                                          void *remoteAddr, size_t dataSize, void *stream, uint32_t flags)
{
    void *local = const_cast<void *>(localAddr);
    return Transfer(handle, &local, remoteUniqueId, &remoteAddr, &dataSize, 1, SMEMB_COPY_L2G, stream, true, flags);
}

MF_EXPORT int32_t smem_trans_batch_read_submit(smem_trans_t handle, void *localAddrs[], const char *remoteUniqueId,
                                               const void *remoteAddrs[], size_t dataSizes[], uint32_t batchSize,
                                               void *stream, uint32_t flags)
{
    return Transfer(handle, localAddrs, remoteUniqueId, const_cast<void **>(remoteAddrs), dataSizes, batchSize,
                    SMEMB_COPY_G2L, stream, true, flags);
}

MF_EXPORT int32_t smem_trans_batch_write_submit(smem_trans_t handle, const void *localAddrs[],
                                                const char *remoteUniqueId, void *remoteAddrs[], size_t dataSizes[],
                                                uint32_t batchSize, void *stream, uint32_t flags)
{
    return Transfer(handle, const_cast<void **>(localAddrs), remoteUniqueId, remoteAddrs, dataSizes, batchSize,
                    SMEMB_COPY_L2G, stream, true, flags);
}
