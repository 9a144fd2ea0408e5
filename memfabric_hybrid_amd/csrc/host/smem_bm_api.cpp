// extern "C" surface of the smem BM layer (declared in include/mf_xcopy_api.h)
// for a world of one rank.  Checks, their order and their return codes follow
// src/smem/csrc/smem_bm/smem_bm.cpp:26-93,120-222,290-380 and
// src/smem/csrc/smem_bm/smem_bm_entry.cpp:256-455; the join/leave exchange,
// the config store and the group engine behind them do not exist here.
#include <cstring>
#include <limits>
#include <map>
#include <memory>
#include <mutex>
#include <shared_mutex>
#include <unordered_map>

#include "../../../include/mf_xcopy_api.h"
#include "copy_direction.h"
#include "gva_layout.h"
#include "mf_log.h"

using namespace mf;

#define MF_EXPORT extern "C" __attribute__((visibility("default")))

namespace {

constexpr uint32_t kDefaultWaitSeconds = 120;
constexpr uint64_t kLocalHbmMax = 64ULL << 30;   // per-rank limits of the reference
constexpr uint64_t kLocalDramMax = 2ULL << 40;   // (src/smem/csrc/common/smem_types.h:55-56)
constexpr uint32_t kBmIdMax = 63;

#define SM_CHECK(cond, code, text)               \
    do {                                         \
        if (!(cond)) {                           \
            MF_FAIL((code), text);               \
        }                                        \
    } while (0)

hybm_data_op_type ToHybmOpTypes(uint32_t smemBits)
{
    uint32_t out = 0;
    if (smemBits & SMEMB_DATA_OP_SDMA) {
        out |= HYBM_DOP_TYPE_SDMA;
    }
    if (smemBits & SMEMB_DATA_OP_DEVICE_RDMA) {
        out |= HYBM_DOP_TYPE_DEVICE_RDMA;
    }
    if (smemBits & SMEMB_DATA_OP_HOST_RDMA) {
        out |= HYBM_DOP_TYPE_HOST_RDMA;
    }
    if (smemBits & SMEMB_DATA_OP_HOST_TCP) {
        out |= HYBM_DOP_TYPE_HOST_TCP;
    }
    if (smemBits & SMEMB_DATA_OP_HOST_URMA) {
        out |= HYBM_DOP_TYPE_HOST_URMA;
    }
    return static_cast<hybm_data_op_type>(out);
}

class BmEntry {
public:
    explicit BmEntry(uint32_t id) : id_(id) {}
    ~BmEntry()
    {
        Release();
    }

    int Initialize(const hybm_options &options)
    {
        if (inited_) {
            return SM_OK;
        }
        entity_ = hybm_create_entity(static_cast<uint16_t>((id_ << 1) + 1U), &options, 0);
        SM_CHECK(entity_ != nullptr, SM_ERROR, "pool entity creation failed");
        if (hybm_reserve_mem_space(entity_, 0) != 0) {
            hybm_destroy_entity(entity_, 0);
            entity_ = nullptr;
            MF_FAIL(SM_ERROR, "pool address space reservation failed");
        }
        if (options.maxHBMSize > 0 &&
            hybm_alloc_local_memory(entity_, HYBM_MEM_TYPE_DEVICE, options.deviceVASpace, 0) == nullptr) {
            Release();
            MF_FAIL(SM_ERROR, "local HBM allocation of " << options.deviceVASpace << " bytes failed");
        }
        if (options.maxDRAMSize > 0 &&
            hybm_alloc_local_memory(entity_, HYBM_MEM_TYPE_HOST, options.hostVASpace, 0) == nullptr) {
            Release();
            MF_FAIL(SM_ERROR, "local DRAM allocation of " << options.hostVASpace << " bytes failed");
        }
        options_ = options;
        host_.base = reinterpret_cast<uint64_t>(hybm_get_memory_ptr(entity_, HYBM_MEM_TYPE_HOST));
        host_.stride = options.maxDRAMSize;
        host_.rankCount = options.rankCount;
        host_.rankSpace = options.hostVASpace;
        device_.base = reinterpret_cast<uint64_t>(hybm_get_memory_ptr(entity_, HYBM_MEM_TYPE_DEVICE));
        device_.stride = options.maxHBMSize;
        device_.rankCount = options.rankCount;
        device_.rankSpace = options.deviceVASpace;
        inited_ = true;
        return SM_OK;
    }

    void Release()
    {
        if (entity_ != nullptr) {
            hybm_destroy_entity(entity_, 0);
            entity_ = nullptr;
        }
        inited_ = false;
    }

    smem_bm_mem_type PoolTypeOf(const void *addr, uint64_t size) const
    {
        const uint64_t a = reinterpret_cast<uint64_t>(addr);
        if (host_.Contains(a, size)) {
            return SMEM_MEM_TYPE_HOST;
        }
        if (device_.Contains(a, size)) {
            return SMEM_MEM_TYPE_DEVICE;
        }
        return SMEM_MEM_TYPE_BUTT;
    }

    int Copy(const void *src, void *dest, uint64_t size, smem_bm_copy_type t, uint32_t flags)
    {
        SM_CHECK(src != nullptr, SM_INVALID_PARAM, "copy source is NULL");
        SM_CHECK(dest != nullptr, SM_INVALID_PARAM, "copy destination is NULL");
        SM_CHECK(size != 0, SM_INVALID_PARAM, "copy size is 0");
        SM_CHECK(t < SMEMB_COPY_BUTT, SM_INVALID_PARAM, "copy type " << t << " is invalid");
        SM_CHECK(inited_, SM_NOT_INITIALIZED, "pool is not initialised");
        hybm_data_copy_direction direction =
            t == SMEMB_COPY_AUTO ? HYBM_DATA_COPY_DIRECTION_AUTO
                                 : TranslateSmemCopy(t, PoolTypeOf(src, size), PoolTypeOf(dest, size));
        SM_CHECK(direction != HYBM_DATA_COPY_DIRECTION_BUTT, SM_INVALID_PARAM,
                 "copy type " << t << " does not fit addresses " << src << " -> " << dest);
        hybm_copy_params p = {const_cast<void *>(src), dest, size};
        return hybm_data_copy(entity_, &p, direction, nullptr, flags);
    }

    int CopyBatch(smem_batch_copy_params *params, smem_bm_copy_type t, uint32_t flags)
    {
        SM_CHECK(params->sources != nullptr, SM_INVALID_PARAM, "batch sources is NULL");
        SM_CHECK(params->destinations != nullptr, SM_INVALID_PARAM, "batch destinations is NULL");
        SM_CHECK(params->batchSize != 0, SM_INVALID_PARAM, "batch is empty");
        SM_CHECK(t < SMEMB_COPY_BUTT, SM_INVALID_PARAM, "copy type " << t << " is invalid");
        SM_CHECK(inited_, SM_NOT_INITIALIZED, "pool is not initialised");
        SM_CHECK(params->dataSizes != nullptr, SM_INVALID_PARAM, "batch dataSizes is NULL");
        // Only element 0 decides the direction; a batch of mixed kinds is a caller error.
        hybm_data_copy_direction direction =
            t == SMEMB_COPY_AUTO
                ? HYBM_DATA_COPY_DIRECTION_AUTO
                : TranslateSmemCopy(t, PoolTypeOf(params->sources[0], params->dataSizes[0]),
                                    PoolTypeOf(params->destinations[0], params->dataSizes[0]));
        SM_CHECK(direction != HYBM_DATA_COPY_DIRECTION_BUTT, SM_INVALID_PARAM,
                 "copy type " << t << " does not fit addresses " << params->sources[0] << " -> "
                              << params->destinations[0]);
        hybm_batch_copy_params p = {params->sources, params->destinations, params->dataSizes, params->batchSize};
        return hybm_data_batch_copy(entity_, &p, direction, nullptr, flags);
    }

    int Wait()
    {
        SM_CHECK(inited_, SM_NOT_INITIALIZED, "pool is not initialised");
        return hybm_wait(entity_);
    }

    uint32_t RankOfGva(const void *gva) const
    {
        const uint64_t a = reinterpret_cast<uint64_t>(gva);
        uint32_t r = host_.RankBySpace(a);
        return r != kNoRank ? r : device_.RankBySpace(a);
    }

    int Join()
    {
        SM_CHECK(inited_, SM_NOT_INITIALIZED, "pool is not initialised");
        joined_ = true;
        return SM_OK;
    }

    int Leave()
    {
        SM_CHECK(inited_, SM_NOT_INITIALIZED, "pool is not initialised");
        joined_ = false;
        return SM_OK;
    }

    const hybm_options &Options() const
    {
        return options_;
    }
    const GvaWindow &Host() const
    {
        return host_;
    }
    const GvaWindow &Device() const
    {
        return device_;
    }
    bool Inited() const
    {
        return inited_;
    }

private:
    uint32_t id_;
    hybm_options options_{};
    hybm_entity_t entity_ = nullptr;
    GvaWindow host_;
    GvaWindow device_;
    bool inited_ = false;
    bool joined_ = false;
};

std::shared_mutex g_lock;
bool g_inited = false;
uint16_t g_deviceId = 0;
std::shared_mutex g_entriesLock;
// Both maps are never destroyed: a pool the caller did not destroy is left to the operating system at
// process exit instead of being torn down (GPU calls included) from a static destructor.
auto &g_entriesById = *new std::map<uint32_t, std::shared_ptr<BmEntry>>();
auto &g_entriesByPtr = *new std::unordered_map<const void *, std::shared_ptr<BmEntry>>();

std::shared_ptr<BmEntry> FindEntry(smem_bm_t handle)
{
    std::shared_lock<std::shared_mutex> guard(g_entriesLock);
    auto it = g_entriesByPtr.find(handle);
    return it == g_entriesByPtr.end() ? nullptr : it->second;
}

bool ConfigValid(const smem_bm_config_t *c)
{
    return c != nullptr && c->unifiedAddressSpace && c->initTimeout != 0 && c->createTimeout != 0 &&
           c->controlOperationTimeout != 0;
}

}  // namespace

MF_EXPORT int32_t smem_bm_config_init(smem_bm_config_t *config)
{
    SM_CHECK(config != nullptr, SM_INVALID_PARAM, "config is NULL");
    std::memset(config, 0, sizeof(*config));
    config->initTimeout = kDefaultWaitSeconds;
    config->createTimeout = kDefaultWaitSeconds;
    config->controlOperationTimeout = kDefaultWaitSeconds;
    config->startConfigStoreServer = true;
    config->unifiedAddressSpace = true;
    config->autoRanking = true;
    config->rankId = std::numeric_limits<uint16_t>::max();
    return SM_OK;
}

MF_EXPORT int32_t smem_bm_init(const char *storeURL, uint32_t worldSize, uint16_t deviceId,
                               const smem_bm_config_t *config)
{
    SM_CHECK(worldSize != 0, SM_INVALID_PARAM, "worldSize is 0");
    SM_CHECK(worldSize <= SMEM_WORLD_SIZE_MAX, SM_INVALID_PARAM, "worldSize is too large");
    SM_CHECK(storeURL != nullptr, SM_INVALID_PARAM, "storeURL is NULL");
    SM_CHECK(ConfigValid(config), SM_INVALID_PARAM, "config is invalid");
    std::unique_lock<std::shared_mutex> guard(g_lock);
    if (g_inited) {
        return SM_OK;
    }
    SM_CHECK(worldSize == 1, SM_ERROR,
             "worldSize " << worldSize << ": this build has no control plane and serves one rank on one GPU");
    int ret = hybm_init(deviceId, config->flags);
    SM_CHECK(ret == 0, SM_ERROR, "GPU data plane start failed: " << ret);
    g_deviceId = deviceId;
    g_inited = true;
    return SM_OK;
}

MF_EXPORT void smem_bm_uninit(uint32_t flags)
{
    (void)flags;
    std::unique_lock<std::shared_mutex> guard(g_lock);
    if (!g_inited) {
        return;
    }
    {
        std::unique_lock<std::shared_mutex> entries(g_entriesLock);
        g_entriesByPtr.clear();
        g_entriesById.clear();  // releases every pool
    }
    hybm_uninit();
    g_inited = false;
}

MF_EXPORT uint32_t smem_bm_get_rank_id(void)
{
    std::shared_lock<std::shared_mutex> guard(g_lock);
    return g_inited ? 0u : UINT32_MAX;
}

MF_EXPORT smem_bm_t smem_bm_create2(uint32_t id, const smem_bm_create_option_t *option)
{
    std::shared_lock<std::shared_mutex> guard(g_lock);
    if (!g_inited) {
        MF_ERROR("smem_bm_create2 before smem_bm_init");
        return nullptr;
    }
    if (option == nullptr || (option->maxDramSize == 0 && option->maxHbmSize == 0) ||
        option->localDRAMSize > kLocalDramMax || option->localHBMSize > kLocalHbmMax ||
        option->maxDramSize < option->localDRAMSize || option->maxHbmSize < option->localHBMSize) {
        MF_ERROR("smem_bm_create2: option is invalid");
        return nullptr;
    }
    constexpr uint32_t kAllOps = SMEMB_DATA_OP_SDMA | SMEMB_DATA_OP_HOST_RDMA | SMEMB_DATA_OP_HOST_URMA |
                                 SMEMB_DATA_OP_HOST_TCP | SMEMB_DATA_OP_DEVICE_RDMA;
    if ((static_cast<uint32_t>(option->dataOpType) & kAllOps) == 0 || id > kBmIdMax) {
        MF_ERROR("smem_bm_create2: no valid data operation type, or id " << id << " > " << kBmIdMax);
        return nullptr;
    }
    if ((option->flags & SMEM_BM_FLAG_CREATE_WITH_SHM) != 0) {
        MF_ERROR("smem_bm_create2: shared-memory-fd backed DRAM pools cannot be mapped to the GPU in this build");
        return nullptr;
    }
    std::shared_ptr<BmEntry> entry;
    {
        std::unique_lock<std::shared_mutex> entries(g_entriesLock);
        if (g_entriesById.count(id) != 0) {
            MF_ERROR("smem_bm_create2: pool id " << id << " exists");
            return nullptr;
        }
        entry = std::make_shared<BmEntry>(id);
        g_entriesById[id] = entry;
        g_entriesByPtr[entry.get()] = entry;
    }
    hybm_options options{};
    options.bmType = HYBM_TYPE_HOST_INITIATE;
    uint32_t memType = 0;
    if (option->maxDramSize != 0) {
        memType |= HYBM_MEM_TYPE_HOST;
    }
    if (option->maxHbmSize != 0) {
        memType |= HYBM_MEM_TYPE_DEVICE;
    }
    options.memType = static_cast<hybm_mem_type>(memType);
    // Whatever transports the caller listed, inside one GPU the copy kernels serve them all.
    options.bmDataOpType =
        static_cast<hybm_data_op_type>(ToHybmOpTypes(option->dataOpType) | static_cast<uint32_t>(HYBM_DOP_TYPE_SDMA));
    options.rankCount = 1;
    options.rankId = 0;
    options.devId = g_deviceId;
    options.maxHBMSize = option->maxHbmSize;
    options.maxDRAMSize = option->maxDramSize;
    options.deviceVASpace = option->localHBMSize;
    options.hostVASpace = option->localDRAMSize;
    options.role = HYBM_ROLE_PEER;
    options.flags = option->flags;
    options.scene = HYBM_SCENE_DEFAULT;
    options.dramShmFd = -1;
    std::memcpy(options.tag, option->tag, sizeof(options.tag));
    std::memcpy(options.tagOpInfo, option->tagOpInfo, sizeof(options.tagOpInfo));
    if (entry->Initialize(options) != SM_OK) {
        std::unique_lock<std::shared_mutex> entries(g_entriesLock);
        g_entriesByPtr.erase(entry.get());
        g_entriesById.erase(id);
        return nullptr;
    }
    return entry.get();
}

MF_EXPORT smem_bm_t smem_bm_create(uint32_t id, uint32_t memberSize, smem_bm_data_op_type dataOpType,
                                   uint64_t localDRAMSize, uint64_t localHBMSize, uint32_t flags)
{
    (void)memberSize;
    smem_bm_create_option_t option{};
    option.maxDramSize = localDRAMSize;
    option.maxHbmSize = localHBMSize;
    option.localDRAMSize = localDRAMSize;
    option.localHBMSize = localHBMSize;
    option.dataOpType = dataOpType;
    option.flags = flags & ~SMEM_BM_FLAG_CREATE_WITH_SHM;
    option.dramShmFd = -1;
    return smem_bm_create2(id, &option);
}

MF_EXPORT void smem_bm_destroy(smem_bm_t handle)
{
    if (handle == nullptr) {
        return;
    }
    std::shared_lock<std::shared_mutex> guard(g_lock);
    if (!g_inited) {
        return;
    }
    std::shared_ptr<BmEntry> entry;
    {
        std::unique_lock<std::shared_mutex> entries(g_entriesLock);
        auto it = g_entriesByPtr.find(handle);
        if (it == g_entriesByPtr.end()) {
            return;
        }
        entry = it->second;
        for (auto e = g_entriesById.begin(); e != g_entriesById.end(); ++e) {
            if (e->second == entry) {
                g_entriesById.erase(e);
                break;
            }
        }
        g_entriesByPtr.erase(it);
    }
    if (entry != nullptr) {
        entry->Release();
    }
}

// Shared prologue of every per-handle call: NULL handle -> INVALID_PARAM, library not
// initialised -> NOT_INITIALIZED, unknown handle -> INVALID_PARAM (in that order).
#define SM_ENTRY_OR_RETURN(handle, entry)                                             \
    SM_CHECK((handle) != nullptr, SM_INVALID_PARAM, "handle is NULL");                \
    std::shared_lock<std::shared_mutex> smGuard_(g_lock);                             \
    SM_CHECK(g_inited, SM_NOT_INITIALIZED, "smem bm not initialized yet");            \
    std::shared_ptr<BmEntry> entry = FindEntry(handle);                               \
    SM_CHECK((entry) != nullptr, SM_INVALID_PARAM, "handle is not a live pool")

MF_EXPORT int32_t smem_bm_join(smem_bm_t handle, uint32_t flags)
{
    (void)flags;
    SM_ENTRY_OR_RETURN(handle, entry);
    return entry->Join();
}

MF_EXPORT int32_t smem_bm_leave(smem_bm_t handle, uint32_t flags)
{
    (void)flags;
    SM_ENTRY_OR_RETURN(handle, entry);
    return entry->Leave();
}

MF_EXPORT uint64_t smem_bm_get_local_mem_size_by_mem_type(smem_bm_t handle, smem_bm_mem_type memType)
{
    if (handle == nullptr) {
        return 0;
    }
    std::shared_ptr<BmEntry> entry = FindEntry(handle);
    if (entry == nullptr) {
        return 0;
    }
    switch (memType) {
        case SMEM_MEM_TYPE_DEVICE:
            return entry->Options().deviceVASpace;
        case SMEM_MEM_TYPE_HOST:
            return entry->Options().hostVASpace;
        default:
            return 0;
    }
}

MF_EXPORT void *smem_bm_ptr_by_mem_type(smem_bm_t handle, smem_bm_mem_type memType, uint16_t peerRankId)
{
    if (handle == nullptr) {
        return nullptr;
    }
    std::shared_lock<std::shared_mutex> guard(g_lock);
    if (!g_inited) {
        return nullptr;
    }
    std::shared_ptr<BmEntry> entry = FindEntry(handle);
    if (entry == nullptr || peerRankId >= entry->Options().rankCount) {
        return nullptr;
    }
    switch (memType) {
        case SMEM_MEM_TYPE_DEVICE:
            return entry->Device().base == 0 ? nullptr : reinterpret_cast<void *>(entry->Device().PtrOfRank(peerRankId));
        case SMEM_MEM_TYPE_HOST:
            return entry->Host().base == 0 ? nullptr : reinterpret_cast<void *>(entry->Host().PtrOfRank(peerRankId));
        default:
            return nullptr;
    }
}

MF_EXPORT int32_t smem_bm_copy(smem_bm_t handle, smem_copy_params *params, smem_bm_copy_type t, uint32_t flags)
{
    SM_CHECK(handle != nullptr, SM_INVALID_PARAM, "handle is NULL");
    SM_CHECK(params != nullptr, SM_INVALID_PARAM, "params is NULL");
    SM_ENTRY_OR_RETURN(handle, entry);
    return entry->Copy(params->src, params->dest, params->dataSize, t, flags);
}

MF_EXPORT int32_t smem_bm_copy_batch(smem_bm_t handle, smem_batch_copy_params *params, smem_bm_copy_type t,
                                     uint32_t flags)
{
    SM_CHECK(handle != nullptr, SM_INVALID_PARAM, "handle is NULL");
    SM_CHECK(params != nullptr, SM_INVALID_PARAM, "params is NULL");
    SM_ENTRY_OR_RETURN(handle, entry);
    return entry->CopyBatch(params, t, flags);
}

MF_EXPORT int32_t smem_bm_wait(smem_bm_t handle)
{
    SM_ENTRY_OR_RETURN(handle, entry);
    return entry->Wait();
}

MF_EXPORT uint32_t smem_bm_get_rank_id_by_gva(smem_bm_t handle, void *gva)
{
    SM_ENTRY_OR_RETURN(handle, entry);
    return entry->RankOfGva(gva);
}

MF_EXPORT int32_t smem_bm_register_user_mem(smem_bm_t handle, uint64_t addr, uint64_t size)
{
    (void)size;
    SM_CHECK(handle != nullptr, SM_INVALID_PARAM, "handle is NULL");
    SM_CHECK(addr != 0, SM_INVALID_PARAM, "addr is 0");
    SM_ENTRY_OR_RETURN(handle, entry);
    // Device memory and pinned host memory are already addressable by the copy kernels; ordinary
    // host memory cannot be pinned after the fact on this platform and goes through staging.
    return SM_OK;
}

MF_EXPORT int32_t smem_bm_unregister_user_mem(smem_bm_t handle, uint64_t addr)
{
    SM_CHECK(handle != nullptr, SM_INVALID_PARAM, "handle is NULL");
    SM_CHECK(addr != 0, SM_INVALID_PARAM, "addr is 0");
    SM_ENTRY_OR_RETURN(handle, entry);
    return SM_OK;
}

MF_EXPORT int32_t smem_set_extern_logger(void (*func)(int level, const char *msg))
{
    SetLogSink(func);
    return SM_OK;
}

MF_EXPORT int32_t smem_set_log_level(int level)
{
    return SetLogLevel(level) == 0 ? SM_OK : SM_INVALID_PARAM;
}

MF_EXPORT const char *smem_get_last_err_msg(void)
{
    return LastError();
}
