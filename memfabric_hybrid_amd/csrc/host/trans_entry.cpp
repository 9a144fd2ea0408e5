#include "trans_entry.h"

#include <arpa/inet.h>

#include <algorithm>
#include <cstring>
#include <limits>

#include "../rt/mf_rt.h"
#include "copy_direction.h"
#include "mem_entity.h"
#include "mf_log.h"

namespace mf {

namespace {

constexpr uint16_t kTransEntityFirst = (16U << 3U) + 1U;   // the reference's transfer entity id
constexpr long kLowestPort = 1024;                        // ports up to this one are refused

bool ParsePort(const std::string &text, long low, uint16_t &port)
{
    if (text.empty() || text.size() > 5) {
        return false;
    }
    long value = 0;
    for (char c : text) {
        if (c < '0' || c > '9') {
            return false;
        }
        value = value * 10 + (c - '0');
    }
    if (value <= low || value > std::numeric_limits<uint16_t>::max()) {
        return false;
    }
    port = static_cast<uint16_t>(value);
    return true;
}

}  // namespace

size_t WorkerKeyHash::operator()(const WorkerKey &k) const
{
    uint64_t h = 0xcbf29ce484222325ull;   // FNV-1a over the 20 bytes
    for (uint8_t b : k) {
        h = (h ^ b) * 0x100000001b3ull;
    }
    return static_cast<size_t>(h);
}

bool ParseWorkerName(const std::string &name, WorkerKey &key)
{
    key.fill(0);
    uint16_t port = 0;
    if (!name.empty() && name[0] == '[') {
        const size_t close = name.find(']');
        if (close == std::string::npos || close + 1 >= name.size() || name[close + 1] != ':') {
            return false;
        }
        in6_addr v6{};
        if (inet_pton(AF_INET6, name.substr(1, close - 1).c_str(), &v6) != 1 ||
            !ParsePort(name.substr(close + 2), 0, port)) {
            return false;
        }
        key[0] = 6;
        std::memcpy(&key[1], v6.s6_addr, 16);
    } else {
        const size_t colon = name.rfind(':');
        if (colon == std::string::npos || colon == 0 || colon > 15) {
            return false;
        }
        in_addr v4{};
        if (inet_pton(AF_INET, name.substr(0, colon).c_str(), &v4) != 1 || v4.s_addr == 0 ||
            !ParsePort(name.substr(colon + 1), kLowestPort, port)) {
            return false;
        }
        key[0] = 4;
        std::memcpy(&key[1], &v4.s_addr, 4);
    }
    key[17] = static_cast<uint8_t>(port >> 8);
    key[18] = static_cast<uint8_t>(port & 0xff);
    return true;
}

std::vector<std::pair<uint64_t, uint64_t>> CombineRanges(std::vector<std::pair<uint64_t, uint64_t>> input)
{
    std::sort(input.begin(), input.end());
    std::vector<std::pair<uint64_t, uint64_t>> runs;
    for (const auto &r : input) {
        if (!runs.empty() && r.first - runs.back().first <= runs.back().second) {
            // starts inside the current run or right at its end: extend it if it reaches further
            const uint64_t reach = r.first - runs.back().first + r.second;
            if (reach >= r.second) {   // no wrap-around
                runs.back().second = std::max(runs.back().second, reach);
                continue;
            }
        }
        runs.push_back(r);
    }
    return runs;
}

int TranslatePeerAddress(const PeerSliceMap &slices, uint64_t remote, uint64_t size, uint64_t &mapped,
                         hybm_mem_type &type)
{
    auto pos = slices.lower_bound(remote);
    if (pos == slices.end()) {
        return SM_INVALID_PARAM;
    }
    const uint64_t offset = remote - pos->first;
    if (offset > pos->second.size || size > pos->second.size - offset) {
        return SM_INVALID_PARAM;
    }
    mapped = pos->second.mapped + offset;
    type = pos->second.type;
    return mapped == 0 ? SM_INVALID_PARAM : SM_OK;
}

// ---- directory ---------------------------------------------------------------------------------

TransDirectory &TransDirectory::Instance()
{
    static TransDirectory *directory = new TransDirectory();   // never destroyed, like the entity registry it refers to
    return *directory;
}

bool TransDirectory::Interested(const TransEntry &watcher, const TransEntry &owner)
{
    // A sender addresses receivers' memory and a receiver senders'
    // (src/smem/csrc/smem_trans/smem_trans_store_helper.cpp:32-38); an object with both roles
    // sees everyone and is seen by everyone, itself included.
    const smem_trans_role_t w = watcher.Role();
    const smem_trans_role_t o = owner.Role();
    if (w == SMEM_TRANS_BOTH || o == SMEM_TRANS_BOTH) {
        return true;
    }
    return (w == SMEM_TRANS_SENDER && o == SMEM_TRANS_RECEIVER) || (w == SMEM_TRANS_RECEIVER && o == SMEM_TRANS_SENDER);
}

int TransDirectory::Join(TransEntry *entry)
{
    std::lock_guard<std::mutex> guard(lock_);
    if (!members_.emplace(entry->Key(), entry).second) {
        return SM_DUPLICATED_OBJECT;
    }
    published_[entry];
    for (auto &other : published_) {
        if (other.first == entry || !Interested(*entry, *other.first)) {
            continue;
        }
        for (const Published &p : other.second) {
            entry->ImportSlice(other.first->Key(), p.base, p.slice);
        }
    }
    return SM_OK;
}

void TransDirectory::Leave(TransEntry *entry)
{
    std::lock_guard<std::mutex> guard(lock_);
    auto mine = published_.find(entry);
    if (mine == published_.end()) {
        return;
    }
    for (auto &member : members_) {
        if (!Interested(*member.second, *entry)) {
            continue;
        }
        for (const Published &p : mine->second) {
            member.second->DropSlice(entry->Key(), p.base);
        }
    }
    published_.erase(mine);
    members_.erase(entry->Key());
}

void TransDirectory::Publish(TransEntry *owner, uint64_t base, const PeerSlice &slice)
{
    std::lock_guard<std::mutex> guard(lock_);
    auto mine = published_.find(owner);
    if (mine == published_.end()) {
        return;
    }
    mine->second.push_back(Published{base, slice});
    for (auto &member : members_) {
        if (Interested(*member.second, *owner)) {
            member.second->ImportSlice(owner->Key(), base, slice);
        }
    }
}

void TransDirectory::Withdraw(TransEntry *owner, uint64_t base)
{
    std::lock_guard<std::mutex> guard(lock_);
    auto mine = published_.find(owner);
    if (mine == published_.end()) {
        return;
    }
    auto &list = mine->second;
    auto it = std::find_if(list.begin(), list.end(), [base](const Published &p) { return p.base == base; });
    if (it == list.end()) {
        return;
    }
    list.erase(it);
    for (auto &member : members_) {
        if (Interested(*member.second, *owner)) {
            member.second->DropSlice(owner->Key(), base);
        }
    }
}

std::shared_ptr<TransEntry> TransDirectory::FindByHandle(const void *handle)
{
    std::shared_lock<std::shared_mutex> guard(handleLock_);
    auto it = handles_.find(handle);
    return it == handles_.end() ? nullptr : it->second;
}

void TransDirectory::Adopt(std::shared_ptr<TransEntry> entry)
{
    std::unique_lock<std::shared_mutex> guard(handleLock_);
    const void *handle = entry.get();
    handles_[handle] = std::move(entry);
}

std::shared_ptr<TransEntry> TransDirectory::Release(const void *handle)
{
    std::unique_lock<std::shared_mutex> guard(handleLock_);
    auto it = handles_.find(handle);
    if (it == handles_.end()) {
        return nullptr;
    }
    auto entry = std::move(it->second);
    handles_.erase(it);
    return entry;
}

uint16_t TransDirectory::NextEntityId()
{
    std::lock_guard<std::mutex> guard(lock_);
    // Ids from the reference's transfer id upwards, wrapping inside the valid id range; an id
    // still in use makes entity creation fail and the caller tries the next one.
    const uint16_t span = static_cast<uint16_t>(kEntityIdMax - kTransEntityFirst + 1);
    const uint16_t id = static_cast<uint16_t>(kTransEntityFirst + nextEntityId_ % span);
    nextEntityId_ = static_cast<uint16_t>((nextEntityId_ + 1) % span);
    return id;
}

// ---- entry -------------------------------------------------------------------------------------

TransEntry::TransEntry(std::string name, const smem_trans_config_t &config) : name_(std::move(name)), config_(config) {}

TransEntry::~TransEntry()
{
    UnInitialize();
}

int TransEntry::Initialize()
{
    if (!ParseWorkerName(name_, key_)) {
        MF_FAIL(SM_INVALID_PARAM, "transfer name '" << name_ << "' is not ip:port (port above 1024) or [ipv6]:port");
    }
    if (config_.role != SMEM_TRANS_SENDER && config_.role != SMEM_TRANS_RECEIVER && config_.role != SMEM_TRANS_BOTH) {
        MF_FAIL(SM_INVALID_PARAM, "transfer role " << config_.role << " is neither sender, receiver nor both");
    }
    hybm_options options{};
    options.bmType = HYBM_TYPE_HOST_INITIATE;
    options.memType = static_cast<hybm_mem_type>(HYBM_MEM_TYPE_DEVICE | HYBM_MEM_TYPE_HOST);
    // Inside one GPU the copy kernels are the engine whatever transports the caller listed.
    options.bmDataOpType = HYBM_DOP_TYPE_SDMA;
    options.rankCount = 1;
    options.rankId = 0;
    options.devId = static_cast<uint16_t>(mfrt_device_id() < 0 ? 0 : mfrt_device_id());
    options.scene = HYBM_SCENE_TRANS;
    options.role = config_.role == SMEM_TRANS_SENDER ? HYBM_ROLE_SENDER : HYBM_ROLE_RECEIVER;
    options.dramShmFd = -1;
    for (uint32_t attempt = 0; attempt < 64 && entity_ == nullptr; ++attempt) {
        const uint16_t id = TransDirectory::Instance().NextEntityId();
        if (EntityRegistry::Instance().FindById(id) == nullptr) {
            entity_ = hybm_create_entity(id, &options, 0);
        }
    }
    if (entity_ == nullptr) {
        MF_FAIL(SM_ERROR, "no entity could be created for transfer object '" << name_ << "'");
    }
    const int ret = TransDirectory::Instance().Join(this);
    if (ret != SM_OK) {
        hybm_destroy_entity(entity_, 0);
        entity_ = nullptr;
        MF_FAIL(ret, "a transfer object named '" << name_ << "' exists already");
    }
    joined_ = true;
    return SM_OK;
}

void TransEntry::UnInitialize()
{
    if (joined_) {
        TransDirectory::Instance().Leave(this);
        joined_ = false;
    }
    if (entity_ != nullptr) {
        hybm_destroy_entity(entity_, 0);   // waits for copies in flight, frees what smem_trans_malloc gave out
        entity_ = nullptr;
    }
    std::lock_guard<std::mutex> guard(localLock_);
    local_.clear();
}

int TransEntry::RegisterOne(uint64_t base, uint64_t size)
{
    hybm_mem_slice_t slice = nullptr;
    hybm_mem_type type = HYBM_MEM_TYPE_BUTT;
    {
        std::lock_guard<std::mutex> guard(localLock_);
        auto next = local_.upper_bound(base);
        if (next != local_.begin()) {
            auto prev = std::prev(next);
            if (prev->first == base && prev->second.size == size) {
                return SM_OK;   // the same run once more
            }
            if (prev->first + prev->second.size > base) {
                MF_FAIL(SM_INVALID_PARAM, "registration overlaps memory registered before");
            }
        }
        if (next != local_.end() && base + size > next->first) {
            MF_FAIL(SM_INVALID_PARAM, "registration overlaps memory registered before");
        }
        slice = hybm_register_local_memory(entity_, reinterpret_cast<const void *>(base), size, 0);
        if (slice == nullptr) {
            MF_FAIL(SM_ERROR, "registration of " << size << " bytes failed: the memory must be HBM or pinned host memory");
        }
        type = static_cast<LocalSlice *>(slice)->memType;
        local_[base] = LocalReg{slice, size, false};
    }
    TransDirectory::Instance().Publish(this, base, PeerSlice{base, size, type});
    return SM_OK;
}

int TransEntry::RegisterLocalMemory(const void *address, uint64_t size, uint32_t flags)
{
    (void)flags;
    if (entity_ == nullptr) {
        MF_FAIL(SM_ERROR, "transfer object has no entity");
    }
    if (address == nullptr || size == 0) {
        MF_FAIL(SM_INVALID_PARAM, "registration needs an address and a size");
    }
    return RegisterOne(reinterpret_cast<uint64_t>(address), size);
}

int TransEntry::RegisterLocalMemories(const std::vector<std::pair<const void *, size_t>> &memories, uint32_t flags)
{
    (void)flags;
    if (entity_ == nullptr) {
        MF_FAIL(SM_ERROR, "transfer object has no entity");
    }
    if (memories.empty()) {
        return SM_OK;
    }
    std::vector<std::pair<uint64_t, uint64_t>> ranges;
    ranges.reserve(memories.size());
    for (const auto &m : memories) {
        if (m.first == nullptr || m.second == 0) {
            MF_FAIL(SM_INVALID_PARAM, "registration needs an address and a size for every element");
        }
        ranges.emplace_back(reinterpret_cast<uint64_t>(m.first), static_cast<uint64_t>(m.second));
    }
    for (const auto &run : CombineRanges(std::move(ranges))) {
        const int ret = RegisterOne(run.first, run.second);
        if (ret != SM_OK) {
            return ret;
        }
    }
    return SM_OK;
}

int TransEntry::DeregisterLocalMemory(const void *address)
{
    const uint64_t base = reinterpret_cast<uint64_t>(address);
    LocalReg reg{};
    {
        std::lock_guard<std::mutex> guard(localLock_);
        auto it = local_.find(base);
        if (it == local_.end() || it->second.allocated) {
            return SM_OK;   // nothing registered under this address: as harmless as in the reference
        }
        reg = it->second;
        local_.erase(it);
    }
    TransDirectory::Instance().Withdraw(this, base);
    (void)hybm_free_local_memory(entity_, reg.slice, 1, 0);
    return SM_OK;
}

void *TransEntry::MallocHost(uint64_t size)
{
    if (size == 0 || size > kTransHostMax) {
        MF_ERROR("transfer allocation of " << size << " bytes: the size must be 1.." << kTransHostMax);
        return nullptr;
    }
    hybm_mem_slice_t slice = hybm_alloc_local_memory(entity_, HYBM_MEM_TYPE_HOST, size, 0);
    if (slice == nullptr) {
        return nullptr;
    }
    auto *ls = static_cast<LocalSlice *>(slice);
    {
        std::lock_guard<std::mutex> guard(localLock_);
        local_[ls->va] = LocalReg{slice, ls->size, true};
    }
    TransDirectory::Instance().Publish(this, ls->va, PeerSlice{ls->va, ls->size, HYBM_MEM_TYPE_HOST});
    return reinterpret_cast<void *>(ls->va);
}

int TransEntry::FreeHost(void *address)
{
    if (address == nullptr) {
        MF_FAIL(SM_INVALID_PARAM, "free of a null address");
    }
    const uint64_t base = reinterpret_cast<uint64_t>(address);
    LocalReg reg{};
    {
        std::lock_guard<std::mutex> guard(localLock_);
        auto it = local_.find(base);
        if (it == local_.end() || !it->second.allocated) {
            MF_FAIL(SM_ERROR, "free of " << address << ": not an address smem_trans_malloc returned");
        }
        reg = it->second;
        local_.erase(it);
    }
    TransDirectory::Instance().Withdraw(this, base);
    return hybm_free_local_memory(entity_, reg.slice, 0, 0);
}

void TransEntry::ImportSlice(const WorkerKey &owner, uint64_t base, const PeerSlice &slice)
{
    auto entity = EntityRegistry::Instance().FindByPtr(entity_);
    if (entity == nullptr) {
        return;
    }
    std::unique_lock<std::shared_mutex> guard(peerLock_);
    auto inserted = peers_[owner].emplace(base, slice);
    if (inserted.second) {
        (void)entity->AddRange(slice.mapped, slice.size, slice.type);
    }
}

void TransEntry::DropSlice(const WorkerKey &owner, uint64_t base)
{
    auto entity = EntityRegistry::Instance().FindByPtr(entity_);
    std::unique_lock<std::shared_mutex> guard(peerLock_);
    auto peer = peers_.find(owner);
    if (peer == peers_.end()) {
        return;
    }
    auto it = peer->second.find(base);
    if (it == peer->second.end()) {
        return;
    }
    if (entity != nullptr) {
        (void)entity->RemoveRange(it->second.mapped);
    }
    peer->second.erase(it);
    if (peer->second.empty()) {
        peers_.erase(peer);
    }
}

int TransEntry::BatchTransfer(void *localAddrs[], const char *remoteName, void *remoteAddrs[], const size_t dataSizes[],
                              uint32_t batchSize, smem_bm_copy_type opcode, void *stream, uint32_t flags)
{
    // Checks and their order: smem_trans_entry.cpp:311-322.
    if (localAddrs == nullptr || remoteAddrs == nullptr || dataSizes == nullptr || batchSize == 0 ||
        !(flags == 0 || flags == COPY_EXTEND_FLAG)) {
        MF_FAIL(SM_INVALID_PARAM, "transfer needs address arrays, sizes, a batch size and flags 0 or COPY_EXTEND_FLAG");
    }
    if (opcode != SMEMB_COPY_L2G && opcode != SMEMB_COPY_G2L) {
        MF_FAIL(SM_INVALID_PARAM, "transfer opcode " << opcode << " is neither write (L2G) nor read (G2L)");
    }
    for (uint32_t i = 0; i < batchSize; ++i) {
        if (localAddrs[i] == nullptr || remoteAddrs[i] == nullptr || dataSizes[i] == 0) {
            MF_FAIL(SM_INVALID_PARAM, "transfer element " << i << " has a null address or size 0");
        }
    }
    // The peer's name in binary form; the last name of this thread is remembered.
    thread_local std::string lastName;
    thread_local WorkerKey lastKey;
    if (lastName.empty() || lastName != remoteName) {
        WorkerKey key;
        if (!ParseWorkerName(remoteName, key)) {
            MF_FAIL(SM_ERROR, "peer name '" << remoteName << "' is not ip:port or [ipv6]:port");
        }
        lastName = remoteName;
        lastKey = key;
    }
    thread_local std::vector<void *> mapped;
    mapped.resize(batchSize);
    hybm_mem_type peerType = HYBM_MEM_TYPE_BUTT;
    {
        std::shared_lock<std::shared_mutex> guard(peerLock_);
        auto peer = peers_.find(lastKey);
        if (peer == peers_.end()) {
            MF_FAIL(SM_INVALID_PARAM, "peer '" << remoteName << "' has registered no memory this object can reach");
        }
        const PeerSliceMap &slices = peer->second;
        // Consecutive elements mostly fall into the run of the one before: try that first.
        uint64_t runBase = 0;
        uint64_t runSize = 0;
        uint64_t runMapped = 0;
        hybm_mem_type runType = HYBM_MEM_TYPE_BUTT;
        for (uint32_t i = 0; i < batchSize; ++i) {
            const uint64_t remote = reinterpret_cast<uint64_t>(remoteAddrs[i]);
            const uint64_t size = dataSizes[i];
            if (!(remote >= runBase && remote - runBase <= runSize && size <= runSize - (remote - runBase))) {
                auto pos = slices.lower_bound(remote);   // greatest start <= remote
                if (pos == slices.end() || remote - pos->first > pos->second.size ||
                    size > pos->second.size - (remote - pos->first) || pos->second.mapped == 0) {
                    MF_FAIL(SM_INVALID_PARAM, "element " << i << ": [" << remoteAddrs[i] << ", +" << size
                                                         << ") is not inside memory '" << remoteName << "' registered");
                }
                runBase = pos->first;
                runSize = pos->second.size;
                runMapped = pos->second.mapped;
                runType = pos->second.type;
            }
            const uint64_t target = runMapped + (remote - runBase);
            if (i == 0) {
                peerType = runType;
            }
            mapped[i] = reinterpret_cast<void *>(target);
        }
    }
    // The direction says what the memory is, taken from element 0 as everywhere in this API:
    // the peer's side from its registration, the local side from the address itself.
    const int localKind = mfrt_pointer_kind(localAddrs[0]);
    const Endpoint local{false, localKind == MFRT_PTR_DEVICE};
    const Endpoint peer{true, peerType == HYBM_MEM_TYPE_DEVICE};
    const bool write = opcode == SMEMB_COPY_L2G;
    const hybm_data_copy_direction direction = write ? ComposeDirection(local, peer) : ComposeDirection(peer, local);
    const uint32_t copyFlags = flags | (stream != nullptr ? ASYNC_COPY_FLAG : 0);
    hybm_batch_copy_params params{};
    params.sources = write ? localAddrs : mapped.data();
    params.destinations = write ? mapped.data() : localAddrs;
    params.dataSizes = reinterpret_cast<const uint64_t *>(dataSizes);
    params.batchSize = batchSize;
    const int ret = hybm_data_batch_copy(entity_, &params, direction, stream, copyFlags);
    if (ret != 0) {
        MF_ERROR("batch transfer of " << batchSize << " elements failed: " << ret);
    }
    return ret;
}

}  // namespace mf
