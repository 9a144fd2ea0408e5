#include "va_manager.h"

#include <mutex>

#include "copy_direction.h"
#include "mf_log.h"

namespace mf {
namespace {

bool LegacyWindowProbe(uint64_t va)
{
    return va >= kLegacyDeviceVaStart && va < kLegacyDeviceVaStart + kLegacyDeviceVaSize;
}

// Entry with the greatest key <= va, or nullptr.
template <class Map>
const typename Map::mapped_type *Floor(const Map &m, uint64_t va)
{
    auto it = m.upper_bound(va);
    if (it == m.begin()) {
        return nullptr;
    }
    --it;
    return &it->second;
}

}  // namespace

VaManager &VaManager::Global()
{
    static VaManager *manager = new VaManager();   // never destroyed: entities that outlive main() may still refer to it
    return *manager;
}

void VaManager::SetDeviceProbe(DeviceProbe probe)
{
    std::unique_lock<std::shared_mutex> guard(lock_);
    probe_ = probe;
}

const VaRange *VaManager::LookupGva(uint64_t va) const
{
    const VaRange *r = Floor(byGva_, va);
    return (r != nullptr && r->HoldsGva(va)) ? r : nullptr;
}

const VaRange *VaManager::LookupLva(uint64_t va) const
{
    const VaRange *r = Floor(byLva_, va);
    return (r != nullptr && r->HoldsLva(va)) ? r : nullptr;
}

int VaManager::Add(const VaRange &range)
{
    if (range.gva == 0) {
        MF_ERROR("address range without a global address rejected, size=" << range.size);
        return BM_ERROR;
    }
    if (range.size == 0) {
        return BM_OK;  // nothing to track
    }
    if (range.memType >= HYBM_MEM_TYPE_BUTT) {
        MF_ERROR("address range with memory type " << range.memType << " rejected");
        return BM_ERROR;
    }
    std::unique_lock<std::shared_mutex> guard(lock_);
    const uint64_t end = range.gva + range.size;
    for (const auto &kv : byGva_) {
        const VaRange &old = kv.second;
        if (old.memType != range.memType) {
            continue;  // ranges of different memory types are checked independently
        }
        const bool startsInside = range.gva >= old.gva && range.gva < old.gva + old.size;
        const bool coversStart = range.gva <= old.gva && end > old.gva;
        if (startsInside || coversStart) {
            if (old.SameAs(range)) {
                return BM_OK;  // re-adding the identical range is a no-op
            }
            MF_ERROR("address range 0x" << std::hex << range.gva << "+0x" << range.size << " overlaps 0x" << old.gva);
            return BM_ERROR;
        }
    }
    byGva_[range.gva] = range;
    byLva_[range.lva] = range;
    return BM_OK;
}

int VaManager::AddOwn(uint64_t gva, uint64_t size, hybm_mem_type t, uint64_t lva, uint32_t localRank)
{
    VaRange r;
    r.gva = gva;
    r.size = size;
    r.memType = t;
    r.lva = lva;
    r.localRank = localRank;
    return Add(r);
}

int VaManager::AddExternal(uint64_t gva, uint64_t size, hybm_mem_type t, uint64_t lva, uint32_t localRank,
                           uint32_t importedRank)
{
    VaRange r;
    r.gva = gva;
    r.size = size;
    r.memType = t;
    r.lva = lva;
    r.localRank = localRank;
    r.importedRank = importedRank;
    r.registered = importedRank == kNoRank;
    return Add(r);
}

void VaManager::Remove(uint64_t va)
{
    uint64_t gva = va;
    if (!IsGva(va)) {
        gva = GvaOfLva(va);
    }
    if (gva == 0) {
        return;
    }
    std::unique_lock<std::shared_mutex> guard(lock_);
    auto it = byGva_.find(gva);
    if (it == byGva_.end()) {
        return;  // only the first address of a range removes it
    }
    auto lv = byLva_.find(it->second.lva);
    if (lv != byLva_.end() && lv->second.gva == gva) {
        byLva_.erase(lv);
    }
    byGva_.erase(it);
}

void VaManager::Clear()
{
    std::unique_lock<std::shared_mutex> guard(lock_);
    byGva_.clear();
    byLva_.clear();
    reserved_.clear();
}

uint64_t VaManager::GvaOfLva(uint64_t lva) const
{
    if (lva == 0) {
        return 0;
    }
    std::shared_lock<std::shared_mutex> guard(lock_);
    const VaRange *r = LookupLva(lva);
    return r == nullptr ? 0 : r->gva + (lva - r->lva);
}

uint64_t VaManager::LvaOfGva(uint64_t gva) const
{
    if (gva == 0) {
        return 0;
    }
    std::shared_lock<std::shared_mutex> guard(lock_);
    const VaRange *r = LookupGva(gva);
    return r == nullptr ? 0 : r->lva + (gva - r->gva);
}

bool VaManager::FindByGva(uint64_t gva, VaRange &out) const
{
    std::shared_lock<std::shared_mutex> guard(lock_);
    const VaRange *r = LookupGva(gva);
    if (r == nullptr) {
        return false;
    }
    out = *r;
    return true;
}

bool VaManager::FindByLva(uint64_t lva, VaRange &out) const
{
    std::shared_lock<std::shared_mutex> guard(lock_);
    const VaRange *r = LookupLva(lva);
    if (r == nullptr) {
        return false;
    }
    out = *r;
    return true;
}

bool VaManager::IsGva(uint64_t va) const
{
    if (va == 0) {
        return false;
    }
    std::shared_lock<std::shared_mutex> guard(lock_);
    return LookupGva(va) != nullptr;
}

bool VaManager::IsKnown(uint64_t va) const
{
    return IsGva(va) || GvaOfLva(va) != 0;
}

hybm_mem_type VaManager::MemTypeOf(uint64_t va) const
{
    if (va == 0) {
        return HYBM_MEM_TYPE_DEVICE;  // the reference's answer for a null probe
    }
    std::shared_lock<std::shared_mutex> guard(lock_);
    if (const VaRange *r = LookupGva(va)) {
        return r->memType;
    }
    if (const VaRange *r = LookupLva(va)) {
        return r->memType;
    }
    if (const ReservedRange *r = Floor(reserved_, va)) {
        if (va >= r->start && va < r->start + r->size) {
            return r->memType;
        }
    }
    return HYBM_MEM_TYPE_BUTT;
}

bool VaManager::RankOf(uint64_t gva, uint32_t &rank) const
{
    rank = 0;
    if (gva == 0) {
        return false;
    }
    std::shared_lock<std::shared_mutex> guard(lock_);
    const VaRange *r = LookupGva(gva);
    if (r == nullptr) {
        return false;
    }
    rank = r->Rank();
    return true;
}

AddressClass VaManager::Classify(uint64_t va) const
{
    const hybm_mem_type t = MemTypeOf(va);
    if (t == HYBM_MEM_TYPE_DEVICE) {
        return AddressClass::POOL_DEVICE;
    }
    if (t == HYBM_MEM_TYPE_HOST) {
        return AddressClass::POOL_HOST;
    }
    DeviceProbe probe;
    {
        std::shared_lock<std::shared_mutex> guard(lock_);
        probe = probe_;
    }
    const bool device = probe != nullptr ? probe(va) : LegacyWindowProbe(va);
    return device ? AddressClass::LOCAL_DEVICE : AddressClass::LOCAL_HOST;
}

hybm_data_copy_direction VaManager::InferDirection(uint64_t srcVa, uint64_t dstVa) const
{
    const AddressClass s = Classify(srcVa);
    const AddressClass d = Classify(dstVa);
    const Endpoint se{s == AddressClass::POOL_DEVICE || s == AddressClass::POOL_HOST,
                      s == AddressClass::POOL_DEVICE || s == AddressClass::LOCAL_DEVICE};
    const Endpoint de{d == AddressClass::POOL_DEVICE || d == AddressClass::POOL_HOST,
                      d == AddressClass::POOL_DEVICE || d == AddressClass::LOCAL_DEVICE};
    return ComposeDirection(se, de);
}

ReservedRange VaManager::Reserve(uint32_t localRank, uint64_t size, hybm_mem_type t)
{
    ReservedRange out;
    if (size == 0 || size > kReserveEnd - kReserveStart) {
        return out;
    }
    std::unique_lock<std::shared_mutex> guard(lock_);
    // First fit over the (address-ordered) reservations.
    uint64_t cursor = kReserveStart;
    bool placed = false;
    for (const auto &kv : reserved_) {
        const ReservedRange &r = kv.second;
        if (r.start < kReserveStart || r.start >= kReserveEnd) {
            continue;
        }
        if (r.start > cursor && r.start - cursor >= size) {
            placed = true;
            break;
        }
        if (r.start + r.size > cursor) {
            cursor = r.start + r.size;
        }
    }
    if (!placed && kReserveEnd - cursor < size) {
        return out;
    }
    out.start = cursor;
    out.size = size;
    out.memType = t;
    out.localRank = localRank;
    reserved_[cursor] = out;
    return out;
}

void VaManager::Unreserve(uint64_t start)
{
    if (start == 0) {
        return;
    }
    std::unique_lock<std::shared_mutex> guard(lock_);
    reserved_.erase(start);
}

size_t VaManager::RangeCount() const
{
    std::shared_lock<std::shared_mutex> guard(lock_);
    return byGva_.size();
}

size_t VaManager::ReservedCount() const
{
    std::shared_lock<std::shared_mutex> guard(lock_);
    return reserved_.size();
}

}  // namespace mf
