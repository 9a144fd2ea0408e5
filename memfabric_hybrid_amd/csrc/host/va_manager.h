// Registry of pooled address ranges: which global address belongs to which
// memory type and rank, and where it is mapped locally.  Behavioural
// counterpart of HybmVaManager
// (src/hybm/csrc/mm/hybm_va_manager.h:175-264, .cpp:34-256), pinned by the
// address known-answer tests in test/ut/testcase/hybm/hybm_va_manager_test.cpp.
#ifndef MF_VA_MANAGER_H
#define MF_VA_MANAGER_H

#include <stdint.h>

#include <map>
#include <shared_mutex>

#include "../../../include/mf_xcopy_types.h"
#include "gva_layout.h"

namespace mf {

// Address-space constants of the pooled VA scheme
// (src/hybm/csrc/common/hybm_define.h:33-34,56-57).
constexpr uint64_t kLegacyDeviceVaStart = 0x100000000000ULL;
constexpr uint64_t kLegacyDeviceVaSize = 0x80000000000ULL;
constexpr uint64_t kReserveStart = 0x280000000000ULL;
constexpr uint64_t kReserveEnd = 0xA80000000000ULL;

struct VaRange {
    uint64_t gva = 0;
    uint64_t size = 0;
    hybm_mem_type memType = HYBM_MEM_TYPE_DEVICE;
    uint64_t lva = 0;            // 0: not addressable from this process
    uint32_t localRank = kNoRank;
    uint32_t importedRank = kNoRank;
    bool registered = false;

    uint32_t Rank() const
    {
        return importedRank != kNoRank ? importedRank : localRank;
    }
    bool HoldsGva(uint64_t a) const
    {
        return a >= gva && a < gva + size;
    }
    bool HoldsLva(uint64_t a) const
    {
        return lva != 0 && a >= lva && a < lva + size;
    }
    bool SameAs(const VaRange &o) const
    {
        return gva == o.gva && size == o.size && Rank() == o.Rank();
    }
};

struct ReservedRange {
    uint64_t start = 0;
    uint64_t size = 0;
    hybm_mem_type memType = HYBM_MEM_TYPE_DEVICE;
    uint32_t localRank = 0;
};

enum class AddressClass : int { POOL_DEVICE = 0, POOL_HOST = 1, LOCAL_DEVICE = 2, LOCAL_HOST = 3 };

class VaManager {
public:
    static VaManager &Global();

    // Decides whether an address outside every pool range is device memory.
    // Default: the fixed device VA window of the reference; the runtime
    // installs a HIP pointer query instead once a GPU is bound.
    using DeviceProbe = bool (*)(uint64_t va);
    void SetDeviceProbe(DeviceProbe probe);

    int Add(const VaRange &range);                       // BM_OK / BM_ERROR
    int AddOwn(uint64_t gva, uint64_t size, hybm_mem_type t, uint64_t lva, uint32_t localRank);
    int AddExternal(uint64_t gva, uint64_t size, hybm_mem_type t, uint64_t lva, uint32_t localRank,
                    uint32_t importedRank = kNoRank);
    void Remove(uint64_t va);
    void Clear();

    uint64_t GvaOfLva(uint64_t lva) const;               // 0 when unknown
    uint64_t LvaOfGva(uint64_t gva) const;               // 0 when unknown
    bool FindByGva(uint64_t gva, VaRange &out) const;
    bool FindByLva(uint64_t lva, VaRange &out) const;
    bool IsGva(uint64_t va) const;
    bool IsKnown(uint64_t va) const;
    hybm_mem_type MemTypeOf(uint64_t va) const;          // HYBM_MEM_TYPE_BUTT when unknown
    bool RankOf(uint64_t gva, uint32_t &rank) const;

    AddressClass Classify(uint64_t va) const;
    hybm_data_copy_direction InferDirection(uint64_t srcVa, uint64_t dstVa) const;

    ReservedRange Reserve(uint32_t localRank, uint64_t size, hybm_mem_type t);
    void Unreserve(uint64_t start);

    size_t RangeCount() const;
    size_t ReservedCount() const;

private:
    VaManager() = default;
    const VaRange *LookupGva(uint64_t va) const;
    const VaRange *LookupLva(uint64_t va) const;

    mutable std::shared_mutex lock_;
    std::map<uint64_t, VaRange> byGva_;
    std::map<uint64_t, VaRange> byLva_;
    std::map<uint64_t, ReservedRange> reserved_;
    DeviceProbe probe_ = nullptr;
};

}  // namespace mf

#endif  // MF_VA_MANAGER_H
