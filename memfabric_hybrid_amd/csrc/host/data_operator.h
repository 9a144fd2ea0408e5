// The C++ operator contract a copy engine implements to be usable by the
// entity layer.  Declared in the reference's own namespace, with the same
// member names, argument types, virtual-member order and noexcept
// qualifiers as DataOperator / ExtOptions in
// src/hybm/csrc/data_operation/hybm_data_operator.h:36-101, so an engine
// written against this header compiles against that one unchanged.
#ifndef MF_DATA_OPERATOR_H
#define MF_DATA_OPERATOR_H

#include <stdint.h>

#include <memory>
#include <unordered_map>
#include <utility>
#include <vector>

#include "../../../include/mf_xcopy_types.h"
#include "gva_layout.h"

namespace ock {
namespace mf {

using Result = int32_t;

struct PairHash {
    std::size_t operator()(const std::pair<uint32_t, uint32_t> &p) const
    {
        return (static_cast<uint64_t>(p.first) << 32ULL) + static_cast<uint64_t>(p.second);
    }
};

struct PairEqual {
    bool operator()(const std::pair<uint32_t, uint32_t> &a, const std::pair<uint32_t, uint32_t> &b) const
    {
        return a.first == b.first && a.second == b.second;
    }
};

// Per-call context handed down by the entity: owner ranks of both sides, the
// caller's stream (nullptr = the operator's per-thread stream), the copy
// flags, and for batches the element indices grouped by (srcRank, dstRank).
struct ExtOptions {
    uint32_t srcRankId;
    uint32_t destRankId;
    void *stream = nullptr;
    uint32_t flags;
    std::unordered_map<std::pair<uint32_t, uint32_t>, std::vector<uint32_t>, PairHash, PairEqual> groupMap;
};

class DataOperator {
public:
    virtual Result Initialize() noexcept = 0;
    virtual void UnInitialize() noexcept = 0;

    virtual Result DataCopy(hybm_copy_params &params, hybm_data_copy_direction direction,
                            const ExtOptions &options) noexcept = 0;
    virtual Result BatchDataCopy(hybm_batch_copy_params &params, hybm_data_copy_direction direction,
                                 const ExtOptions &options) noexcept = 0;
    // 0 on success, > 0 a wait id, < 0 an error.
    virtual Result DataCopyAsync(hybm_copy_params &params, hybm_data_copy_direction direction,
                                 const ExtOptions &options) noexcept = 0;
    virtual Result Wait(int32_t waitId) noexcept = 0;

    virtual ~DataOperator() = default;

    void UpdateGvaSpace(hybm_mem_type type, uint64_t gva, uint64_t localSpaceSize, uint64_t rankCount) noexcept
    {
        if (type >= HYBM_MEM_TYPE_BUTT || localSpaceSize == 0) {
            return;
        }
        gva_[type] = gva;
        localSpaceSize_[type] = localSpaceSize;
        rankCount_[type] = rankCount;
    }

    uint32_t GetRankIdByGva(uint64_t gva) noexcept
    {
        for (int type = 0; type < HYBM_MEM_TYPE_BUTT; ++type) {
            if (localSpaceSize_[type] != 0 && gva >= gva_[type] &&
                gva < gva_[type] + rankCount_[type] * localSpaceSize_[type]) {
                return static_cast<uint32_t>((gva - gva_[type]) / localSpaceSize_[type]);
            }
        }
        return UINT32_MAX;
    }

    virtual void CleanUp() noexcept {}

protected:
    static inline uint64_t gva_[HYBM_MEM_TYPE_BUTT] = {0};
    static inline uint64_t localSpaceSize_[HYBM_MEM_TYPE_BUTT] = {0};
    static inline uint64_t rankCount_[HYBM_MEM_TYPE_BUTT] = {0};
};

using DataOperatorPtr = std::shared_ptr<DataOperator>;

}  // namespace mf
}  // namespace ock

#endif  // MF_DATA_OPERATOR_H
