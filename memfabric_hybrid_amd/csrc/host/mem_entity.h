// One pooled-memory object of this process: its two address windows (HBM and
// pinned host DRAM), the local slices that back them, and the copy engine.
// Single-rank counterpart of MemEntityDefault
// (src/hybm/csrc/entity/hybm_entity_default.cpp:737-827,995-1017,1141-1157) and
// of the handle registry in src/hybm/csrc/entity/hybm_entity_factory.cpp:27-54.
#ifndef MF_MEM_ENTITY_H
#define MF_MEM_ENTITY_H

#include <atomic>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <shared_mutex>
#include <unordered_map>
#include <utility>
#include <vector>

#include "compose_data_op.h"
#include "gva_layout.h"

namespace mf {

constexpr uint64_t kLargePage = 2ull << 20;     // local allocations are multiples of this
constexpr uint32_t kEntityIdMax = 510;

struct LocalSlice {
    hybm_mem_type memType;
    uint64_t va;
    uint64_t size;
    bool ownsMemory = false;    // allocated for this slice alone, released with it
    bool outsideWindow = false; // user memory or a stand-alone allocation, known to the entity as a range
    void *mapping = nullptr;    // physical memory mapped into a reserved window for this slice
    bool released = false;      // given back by the caller, unmapped once every later slice is too
};

class MemEntity {
public:
    MemEntity(uint16_t id, const hybm_options &options);
    ~MemEntity();

    int Initialize(OperatorFactory factory);
    void UnInitialize();

    int ReserveSpace();
    int UnreserveSpace();
    void *WindowBase(hybm_mem_type t) const;
    LocalSlice *AllocLocal(hybm_mem_type t, uint64_t size);
    int FreeLocal(LocalSlice *slice);
    // Memory the caller owns becomes part of the entity (hybm_register_local_memory,
    // src/hybm/csrc/hybm_big_mem_entry.cpp); pageable memory is refused.
    LocalSlice *RegisterLocal(const void *ptr, uint64_t size);
    // Address ranges outside the two windows that belong to the entity: registered user memory
    // and memory of peers made addressable here (what hybm_import yields in the reference's
    // transfer scene).  Ranges are counted, so the same range may be added more than once.
    int AddRange(uint64_t base, uint64_t size, hybm_mem_type t);
    int RemoveRange(uint64_t base);
    uint32_t RangeCount() const
    {
        return rangeCount_.load(std::memory_order_acquire);
    }

    bool CheckAddressInEntity(const void *ptr, uint64_t length) const;
    // Brackets range check and enqueue of one copy (see submitsInFlight_).
    class SubmitScope {
    public:
        explicit SubmitScope(MemEntity &entity) : entity_(entity)
        {
            entity_.submitsInFlight_.fetch_add(1, std::memory_order_seq_cst);
        }
        ~SubmitScope()
        {
            entity_.submitsInFlight_.fetch_sub(1, std::memory_order_release);
        }
        SubmitScope(const SubmitScope &) = delete;
        SubmitScope &operator=(const SubmitScope &) = delete;

    private:
        MemEntity &entity_;
    };
    // The same test for every element of a batch in one pass; the index of the first element that
    // is null or leaves the entity, n when all are inside.
    uint32_t FirstOutside(void *const *ptrs, const uint64_t *lengths, uint32_t n) const;
    void LocateAddrAndRank(void *&src, void *&dest, uint64_t length, std::pair<uint32_t, uint32_t> &ranks) const;

    int CopyData(hybm_copy_params &params, hybm_data_copy_direction direction, void *stream, uint32_t flags);
    int BatchCopyData(hybm_batch_copy_params &params, hybm_data_copy_direction direction, void *stream, uint32_t flags);
    int Wait();

    const hybm_options &Options() const
    {
        return options_;
    }
    uint16_t Id() const
    {
        return id_;
    }

private:
    uint16_t id_;
    hybm_options options_;
    bool initialized_ = false;
    bool reserved_ = false;
    GvaWindow device_;          // stride = maxHBMSize
    GvaWindow host_;            // stride = maxDRAMSize
    // Bytes of the local windows that are real memory.  Written under sliceLock_ (or during
    // Initialize / UnInitialize), read without a lock by the range check of every copy: a map is
    // published with a release store after it exists, an unmap lowers the bound before it waits
    // for the GPU, so no new copy is admitted into memory that is about to go away.
    std::atomic<uint64_t> deviceBacked_{0};
    // copies between their range check and the return of their enqueue: FreeMapped waits for the count to reach zero
    // after it has lowered the bound, so that no copy that passed the old bound is enqueued after the GPU was drained
    std::atomic<uint32_t> submitsInFlight_{0};
    std::atomic<uint64_t> hostBacked_{0};
    std::unique_ptr<LocalSlice> deviceSlice_;
    // Mapped-window mode (the default; MF_HIP_GVA_WINDOW=malloc turns it off): the device window is reserved address space of
    // rankCount * maxHBMSize bytes, and every local allocation maps fresh HBM at the end of the
    // local rank's backed prefix (the reference's HybmDevLegacySegment does the same with its
    // driver's reserve / map calls, src/hybm/csrc/mm/hybm_dev_legacy_segment.cpp:123-181).
    bool deviceMapped_ = false;
    uint64_t deviceWindowBytes_ = 0;
    std::vector<std::unique_ptr<LocalSlice>> mappedSlices_;   // in address order
    LocalSlice *AllocMapped(uint64_t size);
    int FreeMapped(LocalSlice *slice);
    void UnmapAll();
    std::unique_ptr<LocalSlice> hostSlice_;
    std::shared_ptr<ComposeDataOp> dataOperator_;

    struct Range {
        uint64_t size;
        hybm_mem_type type;
        uint32_t uses;
    };
    bool InRanges(uint64_t a, uint64_t length, uint64_t *rangeBase = nullptr, uint64_t *rangeEnd = nullptr) const;
    mutable std::shared_mutex rangeLock_;
    std::map<uint64_t, Range, std::greater<uint64_t>> ranges_;   // by start, descending: lower_bound = covering candidate
    std::atomic<uint32_t> rangeCount_{0};
    std::atomic<uint64_t> rangeEpoch_{1};                        // bumped on every change; invalidates per-thread hits
    std::mutex sliceLock_;
    std::vector<std::unique_ptr<LocalSlice>> looseSlices_;       // slices that are not a window's backing
};

class EntityRegistry {
public:
    static EntityRegistry &Instance();
    std::shared_ptr<MemEntity> Create(uint16_t id, const hybm_options &options, int &result);
    std::shared_ptr<MemEntity> FindById(uint16_t id);
    std::shared_ptr<MemEntity> FindByPtr(const void *handle);
    bool Remove(const void *handle);
    void Clear();
    // Test hook: engines used by entities created afterwards.
    void SetFactory(OperatorFactory factory);

private:
    std::shared_mutex lock_;
    std::map<uint16_t, std::shared_ptr<MemEntity>> byId_;
    std::unordered_map<const void *, std::shared_ptr<MemEntity>> byPtr_;
    OperatorFactory factory_ = OperatorFactory::Default();
};

}  // namespace mf

#endif  // MF_MEM_ENTITY_H
