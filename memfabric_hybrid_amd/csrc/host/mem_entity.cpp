#include "mem_entity.h"

#include <cstdlib>
#if defined(__x86_64__)
#include <immintrin.h>
#endif
#include <cstring>
#include <thread>

#include "../rt/mf_rt.h"
#include "mf_log.h"
#include "va_manager.h"

namespace mf {

using ock::mf::ExtOptions;

namespace {
// The device window is reserved address space into which HBM is mapped piece by piece, so that no
// other allocation can land inside the window.  MF_HIP_GVA_WINDOW=malloc selects the simpler
// form instead: the local rank's share is one ordinary allocation and the rest of the window is
// only arithmetic.
bool WantMappedWindow()
{
    const char *mode = std::getenv("MF_HIP_GVA_WINDOW");
    return mode == nullptr || std::strcmp(mode, "malloc") != 0;
}

// Every entity counts its range epochs in a block of its own, so a per-thread hit remembered for
// an entity that is gone can never match a later entity that reuses its address.
uint64_t NextEpochBlock()
{
    static std::atomic<uint64_t> block{1};
    return block.fetch_add(1, std::memory_order_relaxed) << 32;
}
}  // namespace

MemEntity::MemEntity(uint16_t id, const hybm_options &options) : id_(id), options_(options)
{
    rangeEpoch_.store(NextEpochBlock(), std::memory_order_release);
}

MemEntity::~MemEntity()
{
    UnInitialize();
}

int MemEntity::Initialize(OperatorFactory factory)
{
    if (initialized_) {
        return BM_OK;
    }
    if (options_.bmType != HYBM_TYPE_AI_CORE_INITIATE) {
        dataOperator_ = std::make_shared<ComposeDataOp>(options_, std::move(factory));
        int ret = dataOperator_->Initialize();
        if (ret != BM_OK) {
            dataOperator_ = nullptr;
            MF_FAIL(ret, "copy engine set-up failed: " << ret);
        }
    }
    initialized_ = true;
    return BM_OK;
}

void MemEntity::UnInitialize()
{
    if (!initialized_) {
        return;
    }
    if (dataOperator_ != nullptr) {
        dataOperator_->CleanUp();
        dataOperator_->UnInitialize();
        dataOperator_ = nullptr;
    }
    {
        std::lock_guard<std::mutex> guard(sliceLock_);
        for (auto &slice : looseSlices_) {
            if (slice->ownsMemory) {
                (void)mfrt_free_host(reinterpret_cast<void *>(slice->va));
            }
        }
        looseSlices_.clear();
    }
    {
        std::unique_lock<std::shared_mutex> guard(rangeLock_);
        ranges_.clear();
        rangeCount_.store(0, std::memory_order_release);
        rangeEpoch_.fetch_add(1, std::memory_order_release);
    }
    (void)UnreserveSpace();
    initialized_ = false;
}

int MemEntity::ReserveSpace()
{
    if (!initialized_) {
        return BM_NOT_INITIALIZED;
    }
    if (reserved_) {
        return BM_OK;
    }
    if (mfrt_bind_thread() != 0) {
        MF_FAIL(BM_ERROR, "no GPU bound; call hybm_init first");
    }
    // A world of one: the whole window is this rank's, so it is allocated in
    // one piece now and the address it lands on becomes the window base.
    if ((options_.memType & HYBM_MEM_TYPE_DEVICE) != 0 && options_.maxHBMSize > 0 && WantMappedWindow()) {
        const uint64_t granule = mfrt_window_granularity();
        const uint64_t bytes = options_.maxHBMSize * options_.rankCount;
        void *p = granule != 0 && options_.maxHBMSize % granule == 0 ? mfrt_window_reserve(bytes) : nullptr;
        if (p == nullptr) {
            MF_FAIL(BM_MALLOC_FAILED, "address window of " << bytes << " bytes could not be reserved (granularity "
                                                            << granule << ")");
        }
        device_.base = reinterpret_cast<uint64_t>(p);
        device_.stride = options_.maxHBMSize;
        device_.rankCount = options_.rankCount;
        device_.rankSpace = options_.maxHBMSize;
        deviceBacked_ = 0;
        deviceMapped_ = true;
        deviceWindowBytes_ = bytes;
    } else if ((options_.memType & HYBM_MEM_TYPE_DEVICE) != 0 && options_.deviceVASpace > 0) {
        void *p = mfrt_alloc_device(options_.deviceVASpace);
        if (p == nullptr) {
            MF_FAIL(BM_MALLOC_FAILED, "HBM pool allocation of " << options_.deviceVASpace << " bytes failed");
        }
        device_.base = reinterpret_cast<uint64_t>(p);
        device_.stride = options_.maxHBMSize;
        device_.rankCount = options_.rankCount;
        device_.rankSpace = options_.maxHBMSize;
        deviceBacked_ = options_.deviceVASpace;
    }
    if ((options_.memType & HYBM_MEM_TYPE_HOST) != 0 && options_.hostVASpace > 0) {
        void *p = mfrt_alloc_host(options_.hostVASpace);
        if (p == nullptr) {
            if (device_.base != 0) {
                if (deviceMapped_) {
                    (void)mfrt_window_release(reinterpret_cast<void *>(device_.base), deviceWindowBytes_);
                    deviceMapped_ = false;
                } else {
                    (void)mfrt_free_device(reinterpret_cast<void *>(device_.base));
                }
                device_ = GvaWindow{};
                deviceBacked_ = 0;
            }
            MF_FAIL(BM_MALLOC_FAILED, "pinned DRAM pool allocation of " << options_.hostVASpace << " bytes failed");
        }
        host_.base = reinterpret_cast<uint64_t>(p);
        host_.stride = options_.maxDRAMSize;
        host_.rankCount = options_.rankCount;
        host_.rankSpace = options_.maxDRAMSize;
        hostBacked_ = options_.hostVASpace;
    }
    if (dataOperator_ != nullptr) {
        if (device_.base != 0) {
            dataOperator_->UpdateGvaSpace(HYBM_MEM_TYPE_DEVICE, device_.base, device_.stride, device_.rankCount);
        }
        if (host_.base != 0) {
            dataOperator_->UpdateGvaSpace(HYBM_MEM_TYPE_HOST, host_.base, host_.stride, host_.rankCount);
        }
    }
    reserved_ = true;
    return BM_OK;
}

int MemEntity::UnreserveSpace()
{
    if (!reserved_) {
        return BM_OK;
    }
    if (dataOperator_ != nullptr) {
        dataOperator_->CleanUp();  // nothing may still be reading the pools
    }
    if (deviceSlice_ != nullptr) {
        VaManager::Global().Remove(deviceSlice_->va);
        deviceSlice_ = nullptr;
    }
    if (hostSlice_ != nullptr) {
        VaManager::Global().Remove(hostSlice_->va);
        hostSlice_ = nullptr;
    }
    if (device_.base != 0) {
        (void)mfrt_device_sync();
        if (deviceMapped_) {
            UnmapAll();
            (void)mfrt_window_release(reinterpret_cast<void *>(device_.base), deviceWindowBytes_);
            deviceMapped_ = false;
            deviceWindowBytes_ = 0;
        } else {
            (void)mfrt_free_device(reinterpret_cast<void *>(device_.base));
        }
    }
    if (host_.base != 0) {
        (void)mfrt_free_host(reinterpret_cast<void *>(host_.base));
    }
    device_ = GvaWindow{};
    host_ = GvaWindow{};
    deviceBacked_ = 0;
    hostBacked_ = 0;
    reserved_ = false;
    return BM_OK;
}

void *MemEntity::WindowBase(hybm_mem_type t) const
{
    if (t == HYBM_MEM_TYPE_DEVICE) {
        return reinterpret_cast<void *>(device_.base);
    }
    if (t == HYBM_MEM_TYPE_HOST) {
        return reinterpret_cast<void *>(host_.base);
    }
    return nullptr;
}

LocalSlice *MemEntity::AllocLocal(hybm_mem_type t, uint64_t size)
{
    if (initialized_ && options_.scene == HYBM_SCENE_TRANS) {
        // The transfer scene has no pre-sized window: every allocation is pinned host memory of
        // its own (the reference carves it from a 128 GiB reservation,
        // src/smem/csrc/smem_trans/smem_trans_entry.cpp:33,179-227).
        if (t != HYBM_MEM_TYPE_HOST || size == 0) {
            MF_ERROR("transfer-scene allocation needs host memory type and a size, got type " << t << " size " << size);
            return nullptr;
        }
        if (mfrt_bind_thread() != 0) {
            return nullptr;
        }
        const uint64_t bytes = (size + kLargePage - 1) / kLargePage * kLargePage;
        void *p = mfrt_alloc_host(bytes);
        if (p == nullptr) {
            MF_ERROR("pinned allocation of " << bytes << " bytes failed");
            return nullptr;
        }
        const uint64_t va = reinterpret_cast<uint64_t>(p);
        if (AddRange(va, bytes, HYBM_MEM_TYPE_HOST) != BM_OK) {
            (void)mfrt_free_host(p);
            return nullptr;
        }
        std::lock_guard<std::mutex> guard(sliceLock_);
        looseSlices_.emplace_back(new LocalSlice{HYBM_MEM_TYPE_HOST, va, bytes, true, true});
        return looseSlices_.back().get();
    }
    if (!initialized_ || !reserved_) {
        MF_ERROR("local allocation before the address space was reserved");
        return nullptr;
    }
    if (size == 0 || size % kLargePage != 0) {
        MF_ERROR("local allocation size " << size << " is not a positive multiple of 2 MiB");
        return nullptr;
    }
    const bool device = t == HYBM_MEM_TYPE_DEVICE;
    if (!device && t != HYBM_MEM_TYPE_HOST) {
        MF_ERROR("local allocation with memory type " << t);
        return nullptr;
    }
    if (device && deviceMapped_) {
        return AllocMapped(size);
    }
    const GvaWindow &w = device ? device_ : host_;
    std::unique_ptr<LocalSlice> &slot = device ? deviceSlice_ : hostSlice_;
    const uint64_t backed = device ? deviceBacked_.load(std::memory_order_acquire) : hostBacked_.load(std::memory_order_acquire);
    if (w.base == 0 || slot != nullptr || size > backed) {
        MF_ERROR("local allocation of " << size << " bytes does not fit the reserved window of " << backed);
        return nullptr;
    }
    const uint64_t va = w.PtrOfRank(options_.rankId);
    if (VaManager::Global().AddOwn(va, size, t, va, options_.rankId) != BM_OK) {
        return nullptr;
    }
    slot.reset(new LocalSlice{t, va, size});
    return slot.get();
}

LocalSlice *MemEntity::AllocMapped(uint64_t size)
{
    const uint64_t granule = mfrt_window_granularity();
    std::lock_guard<std::mutex> guard(sliceLock_);   // the backed prefix grows under the lock: two allocations must not pick the same offset
    const uint64_t backed = deviceBacked_.load(std::memory_order_acquire);
    if (granule == 0 || size % granule != 0 || size > options_.maxHBMSize - backed) {
        MF_ERROR("local allocation of " << size << " bytes: not a multiple of " << granule << " or more than the "
                 << options_.maxHBMSize - backed << " bytes left in this rank's window");
        return nullptr;
    }
    if (mfrt_bind_thread() != 0) {
        return nullptr;
    }
    const uint64_t va = device_.PtrOfRank(options_.rankId) + backed;
    void *mapping = mfrt_window_map(reinterpret_cast<void *>(va), size,
                                    reinterpret_cast<void *>(device_.PtrOfRank(options_.rankId)), backed + size);
    if (mapping == nullptr) {
        MF_ERROR("HBM of " << size << " bytes could not be mapped into the window at offset " << backed
                 << " (step and code " << mfrt_window_last_error() << ")");
        return nullptr;
    }
    if (VaManager::Global().AddOwn(va, size, HYBM_MEM_TYPE_DEVICE, va, options_.rankId) != BM_OK) {
        (void)mfrt_window_unmap(reinterpret_cast<void *>(va), size, mapping);
        return nullptr;
    }
    mappedSlices_.emplace_back(new LocalSlice{HYBM_MEM_TYPE_DEVICE, va, size});
    mappedSlices_.back()->mapping = mapping;
    deviceBacked_.store(backed + size, std::memory_order_release);   // published once the mapping exists
    return mappedSlices_.back().get();
}

int MemEntity::FreeMapped(LocalSlice *slice)
{
    std::lock_guard<std::mutex> guard(sliceLock_);
    bool mine = false;
    for (auto &s : mappedSlices_) {
        if (s.get() == slice && !s->released) {
            s->released = true;
            mine = true;
        }
    }
    if (!mine) {
        return BM_INVALID_PARAM;
    }
    // The backed bytes of a rank are one prefix of its window: memory goes back to the GPU from
    // the top, once the slice and everything mapped after it have been released.
    uint64_t going = 0;
    for (auto it = mappedSlices_.rbegin(); it != mappedSlices_.rend() && (*it)->released; ++it) {
        going += (*it)->size;
    }
    if (going == 0) {
        return BM_OK;
    }
    // First the bound comes down, so that no new copy passes the range check for these bytes; then the copies that
    // had passed it before are let through to their enqueue (and those handed to the engine's submit threads to
    // their launch); then the GPU drains; only then the memory goes.  (A copy into a slice that is being freed
    // is a caller error all the same: it may now fail its range check.)
    deviceBacked_.store(deviceBacked_.load(std::memory_order_acquire) - going, std::memory_order_seq_cst);
    while (submitsInFlight_.load(std::memory_order_seq_cst) != 0) {
        std::this_thread::yield();
    }
    if (dataOperator_ != nullptr) {
        dataOperator_->CleanUp();   // also lets the engine's submit threads launch what they still hold
    }
    (void)mfrt_device_sync();
    while (!mappedSlices_.empty() && mappedSlices_.back()->released) {
        LocalSlice &top = *mappedSlices_.back();
        VaManager::Global().Remove(top.va);
        (void)mfrt_window_unmap(reinterpret_cast<void *>(top.va), top.size, top.mapping);
        mappedSlices_.pop_back();
    }
    return BM_OK;
}

void MemEntity::UnmapAll()
{
    std::lock_guard<std::mutex> guard(sliceLock_);
    while (!mappedSlices_.empty()) {
        LocalSlice &top = *mappedSlices_.back();
        VaManager::Global().Remove(top.va);
        (void)mfrt_window_unmap(reinterpret_cast<void *>(top.va), top.size, top.mapping);
        mappedSlices_.pop_back();
    }
    deviceBacked_ = 0;
}

LocalSlice *MemEntity::RegisterLocal(const void *ptr, uint64_t size)
{
    if (!initialized_ || ptr == nullptr || size == 0) {
        MF_ERROR("memory registration needs an initialised entity, an address and a size");
        return nullptr;
    }
    if (mfrt_bind_thread() != 0) {
        return nullptr;
    }
    const uint64_t va = reinterpret_cast<uint64_t>(ptr);
    const int first = mfrt_pointer_kind(ptr);
    const int last = mfrt_pointer_kind(reinterpret_cast<const void *>(va + size - 1));
    if (first == MFRT_PTR_PAGEABLE || first != last) {
        MF_ERROR("memory registration of [" << ptr << ", +" << size << ") refused: it must be one piece of HBM or of "
                 "pinned host memory (ordinary host memory cannot be pinned after the fact here)");
        return nullptr;
    }
    const hybm_mem_type t = first == MFRT_PTR_DEVICE ? HYBM_MEM_TYPE_DEVICE : HYBM_MEM_TYPE_HOST;
    if (AddRange(va, size, t) != BM_OK) {
        return nullptr;
    }
    std::lock_guard<std::mutex> guard(sliceLock_);
    looseSlices_.emplace_back(new LocalSlice{t, va, size, false, true});
    return looseSlices_.back().get();
}

int MemEntity::AddRange(uint64_t base, uint64_t size, hybm_mem_type t)
{
    if (base == 0 || size == 0 || base + size < base) {
        return BM_INVALID_PARAM;
    }
    std::unique_lock<std::shared_mutex> guard(rangeLock_);
    auto it = ranges_.find(base);
    if (it != ranges_.end()) {
        it->second.size = it->second.size > size ? it->second.size : size;
        it->second.uses += 1;
    } else {
        ranges_.emplace(base, Range{size, t, 1});
        rangeCount_.store(static_cast<uint32_t>(ranges_.size()), std::memory_order_release);
    }
    rangeEpoch_.fetch_add(1, std::memory_order_release);
    return BM_OK;
}

int MemEntity::RemoveRange(uint64_t base)
{
    std::unique_lock<std::shared_mutex> guard(rangeLock_);
    auto it = ranges_.find(base);
    if (it == ranges_.end()) {
        return BM_INVALID_PARAM;
    }
    if (--it->second.uses == 0) {
        ranges_.erase(it);
        rangeCount_.store(static_cast<uint32_t>(ranges_.size()), std::memory_order_release);
    }
    rangeEpoch_.fetch_add(1, std::memory_order_release);
    return BM_OK;
}

bool MemEntity::InRanges(uint64_t a, uint64_t length, uint64_t *rangeBase, uint64_t *rangeEnd) const
{
    // Batches walk one or two ranges; the last hit of this thread answers most calls without
    // the lock.  The epoch makes a hit from before any change of the range set worthless.
    struct Hit {
        const MemEntity *owner = nullptr;
        uint64_t epoch = 0;
        uint64_t base = 0;
        uint64_t end = 0;
    };
    thread_local Hit hit;
    const uint64_t epoch = rangeEpoch_.load(std::memory_order_acquire);
    if (hit.owner == this && hit.epoch == epoch && a >= hit.base && a + length <= hit.end && a + length >= a) {
        if (rangeBase != nullptr) {
            *rangeBase = hit.base;
            *rangeEnd = hit.end;
        }
        return true;
    }
    std::shared_lock<std::shared_mutex> guard(rangeLock_);
    auto it = ranges_.lower_bound(a);   // greatest start <= a
    if (it == ranges_.end() || a + length < a || a + length > it->first + it->second.size) {
        return false;
    }
    hit = Hit{this, rangeEpoch_.load(std::memory_order_acquire), it->first, it->first + it->second.size};
    if (rangeBase != nullptr) {
        *rangeBase = hit.base;
        *rangeEnd = hit.end;
    }
    return true;
}

int MemEntity::FreeLocal(LocalSlice *slice)
{
    if (slice != nullptr && slice->outsideWindow) {
        std::unique_ptr<LocalSlice> found;
        {
            std::lock_guard<std::mutex> guard(sliceLock_);
            for (auto it = looseSlices_.begin(); it != looseSlices_.end(); ++it) {
                if (it->get() == slice) {
                    found = std::move(*it);
                    looseSlices_.erase(it);
                    break;
                }
            }
        }
        if (found == nullptr) {
            return BM_INVALID_PARAM;
        }
        (void)RemoveRange(found->va);
        if (found->ownsMemory) {
            if (dataOperator_ != nullptr) {
                dataOperator_->CleanUp();   // nothing may still be copying from or to it
            }
            (void)mfrt_free_host(reinterpret_cast<void *>(found->va));
        }
        return BM_OK;
    }
    if (slice != nullptr && deviceMapped_ && FreeMapped(slice) == BM_OK) {
        return BM_OK;
    }
    for (std::unique_ptr<LocalSlice> *slot : {&deviceSlice_, &hostSlice_}) {
        if (slot->get() == slice && slice != nullptr) {
            VaManager::Global().Remove(slice->va);
            slot->reset();
            return BM_OK;
        }
    }
    return BM_INVALID_PARAM;
}

bool MemEntity::CheckAddressInEntity(const void *ptr, uint64_t length) const
{
    if (!initialized_) {
        return false;
    }
    const uint64_t a = reinterpret_cast<uint64_t>(ptr);
    // Window test as in the reference, narrowed to the bytes that are real
    // memory: an address in the unbacked remainder of a window would fault
    // the GPU instead of failing a remote transfer.
    if (a + length < a) {
        return false;   // wraps round the address space
    }
    if (device_.Contains(a, length)) {
        return a + length <= device_.base + deviceBacked_.load(std::memory_order_acquire) || options_.rankCount > 1;
    }
    if (host_.Contains(a, length)) {
        return a + length <= host_.base + hostBacked_.load(std::memory_order_acquire) || options_.rankCount > 1;
    }
    return rangeCount_.load(std::memory_order_acquire) != 0 && InRanges(a, length);
}

#if defined(__x86_64__)
namespace {
// Whether every [ptrs[i], ptrs[i] + lengths[i]) lies inside [lo1, hi1) or [lo2, hi2), does not wrap and does not start at 0,
// four elements a step.  (The loop below spends 2 ns an element on its six comparisons, twice per batch; with this in front
// of it a call of 122 segments costs the submitting thread 0.8 instead of 1.2 us before the launch on one CPU, 0.05 us less
// on the faster ones of the GPU hosts, where the launch itself, with its 3 KiB of arguments written across the host link,
// is 3 us of the 4.1.)  AVX2 compares 64-bit values as signed ones, so everything is compared with its top bit flipped.
__attribute__((target("avx2"))) bool AllInsideAvx2(void *const *ptrs, const uint64_t *lengths, uint32_t n, uint64_t lo1, uint64_t hi1,
                                                   uint64_t lo2, uint64_t hi2)
{
    const __m256i flip = _mm256_set1_epi64x(static_cast<long long>(0x8000000000000000ull));
    const __m256i vlo1 = _mm256_set1_epi64x(static_cast<long long>(lo1 ^ 0x8000000000000000ull));
    const __m256i vhi1 = _mm256_set1_epi64x(static_cast<long long>(hi1 ^ 0x8000000000000000ull));
    const __m256i vlo2 = _mm256_set1_epi64x(static_cast<long long>(lo2 ^ 0x8000000000000000ull));
    const __m256i vhi2 = _mm256_set1_epi64x(static_cast<long long>(hi2 ^ 0x8000000000000000ull));
    __m256i bad = _mm256_setzero_si256();
    for (uint32_t i = 0; i + 4 <= n; i += 4) {
        const __m256i a = _mm256_loadu_si256(reinterpret_cast<const __m256i *>(ptrs + i));
        const __m256i e = _mm256_add_epi64(a, _mm256_loadu_si256(reinterpret_cast<const __m256i *>(lengths + i)));
        const __m256i af = _mm256_xor_si256(a, flip);
        const __m256i ef = _mm256_xor_si256(e, flip);
        // outside a window: starts below it or ends above it
        const __m256i out1 = _mm256_or_si256(_mm256_cmpgt_epi64(vlo1, af), _mm256_cmpgt_epi64(ef, vhi1));
        const __m256i out2 = _mm256_or_si256(_mm256_cmpgt_epi64(vlo2, af), _mm256_cmpgt_epi64(ef, vhi2));
        const __m256i wraps = _mm256_cmpgt_epi64(af, ef);
        const __m256i null = _mm256_cmpeq_epi64(a, _mm256_setzero_si256());
        bad = _mm256_or_si256(bad, _mm256_or_si256(_mm256_and_si256(out1, out2), _mm256_or_si256(wraps, null)));
    }
    return _mm256_testz_si256(bad, bad) != 0;
}
}  // namespace
#endif

uint32_t MemEntity::FirstOutside(void *const *ptrs, const uint64_t *lengths, uint32_t n) const
{
    if (!initialized_ || options_.rankCount > 1) {
        for (uint32_t i = 0; i < n; ++i) {
            if (ptrs[i] == nullptr || !CheckAddressInEntity(ptrs[i], lengths[i])) {
                return i;
            }
        }
        return n;
    }
    // One rank: an address is inside when it lies in the backed part of one of the two windows
    // (or in a registered range).  The bounds stay in registers for the whole batch.
    const uint64_t devLo = device_.base;
    const uint64_t devBacked = deviceBacked_.load(std::memory_order_acquire);
    const uint64_t hostBacked = hostBacked_.load(std::memory_order_acquire);
    const uint64_t devHi = device_.base == 0 ? 0 : device_.base + (devBacked < device_.Span() ? devBacked : device_.Span());
    const uint64_t hostLo = host_.base;
    const uint64_t hostHi = host_.base == 0 ? 0 : host_.base + (hostBacked < host_.Span() ? hostBacked : host_.Span());
    const bool haveRanges = rangeCount_.load(std::memory_order_acquire) != 0;
    uint64_t rangeLo = 1;   // the registered range the element before lay in (none yet): most of a batch lies in one
    uint64_t rangeHi = 0;
    uint32_t checked = 0;
#if defined(__x86_64__)
    // the usual batch lies in the windows entirely: four elements a step say so; one that does not is found by the loop below
    static const bool haveAvx2 = __builtin_cpu_supports("avx2") != 0;
    if (haveAvx2 && n >= 8 && AllInsideAvx2(ptrs, lengths, n, devLo, devHi, hostLo, hostHi)) {
        checked = n & ~3u;
    }
#endif
    for (uint32_t i = checked; i < n; ++i) {
        const uint64_t a = reinterpret_cast<uint64_t>(ptrs[i]);
        const uint64_t end = a + lengths[i];
        const bool inDevice = a >= devLo && end <= devHi;
        const bool inHost = a >= hostLo && end <= hostHi;
        const bool inRange = a >= rangeLo && end <= rangeHi;
        if (a != 0 && end >= a && (inDevice || inHost || inRange)) {
            continue;
        }
        if (a == 0 || !haveRanges || !InRanges(a, lengths[i], &rangeLo, &rangeHi)) {
            return i;
        }
    }
    return n;
}

void MemEntity::LocateAddrAndRank(void *&src, void *&dest, uint64_t length, std::pair<uint32_t, uint32_t> &ranks) const
{
    auto owner = [&](uint64_t a) -> uint32_t {
        bool inside = false;
        uint32_t r = host_.RankByStride(a, length, options_.rankId, inside);
        if (inside) {
            return r;
        }
        return device_.RankByStride(a, length, options_.rankId, inside);
    };
    ranks.first = owner(reinterpret_cast<uint64_t>(src));
    src = reinterpret_cast<void *>(Mask48(reinterpret_cast<uint64_t>(src)));
    ranks.second = owner(reinterpret_cast<uint64_t>(dest));
    dest = reinterpret_cast<void *>(Mask48(reinterpret_cast<uint64_t>(dest)));
}

int MemEntity::CopyData(hybm_copy_params &params, hybm_data_copy_direction direction, void *stream, uint32_t flags)
{
    if (!initialized_) {
        return BM_NOT_INITIALIZED;
    }
    if (dataOperator_ == nullptr) {
        MF_FAIL(BM_ERROR, "this pool has no host copy engine");
    }
    if (mfrt_bind_thread() != 0) {
        return BM_ERROR;
    }
    std::pair<uint32_t, uint32_t> ranks;
    LocateAddrAndRank(params.src, params.dest, params.dataSize, ranks);
    ExtOptions options{};
    options.flags = flags;
    options.stream = stream;
    options.srcRankId = ranks.first;
    options.destRankId = ranks.second;
    return dataOperator_->DataCopy(params, direction, options);
}

int MemEntity::BatchCopyData(hybm_batch_copy_params &params, hybm_data_copy_direction direction, void *stream,
                             uint32_t flags)
{
    if (!initialized_) {
        return BM_NOT_INITIALIZED;
    }
    if (dataOperator_ == nullptr) {
        MF_FAIL(BM_ERROR, "this pool has no host copy engine");
    }
    if (mfrt_bind_thread() != 0) {
        return BM_ERROR;
    }
    ExtOptions options{};
    options.stream = stream;
    options.flags = flags;
    options.srcRankId = options_.rankId;
    options.destRankId = options_.rankId;
    if (options_.rankCount > 1) {
        for (uint32_t i = 0; i < params.batchSize; ++i) {
            std::pair<uint32_t, uint32_t> ranks;
            LocateAddrAndRank(params.sources[i], params.destinations[i], params.dataSizes[i], ranks);
            options.groupMap[ranks].push_back(i);
        }
    } else {
        // One rank: every element belongs to the pair (rank, rank).  The
        // addresses are still normalised in place as callers may rely on it.
        for (uint32_t i = 0; i < params.batchSize; ++i) {
            params.sources[i] = reinterpret_cast<void *>(Mask48(reinterpret_cast<uint64_t>(params.sources[i])));
            params.destinations[i] =
                reinterpret_cast<void *>(Mask48(reinterpret_cast<uint64_t>(params.destinations[i])));
        }
    }
    return dataOperator_->BatchDataCopy(params, direction, options);
}

int MemEntity::Wait()
{
    if (!initialized_) {
        return BM_NOT_INITIALIZED;
    }
    if (dataOperator_ == nullptr) {
        return BM_ERROR;
    }
    return dataOperator_->Wait(0);
}

EntityRegistry &EntityRegistry::Instance()
{
    static EntityRegistry *registry = new EntityRegistry();   // never destroyed: what is still alive at process exit is left to the operating system, no GPU call runs from a static destructor
    return *registry;
}

void EntityRegistry::SetFactory(OperatorFactory factory)
{
    std::unique_lock<std::shared_mutex> guard(lock_);
    factory_ = std::move(factory);
}

std::shared_ptr<MemEntity> EntityRegistry::Create(uint16_t id, const hybm_options &options, int &result)
{
    std::unique_lock<std::shared_mutex> guard(lock_);
    if (byId_.count(id) != 0) {
        result = BM_ERROR;
        MF_ERROR("pool id " << id << " already exists");
        return nullptr;
    }
    auto entity = std::make_shared<MemEntity>(id, options);
    result = entity->Initialize(factory_);
    if (result != BM_OK) {
        return nullptr;
    }
    byId_[id] = entity;
    byPtr_[entity.get()] = entity;
    return entity;
}

std::shared_ptr<MemEntity> EntityRegistry::FindById(uint16_t id)
{
    std::shared_lock<std::shared_mutex> guard(lock_);
    auto it = byId_.find(id);
    return it == byId_.end() ? nullptr : it->second;
}

std::shared_ptr<MemEntity> EntityRegistry::FindByPtr(const void *handle)
{
    std::shared_lock<std::shared_mutex> guard(lock_);
    auto it = byPtr_.find(handle);
    return it == byPtr_.end() ? nullptr : it->second;
}

bool EntityRegistry::Remove(const void *handle)
{
    std::shared_ptr<MemEntity> victim;
    {
        std::unique_lock<std::shared_mutex> guard(lock_);
        auto it = byPtr_.find(handle);
        if (it == byPtr_.end()) {
            return false;
        }
        victim = it->second;
        byId_.erase(victim->Id());
        byPtr_.erase(it);
    }
    victim->UnInitialize();
    return true;
}

void EntityRegistry::Clear()
{
    std::map<uint16_t, std::shared_ptr<MemEntity>> victims;
    {
        std::unique_lock<std::shared_mutex> guard(lock_);
        victims.swap(byId_);
        byPtr_.clear();
    }
    for (auto &kv : victims) {
        kv.second->UnInitialize();
    }
}

}  // namespace mf
