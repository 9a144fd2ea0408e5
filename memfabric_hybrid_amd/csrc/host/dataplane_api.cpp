// Native C entry points declared in include/mf_hip_dataplane.h and include/mf_hip_dataplane_internal.h.
#include <atomic>
#include <chrono>
#include <cstring>
#include <thread>
#include <vector>

#include <sched.h>

#include "../../../include/mf_hip_dataplane_internal.h"
#include "../../../include/mf_xcopy_types.h"
#include "copy_direction.h"
#include "../rt/mf_rt.h"
#include "gva_layout.h"
#include "mf_log.h"
#include "trans_entry.h"
#include "va_manager.h"
#include "xcopy_engine.h"

using namespace mf;

#define MF_EXPORT extern "C" __attribute__((visibility("default")))

MF_EXPORT int32_t mf_xcopy_batch(const uint64_t *src, const uint64_t *dst, const uint64_t *len, uint32_t n,
                                 int32_t route, void *stream)
{
    if ((n != 0 && (src == nullptr || dst == nullptr || len == nullptr)) || route < 0 || route > MF_ROUTE_FROM_HOST) {
        MF_FAIL(BM_INVALID_PARAM, "mf_xcopy_batch: null array or unknown route " << route);
    }
    return XcopyEngine::Instance().Submit(src, dst, len, n, route, stream, nullptr, 0);
}

MF_EXPORT int32_t mf_xcopy_device_table(const void *triples, uint32_t n, int32_t route, void *stream)
{
    if ((n != 0 && triples == nullptr) || route < 0 || route > MF_ROUTE_FROM_HOST) {
        MF_FAIL(BM_INVALID_PARAM, "mf_xcopy_device_table: null table or unknown route " << route);
    }
    return XcopyEngine::Instance().SubmitDeviceTable(triples, n, route, stream, nullptr, 0);
}

MF_EXPORT int32_t mf_xcopy_device_table_static(const void *triples, uint32_t n, int32_t route, void *stream)
{
    if ((n != 0 && triples == nullptr) || route < 0 || route > MF_ROUTE_FROM_HOST) {
        MF_FAIL(BM_INVALID_PARAM, "mf_xcopy_device_table_static: null table or unknown route " << route);
    }
    return XcopyEngine::Instance().SubmitDeviceTableStatic(triples, n, route, stream);
}

MF_EXPORT int32_t mf_bm_copy_batch_replay(smem_bm_t handle, smem_batch_copy_params *const *batches, uint32_t count,
                                          uint32_t steps, smem_bm_copy_type t, uint32_t flags)
{
    if (batches == nullptr || count == 0) {
        MF_FAIL(SM_INVALID_PARAM, "mf_bm_copy_batch_replay: no batches");
    }
    uint32_t at = 0;
    for (uint32_t i = 0; i < steps; ++i) {
        const int32_t ret = smem_bm_copy_batch(handle, batches[at], t, flags);
        if (ret != 0) {
            return ret;
        }
        at = at + 1 == count ? 0 : at + 1;
    }
    return 0;
}

MF_EXPORT int32_t mf_trans_batch_write_replay(smem_trans_t handle, smem_batch_copy_params *const *batches, uint32_t count,
                                              uint32_t steps, const char *remoteUniqueId, void *stream)
{
    if (batches == nullptr || count == 0) {
        MF_FAIL(SM_INVALID_PARAM, "mf_trans_batch_write_replay: no batches");
    }
    uint32_t at = 0;
    for (uint32_t i = 0; i < steps; ++i) {
        smem_batch_copy_params *b = batches[at];
        const int32_t ret = smem_trans_batch_write_submit(handle, const_cast<const void **>(b->sources), remoteUniqueId, b->destinations,
                                                          const_cast<size_t *>(reinterpret_cast<const size_t *>(b->dataSizes)), b->batchSize,
                                                          stream, 0);
        if (ret != 0) {
            return ret;
        }
        at = at + 1 == count ? 0 : at + 1;
    }
    return 0;
}

MF_EXPORT int32_t mf_bm_copy_batch_replay_threads(smem_bm_t handle, smem_batch_copy_params *const *batches, uint32_t count,
                                                  uint32_t steps, smem_bm_copy_type t, uint32_t threads, double *seconds)
{
    if (batches == nullptr || count == 0 || threads == 0 || threads > 64 || seconds == nullptr) {
        MF_FAIL(SM_INVALID_PARAM, "mf_bm_copy_batch_replay_threads: no batches, no result or 0 / more than 64 threads");
    }
    std::atomic<uint32_t> ready{0};
    std::atomic<bool> go{false};
    std::atomic<int32_t> firstError{0};
    auto body = [&](uint32_t tid) {
        auto fail = [&](int32_t ret) {
            int32_t none = 0;
            firstError.compare_exchange_strong(none, ret);
        };
        // warm-up: the thread's stream and staging exist and have been used before the clock starts
        for (uint32_t i = 0; i < 64 && firstError.load() == 0; ++i) {
            const int32_t ret = smem_bm_copy_batch(handle, batches[(tid * 7 + i) % count], t, ASYNC_COPY_FLAG);
            if (ret != 0) {
                fail(ret);
            }
        }
        (void)smem_bm_wait(handle);
        ready.fetch_add(1, std::memory_order_acq_rel);
        while (!go.load(std::memory_order_acquire)) {
            std::this_thread::yield();
        }
        for (uint32_t i = tid; i < steps && firstError.load(std::memory_order_relaxed) == 0; i += threads) {   // nothing is submitted once anything failed
            const int32_t ret = smem_bm_copy_batch(handle, batches[i % count], t, ASYNC_COPY_FLAG);
            if (ret != 0) {
                fail(ret);
            }
        }
        const int32_t ret = smem_bm_wait(handle);
        if (ret != 0) {
            fail(ret);
        }
    };
    std::vector<std::thread> pool;
    uint32_t started = 0;
    try {
        for (; started < threads; ++started) {
            pool.emplace_back(body, started);
        }
    } catch (...) {   // the system refused another thread: let the ones that run finish, then report
        firstError.store(SM_ERROR);
    }
    while (ready.load(std::memory_order_acquire) < started) {
        std::this_thread::yield();
    }
    const auto t0 = std::chrono::steady_clock::now();
    go.store(true, std::memory_order_release);
    for (auto &th : pool) {
        th.join();
    }
    *seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    return firstError.load();
}

MF_EXPORT void *mf_xcopy_thread_stream(void)
{
    XcopyEngine &engine = XcopyEngine::Instance();
    return engine.Started() ? engine.ThreadStream() : nullptr;
}

MF_EXPORT int32_t mf_xcopy_tune(uint32_t units, uint32_t wgPerCu, uint32_t wgPerCuLink)
{
    XcopyTuning &t = XcopyEngine::Instance().Tuning();
    t.unitsOverride = units;
    t.wgPerCu = wgPerCu;                               // 0: no cap, one workgroup per chunk
    t.wgPerCuLink = wgPerCuLink == 0 ? 1 : wgPerCuLink;
    return BM_OK;
}

MF_EXPORT int32_t mf_xcopy_unordered_streams(uint32_t count)
{
    if (count > XcopyEngine::kFanStreams) {
        MF_FAIL(BM_INVALID_PARAM, "unordered streams: 0 to " << XcopyEngine::kFanStreams << ", got " << count);
    }
    XcopyEngine::Instance().Tuning().unorderedStreams = count;
    return BM_OK;
}

MF_EXPORT uint32_t mf_xcopy_stream_queues(uint32_t *queues, uint32_t capacity)
{
    return XcopyEngine::Instance().StreamQueues(queues, queues == nullptr ? 0 : capacity);
}

MF_EXPORT int32_t mf_xcopy_tune_table(uint32_t stageUnordered, uint32_t deviceTableWgPerCu)
{
    XcopyTuning &t = XcopyEngine::Instance().Tuning();
    t.stageUnordered = stageUnordered != 0;
    t.deviceTableWgPerCu = deviceTableWgPerCu;
    return BM_OK;
}

MF_EXPORT int32_t mf_xcopy_tune_hold(uint32_t deepHold, int32_t pinnedExtraNanos, uint32_t holdOnSideStreams)
{
    XcopyTuning &t = XcopyEngine::Instance().Tuning();
    t.deepHold = deepHold != 0;
    t.holdPinnedExtraNanos = pinnedExtraNanos;
    t.holdOnSideStreams = holdOnSideStreams != 0;
    return BM_OK;
}

MF_EXPORT int32_t mf_xcopy_calibration(int32_t *holdEnabled, int32_t *holdDeltaNanos, uint32_t *windowMBps, uint32_t *windowAlignedMBps,
                                       uint32_t *windowLongMBps, float *micros)
{
    const XcopyCalibration &c = XcopyEngine::Instance().Calibration();
    if (holdEnabled != nullptr) {
        *holdEnabled = c.holdEnabled ? 1 : 0;
    }
    if (holdDeltaNanos != nullptr) {
        *holdDeltaNanos = c.holdDeltaNanos;
    }
    if (windowMBps != nullptr) {
        *windowMBps = XcopyEngine::Instance().Tuning().windowMBps;
    }
    if (windowAlignedMBps != nullptr) {
        *windowAlignedMBps = XcopyEngine::Instance().Tuning().windowAlignedMBps;
    }
    if (windowLongMBps != nullptr) {
        *windowLongMBps = XcopyEngine::Instance().Tuning().windowLongMBps;
    }
    if (micros != nullptr) {
        for (int i = 0; i < 4; ++i) {
            micros[i] = c.batchMicros[i];
        }
        for (int i = 0; i < 4; ++i) {
            micros[4 + i] = c.copyMicros[i];
        }
    }
    return c.ran ? 1 : 0;
}

MF_EXPORT int32_t mf_xcopy_hold_stores(int32_t nanos)
{
    if (nanos < -1) {
        MF_FAIL(BM_INVALID_PARAM, "hold: -1 (the rule), 0 (never) or a time in ns, got " << nanos);
    }
    XcopyEngine::Instance().Tuning().holdNanos = nanos;
    return BM_OK;
}

MF_EXPORT int32_t mf_xcopy_windows(uint32_t megabytesPerSecond)
{
    if (megabytesPerSecond == MF_XCOPY_WINDOWS_OWN_CHOICE) {
        // back to what the library chose: what hybm_init measured on this GPU, else the fitted defaults
        const XcopyCalibration &c = XcopyEngine::Instance().Calibration();
        const XcopyTuning fitted;
        XcopyTuning &t = XcopyEngine::Instance().Tuning();
        t.windowMBps = c.ran ? c.windowMBps : fitted.windowMBps;
        t.windowAlignedMBps = c.ran ? c.windowAlignedMBps : fitted.windowAlignedMBps;
        t.windowLongMBps = c.ran ? c.windowLongMBps : fitted.windowLongMBps;
        return BM_OK;
    }
    if (megabytesPerSecond != 0 && (megabytesPerSecond < 1000000 || megabytesPerSecond > 16000000)) {
        MF_FAIL(BM_INVALID_PARAM, "windows: 0 (never), 1 (the library's own choice) or a rate between 1 000 000 and 16 000 000 MB/s, got "
                                      << megabytesPerSecond);
    }
    XcopyEngine::Instance().Tuning().windowMBps = megabytesPerSecond;
    XcopyEngine::Instance().Tuning().windowAlignedMBps = megabytesPerSecond;   // a rate set by hand holds for every windowed launch
    XcopyEngine::Instance().Tuning().windowLongMBps = megabytesPerSecond;
    return BM_OK;
}

MF_EXPORT uint32_t mf_xcopy_choose_units(uint64_t totalBytes, uint32_t cuCount, int32_t route)
{
    return ChooseUnits(totalBytes, cuCount, route, XcopyEngine::Instance().Tuning());
}

MF_EXPORT uint64_t mf_xcopy_launch_count(void)
{
    return XcopyEngine::Instance().LaunchCount();
}

MF_EXPORT int64_t mf_xcopy_describe_plan(const uint64_t *src, const uint64_t *dst, const uint64_t *len, uint32_t n,
                                         uint32_t units, uint64_t *out, uint64_t capacity, int32_t *inlineForm)
{
    if (units == 0 || units % kXcopyThreads != 0) {
        return 0;
    }
    SegList segs;
    NormalizeSegments(src, dst, len, n, 1ull << 30, segs);
    InlinePlan plan;
    const bool fits = BuildInlinePlan(segs, units, plan);
    if (inlineForm != nullptr) {
        *inlineForm = fits ? 1 : 0;
    }
    {
        // the one-pass planner of the submission path must produce the very same plan
        InlinePlan direct;
        const bool directFits = BuildInlineDirect(src, dst, len, n, units, direct);
        if (directFits && (!fits || std::memcmp(&direct, &plan, sizeof(plan)) != 0)) {
            return -2;
        }
    }
    std::vector<uint64_t> triples(3ull * segs.Size() + 3);
    std::vector<uint32_t> first(segs.Size() + 1);
    const uint64_t nchunk = BuildTablePlan(segs, units, triples.data(), first.data());
    uint64_t count = 0;
    auto emit = [&](uint64_t s, uint64_t d, uint64_t bytes, uint64_t chunk) {
        if (bytes == 0) {
            return;
        }
        if (count < capacity && out != nullptr) {
            out[4 * count] = s;
            out[4 * count + 1] = d;
            out[4 * count + 2] = bytes;
            out[4 * count + 3] = chunk;
        }
        ++count;
    };
    // Walk chunk ids exactly as the kernels do: locate the owner by prefix, then cut by geometry.
    uint32_t seg = 0;
    for (uint64_t c = 0; c < nchunk; ++c) {
        while (seg + 1 <= segs.Size() && first[seg + 1] <= c) {
            ++seg;
        }
        if (fits) {
            // the inline lookup (count of rows whose prefix is <= c, minus one) must agree with the table prefix
            uint32_t below = 0;
            for (uint32_t i = 0; i < kInlineSegs; ++i) {
                below += plan.first[i] <= c ? 1u : 0u;
            }
            if (below - 1 != seg) {
                return -1;
            }
        }
        const uint64_t s = segs.src[seg];
        const uint64_t d = segs.dst[seg];
        const uint64_t l = segs.len[seg];
        const SegGeom g = SegmentGeometry(d, l);
        const uint64_t k = c - first[seg];
        const uint64_t u0 = k * units;
        const uint64_t left = g.body > u0 ? g.body - u0 : 0;
        const uint64_t nunits = left < units ? left : units;
        if (k == 0) {
            emit(s, d, g.head, c);
        }
        emit(s + g.head + u0 * kUnitBytes, d + g.head + u0 * kUnitBytes, nunits * kUnitBytes, c);
        if (u0 + units >= g.body) {
            const uint64_t off = g.head + g.body * kUnitBytes;
            emit(s + off, d + off, g.tail, c);
        }
    }
    if (count > capacity) {
        return -static_cast<int64_t>(count);
    }
    return static_cast<int64_t>(count);
}

/* ---- address registry view ------------------------------------------------ */
MF_EXPORT void mf_va_clear(void)
{
    VaManager::Global().Clear();
}

MF_EXPORT int32_t mf_va_add(uint64_t gva, uint64_t size, int32_t memType, uint64_t lva, uint32_t localRank)
{
    return VaManager::Global().AddOwn(gva, size, static_cast<hybm_mem_type>(memType), lva, localRank);
}

MF_EXPORT int32_t mf_va_add_external(uint64_t gva, uint64_t size, int32_t memType, uint64_t lva, uint32_t localRank,
                                     uint32_t importedRank)
{
    return VaManager::Global().AddExternal(gva, size, static_cast<hybm_mem_type>(memType), lva, localRank, importedRank);
}

MF_EXPORT void mf_va_remove(uint64_t va)
{
    VaManager::Global().Remove(va);
}

MF_EXPORT uint64_t mf_va_gva_of_lva(uint64_t lva)
{
    return VaManager::Global().GvaOfLva(lva);
}

MF_EXPORT uint64_t mf_va_lva_of_gva(uint64_t gva)
{
    return VaManager::Global().LvaOfGva(gva);
}

MF_EXPORT int32_t mf_va_is_gva(uint64_t va)
{
    return VaManager::Global().IsGva(va) ? 1 : 0;
}

MF_EXPORT int32_t mf_va_is_known(uint64_t va)
{
    return VaManager::Global().IsKnown(va) ? 1 : 0;
}

MF_EXPORT int32_t mf_va_mem_type(uint64_t va)
{
    return static_cast<int32_t>(VaManager::Global().MemTypeOf(va));
}

MF_EXPORT int64_t mf_va_rank(uint64_t gva)
{
    uint32_t rank = 0;
    return VaManager::Global().RankOf(gva, rank) ? static_cast<int64_t>(rank) : -1;
}

MF_EXPORT int32_t mf_va_infer_direction(uint64_t srcVa, uint64_t dstVa)
{
    return static_cast<int32_t>(VaManager::Global().InferDirection(srcVa, dstVa));
}

MF_EXPORT uint64_t mf_va_reserve(uint32_t localRank, uint64_t size, int32_t memType)
{
    return VaManager::Global().Reserve(localRank, size, static_cast<hybm_mem_type>(memType)).start;
}

MF_EXPORT void mf_va_unreserve(uint64_t start)
{
    VaManager::Global().Unreserve(start);
}

MF_EXPORT uint64_t mf_va_range_count(void)
{
    return VaManager::Global().RangeCount();
}

MF_EXPORT uint64_t mf_va_reserved_count(void)
{
    return VaManager::Global().ReservedCount();
}

/* ---- direction algebra and window arithmetic views -------------------------- */
MF_EXPORT int32_t mf_dir_compose(int32_t srcPool, int32_t srcDevice, int32_t dstPool, int32_t dstDevice)
{
    return static_cast<int32_t>(
        ComposeDirection(Endpoint{srcPool != 0, srcDevice != 0}, Endpoint{dstPool != 0, dstDevice != 0}));
}

MF_EXPORT int32_t mf_dir_translate_smem(int32_t copyType, int32_t srcPoolType, int32_t dstPoolType)
{
    return static_cast<int32_t>(TranslateSmemCopy(static_cast<smem_bm_copy_type>(copyType),
                                                  static_cast<smem_bm_mem_type>(srcPoolType),
                                                  static_cast<smem_bm_mem_type>(dstPoolType)));
}

MF_EXPORT int32_t mf_dir_checks(int32_t direction)
{
    const auto d = static_cast<hybm_data_copy_direction>(direction);
    return (MustCheckSource(d) ? 1 : 0) | (MustCheckDestination(d) ? 2 : 0);
}

MF_EXPORT int32_t mf_gva_contains(uint64_t base, uint64_t stride, uint64_t rankCount, uint64_t addr, uint64_t size)
{
    GvaWindow w;
    w.base = base;
    w.stride = stride;
    w.rankCount = rankCount;
    return w.Contains(addr, size) ? 1 : 0;
}

MF_EXPORT uint32_t mf_gva_rank(uint64_t base, uint64_t stride, uint64_t rankCount, uint64_t rankSpace, uint64_t addr)
{
    GvaWindow w;
    w.base = base;
    w.stride = stride;
    w.rankCount = rankCount;
    w.rankSpace = rankSpace;
    return w.RankBySpace(addr);
}

MF_EXPORT uint64_t mf_gva_mask48(uint64_t addr)
{
    return Mask48(addr);
}

MF_EXPORT uint32_t mf_trans_combine(const uint64_t *pairs, uint32_t n, uint64_t *out)
{
    if (pairs == nullptr || out == nullptr || n == 0) {
        return 0;
    }
    std::vector<std::pair<uint64_t, uint64_t>> in;
    in.reserve(n);
    for (uint32_t i = 0; i < n; ++i) {
        in.emplace_back(pairs[2 * i], pairs[2 * i + 1]);
    }
    const auto runs = CombineRanges(std::move(in));
    for (size_t k = 0; k < runs.size(); ++k) {
        out[2 * k] = runs[k].first;
        out[2 * k + 1] = runs[k].second;
    }
    return static_cast<uint32_t>(runs.size());
}

MF_EXPORT uint64_t mf_trans_translate(const uint64_t *slices, uint32_t n, uint64_t remote, uint64_t size)
{
    PeerSliceMap map;
    for (uint32_t i = 0; slices != nullptr && i < n; ++i) {
        map.emplace(slices[3 * i], PeerSlice{slices[3 * i + 2], slices[3 * i + 1], HYBM_MEM_TYPE_DEVICE});
    }
    uint64_t mapped = 0;
    hybm_mem_type type = HYBM_MEM_TYPE_BUTT;
    return TranslatePeerAddress(map, remote, size, mapped, type) == SM_OK ? mapped : 0;
}

MF_EXPORT int32_t mf_trans_parse_name(const char *name, uint8_t *key)
{
    WorkerKey k;
    if (name == nullptr || !ParseWorkerName(name, k)) {
        return 0;
    }
    if (key != nullptr) {
        std::memcpy(key, k.data(), k.size());
    }
    return 1;
}

// What one launch with a full argument block costs the calling thread on each CPU it may run on.  On the hosts
// this was built on (16 virtual CPUs, one NUMA node shown) a launch costs 3.1 us from half of the CPUs and 4.3 us
// from the others, whatever the process does, and a thread that the scheduler moves between them changes pace
// mid-run; nothing the operating system reports tells the two kinds apart, so they are measured.
MF_EXPORT int32_t mf_host_launch_costs(uint32_t *cpus, float *micros, uint32_t capacity)
{
    if (cpus == nullptr || micros == nullptr || capacity == 0) {
        MF_FAIL(BM_INVALID_PARAM, "mf_host_launch_costs: no room for the result");
    }
    XcopyEngine &engine = XcopyEngine::Instance();
    if (!engine.Started()) {
        MF_FAIL(BM_NOT_INITIALIZED, "GPU data plane is not running; call hybm_init first");
    }
    if (mfrt_bind_thread() != 0) {
        MF_FAIL(BM_ERROR, "cannot make the GPU current on this thread");
    }
    void *stream = engine.ThreadStream();
    if (stream == nullptr) {
        MF_FAIL(BM_ERROR, "cannot create the thread's stream");
    }
    cpu_set_t allowed;
    if (sched_getaffinity(0, sizeof(allowed), &allowed) != 0) {
        MF_FAIL(BM_ERROR, "cannot read the thread's CPU set");
    }
    // the launch that is timed: the batch kernel with its full argument block, copying 16 bytes
    uint8_t *scratch = static_cast<uint8_t *>(mfrt_alloc_device(4096));
    if (scratch == nullptr) {
        MF_FAIL(BM_MALLOC_FAILED, "mf_host_launch_costs: no device memory");
    }
    const uint64_t src = reinterpret_cast<uint64_t>(scratch);
    const uint64_t dst = src + 2048;
    const uint64_t len = 16;
    InlinePlan tiny;
    if (!BuildInlineDirect(&src, &dst, &len, 1, kXcopyThreads, tiny)) {
        mfrt_free_device(scratch);
        MF_FAIL(BM_ERROR, "mf_host_launch_costs: cannot plan the probe copy");
    }
    constexpr int kWarm = 64;
    constexpr int kTimed = 256;
    uint32_t n = 0;
    int err = 0;
    for (int cpu = 0; cpu < CPU_SETSIZE && n < capacity && err == 0; ++cpu) {
        if (!CPU_ISSET(cpu, &allowed)) {
            continue;
        }
        cpu_set_t one;
        CPU_ZERO(&one);
        CPU_SET(cpu, &one);
        if (sched_setaffinity(0, sizeof(one), &one) != 0) {
            continue;
        }
        for (int i = 0; i < kWarm && err == 0; ++i) {
            err = mfk_xcopy_inline(&tiny, MFRT_ROUTE_HBM, tiny.nchunk, nullptr, 0, stream, 0, 0);
        }
        (void)mfrt_stream_sync(stream);
        const auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < kTimed && err == 0; ++i) {
            err = mfk_xcopy_inline(&tiny, MFRT_ROUTE_HBM, tiny.nchunk, nullptr, 0, stream, 0, 0);
        }
        const auto t1 = std::chrono::steady_clock::now();
        (void)mfrt_stream_sync(stream);
        cpus[n] = static_cast<uint32_t>(cpu);
        micros[n] = static_cast<float>(std::chrono::duration<double, std::micro>(t1 - t0).count() / kTimed);
        ++n;
    }
    (void)sched_setaffinity(0, sizeof(allowed), &allowed);
    (void)mfrt_stream_sync(stream);
    mfrt_free_device(scratch);
    if (err != 0) {
        MF_FAIL(BM_ERROR, "mf_host_launch_costs: launch failed: " << mfrt_error_string(err));
    }
    return static_cast<int32_t>(n);
}

MF_EXPORT int32_t mf_pin_thread_near_gpu(void)
{
    constexpr uint32_t kMaxCpus = 1024;
    std::vector<uint32_t> cpus(kMaxCpus);
    std::vector<float> micros(kMaxCpus);
    const int32_t n = mf_host_launch_costs(cpus.data(), micros.data(), kMaxCpus);
    if (n <= 0) {
        return n;
    }
    float best = micros[0];
    float worst = micros[0];
    for (int32_t i = 1; i < n; ++i) {
        best = micros[i] < best ? micros[i] : best;
        worst = micros[i] > worst ? micros[i] : worst;
    }
    if (worst <= best * 1.25f) {
        return n;   // one kind of CPU (2.5 to 3.0 us on such hosts): the set stays as it is
    }
    cpu_set_t near;
    CPU_ZERO(&near);
    int32_t kept = 0;
    for (int32_t i = 0; i < n; ++i) {
        if (micros[i] <= best * 1.15f) {
            CPU_SET(static_cast<int>(cpus[i]), &near);
            ++kept;
        }
    }
    if (sched_setaffinity(0, sizeof(near), &near) != 0) {
        MF_FAIL(BM_ERROR, "mf_pin_thread_near_gpu: cannot set the thread's CPU set");
    }
    return kept;
}
