// TEST INFRASTRUCTURE ONLY.  A CPU stand-in for the thin runtime layer (csrc/rt/mf_rt.h) so that the
// host stack above it - planner, staging ring, operator fallback, entity and C API - can be
// exercised without a GPU, the way the reference's unit tests run against stub vendor libraries
// (test/ut/mock/acl_stub.cpp of the reference).  "Device" memory is host memory, a launch executes
// its plan at once with the SAME chunk geometry the kernels use (csrc/kernels/xcopy_plan.h), streams
// and events are tokens.  Never linked into the product libraries.
#include <atomic>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>
#include <cstring>
#include <map>
#include <mutex>

#include <sys/mman.h>

#include "../../memfabric_hybrid_amd/csrc/kernels/copy2d_plan.h"
#include "../../memfabric_hybrid_amd/csrc/kernels/xcopy_plan.h"
#include "../../memfabric_hybrid_amd/csrc/rt/mf_rt.h"

namespace {
std::mutex g_lock;
std::map<uint64_t, std::pair<uint64_t, int>> g_allocs;  // base -> (size, kind)
int g_device = -1;
std::atomic<uint64_t> g_launches{0};   // launches may come from the engine's submit threads
std::atomic<uint32_t> g_lastHold{0};
uint32_t g_lastWindow = 0;   // rate of the latest windowed launch, cleared by fake_rt_last_window()     // holdNanos of the latest inline launch
std::atomic<uint64_t> g_chunksRun{0};
bool g_skipCopies = false;       // launches count and check their plans but move nothing (tables of segments no test can back with memory)
uint32_t g_lastTableShift = 0;   // group shift of the latest table launch that used a group map, 0 under a pattern
uint64_t g_groupMapErrors = 0;
uint32_t g_lastTableHold = 0;    // holdNanos of the latest table launch
std::atomic<uint64_t> g_streamsMade{0};   // streams made since mfrt_init

void *Track(uint64_t bytes, int kind)
{
    void *p = nullptr;
    if (posix_memalign(&p, 4096, bytes == 0 ? 4096 : bytes) != 0) {
        return nullptr;
    }
    std::lock_guard<std::mutex> guard(g_lock);
    g_allocs[reinterpret_cast<uint64_t>(p)] = {bytes, kind};
    return p;
}

int Untrack(void *p)
{
    std::lock_guard<std::mutex> guard(g_lock);
    auto it = g_allocs.find(reinterpret_cast<uint64_t>(p));
    if (it == g_allocs.end()) {
        return 1;
    }
    g_allocs.erase(it);
    free(p);
    return 0;
}

void RunChunk(uint64_t src, uint64_t dst, uint64_t len, uint64_t k, uint32_t units)
{
    const mf::SegGeom g = mf::SegmentGeometry(dst, len);
    const uint64_t u0 = k * units;
    const uint64_t left = g.body > u0 ? g.body - u0 : 0;
    const uint64_t n = left < units ? left : units;
    std::memmove(reinterpret_cast<void *>(dst + g.head + u0 * 16), reinterpret_cast<void *>(src + g.head + u0 * 16), n * 16);
    if (k == 0) {
        std::memmove(reinterpret_cast<void *>(dst), reinterpret_cast<void *>(src), g.head);
    }
    if (u0 + units >= g.body) {
        const uint64_t off = g.head + g.body * 16;
        std::memmove(reinterpret_cast<void *>(dst + off), reinterpret_cast<void *>(src + off), g.tail);
    }
    ++g_chunksRun;
}
// Descriptor tables stay "in flight" until something the host has waited for covers their launch:
// an event recorded later, or a stream / device wait.  A table that changed in the meantime was
// rewritten while a kernel could still read it.
struct InFlight {
    uint64_t seq;
    const void *table;
    std::vector<uint8_t> snapshot;
};
std::mutex g_flightLock;
std::vector<InFlight> g_inFlight;
uint64_t g_flightSeq = 0;
uint64_t g_violations = 0;

void TrackTable(const void *table, size_t bytes)
{
    std::lock_guard<std::mutex> guard(g_flightLock);
    InFlight f{++g_flightSeq, table, {}};
    f.snapshot.assign(static_cast<const uint8_t *>(table), static_cast<const uint8_t *>(table) + bytes);
    g_inFlight.push_back(std::move(f));
}

void Retire(uint64_t upTo)
{
    std::lock_guard<std::mutex> guard(g_flightLock);
    size_t keep = 0;
    for (size_t i = 0; i < g_inFlight.size(); ++i) {
        InFlight &f = g_inFlight[i];
        if (f.seq <= upTo) {
            if (std::memcmp(f.table, f.snapshot.data(), f.snapshot.size()) != 0) {
                ++g_violations;
            }
        } else {
            if (keep != i) {
                g_inFlight[keep] = std::move(f);
            }
            ++keep;
        }
    }
    g_inFlight.resize(keep);
}

}  // namespace

extern "C" {
// After this call any allocation, free, mapping or launch aborts: the test binary arms it at the
// end of main() to prove that nothing touches the GPU runtime from static destructors.
static bool g_sealed = false;
void fake_rt_seal(void) { g_sealed = true; }
static void Guard(const char *what)
{
    if (g_sealed) {
        std::fprintf(stderr, "runtime call after main(): %s\n", what);
        std::abort();
    }
}
uint64_t fake_rt_launches(void) { return g_launches; }
uint32_t fake_rt_last_hold(void) { return g_lastHold; }
uint32_t fake_rt_last_window(void) { const uint32_t w = g_lastWindow; g_lastWindow = 0; return w; }
// The next n xcopy launches fail with a runtime error code instead of running.
static int g_failLaunches = 0;
void fake_rt_fail_launches(int n) { g_failLaunches = n; }
uint64_t fake_rt_chunks(void) { return g_chunksRun; }
void fake_rt_skip_copies(int on) { g_skipCopies = on != 0; }
uint32_t fake_rt_last_table_shift(void) { return g_lastTableShift; }
uint64_t fake_rt_group_map_errors(void) { return g_groupMapErrors; }
uint32_t fake_rt_last_table_hold(void) { return g_lastTableHold; }

int mfrt_init(int device)
{
    if (device != 0) {
        return 101;
    }
    g_device = 0;
    g_streamsMade = 0;
    return 0;
}
int mfrt_current_device(void) { return 0; }
int mfrt_bind_thread(void) { return g_device >= 0 ? 0 : 3; }
void mfrt_shutdown(void) { g_device = -1; }
int mfrt_is_initialised(void) { return g_device >= 0; }
int mfrt_device_id(void) { return g_device; }
uint32_t mfrt_cu_count(void) { return 256; }
const char *mfrt_error_string(int) { return "fake runtime error"; }
void *mfrt_alloc_device(uint64_t bytes) { return Track(bytes, MFRT_PTR_DEVICE); }
int mfrt_free_device(void *p) { Guard("mfrt_free_device"); Retire(~0ull); return Untrack(p); }   // hipFree waits for the device
void *mfrt_alloc_host(uint64_t bytes) { return Track(bytes, MFRT_PTR_PINNED_HOST); }
int mfrt_free_host(void *p) { Guard("mfrt_free_host"); Retire(~0ull); return Untrack(p); }
// Address windows: reserved as inaccessible pages, so a touch of an unmapped part ends the test
// with a fault just as it would fault the GPU; mapping makes the pages usable.
uint64_t mfrt_window_granularity(void) { return 2u << 20; }
void *mfrt_window_reserve(uint64_t bytes)
{
    void *p = mmap(nullptr, bytes, PROT_NONE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
    return p == MAP_FAILED ? nullptr : p;
}
int mfrt_window_last_error(void) { return 0; }
int mfrt_window_release(void *base, uint64_t bytes) { Guard("mfrt_window_release"); return munmap(base, bytes) == 0 ? 0 : 1; }
void *mfrt_window_map(void *addr, uint64_t bytes, void *accessBase, uint64_t accessBytes)
{
    if (static_cast<char *>(accessBase) + accessBytes != static_cast<char *>(addr) + bytes) {
        return nullptr;   // the access run must end with the new piece
    }
    if (mprotect(addr, bytes, PROT_READ | PROT_WRITE) != 0) {
        return nullptr;
    }
    std::lock_guard<std::mutex> guard(g_lock);
    g_allocs[reinterpret_cast<uint64_t>(addr)] = {bytes, MFRT_PTR_DEVICE};
    return addr;
}
int mfrt_window_unmap(void *addr, uint64_t bytes, void *handle)
{ Guard("mfrt_window_unmap");
    if (handle != addr) {
        return 1;
    }
    std::lock_guard<std::mutex> guard(g_lock);
    g_allocs.erase(reinterpret_cast<uint64_t>(addr));
    (void)madvise(addr, bytes, MADV_DONTNEED);
    return mprotect(addr, bytes, PROT_NONE) == 0 ? 0 : 1;
}
int mfrt_pointer_kind(const void *p)
{
    std::lock_guard<std::mutex> guard(g_lock);
    const uint64_t a = reinterpret_cast<uint64_t>(p);
    auto it = g_allocs.upper_bound(a);
    if (it == g_allocs.begin()) {
        return MFRT_PTR_PAGEABLE;
    }
    --it;
    return a < it->first + it->second.first ? it->second.second : MFRT_PTR_PAGEABLE;
}
// A stream remembers the how-manieth stream since mfrt_init it is: the stand-in for "which hardware queue the runtime
// put it on" follows the pattern measured on the GPU (queues A B C C B A D C, then round robin).
static int g_queueAnswers = 0;      // 0: by the pattern, 1: not known
void fake_rt_queue_answers(int mode) { g_queueAnswers = mode; }
void *mfrt_stream_create(void)
{
    uint64_t *token = static_cast<uint64_t *>(malloc(8));
    *token = g_streamsMade.fetch_add(1);
    return token;
}
static uint32_t FakeQueueOf(const void *stream)
{
    static const uint32_t first[8] = {0, 1, 2, 2, 1, 0, 3, 2};
    const uint64_t index = *static_cast<const uint64_t *>(stream);
    return index < 8 ? first[index] : static_cast<uint32_t>(index % 4);
}
int mfrt_streams_share_queue(void *a, void *b)
{
    if (g_queueAnswers == 1) {
        return -1;
    }
    return FakeQueueOf(a) == FakeQueueOf(b) ? 1 : 0;
}
int mfrt_stream_destroy(void *s) { Guard("mfrt_stream_destroy"); free(s); return 0; }
uint64_t fake_rt_violations(void) { return g_violations; }
uint64_t fake_rt_in_flight(void)
{
    std::lock_guard<std::mutex> guard(g_flightLock);
    return g_inFlight.size();
}

extern "C" void fake_rt_count_stream_sync(void);
int mfrt_stream_sync(void *) { Guard("mfrt_stream_sync"); Retire(~0ull); fake_rt_count_stream_sync(); return 0; }
int mfrt_device_sync(void) { Guard("mfrt_device_sync"); Retire(~0ull); return 0; }
void *mfrt_event_create(void) { return calloc(1, 8); }
int mfrt_event_destroy(void *e) { Guard("mfrt_event_destroy"); free(e); return 0; }
int mfrt_event_record(void *e, void *)
{
    std::lock_guard<std::mutex> guard(g_flightLock);
    *static_cast<uint64_t *>(e) = g_flightSeq;
    return 0;
}
int mfrt_event_sync(void *e) { Retire(*static_cast<uint64_t *>(e)); return 0; }
static uint64_t g_streamWaits = 0;
extern "C" uint64_t fake_rt_stream_waits(void) { return g_streamWaits; }
int mfrt_stream_wait_event(void *, void *) { ++g_streamWaits; return 0; }
int mfrt_event_done(void *) { return 1; }
float mfrt_event_elapsed_ms(void *, void *) { return 0.0f; }
int mfrt_memcpy(void *dst, const void *src, uint64_t bytes) { std::memmove(dst, src, bytes); return 0; }
int mfrt_memcpy_async(void *dst, const void *src, uint64_t bytes, void *) { std::memmove(dst, src, bytes); return 0; }
int mfrt_memset(void *dst, int value, uint64_t bytes) { std::memset(dst, value, bytes); return 0; }

int mfk_xcopy_inline(const void *inlinePlan, int, uint32_t, void *mask, uint32_t maskValue, void *, int, uint32_t holdNanos)
{
    const mf::InlinePlan &p = *static_cast<const mf::InlinePlan *>(inlinePlan);
    g_lastHold = holdNanos;
    if (g_failLaunches > 0) {
        --g_failLaunches;
        return 719;
    }
    ++g_launches;
    static const bool skip = std::getenv("FAKE_RT_SKIP_COPY") != nullptr;   // host-path timing: the launch is free
    if (skip || g_skipCopies) {
        if (mask != nullptr && g_skipCopies) {
            *static_cast<uint64_t *>(mask) = maskValue;
        }
        return 0;
    }
    for (uint32_t c = 0; c < p.nchunk; ++c) {
        uint32_t below = 0;
        for (uint32_t i = 0; i < mf::kInlineSegs; ++i) {
            below += p.first[i] <= c ? 1u : 0u;
        }
        const uint32_t s = below - 1;
        RunChunk(p.src[s], p.dst[s], p.len[s], c - p.first[s], p.units);
    }
    if (mask != nullptr) {
        *static_cast<uint64_t *>(mask) = maskValue;
    }
    return 0;
}

int mfk_xcopy_windows_available(void) { return 1; }
int mfk_xcopy_prelaunch(void *) { return 0; }
// The calibration "measures" what the test has put here (all zero: nothing measured, the defaults stay).
static float g_calibration[8] = {};
static uint32_t g_calibrationHolds[3] = {};
extern "C" void fake_rt_set_calibration(const float *us) { std::memcpy(g_calibration, us, sizeof(g_calibration)); }
extern "C" const uint32_t *fake_rt_calibration_holds(void) { return g_calibrationHolds; }
int mfk_xcopy_calibrate(void *, const uint32_t *holdNanos, const uint32_t *, float *out)
{
    std::memcpy(g_calibrationHolds, holdNanos, sizeof(g_calibrationHolds));
    std::memcpy(out, g_calibration, sizeof(g_calibration));
    return 0;
}
uint32_t mfk_xcopy_window_units(void) { return 1024; }
uint32_t mfk_xcopy_window_waves(void) { return 4096; }
int mfk_xcopy_windowed(const void *inlinePlan, uint32_t windowMBps, void *mask, uint32_t maskValue, void *stream)
{
    const mf::InlinePlan &p = *static_cast<const mf::InlinePlan *>(inlinePlan);
    if (p.units != 1024 || p.nchunk == 0 || windowMBps == 0) {
        return -1;
    }
    g_lastWindow = windowMBps;
    return mfk_xcopy_inline(inlinePlan, 0, p.nchunk, mask, maskValue, stream, 0, 0);
}

// As the kernel: chunk count, group shift and pattern out of the header when there is one; the owner of a
// chunk by division under a pattern, else from the two group-map entries around it and the prefix between
// them.  A map whose entries do not bracket the owner fails the launch.
int mfk_xcopy_table(const void *tablePlan, int, uint32_t grid, void *mask, uint32_t maskValue, void *, uint32_t holdNanos)
{
    g_lastTableHold = holdNanos;
    const mf::TablePlan &plan = *static_cast<const mf::TablePlan *>(tablePlan);
    const uint64_t *t = plan.triples;
    const uint32_t *f = plan.first;
    uint32_t total = plan.nchunk;
    uint32_t shift = plan.groupShift;
    mf::ChunkPattern pat = plan.pattern;
    if (plan.nseg == 0 || grid == 0 || t == nullptr) {
        return -1;
    }
    if (plan.header != nullptr) {
        total = plan.header->nchunk;
        shift = plan.header->groupShift;
        pat = plan.header->pattern;
    } else if (pat.period != 0 && (pat.period > mf::kMaxPeriod || mf::PatternChunks(pat, plan.nseg) != total)) {
        return -1;
    }
    if (pat.period == 0 && (f == nullptr || plan.group == nullptr || shift < mf::kGroupShiftMin || shift > 31)) {
        return -1;
    }
    if (g_failLaunches > 0) {
        --g_failLaunches;
        return 719;
    }
    ++g_launches;
    g_lastTableShift = pat.period != 0 ? 0 : shift;
    TrackTable(t, 24ull * plan.nseg);
    if (g_skipCopies) {
        if (mask != nullptr) {
            *static_cast<uint64_t *>(mask) = maskValue;
        }
        return 0;
    }
    for (uint32_t c = 0; pat.period != 0 && c < total; ++c) {
        uint32_t seg = 0;
        uint32_t k = 0;
        mf::PatternOwner(pat, c, seg, k);
        RunChunk(t[3 * seg], t[3 * seg + 1], t[3 * seg + 2], k, plan.units);
    }
    for (uint32_t c = 0; pat.period == 0 && c < total; ++c) {
        const uint32_t lo = plan.group[c >> shift];
        const uint32_t hiEx = plan.group[(c >> shift) + 1] + 1;
        if (lo >= hiEx || hiEx > plan.nseg || f[lo] > c || f[hiEx] <= c) {
            ++g_groupMapErrors;
            return 720;
        }
        uint32_t s = lo;
        while (s + 1 < hiEx && f[s + 1] <= c) {
            ++s;
        }
        RunChunk(t[3 * s], t[3 * s + 1], t[3 * s + 2], c - f[s], plan.units);
    }
    if (mask != nullptr) {
        *static_cast<uint64_t *>(mask) = maskValue;
    }
    return 0;
}

uint64_t mfk_xcopy_plan_scratch_words(uint32_t nseg, uint32_t groupCapacity)
{
    return mf::ScratchLayoutFor(nseg, groupCapacity).words;
}

// The device-side planner restated: same scratch layout, same header, prefix, group map and pattern rule.
int mfk_xcopy_plan(const void *triples, uint32_t nseg, uint32_t units, void *scratch, uint32_t groupCapacity, void *tablePlan,
                   void *)
{
    if (nseg == 0 || scratch == nullptr || groupCapacity < 2 || tablePlan == nullptr) {
        return -1;
    }
    const uint64_t *t = static_cast<const uint64_t *>(triples);
    uint32_t *words = static_cast<uint32_t *>(scratch);
    const mf::ScratchLayout at = mf::ScratchLayoutFor(nseg, groupCapacity);
    uint32_t *f = words + at.first;
    uint32_t run = 0;
    uint32_t alive = 0x1FEu;
    std::vector<uint32_t> counts(nseg);
    for (uint32_t i = 0; i < nseg; ++i) {
        f[i] = run;
        counts[i] = static_cast<uint32_t>(mf::SegmentChunks(t[3 * i + 1], t[3 * i + 2], units));
        for (uint32_t p = 1; p <= mf::kMaxPeriod; ++p) {
            if (i >= p && counts[i - p] != counts[i]) {
                alive &= ~(1u << p);
            }
        }
        run += counts[i];
    }
    f[nseg] = run;
    mf::TableHeader *header = reinterpret_cast<mf::TableHeader *>(words);
    *header = mf::TableHeader{};
    header->nchunk = run;
    header->groupShift = mf::GroupShiftFor(run, groupCapacity);
    if (run != 0) {
        header->groupShift = mf::BuildGroupMap(f, nseg, words + at.group, groupCapacity);
    }
    if (alive != 0 && run != 0) {
        const uint32_t period = static_cast<uint32_t>(__builtin_ctz(alive));
        uint32_t sum = 0;
        for (uint32_t q = 0; q < period; ++q) {
            header->pattern.start[q] = sum;
            sum += counts[q];
        }
        header->pattern.start[period] = sum;
        if (sum != 0) {
            header->pattern.period = period;
            header->pattern.chunksPerPeriod = sum;
        } else {
            header->pattern = mf::ChunkPattern{};
        }
    }
    mf::TablePlan &plan = *static_cast<mf::TablePlan *>(tablePlan);
    plan = mf::TablePlan{};
    plan.triples = t;
    plan.first = f;
    plan.group = words + at.group;
    plan.header = header;
    plan.nseg = nseg;
    plan.units = units;
    ++g_launches;
    return 0;
}

static uint64_t g_signals = 0;
static uint64_t g_streamSyncs = 0;
extern "C" uint64_t fake_rt_signals() { return g_signals; }
extern "C" uint64_t fake_rt_stream_syncs() { return g_streamSyncs; }
extern "C" void fake_rt_count_stream_sync(void) { ++g_streamSyncs; }
int mfk_xcopy_signal(void *word, uint32_t value, void *)
{
    // not counted: fake_rt_launches() counts the launches that move data
    ++g_signals;
    __atomic_store_n(static_cast<uint64_t *>(word), static_cast<uint64_t>(value), __ATOMIC_RELEASE);
    return 0;
}
int mfk_xcopy_static_setup(void) { return 0; }
int mfk_xcopy_table_static(const void *triples, uint32_t nseg, uint32_t units, int route, uint32_t grid, void *stream)
{
    static std::vector<uint32_t> scratch(mf::ScratchLayoutFor(MFK_STATIC_TABLE_SEGMENTS, MFK_STATIC_TABLE_SEGMENTS).words);
    if (nseg == 0 || nseg > MFK_STATIC_TABLE_SEGMENTS) {
        return -1;
    }
    mf::TablePlan plan;
    int err = mfk_xcopy_plan(triples, nseg, units, scratch.data(), MFK_STATIC_TABLE_SEGMENTS, &plan, stream);
    return err != 0 ? err : mfk_xcopy_table(&plan, route, grid, nullptr, 0, stream, 0);
}

static uint32_t g_lastRectMates = 0;
extern "C" uint32_t fake_rt_last_rect_mates() { return g_lastRectMates; }

// Walks the chunks as the kernel's workgroups do, so a wrong chunk-to-rectangle rule leaves rows uncopied.
int mfk_copy2d(const void *rectPlan, uint32_t, void *)
{
    const mf::RectPlan &p = *static_cast<const mf::RectPlan *>(rectPlan);
    ++g_launches;
    g_lastRectMates = 0;
    for (uint32_t r = 0; r < mf::kRectInline; ++r) {
        g_lastRectMates += p.mate[r] != 0 ? 1u : 0u;
    }
    for (uint32_t c = 0; c < p.nchunk; ++c) {
        uint32_t r = 0;
        uint32_t k = 0;
        mf::RectOfChunk(p, c, r, k);
        const uint32_t row0 = k * p.rowsPerChunk[r];
        for (uint32_t row = row0; row < row0 + p.rowsPerChunk[r] && row < p.height[r]; ++row) {
            std::memmove(reinterpret_cast<void *>(p.dst[r] + 16ull * p.dpitchUnits[r] * row),
                         reinterpret_cast<void *>(p.src[r] + 16ull * p.spitchUnits[r] * row), 16ull * p.widthUnits[r]);
        }
    }
    return 0;
}

// The windowed form: chunks of kRectWindowUnits units of the payload taken row-major, unit by unit as the kernel's lanes do.
static uint32_t g_rectWindowed = 0;
extern "C" uint32_t fake_rt_rect_windowed_launches() { return g_rectWindowed; }
int mfk_copy2d_windowed(const void *rectPlan, uint32_t windowMBps, void *)
{
    const mf::RectPlan &p = *static_cast<const mf::RectPlan *>(rectPlan);
    if (windowMBps == 0) {
        return -1;
    }
    ++g_launches;
    ++g_rectWindowed;
    for (uint32_t c = 0; c < p.nchunk; ++c) {
        uint32_t r = 0;
        uint32_t k = 0;
        mf::RectOfChunk(p, c, r, k);
        const uint32_t wu = p.widthUnits[r];
        const uint32_t base = k * mf::kRectWindowUnits;
        const uint32_t total = p.height[r] * wu;
        const uint32_t row0 = base / wu;
        const uint32_t col0 = base - row0 * wu;
        for (uint32_t u = 0; u < mf::kRectWindowUnits && base + u < total; ++u) {
            uint32_t row = 0;
            uint32_t col = 0;
            mf::RectWindowRowCol(col0 + u, wu, p.magic[r], row, col);
            std::memmove(reinterpret_cast<void *>(p.dst[r] + 16ull * (static_cast<uint64_t>(p.dpitchUnits[r]) * (row0 + row) + col)),
                         reinterpret_cast<void *>(p.src[r] + 16ull * (static_cast<uint64_t>(p.spitchUnits[r]) * (row0 + row) + col)), 16);
        }
    }
    return 0;
}
int mfk_copy2d_prelaunch(void *) { return 0; }

uint64_t mfk_moe_workspace_bytes(uint32_t, uint32_t, uint32_t) { return 0; }
int mfk_moe_dispatch(const void *, const void *, uint32_t, uint32_t, uint32_t, uint32_t, void *, void *, void *, void *, void *,
                     void *, void *) { return -1; }
static int g_lastCombinePaced = -1;
extern "C" int fake_rt_last_combine_paced() { return g_lastCombinePaced; }
int mfk_moe_combine(const void *, const void *, const void *, uint32_t, uint32_t, uint32_t, void *, void *, int paced)
{
    g_lastCombinePaced = paced;
    return 0;
}
void mfk_moe_combine_windows(uint32_t, uint32_t) {}
int mfk_moe_setup(void) { return 0; }
int mfk_moe_xcd_streams(void) { return 0; }
}
