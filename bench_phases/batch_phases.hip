// mf_batch_phases: a stand-alone measurement program (not part of the data plane, nothing links it).
// It takes KV-block batches apart on one GPU: what a launch that waits for its predecessor costs, what the
// descriptor lookup, the loads and the stores of a batch add, and what the product kernels need, each as
// the period per launch of dependent launches on one stream.  A batch holds the blocks of `requests`
// requests (122 segments of 128 KiB and 16 KiB in turn per request, 8 994 816 bytes): one request is the
// form whose descriptors travel in the kernel-argument block, several requests take the table form, whose
// descriptors are fetched from pinned host memory (what the library does for such a batch) or from HBM.
// Every kernel is first run from the host loop (period by HIP events; cheap kernels are bound by the host
// there) and then replayed from a HIP graph of the same launches, where the host does not set the pace.
//
//   mf_batch_phases [requests ...]      default: 1 4
//
// Prints one JSON object per line.  The product kernels are compiled in from their source
// (xcopy.hip is found through the include path), so what is timed is the code the library runs.
#include "xcopy.hip"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <functional>
#include <random>
#include <string>
#include <vector>

using namespace mf;

#define MF_CHECK(call)                                                                                      \
    do {                                                                                                    \
        hipError_t err_ = (call);                                                                           \
        if (err_ != hipSuccess) {                                                                           \
            std::fprintf(stderr, "%s failed: %s (%s:%d)\n", #call, hipGetErrorString(err_), __FILE__, __LINE__); \
            std::exit(1);                                                                                   \
        }                                                                                                   \
    } while (0)

namespace mf {
namespace {

// phase 0: nothing; 1: the table out of the argument block and the owner lookup; 2: + the chunk's loads;
// 3: the lookup and the chunk's stores.  Whole 4 KiB chunks at 16-byte aligned addresses only.
template <int kPhase>
__global__ __launch_bounds__(64) void PhaseKernel(const InlinePlan p, uint32_t *__restrict__ sink)
{
    if (kPhase == 0) {
        if (p.nchunk == 0xFFFFFFFFu) {
            sink[0] = 1;   // never: keeps the argument alive
        }
        return;
    }
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t f0 = p.first[lane];
    const uint32_t f1 = p.first[lane + 64];
    const uint64_t s0 = p.src[lane];
    const uint64_t s1 = p.src[lane + 64];
    const uint64_t d0 = p.dst[lane];
    const uint64_t d1 = p.dst[lane + 64];
    const uint32_t c = blockIdx.x;
    const uint32_t below = __popcll(__ballot(f0 <= c)) + __popcll(__ballot(f1 <= c));
    const uint32_t owner = below - 1;
    const uint32_t row = owner & 63u;
    uint64_t src;
    uint64_t dst;
    uint32_t first;
    if (owner < 64) {
        src = ReadLane64(s0, row);
        dst = ReadLane64(d0, row);
        first = __builtin_amdgcn_readlane(f0, row);
    } else {
        src = ReadLane64(s1, row);
        dst = ReadLane64(d1, row);
        first = __builtin_amdgcn_readlane(f1, row);
    }
    const uint32_t k = c - first;
    if (kPhase == 1) {
        if (src + dst + k == 0x123456789ull) {
            sink[0] = 1;
        }
        return;
    }
    const uint64_t s = src + static_cast<uint64_t>(k) * 4096 + lane * 16;
    const uint64_t d = dst + static_cast<uint64_t>(k) * 4096 + lane * 16;
    if (kPhase == 2) {
        u32x4 acc = {0, 0, 0, 0};
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            acc ^= LoadUnit<true>(s + j * 1024);
        }
        if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9E3779B9u && acc.x == 77u) {
            sink[0] = acc.x;
        }
        return;
    }
    const u32x4 v = {lane, c, 3u, 4u};
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
        StoreUnit<kStoreStream>(d + j * 1024, v);
    }
}

// The same phases for the table form under a pattern: 1: owner by division and its descriptor out of `triples`
// (pinned host memory or HBM); 2: + the chunk's loads; 3: descriptor and the chunk's stores.
template <int kPhase>
__global__ __launch_bounds__(64) void TablePhaseKernel(const uint64_t *__restrict__ triples, const ChunkPattern pattern,
                                                       uint32_t *__restrict__ sink)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t c = blockIdx.x;
    uint32_t seg;
    uint32_t k;
    PatternOwner(pattern, c, seg, k);
    const uint64_t *t = triples + 3ull * seg;
    const uint64_t src = t[0];
    const uint64_t dst = t[1];
    if (kPhase == 1) {
        if (src + dst + k == 0x123456789ull) {
            sink[0] = 1;
        }
        return;
    }
    const uint64_t s = src + static_cast<uint64_t>(k) * 4096 + lane * 16;
    const uint64_t d = dst + static_cast<uint64_t>(k) * 4096 + lane * 16;
    if (kPhase == 2) {
        u32x4 acc = {0, 0, 0, 0};
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            acc ^= LoadUnit<true>(s + j * 1024);
        }
        if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9E3779B9u && acc.x == 77u) {
            sink[0] = acc.x;
        }
        return;
    }
    const u32x4 v = {lane, c, 3u, 4u};
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
        StoreUnit<kStoreStream>(d + j * 1024, v);
    }
}

}  // namespace
}  // namespace mf

namespace {

uint32_t *g_sink = nullptr;

// One batch in every form the rows below launch it in.
struct Batch {
    InlinePlan inlinePlan;              // requests == 1 only
    std::vector<InlinePlan> slices;     // the batch cut into launches of up to 128 segments
    TablePlan pinned;                   // triples in pinned host memory, owner by pattern
    TablePlan hbm;                      // triples in HBM, owner by pattern
    TablePlan grouped;                  // triples, prefix and group map in HBM, no pattern
    TablePlan deepPinned;               // chunks of 16 KiB (what the library takes for 24 to 64 MiB), triples in pinned memory
    TablePlan deepHbm;                  // the same with the triples in HBM
    uint32_t nchunk;
};

typedef std::function<void(const Batch &, hipStream_t)> LaunchFn;

double Median(std::vector<double> v)
{
    std::sort(v.begin(), v.end());
    return v[v.size() / 2];
}

// Period per launch from the host loop: `reps` repetitions of `launches` batches between two events.
double FromHostLoop(const LaunchFn &fn, const std::vector<Batch> &batches, int launches, hipStream_t s)
{
    hipEvent_t e0;
    hipEvent_t e1;
    MF_CHECK(hipEventCreate(&e0));
    MF_CHECK(hipEventCreate(&e1));
    for (int i = 0; i < 3 * launches; ++i) {
        fn(batches[i % batches.size()], s);
    }
    MF_CHECK(hipStreamSynchronize(s));
    std::vector<double> periods;
    for (int r = 0; r < 11; ++r) {
        MF_CHECK(hipEventRecord(e0, s));
        for (int i = 0; i < launches; ++i) {
            fn(batches[i % batches.size()], s);
        }
        MF_CHECK(hipEventRecord(e1, s));
        MF_CHECK(hipStreamSynchronize(s));
        float ms = 0.0f;
        MF_CHECK(hipEventElapsedTime(&ms, e0, e1));
        periods.push_back(ms * 1e3 / launches);
    }
    MF_CHECK(hipEventDestroy(e0));
    MF_CHECK(hipEventDestroy(e1));
    return Median(periods);
}

// The same launches captured once and replayed: the GPU's own period for dependent launches of one queue.
double FromGraph(const LaunchFn &fn, const std::vector<Batch> &batches, int nodes, hipStream_t s)
{
    hipGraph_t graph;
    hipGraphExec_t exec;
    MF_CHECK(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
    for (int i = 0; i < nodes; ++i) {
        fn(batches[i % batches.size()], s);
    }
    MF_CHECK(hipStreamEndCapture(s, &graph));
    MF_CHECK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
    for (int i = 0; i < 5; ++i) {
        MF_CHECK(hipGraphLaunch(exec, s));
    }
    MF_CHECK(hipStreamSynchronize(s));
    hipEvent_t e0;
    hipEvent_t e1;
    MF_CHECK(hipEventCreate(&e0));
    MF_CHECK(hipEventCreate(&e1));
    std::vector<double> periods;
    for (int r = 0; r < 11; ++r) {
        MF_CHECK(hipEventRecord(e0, s));
        for (int i = 0; i < 4; ++i) {
            MF_CHECK(hipGraphLaunch(exec, s));
        }
        MF_CHECK(hipEventRecord(e1, s));
        MF_CHECK(hipStreamSynchronize(s));
        float ms = 0.0f;
        MF_CHECK(hipEventElapsedTime(&ms, e0, e1));
        periods.push_back(ms * 1e3 / (4 * nodes));
    }
    MF_CHECK(hipEventDestroy(e0));
    MF_CHECK(hipEventDestroy(e1));
    MF_CHECK(hipGraphExecDestroy(exec));
    MF_CHECK(hipGraphDestroy(graph));
    return Median(periods);
}

// `count` batches of `requests` x 61 x (128 KiB + 16 KiB) at random 4 KiB-aligned places of the pool, no two segments
// of a batch overlapping.  The tables of all batches sit in one pinned and one device allocation.
std::vector<Batch> MakeBatches(char *pool, uint64_t poolBytes, int count, uint32_t requests)
{
    std::mt19937_64 rng(0xC1 + requests);
    const uint64_t slotBytes = 256 << 10;
    const uint64_t slots = poolBytes / slotBytes;
    const uint32_t nseg = 122 * requests;
    const uint32_t nchunk = 2196 * requests;
    const uint32_t ngroups = GroupCount(nchunk, kGroupShiftMin);
    const uint64_t tableWords64 = 3ull * nseg;                                     // triples
    const uint64_t tableBytes = (tableWords64 * 8 + 4ull * (nseg + 1) + 4ull * (ngroups + 1) + 255) & ~255ull;
    char *hostTables = nullptr;
    char *devTables = nullptr;
    MF_CHECK(hipHostMalloc(&hostTables, tableBytes * count, hipHostMallocDefault));
    MF_CHECK(hipMalloc(&devTables, tableBytes * count));
    std::vector<Batch> batches(count);
    for (int b = 0; b < count; ++b) {
        std::vector<uint32_t> pick;
        std::vector<bool> taken(slots, false);
        while (pick.size() < 2 * nseg) {
            const uint32_t s = static_cast<uint32_t>(rng() % slots);
            if (!taken[s]) {
                taken[s] = true;
                pick.push_back(s);
            }
        }
        uint64_t *triples = reinterpret_cast<uint64_t *>(hostTables + b * tableBytes);
        uint32_t *first = reinterpret_cast<uint32_t *>(triples + tableWords64);
        uint32_t *group = first + nseg + 1;
        uint32_t run = 0;
        for (uint32_t i = 0; i < nseg; ++i) {
            const uint32_t len = (i & 1) != 0 ? 16384 : 131072;
            const uint64_t shift = (rng() % 32) * 4096;
            triples[3 * i] = reinterpret_cast<uint64_t>(pool) + pick[2 * i] * slotBytes + shift;
            triples[3 * i + 1] = reinterpret_cast<uint64_t>(pool) + pick[2 * i + 1] * slotBytes + shift;
            triples[3 * i + 2] = len;
            first[i] = run;
            run += len / 4096;
        }
        first[nseg] = run;
        const uint32_t shiftUsed = BuildGroupMap(first, nseg, group, ngroups + 1);
        Batch &batch = batches[b];
        batch.nchunk = run;
        for (uint32_t at = 0; at < nseg; at += kInlineSegs) {
            InlinePlan plan;
            const uint32_t m = std::min(kInlineSegs, nseg - at);
            uint32_t sliceRun = 0;
            for (uint32_t i = 0; i < kInlineSegs; ++i) {
                if (i < m) {
                    plan.src[i] = triples[3 * (at + i)];
                    plan.dst[i] = triples[3 * (at + i) + 1];
                    plan.len[i] = static_cast<uint32_t>(triples[3 * (at + i) + 2]);
                    plan.first[i] = sliceRun;
                    sliceRun += plan.len[i] / 4096;
                } else {
                    plan.src[i] = plan.dst[i] = 0;
                    plan.len[i] = 0;
                    plan.first[i] = kNoChunk;
                }
            }
            plan.nchunk = sliceRun;
            plan.units = 256;
            batch.slices.push_back(plan);
        }
        batch.inlinePlan = batch.slices[0];
        ChunkPattern pattern{};
        pattern.period = 2;
        pattern.chunksPerPeriod = 36;
        pattern.start[0] = 0;
        pattern.start[1] = 32;
        pattern.start[2] = 36;
        TablePlan plan{};
        plan.nseg = nseg;
        plan.nchunk = run;
        plan.units = 256;
        plan.pattern = pattern;
        plan.triples = triples;
        batch.pinned = plan;
        const char *dev = devTables + b * tableBytes;
        plan.triples = reinterpret_cast<const uint64_t *>(dev);
        batch.hbm = plan;
        {
            TablePlan deep = batch.pinned;
            deep.units = kDeepUnits;
            deep.pattern.chunksPerPeriod = 9;      // 128 KiB: eight chunks of 16 KiB, 16 KiB: one
            deep.pattern.start[1] = 8;
            deep.pattern.start[2] = 9;
            deep.nchunk = nseg / 2 * 9;
            batch.deepPinned = deep;
            deep.triples = reinterpret_cast<const uint64_t *>(dev);
            batch.deepHbm = deep;
        }
        plan.pattern = ChunkPattern{};
        plan.first = reinterpret_cast<const uint32_t *>(dev + tableWords64 * 8);
        plan.group = plan.first + nseg + 1;
        plan.groupShift = shiftUsed;
        batch.grouped = plan;
    }
    MF_CHECK(hipMemcpy(devTables, hostTables, tableBytes * count, hipMemcpyHostToDevice));
    return batches;
}

struct Row {
    std::string name;
    LaunchFn fn;
    bool graph;     // also replayed from a graph
};

template <int kPhase>
void LaunchInlinePhase(const Batch &b, hipStream_t s, uint32_t grid)
{
    hipLaunchKernelGGL((PhaseKernel<kPhase>), dim3(grid != 0 ? grid : b.inlinePlan.nchunk), dim3(64), 0, s, b.inlinePlan, g_sink);
}

template <int kPhase>
void LaunchTablePhase(const TablePlan &plan, hipStream_t s)
{
    hipLaunchKernelGGL((TablePhaseKernel<kPhase>), dim3(plan.nchunk), dim3(64), 0, s, plan.triples, plan.pattern, g_sink);
}

void LaunchInlineProduct(const InlinePlan &plan, hipStream_t s, bool held, bool anyOrder)
{
    const uint32_t ticks = held ? HoldTicks(HoldNanosFor(plan.nchunk, plan.nchunk, plan.units, false)) : 0u;
    if (anyOrder) {   // never under stream capture
        hipExtLaunchKernelGGL((XcopyInlineKernel<true, kStoreStream>), dim3(plan.nchunk), dim3(64), 0, s, nullptr, nullptr,
                              hipExtAnyOrderLaunch, plan, 0u);
    } else if (ticks != 0) {
        hipLaunchKernelGGL((XcopyInlineKernel<true, kStoreStream, true>), dim3(plan.nchunk), dim3(64), 0, s, plan, ticks);
    } else {
        hipLaunchKernelGGL((XcopyInlineKernel<true, kStoreStream>), dim3(plan.nchunk), dim3(64), 0, s, plan, 0u);
    }
}

// What the library launches for a batch of 24 to 64 MiB: 16 KiB per wave, sixteen loads per lane, stores held back
// (2.4 us longer where every workgroup first fetches its descriptor over the link).
void LaunchTableDeep(const TablePlan &plan, hipStream_t s, bool pinned)
{
    const uint32_t nanos = HoldNanosFor(plan.nchunk, plan.nchunk, plan.units, false);
    const uint32_t ticks = HoldTicks(nanos != 0 && pinned ? nanos + 2400 : nanos);
    hipLaunchKernelGGL((XcopyTableKernel<true, kStoreStream, false, kHoldDeep>), dim3(plan.nchunk), dim3(64), 0, s, plan, ticks);
}

void LaunchTableProduct(const TablePlan &plan, hipStream_t s)
{
    hipLaunchKernelGGL((XcopyTableKernel<true, kStoreStream, false>), dim3(plan.nchunk), dim3(64), 0, s, plan, 0u);
}

void Measure(uint32_t requests, char *pool, uint64_t poolBytes, hipStream_t s)
{
    const int tables = requests <= 2 ? 64 : 16;    // the touched set stays beyond the 256 MiB last-level cache
    const std::vector<Batch> batches = MakeBatches(pool, poolBytes, tables, requests);
    std::vector<Row> rows;
    if (requests == 1) {
        rows.push_back({"empty_kernel_one_workgroup", [](const Batch &b, hipStream_t st) { LaunchInlinePhase<0>(b, st, 1); }, true});
        rows.push_back({"empty_kernel", [](const Batch &b, hipStream_t st) { LaunchInlinePhase<0>(b, st, 0); }, true});
        rows.push_back({"descriptor_lookup", [](const Batch &b, hipStream_t st) { LaunchInlinePhase<1>(b, st, 0); }, true});
        rows.push_back({"lookup_and_loads", [](const Batch &b, hipStream_t st) { LaunchInlinePhase<2>(b, st, 0); }, true});
        rows.push_back({"lookup_and_stores", [](const Batch &b, hipStream_t st) { LaunchInlinePhase<3>(b, st, 0); }, true});
        rows.push_back({"product_kernel_stores_not_held",
                        [](const Batch &b, hipStream_t st) { LaunchInlineProduct(b.inlinePlan, st, false, false); }, true});
        rows.push_back({"product_kernel", [](const Batch &b, hipStream_t st) { LaunchInlineProduct(b.inlinePlan, st, true, false); }, true});
    } else {
        rows.push_back({"empty_kernel", [](const Batch &b, hipStream_t st) {
                            hipLaunchKernelGGL((PhaseKernel<0>), dim3(b.nchunk), dim3(64), 0, st, b.inlinePlan, g_sink);
                        }, true});
        rows.push_back({"descriptor_from_pinned_host", [](const Batch &b, hipStream_t st) { LaunchTablePhase<1>(b.pinned, st); }, true});
        rows.push_back({"descriptor_from_hbm", [](const Batch &b, hipStream_t st) { LaunchTablePhase<1>(b.hbm, st); }, true});
        rows.push_back({"hbm_descriptor_and_loads", [](const Batch &b, hipStream_t st) { LaunchTablePhase<2>(b.hbm, st); }, true});
        rows.push_back({"hbm_descriptor_and_stores", [](const Batch &b, hipStream_t st) { LaunchTablePhase<3>(b.hbm, st); }, true});
        rows.push_back({"pinned_descriptor_and_loads", [](const Batch &b, hipStream_t st) { LaunchTablePhase<2>(b.pinned, st); }, true});
        rows.push_back({"product_table_kernel_pinned_descriptors",
                        [](const Batch &b, hipStream_t st) { LaunchTableProduct(b.pinned, st); }, true});
        rows.push_back({"product_table_kernel_hbm_descriptors", [](const Batch &b, hipStream_t st) { LaunchTableProduct(b.hbm, st); }, true});
        rows.push_back({"product_table_kernel_group_map", [](const Batch &b, hipStream_t st) { LaunchTableProduct(b.grouped, st); }, true});
        rows.push_back({"product_table_kernel_16KiB_chunks_held_pinned_descriptors",
                        [](const Batch &b, hipStream_t st) { LaunchTableDeep(b.deepPinned, st, true); }, true});
        rows.push_back({"product_table_kernel_16KiB_chunks_held_hbm_descriptors",
                        [](const Batch &b, hipStream_t st) { LaunchTableDeep(b.deepHbm, st, false); }, true});
        rows.push_back({"inline_launches_first_ordered_rest_any_order", [](const Batch &b, hipStream_t st) {
                            for (size_t i = 0; i < b.slices.size(); ++i) {
                                LaunchInlineProduct(b.slices[i], st, false, i != 0);
                            }
                        }, false});
        rows.push_back({"inline_launches_ordered_held", [](const Batch &b, hipStream_t st) {
                            for (size_t i = 0; i < b.slices.size(); ++i) {
                                LaunchInlineProduct(b.slices[i], st, true, false);
                            }
                        }, true});
    }
    const int launches = requests <= 2 ? 400 : 200;
    std::printf("{\"workload\": \"KV blocks of %u request(s) per batch: %u segments, %u bytes, %d tables in a 4 GiB pool, %u single-wave "
                "workgroups\", \"unit\": \"us per batch, dependent launches on one stream\", \"phases\": {",
                requests, 122 * requests, 8994816 * requests, tables, batches[0].nchunk);
    bool firstRow = true;
    for (const Row &row : rows) {
        const double host = FromHostLoop(row.fn, batches, launches, s);   // also the first launches of the kernel: a graph is only captured afterwards
        std::printf("%s\"%s\": {\"host_loop\": %.2f", firstRow ? "" : ", ", row.name.c_str(), host);
        if (row.graph) {
            std::printf(", \"graph_replay\": %.2f", FromGraph(row.fn, batches, 256 / static_cast<int>(requests), s));
        }
        std::printf("}");
        std::fflush(stdout);
        firstRow = false;
    }
    std::printf("}}\n");
    std::fflush(stdout);
    MF_CHECK(hipStreamSynchronize(s));
}

}  // namespace

int main(int argc, char **argv)
{
    std::vector<uint32_t> requests;
    for (int i = 1; i < argc; ++i) {
        const long r = std::strtol(argv[i], nullptr, 10);
        if (r < 1 || r > 16) {
            std::fprintf(stderr, "requests per batch: 1 ... 16, got %s\n", argv[i]);
            return 2;
        }
        requests.push_back(static_cast<uint32_t>(r));
    }
    if (requests.empty()) {
        requests = {1, 4};
    }
    MF_CHECK(hipSetDevice(0));
    const uint64_t poolBytes = 4ull << 30;
    char *pool = nullptr;
    MF_CHECK(hipMalloc(&pool, poolBytes));
    MF_CHECK(hipMemset(pool, 0x5A, poolBytes));
    MF_CHECK(hipMalloc(&g_sink, 256));
    MF_CHECK(hipDeviceSynchronize());
    hipStream_t s;
    MF_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    for (uint32_t r : requests) {
        Measure(r, pool, poolBytes, s);
    }
    MF_CHECK(hipStreamSynchronize(s));
    MF_CHECK(hipFree(g_sink));
    MF_CHECK(hipFree(pool));
    return 0;
}
