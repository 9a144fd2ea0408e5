// mf_batch_phases: a stand-alone measurement program (not part of the data plane, nothing links it).
// It takes the 122-segment KV batch apart on one GPU: what a launch that waits for its predecessor costs,
// what the descriptor lookup, the loads and the stores of a 9 MB batch add, and what the product kernel
// needs (with its stores held back until the loads of the launch are out, as the library launches this
// batch, and without), each as the period per launch of dependent launches on one stream.  Every kernel is first run
// from the host loop (period by HIP events; cheap kernels are bound by the host there) and then
// replayed from a HIP graph of the same launches, where the host does not set the pace.
// Prints one JSON object.  The product kernel is compiled in from its source, so what is timed is the
// code the library runs.
#include "xcopy.hip"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <random>
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

}  // namespace
}  // namespace mf

namespace {

uint32_t *g_sink = nullptr;

typedef void (*LaunchFn)(const InlinePlan &, uint32_t grid, hipStream_t);
template <int kPhase>
void LaunchPhase(const InlinePlan &plan, uint32_t grid, hipStream_t s)
{
    hipLaunchKernelGGL((PhaseKernel<kPhase>), dim3(grid != 0 ? grid : plan.nchunk), dim3(64), 0, s, plan, g_sink);
}
void LaunchProduct(const InlinePlan &plan, uint32_t grid, hipStream_t s)
{
    hipLaunchKernelGGL((XcopyInlineKernel<true, kStoreStream>), dim3(grid != 0 ? grid : plan.nchunk), dim3(64), 0, s, plan, 0u);
}
// the same with the stores held back for as long as the library's rule says for this grid
void LaunchProductHeld(const InlinePlan &plan, uint32_t grid, hipStream_t s)
{
    const uint32_t ticks = HoldTicks(HoldNanosFor(plan.nchunk, plan.nchunk, plan.units, false));
    hipLaunchKernelGGL((XcopyInlineKernel<true, kStoreStream, true>), dim3(grid != 0 ? grid : plan.nchunk), dim3(64), 0, s, plan, ticks);
}

double Median(std::vector<double> v)
{
    std::sort(v.begin(), v.end());
    return v[v.size() / 2];
}

// Period per launch from the host loop: `reps` repetitions of `launches` launches between two events.
double FromHostLoop(LaunchFn fn, const std::vector<InlinePlan> &plans, uint32_t grid, hipStream_t s)
{
    hipEvent_t e0;
    hipEvent_t e1;
    MF_CHECK(hipEventCreate(&e0));
    MF_CHECK(hipEventCreate(&e1));
    const int launches = 400;
    for (int i = 0; i < 1500; ++i) {
        fn(plans[i % plans.size()], grid, s);
    }
    MF_CHECK(hipStreamSynchronize(s));
    std::vector<double> periods;
    for (int r = 0; r < 11; ++r) {
        MF_CHECK(hipEventRecord(e0, s));
        for (int i = 0; i < launches; ++i) {
            fn(plans[i % plans.size()], grid, s);
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
double FromGraph(LaunchFn fn, const std::vector<InlinePlan> &plans, uint32_t grid, hipStream_t s)
{
    const int nodes = 256;
    hipGraph_t graph;
    hipGraphExec_t exec;
    MF_CHECK(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
    for (int i = 0; i < nodes; ++i) {
        fn(plans[i % plans.size()], grid, s);
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

// 64 tables of 61 x (128 KiB + 16 KiB) at random 4 KiB-aligned places of the pool, no two segments of a table overlapping.
std::vector<InlinePlan> MakePlans(char *pool, uint64_t poolBytes, int count)
{
    std::mt19937_64 rng(0xC1);
    const uint64_t slotBytes = 256 << 10;
    const uint64_t slots = poolBytes / slotBytes;
    std::vector<InlinePlan> plans(count);
    for (int b = 0; b < count; ++b) {
        std::vector<uint32_t> pick;
        while (pick.size() < 244) {
            const uint32_t s = static_cast<uint32_t>(rng() % slots);
            if (std::find(pick.begin(), pick.end(), s) == pick.end()) {
                pick.push_back(s);
            }
        }
        InlinePlan &plan = plans[b];
        uint32_t run = 0;
        for (uint32_t i = 0; i < kInlineSegs; ++i) {
            if (i < 122) {
                const uint32_t len = (i & 1) != 0 ? 16384 : 131072;
                const uint64_t shift = (rng() % 32) * 4096;
                plan.src[i] = reinterpret_cast<uint64_t>(pool) + pick[2 * i] * slotBytes + shift;
                plan.dst[i] = reinterpret_cast<uint64_t>(pool) + pick[2 * i + 1] * slotBytes + shift;
                plan.len[i] = len;
                plan.first[i] = run;
                run += len / 4096;
            } else {
                plan.src[i] = plan.dst[i] = 0;
                plan.len[i] = 0;
                plan.first[i] = kNoChunk;
            }
        }
        plan.nchunk = run;
        plan.units = 256;
    }
    return plans;
}

}  // namespace

int main()
{
    MF_CHECK(hipSetDevice(0));
    const uint64_t poolBytes = 4ull << 30;
    char *pool = nullptr;
    MF_CHECK(hipMalloc(&pool, poolBytes));
    MF_CHECK(hipMemset(pool, 0x5A, poolBytes));
    MF_CHECK(hipMalloc(&g_sink, 256));
    MF_CHECK(hipDeviceSynchronize());
    hipStream_t s;
    MF_CHECK(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    const std::vector<InlinePlan> plans = MakePlans(pool, poolBytes, 64);
    struct Row {
        const char *name;
        LaunchFn fn;
        uint32_t grid;
    };
    const Row rows[] = {
        {"empty_kernel_one_workgroup", LaunchPhase<0>, 1},   {"empty_kernel", LaunchPhase<0>, 0},
        {"descriptor_lookup", LaunchPhase<1>, 0},            {"lookup_and_loads", LaunchPhase<2>, 0},
        {"lookup_and_stores", LaunchPhase<3>, 0},            {"product_kernel_stores_not_held", LaunchProduct, 0},
        {"product_kernel", LaunchProductHeld, 0},
    };
    std::printf("{\"workload\": \"122-segment KV batch, 64 tables in a 4 GiB pool, grid %u single-wave workgroups\", "
                "\"unit\": \"us per launch, dependent launches on one stream\", \"phases\": {", plans[0].nchunk);
    bool firstRow = true;
    for (const Row &row : rows) {
        const double host = FromHostLoop(row.fn, plans, row.grid, s);   // also the first launches of the kernel: a graph is only captured afterwards
        const double graph = FromGraph(row.fn, plans, row.grid, s);
        std::printf("%s\"%s\": {\"host_loop\": %.2f, \"graph_replay\": %.2f}", firstRow ? "" : ", ", row.name, host, graph);
        firstRow = false;
    }
    std::printf("}}\n");
    MF_CHECK(hipStreamSynchronize(s));
    MF_CHECK(hipFree(g_sink));
    MF_CHECK(hipFree(pool));
    return 0;
}
