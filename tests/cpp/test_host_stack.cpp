// CPU unit tests of the host stack over the fake runtime (tests/cpp/fake_rt.cpp).
// Part 1 restates the behaviours the reference pins for its operator set in
// test/ut/testcase/hybm/data_operator/hybm_compose_data_op_test.cpp (init order and rollback,
// intra-node engine first, fallback to the next engine on failure for copy / batch / async,
// Wait only through the intra-node engine).  Part 2 drives the C API end to end and compares
// bytes with memcpy.  Part 3 does the same for the transfer front-end.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <atomic>
#include <thread>
#include <vector>

#include <sched.h>

#include "../../include/mf_hip_dataplane_internal.h"
#include "../../include/mf_xcopy_api.h"
#include "../../memfabric_hybrid_amd/csrc/host/compose_data_op.h"
#include "../../memfabric_hybrid_amd/csrc/host/mf_log.h"
#include "../../memfabric_hybrid_amd/csrc/host/xcopy_engine.h"
#include "../../memfabric_hybrid_amd/csrc/host/host_copy.h"

extern "C" uint64_t fake_rt_launches(void);
extern "C" uint32_t fake_rt_last_hold(void);
extern "C" uint32_t fake_rt_last_rect_mates(void);
extern "C" uint32_t fake_rt_rect_windowed_launches(void);
extern "C" void fake_rt_queue_answers(int mode);
extern "C" int fake_rt_last_combine_paced(void);
extern "C" uint64_t fake_rt_signals(void);
extern "C" uint64_t fake_rt_stream_syncs(void);
extern "C" uint32_t fake_rt_last_window(void);
extern "C" void fake_rt_seal(void);
extern "C" void fake_rt_fail_launches(int n);
#include "../../include/mf_hip_copy_extend.h"
extern "C" uint64_t fake_rt_violations(void);
extern "C" void fake_rt_skip_copies(int on);
extern "C" uint64_t fake_rt_stream_waits(void);
extern "C" void fake_rt_set_calibration(const float *us);
extern "C" const uint32_t *fake_rt_calibration_holds(void);
extern "C" uint32_t fake_rt_last_table_shift(void);
extern "C" uint32_t fake_rt_last_table_hold(void);
extern "C" uint64_t fake_rt_group_map_errors(void);
extern "C" uint64_t fake_rt_in_flight(void);

using namespace mf;
using ock::mf::DataOperatorPtr;
using ock::mf::ExtOptions;

static int g_failed = 0;
#define CHECK(cond)                                                             \
    do {                                                                        \
        if (!(cond)) {                                                          \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);       \
            ++g_failed;                                                         \
        }                                                                       \
    } while (0)

struct MockOp : ock::mf::DataOperator {
    int initRet = 0, copyRet = 0, batchRet = 0, asyncRet = 0, waitRet = 0;
    int inits = 0, uninits = 0, copies = 0, batches = 0, asyncs = 0, waits = 0, cleanups = 0;
    uint32_t lastBatchSize = 0, lastSrcRank = 99, lastDstRank = 99;
    ock::mf::Result Initialize() noexcept override { ++inits; return initRet; }
    void UnInitialize() noexcept override { ++uninits; }
    ock::mf::Result DataCopy(hybm_copy_params &, hybm_data_copy_direction, const ExtOptions &) noexcept override { ++copies; return copyRet; }
    ock::mf::Result BatchDataCopy(hybm_batch_copy_params &p, hybm_data_copy_direction, const ExtOptions &o) noexcept override
    {
        ++batches;
        lastBatchSize = p.batchSize;
        lastSrcRank = o.srcRankId;
        lastDstRank = o.destRankId;
        return batchRet;
    }
    ock::mf::Result DataCopyAsync(hybm_copy_params &, hybm_data_copy_direction, const ExtOptions &) noexcept override { ++asyncs; return asyncRet; }
    ock::mf::Result Wait(int32_t) noexcept override { ++waits; return waitRet; }
    void CleanUp() noexcept override { ++cleanups; }
};

static hybm_options Options(uint32_t ops)
{
    hybm_options o{};
    o.bmType = HYBM_TYPE_HOST_INITIATE;
    o.bmDataOpType = static_cast<hybm_data_op_type>(ops);
    o.rankCount = 1;
    return o;
}

static void TestCompose()
{
    auto a = std::make_shared<MockOp>();
    auto b = std::make_shared<MockOp>();
    auto c = std::make_shared<MockOp>();
    OperatorFactory f;
    f.intraNode = [&]() -> DataOperatorPtr { return a; };
    f.deviceRdma = [&]() -> DataOperatorPtr { return b; };
    f.hostNet = [&]() -> DataOperatorPtr { return c; };
    const uint32_t all = HYBM_DOP_TYPE_SDMA | HYBM_DOP_TYPE_DEVICE_RDMA | HYBM_DOP_TYPE_HOST_RDMA;
    hybm_copy_params cp{reinterpret_cast<void *>(0x1000), reinterpret_cast<void *>(0x2000), 16};
    void *srcs[3] = {cp.src, cp.src, cp.src};
    void *dsts[3] = {cp.dest, cp.dest, cp.dest};
    uint64_t lens[3] = {1, 2, 3};
    hybm_batch_copy_params bp{srcs, dsts, lens, 3};
    ExtOptions opt{};
    opt.srcRankId = 0;
    opt.destRankId = 0;
    {
        // only requested engines are created; device-initiated pools create none
        ComposeDataOp only(Options(HYBM_DOP_TYPE_SDMA), f);
        CHECK(only.Initialize() == BM_OK && a->inits == 1 && b->inits == 0 && c->inits == 0);
        hybm_options ai = Options(all);
        ai.bmType = HYBM_TYPE_AI_CORE_INITIATE;
        ComposeDataOp none(ai, f);
        CHECK(none.Initialize() == BM_OK && a->inits == 1);
        CHECK(none.DataCopy(cp, HYBM_GLOBAL_DEVICE_TO_GLOBAL_DEVICE, opt) == BM_INVALID_PARAM);
        CHECK(none.Wait(0) == BM_ERROR);
    }
    {
        // a later engine failing to start drops the earlier ones and reports its code
        *a = MockOp{};
        *b = MockOp{};
        *c = MockOp{};
        c->initRet = BM_ERROR;
        ComposeDataOp op(Options(all), f);
        CHECK(op.Initialize() == BM_ERROR);
        CHECK(a->inits == 1 && b->inits == 1 && c->inits == 1);
        CHECK(op.DataCopy(cp, HYBM_GLOBAL_DEVICE_TO_GLOBAL_DEVICE, opt) == BM_INVALID_PARAM);  // nothing left
    }
    {
        *a = MockOp{};
        *b = MockOp{};
        *c = MockOp{};
        ComposeDataOp op(Options(all), f);
        CHECK(op.Initialize() == BM_OK);
        // first engine wins
        CHECK(op.DataCopy(cp, HYBM_GLOBAL_DEVICE_TO_GLOBAL_DEVICE, opt) == BM_OK);
        CHECK(a->copies == 1 && b->copies == 0 && c->copies == 0);
        // failure falls through, in order
        a->copyRet = BM_ERROR;
        CHECK(op.DataCopy(cp, HYBM_GLOBAL_DEVICE_TO_GLOBAL_DEVICE, opt) == BM_OK);
        CHECK(a->copies == 2 && b->copies == 1 && c->copies == 0);
        b->copyRet = BM_TIMEOUT;
        CHECK(op.DataCopy(cp, HYBM_GLOBAL_DEVICE_TO_GLOBAL_DEVICE, opt) == BM_OK);
        CHECK(c->copies == 1);
        c->copyRet = BM_NOT_SUPPORTED;
        CHECK(op.DataCopy(cp, HYBM_GLOBAL_DEVICE_TO_GLOBAL_DEVICE, opt) == BM_NOT_SUPPORTED);  // last error is reported
        // batch: whole batch to the intra-node engine, per rank pair to the others
        CHECK(op.BatchDataCopy(bp, HYBM_GLOBAL_DEVICE_TO_GLOBAL_DEVICE, opt) == BM_OK);
        CHECK(a->batches == 1 && a->lastBatchSize == 3 && b->batches == 0);
        a->batchRet = BM_ERROR;
        ExtOptions grouped = opt;
        grouped.groupMap[{0, 1}] = {0, 2};
        grouped.groupMap[{2, 0}] = {1};
        CHECK(op.BatchDataCopy(bp, HYBM_GLOBAL_DEVICE_TO_GLOBAL_DEVICE, grouped) == BM_OK);
        CHECK(b->batches == 2 && c->batches == 0);
        b->batchRet = BM_ERROR;
        CHECK(op.BatchDataCopy(bp, HYBM_GLOBAL_DEVICE_TO_GLOBAL_DEVICE, grouped) == BM_OK);
        CHECK(c->batches == 2);
        // an ungrouped batch reaches a network engine whole, between the two ranks named
        c->batches = 0;
        CHECK(op.BatchDataCopy(bp, HYBM_GLOBAL_DEVICE_TO_GLOBAL_DEVICE, opt) == BM_OK);
        CHECK(c->batches == 1 && c->lastBatchSize == 3 && c->lastSrcRank == 0 && c->lastDstRank == 0);
        // async: same fallback
        CHECK(op.DataCopyAsync(cp, HYBM_GLOBAL_DEVICE_TO_GLOBAL_DEVICE, opt) == BM_OK && a->asyncs == 1 && b->asyncs == 0);
        a->asyncRet = BM_ERROR;
        CHECK(op.DataCopyAsync(cp, HYBM_GLOBAL_DEVICE_TO_GLOBAL_DEVICE, opt) == BM_OK && b->asyncs == 1);
        // wait is routed to the intra-node engine only
        CHECK(op.Wait(7) == BM_OK && a->waits == 1 && b->waits == 0 && c->waits == 0);
        a->waitRet = BM_TIMEOUT;
        CHECK(op.Wait(7) == BM_TIMEOUT);
        op.CleanUp();
        CHECK(a->cleanups == 1 && b->cleanups == 1 && c->cleanups == 1);
        op.UnInitialize();
        CHECK(a->uninits == 1 && b->uninits == 1 && c->uninits == 1);
    }
    {
        // without the intra-node engine there is nothing to wait on
        *b = MockOp{};
        ComposeDataOp op(Options(HYBM_DOP_TYPE_DEVICE_RDMA), f);
        CHECK(op.Initialize() == BM_OK);
        CHECK(op.Wait(0) == BM_ERROR);
        CHECK(op.DataCopy(cp, HYBM_GLOBAL_DEVICE_TO_GLOBAL_DEVICE, opt) == BM_OK && b->copies == 1);
    }
}

static void Fill(std::vector<uint8_t> &v, uint32_t seed)
{
    std::mt19937 rng(seed);
    for (auto &x : v) {
        x = static_cast<uint8_t>(rng());
    }
}

static void TestCApi()
{
    const uint64_t pool = 64ull << 20;
    smem_bm_config_t cfg;
    CHECK(smem_bm_config_init(&cfg) == SM_OK);
    CHECK(smem_bm_init("tcp://127.0.0.1:1", 2, 0, &cfg) == SM_ERROR);  // a world of one only
    CHECK(smem_bm_init("tcp://127.0.0.1:1", 1, 0, &cfg) == SM_OK);
    CHECK(smem_bm_init("tcp://127.0.0.1:1", 1, 0, &cfg) == SM_OK);     // idempotent
    CHECK(smem_bm_get_rank_id() == 0);
    smem_bm_t bm = smem_bm_create(2, 1, SMEMB_DATA_OP_SDMA, pool, pool, 0);
    CHECK(bm != nullptr);
    CHECK(smem_bm_create(2, 1, SMEMB_DATA_OP_SDMA, pool, pool, 0) == nullptr);
    CHECK(smem_bm_join(bm, 0) == SM_OK);
    uint8_t *dev = static_cast<uint8_t *>(smem_bm_ptr_by_mem_type(bm, SMEM_MEM_TYPE_DEVICE, 0));
    uint8_t *host = static_cast<uint8_t *>(smem_bm_ptr_by_mem_type(bm, SMEM_MEM_TYPE_HOST, 0));
    CHECK(dev != nullptr && host != nullptr);
    CHECK(smem_bm_ptr_by_mem_type(bm, SMEM_MEM_TYPE_DEVICE, 1) == nullptr);
    CHECK(smem_bm_get_local_mem_size_by_mem_type(bm, SMEM_MEM_TYPE_HOST) == pool);
    CHECK(smem_bm_get_rank_id_by_gva(bm, dev + 5) == 0);
    CHECK(smem_bm_get_rank_id_by_gva(bm, &cfg) == UINT32_MAX);
    CHECK(mf_va_infer_direction(reinterpret_cast<uint64_t>(host), reinterpret_cast<uint64_t>(dev)) == HYBM_GLOBAL_HOST_TO_GLOBAL_DEVICE);

    std::vector<uint8_t> ref(pool);
    Fill(ref, 1);
    std::memcpy(host, ref.data(), pool);
    std::memset(dev, 0, pool);
    std::vector<uint8_t> model(pool, 0);

    // 300 ragged segments (table form) host pool -> device pool
    std::mt19937_64 rng(7);
    std::vector<void *> s, d;
    std::vector<uint64_t> l;
    uint64_t cursor = 0;
    for (int i = 0; i < 300; ++i) {
        uint64_t len = i % 11 == 0 ? 0 : rng() % 50000;
        uint64_t so = rng() % (pool - 60000);
        s.push_back(host + so);
        d.push_back(dev + cursor + (i % 16));
        l.push_back(len);
        std::memcpy(model.data() + cursor + (i % 16), ref.data() + so, len);
        cursor += len + 64;
    }
    smem_batch_copy_params bp{s.data(), d.data(), l.data(), 300};
    const uint64_t before = fake_rt_launches();
    CHECK(smem_bm_copy_batch(bm, &bp, SMEMB_COPY_G2G, 0) == SM_OK);
    CHECK(fake_rt_launches() - before == 2);  // descriptor staging + table kernel
    CHECK(std::memcmp(dev, model.data(), pool) == 0);
    // the same as an inline batch (first 100), asynchronous + wait, AUTO direction
    std::memset(dev, 0, pool);
    bp.batchSize = 100;
    CHECK(smem_bm_copy_batch(bm, &bp, SMEMB_COPY_AUTO, ASYNC_COPY_FLAG) == SM_OK);
    CHECK(smem_bm_wait(bm) == SM_OK);
    std::vector<uint8_t> model2(pool, 0);
    for (int i = 0; i < 100; ++i) {
        std::memcpy(model2.data() + (static_cast<uint8_t *>(d[i]) - dev), ref.data() + (static_cast<uint8_t *>(s[i]) - host), l[i]);
    }
    CHECK(std::memcmp(dev, model2.data(), pool) == 0);
    // pageable local memory: staged in rounds (70 MiB through a 32 MiB area would not fit the pool; use 40 MiB)
    std::vector<uint8_t> big(40u << 20);
    Fill(big, 3);
    smem_copy_params one{big.data(), dev + 3, big.size()};
    CHECK(smem_bm_copy(bm, &one, SMEMB_COPY_H2G, 0) == SM_OK);
    CHECK(std::memcmp(dev + 3, big.data(), big.size()) == 0);
    std::vector<uint8_t> back(big.size());
    smem_copy_params two{dev + 3, back.data(), back.size()};
    CHECK(smem_bm_copy(bm, &two, SMEMB_COPY_G2H, 0) == SM_OK);
    CHECK(back == big);
    // host pool <-> pageable: plain CPU copy
    smem_copy_params three{big.data(), host + 9, 1000};
    CHECK(smem_bm_copy(bm, &three, SMEMB_COPY_H2GH, 0) == SM_OK);
    CHECK(std::memcmp(host + 9, big.data(), 1000) == 0);
    // errors
    smem_copy_params bad{dev, dev + pool - 8, 16};
    CHECK(smem_bm_copy(bm, &bad, SMEMB_COPY_G2G, 0) == SM_INVALID_PARAM);  // leaves the window: unclassifiable
    bad = {dev, host, 0};
    CHECK(smem_bm_copy(bm, &bad, SMEMB_COPY_G2G, 0) == SM_INVALID_PARAM);
    bad = {&cfg, host, 16};
    CHECK(smem_bm_copy(bm, &bad, SMEMB_COPY_L2GH, 0) == SM_INVALID_PARAM);  // L2GH does not override the source
    CHECK(smem_bm_copy(bm, &bad, SMEMB_COPY_BUTT, 0) == SM_INVALID_PARAM);
    // a size that wraps round the address space is refused, not cut into 2^34 pieces
    bad = {dev + 4096, host, ~0ull - reinterpret_cast<uint64_t>(dev) - 100};
    CHECK(smem_bm_copy(bm, &bad, SMEMB_COPY_G2G, 0) == SM_INVALID_PARAM);
    bad = {dev + 4096, host, ~0ull};
    CHECK(smem_bm_copy(bm, &bad, SMEMB_COPY_G2G, 0) == SM_INVALID_PARAM);
    {
        void *ws[1] = {dev + 4096};
        void *wd[1] = {host};
        uint64_t wl[1] = {~0ull - 5};
        smem_batch_copy_params wrap{ws, wd, wl, 1};
        CHECK(smem_bm_copy_batch(bm, &wrap, SMEMB_COPY_G2G, 0) != SM_OK);
    }
    // 2-D copy, aligned and unaligned geometry
    std::memset(dev, 0, pool);
    mf_copy2d_desc rects[2] = {
        {reinterpret_cast<uint64_t>(host), reinterpret_cast<uint64_t>(dev), 896, 100, 896, 1792},
        {reinterpret_cast<uint64_t>(host) + 5, reinterpret_cast<uint64_t>(dev) + (1u << 20) + 3, 100, 50, 160, 300},
    };
    CHECK(mf_xcopy_2d_batch(rects, 2, MF_ROUTE_FROM_HOST, nullptr) == BM_OK);
    bool ok = true;
    for (int r = 0; r < 100; ++r) {
        ok = ok && std::memcmp(dev + r * 1792, host + r * 896, 896) == 0;
    }
    for (int r = 0; r < 50; ++r) {
        ok = ok && std::memcmp(dev + (1u << 20) + 3 + r * 300, host + 5 + r * 160, 100) == 0;
    }
    CHECK(ok);
    // two rectangles side by side in the destination become mates and share their chunks in turn; a third of another
    // height and one whose destination does not continue the row stay alone; every row still arrives
    std::memset(dev, 0, pool);
    const uint64_t h0 = reinterpret_cast<uint64_t>(host);
    const uint64_t d0 = reinterpret_cast<uint64_t>(dev);
    mf_copy2d_desc sideBySide[5] = {
        {h0, d0, 896, 101, 896, 1792},
        {h0 + 101 * 896, d0 + 896, 896, 101, 896, 1792},
        {h0 + 202 * 896, d0 + (1u << 20), 896, 77, 896, 1792},
        {h0 + 300 * 896, d0 + (1u << 20) + 896, 896, 76, 896, 1792},
        {h0 + 400 * 896, d0 + (2u << 20), 4736, 9, 4736, 9472},
    };
    CHECK(mf_xcopy_2d_batch(sideBySide, 5, MF_ROUTE_FROM_HOST, nullptr) == BM_OK);
    CHECK(fake_rt_last_rect_mates() == 2);
    ok = true;
    for (int r = 0; r < 101; ++r) {
        ok = ok && std::memcmp(dev + r * 1792, host + r * 896, 896) == 0;
        ok = ok && std::memcmp(dev + r * 1792 + 896, host + (101 + r) * 896, 896) == 0;
    }
    for (int r = 0; r < 77; ++r) {
        ok = ok && std::memcmp(dev + (1u << 20) + r * 1792, host + (202 + r) * 896, 896) == 0;
    }
    for (int r = 0; r < 76; ++r) {
        ok = ok && std::memcmp(dev + (1u << 20) + 896 + r * 1792, host + (300 + r) * 896, 896) == 0;
    }
    for (int r = 0; r < 9; ++r) {
        ok = ok && std::memcmp(dev + (2u << 20) + r * 9472, host + 400 * 896 + r * 4736, 4736) == 0;
    }
    CHECK(ok);
    CHECK(smem_bm_leave(bm, 0) == SM_OK);
    smem_bm_destroy(bm);
    CHECK(smem_bm_wait(bm) == SM_INVALID_PARAM);  // handle is gone
    smem_bm_uninit(0);
    CHECK(smem_bm_wait(bm) == SM_NOT_INITIALIZED);
}

// Part 3: the transfer front-end.  Error codes are those the reference's unit tests pin
// (test/ut/testcase/smem/smem_trans_test.cpp:145-168 create, :170-219 register, :1016-1098 batch
// write); the data cases follow its two-object write / read tests (:272-373, :655-779) with both
// objects in this process.
// Launch cost per CPU and the pinning built on it: every CPU of the thread's set is measured, the set is put back,
// and the pinned set is a part of it.
static void TestHostLaunchCosts()
{
    CHECK(hybm_init(0, 0) == BM_OK);
    cpu_set_t before;
    CHECK(sched_getaffinity(0, sizeof(before), &before) == 0);
    uint32_t cpus[1024];
    float micros[1024];
    const int32_t n = mf_host_launch_costs(cpus, micros, 1024);
    CHECK(n == CPU_COUNT(&before));
    cpu_set_t after;
    CHECK(sched_getaffinity(0, sizeof(after), &after) == 0);
    CHECK(CPU_EQUAL(&before, &after));
    for (int32_t i = 0; i < n; ++i) {
        CHECK(CPU_ISSET(static_cast<int>(cpus[i]), &before) && micros[i] >= 0.0f);
    }
    CHECK(mf_host_launch_costs(cpus, micros, 1) == 1);          // no more than there is room for
    CHECK(mf_host_launch_costs(nullptr, micros, 4) == BM_INVALID_PARAM);
    const int32_t kept = mf_pin_thread_near_gpu();
    CHECK(kept >= 1 && kept <= n);
    CHECK(sched_getaffinity(0, sizeof(after), &after) == 0);
    CHECK(CPU_COUNT(&after) == kept);
    for (int cpu = 0; cpu < CPU_SETSIZE; ++cpu) {
        CHECK(!CPU_ISSET(cpu, &after) || CPU_ISSET(cpu, &before));
    }
    CHECK(sched_setaffinity(0, sizeof(before), &before) == 0);
    hybm_uninit();
}

// A wait behind a short queue of copies polls a word that a one-lane launch stores; behind a long queue, behind
// kernels of the other entry points and behind tables of unknown size it sleeps on the stream.
static void TestWaitOfShortQueues()
{
    CHECK(hybm_init(0, 0) == BM_OK);
    XcopyEngine &engine = XcopyEngine::Instance();
    void *stream = engine.ThreadStream();
    CHECK(stream != nullptr);
    std::vector<uint8_t> from(1 << 20, 7), to(1 << 20, 0);
    uint64_t s = reinterpret_cast<uint64_t>(from.data()), d = reinterpret_cast<uint64_t>(to.data()), l = from.size();
    for (int i = 0; i < 3; ++i) {
        CHECK(engine.Submit(&s, &d, &l, 1, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
    }
    uint64_t signals = fake_rt_signals(), syncs = fake_rt_stream_syncs();
    CHECK(engine.DrainThread() == BM_OK);
    CHECK(fake_rt_signals() == signals + 1 && fake_rt_stream_syncs() == syncs);       // polled
    CHECK(to == from);
    signals = fake_rt_signals();
    syncs = fake_rt_stream_syncs();
    CHECK(engine.DrainThread() == BM_OK);                                               // nothing queued: the stream wait
    CHECK(fake_rt_signals() == signals && fake_rt_stream_syncs() == syncs + 1);
    // more than the polling limit in the queue
    uint64_t big = XcopyEngine::kSpinBytes / 2 + 4096;
    std::vector<uint8_t> wide(big, 1), wide2(big, 0);
    uint64_t ws = reinterpret_cast<uint64_t>(wide.data()), wd = reinterpret_cast<uint64_t>(wide2.data());
    CHECK(engine.Submit(&ws, &wd, &big, 1, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
    CHECK(engine.Submit(&ws, &wd, &big, 1, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
    signals = fake_rt_signals();
    syncs = fake_rt_stream_syncs();
    CHECK(engine.DrainThread() == BM_OK);
    CHECK(fake_rt_signals() == signals && fake_rt_stream_syncs() == syncs + 1);
    // a copy on another stream is not this thread's queue
    int other = 0;
    CHECK(engine.Submit(&s, &d, &l, 1, MF_ROUTE_HBM, &other, nullptr, 0) == BM_OK);
    signals = fake_rt_signals();
    syncs = fake_rt_stream_syncs();
    CHECK(engine.DrainThread() == BM_OK);
    CHECK(fake_rt_signals() == signals && fake_rt_stream_syncs() == syncs + 1);
    // kernels of the other entry points behind a short copy
    CHECK(engine.Submit(&s, &d, &l, 1, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
    alignas(16) static uint8_t moeBuf[64];
    CHECK(mf_moe_combine(moeBuf, reinterpret_cast<const int32_t *>(moeBuf), reinterpret_cast<const float *>(moeBuf), 1, 8, 1,
                         moeBuf + 16, nullptr) == BM_OK);
    signals = fake_rt_signals();
    syncs = fake_rt_stream_syncs();
    CHECK(engine.DrainThread() == BM_OK);
    CHECK(fake_rt_signals() == signals && fake_rt_stream_syncs() == syncs + 1);
    // a blocking call drains the queue, so the wait after it has nothing to poll for
    CHECK(engine.Submit(&s, &d, &l, 1, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
    CHECK(engine.WaitStream(stream, l) == BM_OK);
    signals = fake_rt_signals();
    syncs = fake_rt_stream_syncs();
    CHECK(engine.DrainThread() == BM_OK);
    CHECK(fake_rt_signals() == signals && fake_rt_stream_syncs() == syncs + 1);
    hybm_uninit();
}

static void TestTrans()
{
    const char *store = "tcp://127.0.0.1:5432";
    const char *senderName = "127.0.0.1:5321";
    const char *receiverName = "127.0.0.1:5322";
    smem_trans_config_t sendCfg{};
    CHECK(smem_trans_config_init(nullptr) == SM_INVALID_PARAM);
    CHECK(smem_trans_config_init(&sendCfg) == SM_OK);
    CHECK(sendCfg.role == SMEM_TRANS_SENDER && sendCfg.initTimeout == 120 && sendCfg.deviceId == UINT32_MAX &&
          !sendCfg.startConfigServer);
    sendCfg.deviceId = 0;
    sendCfg.dataOpType = SMEMB_DATA_OP_SDMA;
    smem_trans_config_t recvCfg = sendCfg;
    recvCfg.role = SMEM_TRANS_RECEIVER;

    CHECK(smem_trans_create(store, senderName, &sendCfg) == nullptr);   // not initialised
    CHECK(smem_trans_init(nullptr) == SM_INVALID_PARAM);
    CHECK(smem_trans_init(&sendCfg) == SM_OK);
    CHECK(smem_trans_init(&sendCfg) == SM_OK);
    CHECK(smem_trans_create(nullptr, senderName, &sendCfg) == nullptr);
    CHECK(smem_trans_create(store, nullptr, &sendCfg) == nullptr);
    CHECK(smem_trans_create(store, senderName, nullptr) == nullptr);
    CHECK(smem_trans_create("", senderName, &sendCfg) == nullptr);
    CHECK(smem_trans_create(store, "", &sendCfg) == nullptr);
    CHECK(smem_trans_create(store, "127.0.0.1:80", &sendCfg) == nullptr);     // port not above 1024
    CHECK(smem_trans_create(store, "0.0.0.0:5321", &sendCfg) == nullptr);
    CHECK(smem_trans_create(store, "not-a-name", &sendCfg) == nullptr);

    smem_trans_t sender = smem_trans_create(store, senderName, &sendCfg);
    smem_trans_t receiver = smem_trans_create(store, receiverName, &recvCfg);
    smem_trans_t v6 = smem_trans_create("tcp://[::1]:5432", "[::1]:5321", &recvCfg);
    CHECK(sender != nullptr && receiver != nullptr && v6 != nullptr);
    CHECK(smem_trans_create(store, senderName, &sendCfg) == nullptr);   // name taken

    const size_t n = 3u << 20;
    uint8_t *src = static_cast<uint8_t *>(mfrt_alloc_device(n));
    uint8_t *dst = static_cast<uint8_t *>(mfrt_alloc_device(n));
    uint8_t *pinned = static_cast<uint8_t *>(mfrt_alloc_host(n));
    std::vector<uint8_t> pageable(n), pattern(n);
    Fill(pattern, 77);
    std::memcpy(src, pattern.data(), n);

    CHECK(smem_trans_register_mem(nullptr, dst, n, 0) == SM_INVALID_PARAM);
    CHECK(smem_trans_register_mem(receiver, nullptr, n, 0) == SM_INVALID_PARAM);
    CHECK(smem_trans_register_mem(receiver, dst, 0, 0) == SM_INVALID_PARAM);
    CHECK(smem_trans_register_mem(receiver, pageable.data(), n, 0) == SM_ERROR);   // cannot be pinned afterwards
    CHECK(smem_trans_register_mem(receiver, dst + 4096, n - 8192, 0) == SM_OK);
    CHECK(smem_trans_register_mem(receiver, dst + 4096, n - 8192, 0) == SM_OK);   // the same run again
    CHECK(smem_trans_register_mem(receiver, dst, 8192, 0) == SM_INVALID_PARAM);    // overlaps it

    const void *locals[3] = {src, src + 70001, src + (1u << 20)};
    void *remotes[3] = {dst + 4096, dst + 200003, dst + (2u << 20)};
    size_t sizes[3] = {70001, 4095, 1u << 19};
    CHECK(smem_trans_batch_write(nullptr, locals, receiverName, remotes, sizes, 3, 0) == SM_INVALID_PARAM);
    CHECK(smem_trans_batch_write(sender, nullptr, receiverName, remotes, sizes, 3, 0) == SM_INVALID_PARAM);
    CHECK(smem_trans_batch_write(sender, locals, nullptr, remotes, sizes, 3, 0) == SM_INVALID_PARAM);
    CHECK(smem_trans_batch_write(sender, locals, receiverName, nullptr, sizes, 3, 0) == SM_INVALID_PARAM);
    CHECK(smem_trans_batch_write(sender, locals, receiverName, remotes, nullptr, 3, 0) == SM_INVALID_PARAM);
    CHECK(smem_trans_batch_write(sender, locals, receiverName, remotes, sizes, 0, 0) == SM_INVALID_PARAM);
    CHECK(smem_trans_batch_write(sender, locals, receiverName, remotes, sizes, 3, ASYNC_COPY_FLAG) == SM_INVALID_PARAM);
    CHECK(smem_trans_batch_write(sender, locals, "127.0.0.1:9999", remotes, sizes, 3, 0) == SM_INVALID_PARAM);   // unknown peer
    CHECK(smem_trans_batch_write(sender, locals, "garbage", remotes, sizes, 3, 0) == SM_ERROR);
    CHECK(smem_trans_batch_write(sender, locals, senderName, remotes, sizes, 3, 0) == SM_INVALID_PARAM);   // senders see receivers only
    CHECK(smem_trans_batch_write_submit(sender, locals, receiverName, remotes, sizes, 3, nullptr, 0) == SM_INVALID_PARAM);

    std::memset(dst, 0, n);
    const uint64_t before = fake_rt_launches();
    CHECK(smem_trans_batch_write(sender, locals, receiverName, remotes, sizes, 3, 0) == SM_OK);
    CHECK(fake_rt_launches() == before + 1);   // one fused launch for the batch
    bool ok = true;
    for (int i = 0; i < 3; ++i) {
        ok = ok && std::memcmp(remotes[i], locals[i], sizes[i]) == 0;
    }
    CHECK(ok && dst[4095] == 0 && dst[4096 + 70001] == 0);

    // ranges that leave the registered run: before it, past its end, and across its end
    void *outside[1] = {dst};
    size_t one[1] = {16};
    const void *oneLocal[1] = {src};
    CHECK(smem_trans_batch_write(sender, oneLocal, receiverName, outside, one, 1, 0) == SM_INVALID_PARAM);
    outside[0] = dst + n - 4096;
    CHECK(smem_trans_batch_write(sender, oneLocal, receiverName, outside, one, 1, 0) == SM_INVALID_PARAM);
    outside[0] = dst + n - 4096 - 8;
    CHECK(smem_trans_batch_write(sender, oneLocal, receiverName, outside, one, 1, 0) == SM_INVALID_PARAM);
    one[0] = 8;
    CHECK(smem_trans_batch_write(sender, oneLocal, receiverName, outside, one, 1, 0) == SM_OK);           // ends exactly at the end

    // read back through the single-element calls, into pinned and into pageable memory
    CHECK(smem_trans_read(sender, pinned, receiverName, dst + 4096, 70001, 0) == SM_OK);
    CHECK(std::memcmp(pinned, src, 70001) == 0);
    CHECK(smem_trans_read(sender, pageable.data(), receiverName, dst + (2u << 20), 1u << 19, 0) == SM_OK);
    CHECK(std::memcmp(pageable.data(), src + (1u << 20), 1u << 19) == 0);
    CHECK(smem_trans_write(sender, pageable.data(), receiverName, dst + 8192, 1000, 0) == SM_OK);
    CHECK(std::memcmp(dst + 8192, pageable.data(), 1000) == 0);
    void *stream = mfrt_stream_create();
    CHECK(smem_trans_write_submit(sender, src + 5, receiverName, dst + 300000, 12345, stream, 0) == SM_OK);
    CHECK(mfrt_stream_sync(stream) == 0 && std::memcmp(dst + 300000, src + 5, 12345) == 0);
    CHECK(smem_trans_read_submit(sender, pinned, receiverName, dst + 300000, 12345, stream, 0) == SM_OK);
    CHECK(mfrt_stream_sync(stream) == 0 && std::memcmp(pinned, src + 5, 12345) == 0);
    mfrt_stream_destroy(stream);

    // host memory from the object itself; batch registration merges touching pieces into one run
    uint8_t *given = static_cast<uint8_t *>(smem_trans_malloc(v6, 1000));
    CHECK(given != nullptr && mfrt_pointer_kind(given) == 2);
    CHECK(smem_trans_malloc(nullptr, 1000) == nullptr && smem_trans_malloc(v6, 0) == nullptr);
    CHECK(smem_trans_write(sender, src, "[::1]:5321", given + 100, 900, 0) == SM_OK && std::memcmp(given + 100, src, 900) == 0);
    uint8_t *second = static_cast<uint8_t *>(mfrt_alloc_device(n));
    void *pieces[3] = {second + 8192, second, second + 4096};
    size_t pieceSizes[3] = {4096, 4096, 4096};
    CHECK(smem_trans_batch_register_mem(v6, pieces, pieceSizes, 3, 0) == SM_OK);
    CHECK(smem_trans_batch_register_mem(v6, pieces, pieceSizes, 0, 0) == SM_INVALID_PARAM);
    pieces[1] = nullptr;
    CHECK(smem_trans_batch_register_mem(v6, pieces, pieceSizes, 3, 0) == SM_INVALID_PARAM);
    CHECK(smem_trans_write(sender, src, "[::1]:5321", second + 100, 12000, 0) == SM_OK);   // spans all three pieces
    CHECK(std::memcmp(second + 100, src, 12000) == 0);
    CHECK(smem_trans_write(sender, src, "[::1]:5321", second + 100, 12289 - 100, 0) == SM_INVALID_PARAM);

    // withdrawing memory ends access to it; so does destroying its owner
    CHECK(smem_trans_deregister_mem(receiver, nullptr) == SM_INVALID_PARAM);
    CHECK(smem_trans_deregister_mem(receiver, dst + 4096) == SM_OK);
    one[0] = 8;
    outside[0] = dst + 8192;
    CHECK(smem_trans_batch_write(sender, oneLocal, receiverName, outside, one, 1, 0) == SM_INVALID_PARAM);
    CHECK(smem_trans_free(v6, nullptr) == SM_INVALID_PARAM);
    CHECK(smem_trans_free(v6, second) == SM_ERROR);    // registered, not allocated by the object
    CHECK(smem_trans_free(v6, given) == SM_OK);
    smem_trans_destroy(v6, 0);
    CHECK(smem_trans_write(sender, src, "[::1]:5321", second + 100, 100, 0) == SM_INVALID_PARAM);
    CHECK(smem_trans_register_mem(v6, second, 16, 0) == SM_OBJECT_NOT_EXISTS);
    smem_trans_destroy(nullptr, 0);
    smem_trans_destroy(sender, 0);
    smem_trans_destroy(receiver, 0);
    smem_trans_uninit(0);
    CHECK(smem_trans_register_mem(receiver, dst, 16, 0) == SM_INVALID_PARAM);   // not initialised
    mfrt_free_device(src);
    mfrt_free_device(dst);
    mfrt_free_device(second);
    mfrt_free_host(pinned);
}

// Per-thread GPU resources are leased from the engine: a thread that ends hands its stream back
// without touching the runtime, the next new thread takes it over, and a stop / start cycle of the
// library invalidates every lease, also those of threads that are still alive.
static void TestLeases()
{
    CHECK(hybm_init(0, 0) == BM_OK);
    void *mine = mf_xcopy_thread_stream();
    CHECK(mine != nullptr && mf_xcopy_thread_stream() == mine);
    void *first = nullptr, *second = nullptr;
    std::thread([&] { first = mf_xcopy_thread_stream(); }).join();
    std::thread([&] { second = mf_xcopy_thread_stream(); }).join();
    CHECK(first != nullptr && first != mine && second == first);
    void *a = nullptr, *b = nullptr;
    std::thread ta([&] { a = mf_xcopy_thread_stream(); });
    ta.join();
    std::thread tb([&] {
        b = mf_xcopy_thread_stream();
        std::thread inner([&] { a = mf_xcopy_thread_stream(); });   // tb still holds its lease
        inner.join();
    });
    tb.join();
    CHECK(a != nullptr && b != nullptr && a != b);
    hybm_uninit();
    CHECK(mf_xcopy_thread_stream() == nullptr);   // not started
    CHECK(hybm_init(0, 0) == BM_OK);
    void *again = mf_xcopy_thread_stream();
    CHECK(again != nullptr);
    CHECK(hybm_wait(nullptr) == BM_INVALID_PARAM);
    hybm_uninit();
}

// Mapped-window mode: the device window is reserved address space, local allocations map HBM
// into it piece by piece, and only the mapped prefix passes the pool-side range check.
static void TestMappedWindow()
{
    CHECK(hybm_init(0, 0) == BM_OK);
    const uint64_t page = 2u << 20;
    hybm_options o{};
    o.bmType = HYBM_TYPE_HOST_INITIATE;
    o.memType = HYBM_MEM_TYPE_DEVICE;
    o.bmDataOpType = HYBM_DOP_TYPE_SDMA;
    o.rankCount = 1;
    o.maxHBMSize = 64 * page;      // window
    o.deviceVASpace = 8 * page;    // what the caller intends to back
    o.scene = HYBM_SCENE_DEFAULT;
    o.dramShmFd = -1;
    hybm_entity_t e = hybm_create_entity(300, &o, 0);
    CHECK(e != nullptr);
    CHECK(hybm_reserve_mem_space(e, 0) == BM_OK);
    uint8_t *base = static_cast<uint8_t *>(hybm_get_memory_ptr(e, HYBM_MEM_TYPE_DEVICE));
    CHECK(base != nullptr);
    std::vector<uint8_t> local(4 * page);
    Fill(local, 9);
    hybm_copy_params cp{local.data(), base, page};
    CHECK(hybm_data_copy(e, &cp, HYBM_LOCAL_HOST_TO_GLOBAL_DEVICE, nullptr, 0) == BM_INVALID_PARAM);   // nothing mapped yet
    CHECK(hybm_alloc_local_memory(e, HYBM_MEM_TYPE_DEVICE, page + 4096, 0) == nullptr);               // not a granule multiple
    hybm_mem_slice_t s1 = hybm_alloc_local_memory(e, HYBM_MEM_TYPE_DEVICE, 2 * page, 0);
    hybm_mem_slice_t s2 = hybm_alloc_local_memory(e, HYBM_MEM_TYPE_DEVICE, 3 * page, 0);
    CHECK(s1 != nullptr && s2 != nullptr);
    CHECK(hybm_get_slice_va(e, s1) == base && hybm_get_slice_va(e, s2) == base + 2 * page);
    CHECK(hybm_alloc_local_memory(e, HYBM_MEM_TYPE_DEVICE, 60 * page, 0) == nullptr);                  // window exhausted
    cp = {local.data(), base + page, 3 * page};                                                         // spans both slices
    CHECK(hybm_data_copy(e, &cp, HYBM_LOCAL_HOST_TO_GLOBAL_DEVICE, nullptr, 0) == BM_OK);
    CHECK(std::memcmp(base + page, local.data(), 3 * page) == 0);
    cp = {local.data(), base + 4 * page, 2 * page};                                                     // one page past the mapped prefix
    CHECK(hybm_data_copy(e, &cp, HYBM_LOCAL_HOST_TO_GLOBAL_DEVICE, nullptr, 0) == BM_INVALID_PARAM);
    CHECK(mf_va_infer_direction(reinterpret_cast<uint64_t>(base + 3 * page), reinterpret_cast<uint64_t>(local.data())) ==
          HYBM_GLOBAL_DEVICE_TO_LOCAL_HOST);
    // the lower slice stays mapped while the upper one is in use; both go when the upper is released
    CHECK(hybm_free_local_memory(e, s1, 1, 0) == BM_OK);
    cp = {base, local.data(), page};
    CHECK(hybm_data_copy(e, &cp, HYBM_GLOBAL_DEVICE_TO_LOCAL_HOST, nullptr, 0) == BM_OK);
    CHECK(hybm_free_local_memory(e, s1, 1, 0) == BM_INVALID_PARAM);
    CHECK(hybm_free_local_memory(e, s2, 1, 0) == BM_OK);
    CHECK(hybm_data_copy(e, &cp, HYBM_GLOBAL_DEVICE_TO_LOCAL_HOST, nullptr, 0) == BM_INVALID_PARAM);
    hybm_mem_slice_t s3 = hybm_alloc_local_memory(e, HYBM_MEM_TYPE_DEVICE, page, 0);
    CHECK(s3 != nullptr && hybm_get_slice_va(e, s3) == base);
    {
        // A thread keeps copying into a slice while it is freed: every copy either was enqueued before the memory went (the stand-in
        // runtime executes it at once; a late one would touch a page without access rights and end the test) or fails its range check.
        // With the copies unordered and handed to submit threads, which launch them later than the call returns.
        for (uint32_t submitters : {0u, 2u}) {
            CHECK(mf_xcopy_unordered_streams(submitters) == BM_OK);
            hybm_mem_slice_t top = hybm_alloc_local_memory(e, HYBM_MEM_TYPE_DEVICE, 2 * page, 0);
            CHECK(top != nullptr && hybm_get_slice_va(e, top) == base + page);
            std::atomic<int> phase{0};
            std::atomic<uint64_t> done{0};
            std::atomic<uint64_t> refused{0};
            std::atomic<uint64_t> other{0};
            std::thread hammer([&] {
                // copies that are declared independent must be: 32 destinations in turn, so that copies with the same
                // destination always reach the same one of the two submit threads
                uint64_t turn = 0;
                while (phase.load() != 2) {
                    hybm_copy_params p{base, base + page + 4096 + (turn++ % 32) * 65536, 65536};
                    const int ret = hybm_data_copy(e, &p, HYBM_GLOBAL_DEVICE_TO_GLOBAL_DEVICE, nullptr, ASYNC_COPY_FLAG | MF_COPY_UNORDERED_FLAG);
                    (ret == BM_OK ? done : (ret == BM_INVALID_PARAM ? refused : other)).fetch_add(1);
                    if (done.load() > 50) {
                        { int zero = 0; phase.compare_exchange_strong(zero, 1); }
                    }
                }
                (void)hybm_wait(e);
            });
            while (phase.load() == 0) {
                std::this_thread::yield();
            }
            CHECK(hybm_free_local_memory(e, top, 1, 0) == BM_OK);
            const uint64_t refusedAtFree = refused.load();
            while (refused.load() < refusedAtFree + 50) {
                std::this_thread::yield();
            }
            phase.store(2);
            hammer.join();
            CHECK(done.load() > 50 && other.load() == 0);
        }
        CHECK(mf_xcopy_unordered_streams(0) == BM_OK);
    }
    hybm_destroy_entity(e, 0);
    hybm_uninit();
}

// The one-pass planners must produce exactly what normalisation followed by planning produces.
static void TestPlanners()
{
    std::mt19937_64 rng(0x9142);
    for (int trial = 0; trial < 400; ++trial) {
        const uint32_t n = 1 + rng() % (trial % 3 == 0 ? 600 : 140);
        const uint32_t units = 64u << (rng() % 6);
        std::vector<uint64_t> src(n), dst(n), len(n);
        uint64_t s = 0x7f1000000000ull + rng() % 4096, d = 0x7f8000000000ull + rng() % 4096;
        const bool pages = trial % 5 == 4;   // equal-size segments at page-aligned places
        const bool turns = trial % 5 == 3;   // a few sizes taking turns (K and V blocks)
        const uint64_t pageBytes = 4096ull << (rng() % 5);
        const uint32_t sizes = 2 + static_cast<uint32_t>(rng() % 7);
        uint64_t turnBytes[8];
        for (auto &t : turnBytes) {
            t = 4096ull * (1 + rng() % 40);
        }
        for (uint32_t i = 0; i < n; ++i) {
            if (pages || turns) {
                len[i] = pages ? pageBytes : turnBytes[i % sizes];
                src[i] = 0x7f1000000000ull + 4096ull * (400 * (rng() % 100000));
                dst[i] = 0x7f8000000000ull + 4096ull * (400 * i);
                continue;
            }
            const uint32_t kind = rng() % 8;
            len[i] = kind == 0 ? 0 : (kind == 1 ? rng() % 40 : rng() % 300000);
            if (kind != 2) {   // kind 2: continue the previous segment on both sides
                s += rng() % 70000;
                d += rng() % 70000;
            }
            src[i] = s;
            dst[i] = d;
            s += len[i];
            d += len[i];
        }
        SegList segs;
        NormalizeSegments(src.data(), dst.data(), len.data(), n, 0, segs);
        std::vector<uint64_t> t1(3 * segs.Size() + 3), t2(3 * n + 3);
        std::vector<uint32_t> f1(segs.Size() + 1), f2(n + 1);
        const uint64_t c1 = BuildTablePlan(segs, units, t1.data(), f1.data());
        uint32_t count = 0;
        ChunkPattern pattern;
        pattern.period = 99;
        const uint64_t c2 = BuildTableDirect(src.data(), dst.data(), len.data(), n, units, t2.data(), f2.data(), count,
                                             &pattern);
        uint32_t expectPeriod = 0;
        for (uint32_t p = 1; p <= kMaxPeriod && expectPeriod == 0 && segs.Size() != 0; ++p) {
            bool repeats = true;
            for (uint32_t i = p; i < segs.Size() && repeats; ++i) {
                repeats = f1[i + 1] - f1[i] == f1[i + 1 - p] - f1[i - p];
            }
            expectPeriod = repeats ? p : 0;
        }
        CHECK(pattern.period == expectPeriod);
        CHECK(!pages || pattern.period == 1);
        CHECK(!turns || pattern.period != 0);
        if (pattern.period != 0) {
            CHECK(PatternChunks(pattern, segs.Size()) == c1);
            uint32_t seg = 0;
            for (uint32_t c = 0; c < c1; ++c) {   // every chunk lands on the segment the prefix names
                while (f1[seg + 1] <= c) {
                    ++seg;
                }
                uint32_t gotSeg = 0;
                uint32_t gotK = 0;
                PatternOwner(pattern, c, gotSeg, gotK);
                if (gotSeg != seg || gotK != c - f1[seg]) {
                    CHECK(false);
                    break;
                }
            }
        }
        bool same = c1 == c2 && count == segs.Size();
        for (uint32_t i = 0; same && i < count; ++i) {
            same = t1[3 * i] == t2[3 * i] && t1[3 * i + 1] == t2[3 * i + 1] && t1[3 * i + 2] == t2[3 * i + 2] && f1[i] == f2[i];
        }
        same = same && f1[segs.Size()] == f2[count];
        CHECK(same);
        if (c1 != 0) {
            // the group map brackets the owner of every chunk, at the finest shift its room allows
            const uint32_t room[] = {GroupCapacityFor(count), static_cast<uint32_t>(c1 / 64 + 2), 17, 2};
            for (uint32_t capacity : room) {
                std::vector<uint32_t> group(capacity, 0xFFFFFFFFu);
                const uint32_t shift = BuildGroupMap(f1.data(), segs.Size(), group.data(), capacity);
                bool ok = shift >= kGroupShiftMin && GroupCount(c1, shift) + 1 <= capacity &&
                          (shift == kGroupShiftMin || GroupCount(c1, shift - 1) + 1 > capacity);
                uint32_t seg = 0;
                for (uint32_t c = 0; ok && c < c1; ++c) {
                    while (f1[seg + 1] <= c) {
                        ++seg;
                    }
                    const uint32_t lo = group[c >> shift];
                    const uint32_t hi = group[(c >> shift) + 1];
                    ok = lo <= seg && seg <= hi && hi < segs.Size();
                    if (shift == kGroupShiftMin) {
                        ok = ok && hi - lo < 64;     // no empty segments after normalisation: one probe round
                    }
                }
                CHECK(ok);
            }
        }
        InlinePlan a, b;
        NormalizeSegments(src.data(), dst.data(), len.data(), n, 1ull << 30, segs);
        const bool fitsA = BuildInlinePlan(segs, units, a);
        const bool fitsB = BuildInlineDirect(src.data(), dst.data(), len.data(), n, units, b);
        CHECK(fitsA == fitsB);
        if (fitsA && fitsB) {
            CHECK(std::memcmp(&a, &b, sizeof(a)) == 0);
        }
    }
}

// The choice hybm_init makes from what it measures on its GPU.
static void TestCalibration()
{
    const uint32_t rate = XcopyTuning{}.windowMBps;
    const uint32_t alignedRate = XcopyTuning{}.windowAlignedMBps;
    const uint32_t longRate = XcopyTuning{}.windowLongMBps;
    XcopyCalibration c;
    {   // the usual picture: the rule's wait is best, held stores gain 14 %, windows 7 %, one long segment holds the higher rate
        const float batch[4] = {5.30f, 4.62f, 4.55f, 4.60f};
        const float copy[4] = {172.0f, 160.0f, 163.0f, 149.0f};
        ChooseCalibration(batch, copy, rate, alignedRate, longRate, c);
        CHECK(c.ran && c.holdEnabled && c.holdDeltaNanos == 0 && c.windowMBps == rate && c.windowAlignedMBps == alignedRate && c.windowLongMBps == longRate);
    }
    {   // the higher rate does not hold here (no better than the default by 2 %): long segments take the default too
        const float batch[4] = {5.30f, 4.62f, 4.55f, 4.60f};
        const float copy[4] = {172.0f, 160.0f, 163.0f, 158.5f};
        ChooseCalibration(batch, copy, rate, alignedRate, longRate, c);
        CHECK(c.windowMBps == rate && c.windowAlignedMBps == rate && c.windowLongMBps == rate);
    }
    {   // a GPU whose loads land later: the longer wait wins clearly; windows only hold at the lower rate
        const float batch[4] = {5.30f, 4.95f, 4.80f, 4.60f};
        const float copy[4] = {172.0f, 171.0f, 161.0f, 176.0f};
        ChooseCalibration(batch, copy, rate, alignedRate, longRate, c);
        CHECK(c.holdEnabled && c.holdDeltaNanos == kCalibrateHoldStepNanos && c.windowMBps == static_cast<uint32_t>(static_cast<uint64_t>(rate) * 94 / 100) &&
              c.windowAlignedMBps == c.windowMBps && c.windowLongMBps == c.windowMBps);
    }
    {   // a neighbour that is better by less than 1 % does not move the wait
        const float batch[4] = {5.30f, 4.53f, 4.55f, 4.60f};
        const float copy[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        ChooseCalibration(batch, copy, rate, alignedRate, longRate, c);
        CHECK(c.ran && c.holdDeltaNanos == 0 && c.windowMBps == rate && c.windowAlignedMBps == alignedRate && c.windowLongMBps == longRate);   // windows not measured: the defaults stay
    }
    {   // a busy or capped chip: holding gains 2 %, windows lose: both off
        const float batch[4] = {5.30f, 5.25f, 5.20f, 5.28f};
        const float copy[4] = {172.0f, 175.0f, 174.0f, 169.0f};
        ChooseCalibration(batch, copy, rate, alignedRate, longRate, c);
        CHECK(c.ran && !c.holdEnabled && c.windowMBps == 0 && c.windowAlignedMBps == 0 && c.windowLongMBps == 0);
    }
    {   // nothing measured
        const float none[4] = {0, 0, 0, 0};
        ChooseCalibration(none, none, rate, alignedRate, longRate, c);
        CHECK(!c.ran && c.holdEnabled && c.holdDeltaNanos == 0 && c.windowMBps == rate);
    }
    // through hybm_init: the engine applies what it chose, and mf_xcopy_hold_stores(-1) means the calibrated rule
    const float shorter[8] = {5.30f, 4.40f, 4.60f, 4.70f, 172.0f, 160.0f, 163.0f, 150.0f};
    fake_rt_set_calibration(shorter);
    CHECK(hybm_init(0, 0) == BM_OK);
    const uint32_t rule = HoldNanosFor(2196, 2196, 256, false);
    CHECK(fake_rt_calibration_holds()[0] == rule - 200 && fake_rt_calibration_holds()[1] == rule && fake_rt_calibration_holds()[2] == rule + 200);
    int32_t enabled = -1;
    int32_t delta = 0;
    uint32_t mbps = 0;
    uint32_t alignedMbps = 0;
    uint32_t longMbps = 0;
    float micros[8] = {};
    CHECK(mf_xcopy_calibration(&enabled, &delta, &mbps, &alignedMbps, &longMbps, micros) == 1);
    CHECK(enabled == 1 && delta == -200 && mbps == rate && alignedMbps == alignedRate && longMbps == longRate && micros[1] == 4.40f && micros[5] == 160.0f && micros[7] == 150.0f);
    {
        std::vector<uint8_t> from(12 << 20), to(12 << 20);
        const uint64_t fromBase = (reinterpret_cast<uint64_t>(from.data()) + 4095) & ~4095ull;
        const uint64_t toBase = (reinterpret_cast<uint64_t>(to.data()) + 4095) & ~4095ull;
        std::vector<uint64_t> s(122), d(122), l(122);
        uint64_t at = 0;
        for (uint32_t i = 0; i < 122; ++i) {
            l[i] = (i & 1) != 0 ? 16384 : 131072;
            s[i] = fromBase + at + 4096;    // a page between neighbours on one side: no merging
            d[i] = toBase + at;
            at += l[i] + 4096 * (1 + i % 2);
        }
        CHECK(XcopyEngine::Instance().Submit(s.data(), d.data(), l.data(), 122, MF_ROUTE_HBM, nullptr, nullptr, 0) == BM_OK);
        CHECK(fake_rt_last_hold() == HoldNanosFor(2196, 2196, 256, false) - 200);
    }
    hybm_uninit();
    const float lost[8] = {5.30f, 5.29f, 5.31f, 5.30f, 172.0f, 175.0f, 176.0f, 177.0f};
    fake_rt_set_calibration(lost);
    CHECK(hybm_init(0, 0) == BM_OK);
    CHECK(mf_xcopy_calibration(&enabled, &delta, &mbps, &alignedMbps, &longMbps, nullptr) == 1 && enabled == 0 && mbps == 0 && alignedMbps == 0 && longMbps == 0);
    hybm_uninit();
    setenv("MF_HIP_CALIBRATE", "0", 1);
    CHECK(hybm_init(0, 0) == BM_OK);
    CHECK(mf_xcopy_calibration(&enabled, &delta, &mbps, &alignedMbps, &longMbps, nullptr) == 0 && enabled == 1 && delta == 0 && mbps == rate &&
          alignedMbps == alignedRate && longMbps == longRate);
    hybm_uninit();
    unsetenv("MF_HIP_CALIBRATE");
    const float none[8] = {};
    fake_rt_set_calibration(none);
}

// Unordered batches handed to submit threads: the thread's stream is made to wait for them exactly when something ordered follows.
static void TestUnorderedFanOut()
{
    CHECK(hybm_init(0, 0) == BM_OK);
    XcopyEngine &engine = XcopyEngine::Instance();
    std::vector<uint8_t> from(1 << 20), to(1 << 20, 0);
    Fill(from, 77);
    auto batch = [&](uint32_t piece, bool unordered, void *stream) {
        uint64_t s = reinterpret_cast<uint64_t>(from.data()) + piece * 4096;
        uint64_t d = reinterpret_cast<uint64_t>(to.data()) + piece * 4096;
        uint64_t l = 4096;
        return engine.Submit(&s, &d, &l, 1, MF_ROUTE_HBM, stream, nullptr, 0, unordered);
    };
    CHECK(mf_xcopy_unordered_streams(9) == BM_INVALID_PARAM);
    CHECK(mf_xcopy_unordered_streams(3) == BM_OK);
    uint64_t waits = fake_rt_stream_waits();
    for (uint32_t i = 0; i < 7; ++i) {
        CHECK(batch(i, true, nullptr) == BM_OK);
    }
    CHECK(fake_rt_stream_waits() == waits);                     // nothing ordered yet: nothing joined
    CHECK(batch(7, false, nullptr) == BM_OK);                   // an ordered copy: the three side streams are joined first
    CHECK(fake_rt_stream_waits() == waits + 3);
    CHECK(batch(8, false, nullptr) == BM_OK);
    CHECK(fake_rt_stream_waits() == waits + 3);                 // nothing new to join
    CHECK(batch(9, true, nullptr) == BM_OK);
    CHECK(engine.DrainThread() == BM_OK);                       // the wait joins the one side stream that was used
    CHECK(fake_rt_stream_waits() == waits + 4);
    CHECK(batch(10, true, nullptr) == BM_OK);
    CHECK(mf_xcopy_thread_stream() != nullptr);                 // fetching the thread's stream joins as well
    CHECK(fake_rt_stream_waits() == waits + 5);
    void *own = mfrt_stream_create();
    CHECK(batch(11, true, own) == BM_OK);                       // a caller's stream is never fanned out
    CHECK(engine.DrainThread() == BM_OK);
    CHECK(fake_rt_stream_waits() == waits + 5);
    CHECK(mf_xcopy_unordered_streams(0) == BM_OK);
    CHECK(batch(12, true, nullptr) == BM_OK);
    CHECK(engine.DrainThread() == BM_OK);
    CHECK(fake_rt_stream_waits() == waits + 5);
    CHECK(std::memcmp(from.data(), to.data(), 13 * 4096) == 0);
    mfrt_stream_destroy(own);
    hybm_uninit();
}

// Tables the engine cannot back with memory in a test: the launches are planned and checked, nothing is moved.
// Rectangles of a launch that moves 512 MiB and more between device addresses take the windowed form: chunks of
// 1024 units of the payload taken row-major.  Mates, rows narrower and wider than a chunk, a single column of units;
// every row arrives, nothing lands between the rows.
static void TestWindowedRectangles()
{
    CHECK(hybm_init(0, 0) == BM_OK);
    CHECK(mf_xcopy_windows(6800000) == BM_OK);
    const uint64_t rowsA = 57000;                      // 2 x 57000 rows of 4736 bytes: 540 MB
    struct Shape { uint64_t width, height, spitch, dpitch; };
    const Shape shapes[5] = {{4736, rowsA, 4736, 9472}, {4736, rowsA, 4736, 9472}, {48, 1000, 64, 80}, {40000, 50, 40016, 40032},
                             {16, 3000, 16, 32}};
    uint64_t srcBytes = 0;
    uint64_t dstBytes = 0;
    uint64_t srcAt[5];
    uint64_t dstAt[5];
    for (int i = 0; i < 5; ++i) {
        srcAt[i] = srcBytes;
        srcBytes += shapes[i].spitch * shapes[i].height;
        if (i == 1) {
            dstAt[i] = dstAt[0] + shapes[0].width;     // side by side with the first in the destination
            continue;
        }
        dstAt[i] = dstBytes;
        dstBytes += shapes[i].dpitch * shapes[i].height;
    }
    std::vector<unsigned char> src(srcBytes + 16);
    std::vector<unsigned char> dst(dstBytes + 16, 0xEE);
    for (uint64_t i = 0; i < srcBytes; i += 8) {
        const uint64_t word = i * 0x9E3779B97F4A7C15ull + 1;
        std::memcpy(&src[i], &word, 8);
    }
    const uint64_t s0 = (reinterpret_cast<uint64_t>(src.data()) + 15) & ~15ull;
    const uint64_t d0 = (reinterpret_cast<uint64_t>(dst.data()) + 15) & ~15ull;
    mf_copy2d_desc rects[5];
    for (int i = 0; i < 5; ++i) {
        rects[i] = {s0 + srcAt[i], d0 + dstAt[i], shapes[i].width, shapes[i].height, shapes[i].spitch, shapes[i].dpitch};
    }
    const uint32_t before = fake_rt_rect_windowed_launches();
    CHECK(mf_xcopy_2d_batch(rects, 5, MF_ROUTE_HBM, nullptr) == BM_OK);
    CHECK(fake_rt_rect_windowed_launches() == before + 1);
    bool ok = true;
    for (int i = 0; i < 5 && ok; ++i) {
        const unsigned char *s = reinterpret_cast<const unsigned char *>(rects[i].src);
        const unsigned char *d = reinterpret_cast<const unsigned char *>(rects[i].dst);
        for (uint64_t r = 0; r < shapes[i].height && ok; ++r) {
            ok = std::memcmp(d + r * shapes[i].dpitch, s + r * shapes[i].spitch, shapes[i].width) == 0;
            // the gap behind a row (for the mates: behind the pair) is untouched
            const uint64_t gapAt = i == 0 ? 2 * shapes[i].width : shapes[i].width;
            if (i != 1 && gapAt < shapes[i].dpitch) {
                ok = ok && d[r * shapes[i].dpitch + gapAt] == 0xEE && d[(r + 1) * shapes[i].dpitch - 1] == 0xEE;
            }
        }
        CHECK(ok);
    }
    // the same call below the size takes the kernel of whole rows
    rects[0].height = rects[1].height = 1000;
    CHECK(mf_xcopy_2d_batch(rects, 5, MF_ROUTE_HBM, nullptr) == BM_OK);
    CHECK(fake_rt_rect_windowed_launches() == before + 1);
    // and so does a route over the host link
    rects[0].height = rects[1].height = rowsA;
    CHECK(mf_xcopy_2d_batch(rects, 5, MF_ROUTE_TO_HOST, nullptr) == BM_OK);
    CHECK(fake_rt_rect_windowed_launches() == before + 1);
    hybm_uninit();
}

// Streams are dealt out one per hardware queue before the second of any.  The stand-in runtime puts the first eight
// streams of a process on queues A B C C B A D C, as the GPU did.
static void TestStreamDeck()
{
    CHECK(hybm_init(0, 0) == BM_OK);
    uint32_t queues[16] = {};
    CHECK(mf_xcopy_stream_queues(queues, 16) == 8);
    const uint32_t expect[8] = {0, 1, 2, 3, 0, 1, 2, 2};
    for (int i = 0; i < 8; ++i) {
        CHECK(queues[i] == expect[i]);
    }
    // the calling thread holds the first; four submit threads then sit on four different queues
    void *mine = mf_xcopy_thread_stream();
    CHECK(mine != nullptr);
    CHECK(mf_xcopy_stream_queues(nullptr, 0) == 8);
    hybm_uninit();
    // no answer from the GPU: every stream a queue of its own, the order they were made in
    fake_rt_queue_answers(1);
    CHECK(hybm_init(0, 0) == BM_OK);
    CHECK(mf_xcopy_stream_queues(queues, 16) == 8);
    for (uint32_t i = 0; i < 8; ++i) {
        CHECK(queues[i] == i);
    }
    hybm_uninit();
    fake_rt_queue_answers(0);
}

static void TestLongSegments()
{
    CHECK(hybm_init(0, 0) == BM_OK);
    XcopyEngine &engine = XcopyEngine::Instance();
    void *stream = mf_xcopy_thread_stream();
    fake_rt_skip_copies(1);
    const uint64_t gib = 1ull << 30;
    const uint64_t base = 0x7f0000000000ull;
    const uint64_t errorsBefore = fake_rt_group_map_errors();
    {
        // 128 segments that do not merge, one of them 4 GiB: cut into 1 GiB pieces it no longer fits the kernel-argument
        // form, and its average length makes it a candidate for slicing.  It goes to the table form, once.
        for (uint32_t n : {126u, 128u, 100u}) {
            std::vector<uint64_t> src(n), dst(n), len(n, 4096);
            for (uint32_t i = 0; i < n; ++i) {
                src[i] = base + i * 16 * gib;
                dst[i] = base + (2048 + i) * 16 * gib + 7;
            }
            len[n / 2] = 4 * gib;
            const uint64_t before = mf_xcopy_launch_count();
            CHECK(engine.Submit(src.data(), dst.data(), len.data(), n, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
            CHECK(mf_xcopy_launch_count() - before <= 2);
        }
    }
    {
        // one segment beyond what 128 pieces of 1 GiB hold
        uint64_t src = base;
        uint64_t dst = base + 4096 * gib + 384;
        uint64_t len = 129 * gib + 5;
        const uint64_t before = mf_xcopy_launch_count();
        CHECK(engine.Submit(&src, &dst, &len, 1, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
        CHECK(mf_xcopy_launch_count() - before == 258);        // windowed launches of 512 MiB, however long the segment
        CHECK(fake_rt_last_window() != 0);
        // declared independent of what is in flight it takes no windows: one launch of the table form, a pattern of period 1, no upload
        const uint64_t again = mf_xcopy_launch_count();
        CHECK(engine.Submit(&src, &dst, &len, 1, MF_ROUTE_HBM, stream, nullptr, 0, true) == BM_OK);
        CHECK(mf_xcopy_launch_count() - again == 1);
    }
    {
        // 600 long segments are cut into slices of 128; the slice with the 5 GiB segment has more chunks than the kernel-argument
        // form counts and goes through the table (upload + launch); everything in windows, the completion word behind the last launch
        const uint32_t n = 600;
        std::vector<uint64_t> src(n), dst(n), len(n, 8u << 20);
        for (uint32_t i = 0; i < n; ++i) {
            src[i] = base + i * 16 * gib;
            dst[i] = base + (2048 + i) * 16 * gib + 512;
        }
        len[300] = 5 * gib;
        uint64_t word = 0;
        const uint64_t before = mf_xcopy_launch_count();
        (void)fake_rt_last_window();
        CHECK(engine.Submit(src.data(), dst.data(), len.data(), n, MF_ROUTE_HBM, stream, &word, 32) == BM_OK);
        // 128 + 128 + (upload + table) + 128 + 88
        CHECK(mf_xcopy_launch_count() - before == 6);
        CHECK(word == 32);
        CHECK(fake_rt_last_window() != 0);
    }
    {
        // a ragged table whose chunks outnumber the room of its map: coarser groups, the owner still bracketed
        const uint32_t n = 500;     // beyond what is cut into launches of 128 segments
        std::vector<uint64_t> src(n), dst(n), len(n);
        for (uint32_t i = 0; i < n; ++i) {
            src[i] = base + i * 64 * gib;
            dst[i] = base + (2048 + i) * 64 * gib + (i % 16);
            len[i] = (i % 7 == 0 ? 3 * gib : 70000) + i;
        }
        CHECK(mf_xcopy_windows(0) == BM_OK);                   // no slicing: one table
        CHECK(engine.Submit(src.data(), dst.data(), len.data(), n, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
        CHECK(fake_rt_last_table_shift() > kGroupShiftMin);
        CHECK(mf_xcopy_windows(6800000) == BM_OK);
    }
    CHECK(fake_rt_group_map_errors() == errorsBefore);
    CHECK(engine.DrainThread() == BM_OK);
    fake_rt_skip_copies(0);
    {
        // the planner of a device-resident table, restated by the stand-in runtime: empty segments in runs longer than a
        // probe round, a pattern with an empty member, a table of nothing but empty segments
        std::mt19937_64 rng(0x6A09);
        for (int trial = 0; trial < 60; ++trial) {
            const uint32_t n = 1 + rng() % 700;
            std::vector<uint8_t> from(1 << 20), to(1 << 20, 0), expect(1 << 20, 0);
            for (auto &b : from) {
                b = static_cast<uint8_t>(rng());
            }
            std::vector<uint64_t> triples(3 * n);
            uint64_t at = 0;
            for (uint32_t i = 0; i < n; ++i) {
                uint64_t l = trial % 4 == 0 ? (i % 3 == 1 ? 0 : 1024) : (rng() % 5 == 0 ? rng() % 3000 : 0);
                if (trial % 7 == 6) {
                    l = 0;
                }
                if (at + l + 64 > from.size()) {
                    l = 0;
                }
                triples[3 * i] = reinterpret_cast<uint64_t>(from.data()) + at + (rng() % 16);
                triples[3 * i + 1] = reinterpret_cast<uint64_t>(to.data()) + at;
                triples[3 * i + 2] = l;
                std::memcpy(expect.data() + at, reinterpret_cast<void *>(triples[3 * i]), l);
                at += l + (rng() % 48);
            }
            const uint64_t errors = fake_rt_group_map_errors();
            CHECK(mf_xcopy_device_table(triples.data(), n, MF_ROUTE_HBM, stream) == BM_OK);
            CHECK(fake_rt_group_map_errors() == errors);
            CHECK(engine.DrainThread() == BM_OK);
            CHECK(to == expect);
        }
    }
    hybm_uninit();
}

// Copies shared with the helper thread move exactly the bytes memcpy would, also when two
// callers compete for the helper and when pieces are just below and above the split size.
static void TestHostCopy()
{
    HostCopyHelper &helper = HostCopyHelper::Instance();
    auto worker = [&](uint64_t seed, int rounds) {
        std::mt19937_64 rng(seed);
        std::vector<uint8_t> src(5u << 20), dst(5u << 20), expect(5u << 20);
        for (auto &b : src) {
            b = static_cast<uint8_t>(rng());
        }
        for (int r = 0; r < rounds; ++r) {
            const size_t edge = HostCopyHelper::kSplitMin;
            const size_t lens[] = {0, 1, 4095, edge - 1, edge, edge + 1, (2u << 20), (2u << 20) + 77, 3000001};
            const size_t len = lens[r % 9];
            const size_t so = rng() % 4097, dof = rng() % 4097;
            std::memset(dst.data(), 0xCD, dst.size());
            std::memset(expect.data(), 0xCD, expect.size());
            std::memcpy(expect.data() + dof, src.data() + so, len);
            helper.Copy(dst.data() + dof, src.data() + so, len);
            CHECK(dst == expect);
        }
    };
    worker(1, 27);
    CHECK(helper.SharedCopies() > 0);
    // sets of pieces: the cut falls between pieces, inside one, and after empty ones
    {
        std::mt19937_64 rng(9);
        std::vector<uint8_t> src(6u << 20), dst(6u << 20), expect(6u << 20);
        for (auto &b : src) {
            b = static_cast<uint8_t>(rng());
        }
        for (int trial = 0; trial < 40; ++trial) {
            std::vector<HostCopyHelper::Task> set;
            std::memset(dst.data(), 0xEE, dst.size());
            std::memset(expect.data(), 0xEE, expect.size());
            size_t at = 0;
            const int pieces = 1 + static_cast<int>(rng() % 40);
            for (int i = 0; i < pieces && at < (5u << 20); ++i) {
                const uint32_t kind = static_cast<uint32_t>(rng() % 6);
                const size_t len = kind == 0 ? 0 : (kind == 1 ? 1u << 20 : rng() % 200000);
                const size_t so = rng() % ((6u << 20) - len);
                set.push_back(HostCopyHelper::Task{dst.data() + at, src.data() + so, len});
                std::memcpy(expect.data() + at, src.data() + so, len);
                at += len + rng() % 64;
            }
            helper.CopySet(set.data(), set.size());
            CHECK(dst == expect);
        }
        helper.CopySet(nullptr, 0);
    }
    std::thread other(worker, 2, 27);
    worker(3, 27);
    other.join();
}

// Descriptor staging slots are recycled behind events that several launches share.  The stand-in
// runtime keeps every table "in flight" until a wait covers its launch and counts tables that were
// rewritten before that.
static void TestSlotRing()
{
    CHECK(hybm_init(0, 0) == BM_OK);
    const size_t pool = 8u << 20;
    uint8_t *a = static_cast<uint8_t *>(mfrt_alloc_device(pool));
    uint8_t *b = static_cast<uint8_t *>(mfrt_alloc_device(pool));
    std::mt19937_64 rng(0x51);
    for (size_t i = 0; i < pool; ++i) {
        a[i] = static_cast<uint8_t>(rng());
    }
    std::memset(b, 0, pool);
    std::vector<uint8_t> model(pool, 0);
    auto batch = [&](uint32_t n, bool pages, void *stream) {
        std::vector<uint64_t> s(n), d(n), l(n);
        const uint64_t slot = pool / n / 64 * 64;
        for (uint32_t i = 0; i < n; ++i) {
            l[i] = pages ? 4096 : 1 + rng() % (slot - 1);
            s[i] = reinterpret_cast<uint64_t>(a) + (rng() % n) * slot;
            d[i] = reinterpret_cast<uint64_t>(b) + static_cast<uint64_t>(i) * slot;
            std::memcpy(model.data() + static_cast<uint64_t>(i) * slot, reinterpret_cast<const void *>(s[i]), l[i]);
        }
        CHECK(mf_xcopy_batch(s.data(), d.data(), l.data(), n, MF_ROUTE_HBM, stream) == BM_OK);
    };
    const uint64_t before = fake_rt_violations();
    for (int i = 0; i < 45; ++i) {   // the ring wraps five times; forms with and without a chunk prefix alternate irregularly
        batch(200 + static_cast<uint32_t>(rng() % 300), i % 3 == 1, nullptr);
    }
    CHECK(fake_rt_in_flight() > 0);      // nothing waited for the last launches yet
    void *other = mfrt_stream_create();  // a caller's stream: every launch is followed by its own event
    for (int i = 0; i < 20; ++i) {
        batch(300, i % 2 == 0, i % 4 < 2 ? other : nullptr);
    }
    CHECK(mfrt_stream_sync(mf_xcopy_thread_stream()) == 0);
    CHECK(mfrt_stream_sync(other) == 0);
    CHECK(fake_rt_in_flight() == 0);
    CHECK(fake_rt_violations() == before);
    CHECK(std::memcmp(b, model.data(), pool) == 0);
    // a thread that ends with launches queued hands its lease to the next thread
    std::thread first([&] {
        mfrt_bind_thread();
        for (int i = 0; i < 3; ++i) {
            batch(260, false, nullptr);
        }
    });
    first.join();
    std::thread second([&] {
        mfrt_bind_thread();
        for (int i = 0; i < 12; ++i) {
            batch(260, i % 2 == 0, nullptr);
        }
        CHECK(mfrt_stream_sync(mf_xcopy_thread_stream()) == 0);
    });
    second.join();
    CHECK(mfrt_device_sync() == 0);
    CHECK(fake_rt_violations() == before);
    CHECK(std::memcmp(b, model.data(), pool) == 0);
    mfrt_stream_destroy(other);
    mfrt_free_device(a);
    mfrt_free_device(b);
    hybm_uninit();
}

// The two-symbol plugin over the same engine: the completion word of a table the CPU can read is
// stored before the call returns; a failed launch leaves the word alone and is counted.
static void TestPlugin()
{
    CHECK(hybm_init(0, 0) == BM_OK);
    const uint64_t n = 1u << 20;
    uint8_t *a = static_cast<uint8_t *>(mfrt_alloc_device(n));
    uint8_t *b = static_cast<uint8_t *>(mfrt_alloc_device(n));
    uint64_t *slot = static_cast<uint64_t *>(mfrt_alloc_host(16384 * 24 + 64));
    uint64_t *devWord = static_cast<uint64_t *>(mfrt_alloc_device(64));
    CHECK(a != nullptr && b != nullptr && slot != nullptr && devWord != nullptr);
    std::vector<uint8_t> ref(n);
    Fill(ref, 21);
    std::memcpy(a, ref.data(), n);
    std::memset(b, 0, n);
    for (uint32_t i = 0; i < 64; ++i) {
        slot[3 * i] = reinterpret_cast<uint64_t>(a) + i * 4096 + 3;
        slot[3 * i + 1] = reinterpret_cast<uint64_t>(b) + i * 4096 + 5;
        slot[3 * i + 2] = 3000;
    }
    uint64_t *word = slot + 16384 * 3;
    *word = 0;
    const uint64_t failuresBefore = mf_copy_extend_failures();
    uint64_t launches = fake_rt_launches();
    hybm_batch_copy_extend(slot, 64, word, 32, nullptr);
    CHECK(*word == 32);
    CHECK(fake_rt_launches() - launches == 1);          // no launch of its own for the word
    bool ok = true;
    for (uint32_t i = 0; i < 64; ++i) {
        ok = ok && std::memcmp(b + i * 4096 + 5, ref.data() + i * 4096 + 3, 3000) == 0;
    }
    CHECK(ok);
    CHECK(mf_copy_extend_failures() == failuresBefore);
    // a word in device memory is stored by the launch path
    *devWord = 0;
    hybm_batch_copy_extend(slot, 64, devWord, 32, nullptr);
    CHECK(*devWord == 32);
    // a launch that fails: counted, word untouched
    *word = 0;
    fake_rt_fail_launches(1);
    hybm_batch_copy_extend(slot, 64, word, 32, nullptr);
    CHECK(*word == 0);
    CHECK(mf_copy_extend_failures() == failuresBefore + 1);
    fake_rt_fail_launches(1);
    hybm_copy_extend(a, b, 100, 32, nullptr);
    CHECK(mf_copy_extend_failures() == failuresBefore + 2);
    hybm_batch_copy_extend(nullptr, 64, word, 32, nullptr);
    CHECK(*word == 0 && mf_copy_extend_failures() == failuresBefore + 3);
    // and the next one works again
    hybm_batch_copy_extend(slot, 64, word, 32, nullptr);
    CHECK(*word == 32);
    mfrt_free_device(a);
    mfrt_free_device(b);
    mfrt_free_device(devWord);
    mfrt_free_host(slot);
    hybm_uninit();
}

// Which launches are told to hold their stores back, and for how long.
static void TestHeldStores()
{
    CHECK(HoldNanosFor(959, 959, 256, false) == 0 && HoldNanosFor(960, 960, 256, false) == 640 + 576);
    CHECK(HoldNanosFor(2196, 2196, 256, false) == 640 + 1317);
    CHECK(HoldNanosFor(3904, 3904, 256, false) == 2982 && HoldNanosFor(3905, 3905, 256, false) == 2982);
    CHECK(HoldNanosFor(6144, 6144, 256, false) == 2982 + 739 && HoldNanosFor(6145, 6145, 256, false) == 0);
    CHECK(HoldNanosFor(2196, 2195, 256, false) == 0);    // a workgroup with two chunks
    CHECK(HoldNanosFor(2196, 2196, 512, false) == 0);    // chunks of 8 KiB
    CHECK(HoldNanosFor(1399, 1399, 256, true) == 0 && HoldNanosFor(1400, 1400, 256, true) == 100 + 798);
    CHECK(HoldNanosFor(6144, 6144, 256, true) == 100 + 3502 && HoldNanosFor(6145, 6145, 256, true) == 0);
    for (int single = 0; single < 2; ++single) {  // never shorter for more chunks, and one segment never waits longer than many
        uint32_t last = 0;
        for (uint32_t n = 960; n <= 6144; ++n) {
            const uint32_t h = HoldNanosFor(n, n, 256, single != 0);
            CHECK(h >= last && h < 4000);
            CHECK(single == 0 || h < HoldNanosFor(n, n, 256, false));
            last = h;
        }
    }

    CHECK(hybm_init(0, 0) == BM_OK);
    const uint64_t seg = 128u << 10;
    const uint32_t count = 32;                    // 32 x 128 KiB = 1024 chunks of 4 KiB
    std::vector<uint8_t> from(seg * count), to(seg * count, 0);
    for (size_t i = 0; i < from.size(); ++i) {
        from[i] = static_cast<uint8_t>(i * 31 + (i >> 12));
    }
    std::vector<uint64_t> src(count), dst(count), len(count, seg);
    for (uint32_t i = 0; i < count; ++i) {
        src[i] = reinterpret_cast<uint64_t>(from.data()) + i * seg;
        dst[i] = reinterpret_cast<uint64_t>(to.data()) + (count - 1 - i) * seg;
    }
    XcopyEngine &engine = XcopyEngine::Instance();
    void *stream = mf_xcopy_thread_stream();
    CHECK(engine.Submit(src.data(), dst.data(), len.data(), count, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
    CHECK(fake_rt_last_hold() == HoldNanosFor(1024, 1024, 256, false));
    CHECK(engine.Submit(src.data(), dst.data(), len.data(), count, MF_ROUTE_HBM, stream, nullptr, 0, true) == BM_OK);
    CHECK(fake_rt_last_hold() == 0);              // unordered launches overlap on purpose
    CHECK(engine.Submit(src.data(), dst.data(), len.data(), count, MF_ROUTE_TO_HOST, stream, nullptr, 0) == BM_OK);
    CHECK(fake_rt_last_hold() == 0);              // the host link is the bound there, not HBM
    {
        const uint64_t one = seg * count;          // the same bytes as one segment of 1024 chunks, then as one of 2048
        uint64_t s1 = src[0], d1 = reinterpret_cast<uint64_t>(to.data()), l1 = one;
        CHECK(engine.Submit(&s1, &d1, &l1, 1, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
        CHECK(fake_rt_last_hold() == 0);          // below the 1400 chunks from which a single segment gains
        std::vector<uint8_t> wider(4 * one);
        s1 = reinterpret_cast<uint64_t>(wider.data());
        d1 = s1 + 2 * one;
        l1 = 2 * one;
        CHECK(engine.Submit(&s1, &d1, &l1, 1, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
        CHECK(fake_rt_last_hold() == HoldNanosFor(2048, 2048, 256, true));
        CHECK(engine.DrainThread() == BM_OK);
    }
    {
        // 5120 chunks: held while this thread is the only submitter, not while a second thread has a stream
        std::vector<uint8_t> big(40u << 20);
        uint64_t s5[2], d5[2], l5[2] = {10u << 20, 10u << 20};
        for (int i = 0; i < 2; ++i) {
            s5[i] = reinterpret_cast<uint64_t>(big.data()) + (static_cast<uint64_t>(i) << 20) * 10;
            d5[i] = s5[i] + (20u << 20);
        }
        std::swap(d5[0], d5[1]);   // not one run
        CHECK(engine.Submit(s5, d5, l5, 2, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
        CHECK(fake_rt_last_hold() == HoldNanosFor(5120, 5120, 256, false));
        std::atomic<int> phase{0};
        std::thread other([&] {
            (void)mf_xcopy_thread_stream();
            phase.store(1);
            while (phase.load() != 2) {
                std::this_thread::yield();
            }
        });
        while (phase.load() != 1) {
            std::this_thread::yield();
        }
        CHECK(engine.Submit(s5, d5, l5, 2, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
        CHECK(fake_rt_last_hold() == 0);
        CHECK(engine.Submit(src.data(), dst.data(), len.data(), count, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
        CHECK(fake_rt_last_hold() == HoldNanosFor(1024, 1024, 256, false));   // small launches keep the wait
        // the MoE combine leaves its paced form alone as long as the second thread has its stream
        alignas(16) static uint8_t moeBuf[64];
        CHECK(mf_moe_combine(moeBuf, reinterpret_cast<const int32_t *>(moeBuf), reinterpret_cast<const float *>(moeBuf), 1, 8, 1,
                             moeBuf + 16, nullptr) == BM_OK);
        CHECK(fake_rt_last_combine_paced() == 0);
        phase.store(2);
        other.join();
        CHECK(mf_moe_combine(moeBuf, reinterpret_cast<const int32_t *>(moeBuf), reinterpret_cast<const float *>(moeBuf), 1, 8, 1,
                             moeBuf + 16, nullptr) == BM_OK);
        CHECK(fake_rt_last_combine_paced() == 1);
        CHECK(engine.Submit(s5, d5, l5, 2, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
        CHECK(fake_rt_last_hold() == HoldNanosFor(5120, 5120, 256, false));
        CHECK(engine.DrainThread() == BM_OK);
    }
    CHECK(engine.Submit(src.data(), dst.data(), len.data(), count, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
    CHECK(mf_xcopy_hold_stores(2500) == BM_OK);
    CHECK(engine.Submit(src.data(), dst.data(), len.data(), count, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
    CHECK(fake_rt_last_hold() == 2500);
    CHECK(engine.Submit(src.data(), dst.data(), len.data(), 4, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
    CHECK(fake_rt_last_hold() == 0);              // 128 chunks: the fixed time applies only where the rule does
    CHECK(mf_xcopy_hold_stores(0) == BM_OK);
    CHECK(engine.Submit(src.data(), dst.data(), len.data(), count, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
    CHECK(fake_rt_last_hold() == 0);
    CHECK(mf_xcopy_hold_stores(-2) == BM_INVALID_PARAM);
    CHECK(mf_xcopy_hold_stores(-1) == BM_OK);
    CHECK(engine.DrainThread() == BM_OK);
    bool ok = true;
    for (uint32_t i = 0; i < count; ++i) {
        ok = ok && std::memcmp(to.data() + (count - 1 - i) * seg, from.data() + i * seg, seg) == 0;
    }
    CHECK(ok);
    {
        // Tables (more than 128 segments) hold their stores too, a little longer than the kernel-argument form: K and V blocks in
        // turn (a pattern: descriptors out of the pinned slot) and ragged segments (descriptors through the group map), on 4 KiB
        // chunks below 24 MiB and on 16 KiB chunks from there to 64 MiB.
        const uint64_t k = 128u << 10;
        const uint64_t v = 16u << 10;
        std::vector<uint8_t> a(80u << 20), b(80u << 20);
        const uint64_t sa = (reinterpret_cast<uint64_t>(a.data()) + 4095) & ~4095ull;
        const uint64_t sb = (reinterpret_cast<uint64_t>(b.data()) + 4095) & ~4095ull;
        auto submit = [&](uint32_t n, bool ragged) {
            std::vector<uint64_t> s(n), d(n), l(n);
            uint64_t at = 0;
            for (uint32_t i = 0; i < n; ++i) {
                l[i] = ragged ? 4096u * (1 + (i * 2654435761u >> 27)) + 4096u * (i % 3) : (i % 2 == 0 ? k : v);
                s[i] = sa + at;
                d[i] = sb + at + 4096;
                at += l[i] + 8192;
            }
            CHECK(at + 8192 < (76u << 20));
            CHECK(engine.Submit(s.data(), d.data(), l.data(), n, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
            CHECK(engine.DrainThread() == BM_OK);
            uint64_t chunks4 = 0;
            uint64_t chunks16 = 0;
            uint64_t total = 0;
            for (uint32_t i = 0; i < n; ++i) {
                chunks4 += (l[i] + 4095) / 4096;
                chunks16 += (l[i] + 16383) / 16384;
                total += l[i];
            }
            const bool deep = total > (24u << 20);
            const uint32_t chunks = static_cast<uint32_t>(deep ? chunks16 : chunks4);
            return HoldNanosFor(chunks, chunks, deep ? 1024 : 256, false);
        };
        uint32_t rule = submit(244, false);                 // 17.6 MB: 4 KiB chunks
        CHECK(rule != 0 && fake_rt_last_table_hold() == rule + 1600);
        rule = submit(488, false);                          // 35 MB: 16 KiB chunks
        CHECK(rule != 0 && fake_rt_last_table_hold() == rule + 1600 + kHoldPinnedDeepExtraNanos);
        rule = submit(300, true);                           // ragged, some 20 MB
        CHECK(rule != 0 && fake_rt_last_table_hold() == rule + kHoldLookupExtraNanos);
        rule = submit(600, true);                           // ragged, some 40 MB
        CHECK(rule != 0 && fake_rt_last_table_hold() == rule + kHoldLookupDeepExtraNanos);
    }
    hybm_uninit();
}

// Which batches take the form with read and write windows.
static void TestWindows()
{
    {
        // the clock value a wave restores from the 40 published bits is the one nearest to its own clock, across a wrap of those bits
        const uint64_t span = 1ull << 40;
        const uint64_t nows[] = {5, span - 3, span + 7, 3 * span + 11, 7 * span - 1, (1ull << 63) + 12345};
        for (uint64_t now : nows) {
            for (int64_t off : {-2000ll, -64ll, 0ll, 64ll, 250000ll, -250000ll}) {
                if (off < 0 && static_cast<uint64_t>(-off) > now) {
                    continue;
                }
                const uint64_t start = now + static_cast<uint64_t>(off);
                CHECK(NearClock(now, start & (span - 1)) == start);
            }
        }
    }
    CHECK(hybm_init(0, 0) == BM_OK);
    const uint64_t gib = 1ull << 30;
    std::vector<uint8_t> mem(2 * gib + 1024);
    uint64_t s1 = (reinterpret_cast<uint64_t>(mem.data()) + 127) & ~127ull;      // on a cache line
    uint8_t *from = reinterpret_cast<uint8_t *>(s1);
    for (uint64_t i = 0; i < gib; i += 4093) {
        from[i] = static_cast<uint8_t>(i * 7 + 1);
    }
    XcopyEngine &engine = XcopyEngine::Instance();
    void *stream = mf_xcopy_thread_stream();
    uint64_t d1 = s1 + gib + 256;
    uint64_t l1 = gib;
    (void)fake_rt_last_window();
    uint64_t launchesBefore = mf_xcopy_launch_count();
    CHECK(engine.Submit(&s1, &d1, &l1, 1, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
    CHECK(fake_rt_last_window() == 7400000);                   // source and destination on cache lines: the higher rate
    CHECK(mf_xcopy_launch_count() - launchesBefore == 2);      // twice the minimum: two launches of 512 MiB, a schedule each
    CHECK(engine.DrainThread() == BM_OK);
    bool ok = true;
    for (uint64_t i = 0; i < gib; i += 4093) {
        ok = ok && from[gib + 256 + i] == static_cast<uint8_t>(i * 7 + 1);
    }
    CHECK(ok && from[gib + 256 + gib - 1] == from[gib - 1]);
    {
        // odd addresses that agree modulo 16 (head and tail bytes): windows at the general rate;
        // addresses that differ modulo 16: no windows, one launch
        uint64_t so = s1 + 3;
        uint64_t dO = s1 + gib + 256 + 19;
        uint64_t lo = gib - 64;
        std::memset(from + gib, 0, gib + 512);
        launchesBefore = mf_xcopy_launch_count();
        CHECK(engine.Submit(&so, &dO, &lo, 1, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
        CHECK(fake_rt_last_window() == 6800000);
        CHECK(mf_xcopy_launch_count() - launchesBefore == 1);      // 64 bytes short of twice the minimum
        CHECK(engine.DrainThread() == BM_OK);
        CHECK(std::memcmp(from + gib + 256 + 19, from + 3, lo) == 0 && from[gib + 256 + 18] == 0 && from[gib + 256 + 19 + lo] == 0);
        dO = s1 + gib + 256 + 5;
        std::memset(from + gib, 0, gib + 512);
        launchesBefore = mf_xcopy_launch_count();
        CHECK(engine.Submit(&so, &dO, &lo, 1, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
        CHECK(fake_rt_last_window() == 0);
        CHECK(mf_xcopy_launch_count() - launchesBefore == 1);
        CHECK(engine.DrainThread() == BM_OK);
        CHECK(std::memcmp(from + gib + 256 + 5, from + 3, lo) == 0 && from[gib + 256 + 4] == 0 && from[gib + 256 + 5 + lo] == 0);
    }
    {
        // three segments, 600 + 24 + 400 MiB: the first piece ends inside the long segment, at a multiple of 1 MiB, the
        // second takes its rest and the others; then 64 segments of 16 MiB: pieces end where segments end
        const uint64_t mib = 1ull << 20;
        std::memset(from + gib, 0, gib);
        uint64_t src3[3] = {s1, s1 + 600 * mib, s1 + 624 * mib};
        uint64_t dst3[3] = {s1 + gib, s1 + gib + 600 * mib, s1 + gib + 624 * mib};
        uint64_t len3[3] = {600 * mib, 24 * mib, 400 * mib};
        uint64_t word = 0;
        launchesBefore = mf_xcopy_launch_count();
        CHECK(engine.Submit(src3, dst3, len3, 3, MF_ROUTE_HBM, stream, &word, 32) == BM_OK);
        CHECK(mf_xcopy_launch_count() - launchesBefore == 2 && word == 32);
        CHECK(engine.DrainThread() == BM_OK);
        bool same = true;
        for (uint64_t i = 0; i < gib; i += 4093) {
            same = same && from[gib + i] == from[i];
        }
        CHECK(same && from[2 * gib - 1] == from[gib - 1]);
        std::memset(from + gib, 0, gib);
        std::vector<uint64_t> src64(64), dst64(64), len64(64, 16 * mib - 4096);
        for (uint32_t i = 0; i < 64; ++i) {
            src64[i] = s1 + i * 16 * mib;
            dst64[i] = s1 + gib + ((i * 5) % 64) * 16 * mib + 48;     // as the sources modulo 16, not on cache lines
        }
        launchesBefore = mf_xcopy_launch_count();
        CHECK(engine.Submit(src64.data(), dst64.data(), len64.data(), 64, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
        CHECK(mf_xcopy_launch_count() - launchesBefore == 1);      // 1023.75 MiB: below twice the minimum, one launch
        CHECK(engine.DrainThread() == BM_OK);
        same = true;
        for (uint32_t i = 0; i < 64 && same; ++i) {
            same = std::memcmp(reinterpret_cast<void *>(dst64[i]), reinterpret_cast<void *>(src64[i]), len64[i]) == 0;
        }
        CHECK(same);
        CHECK(fake_rt_last_window() == 6800000);       // destinations between cache lines: the general rate
        for (uint32_t i = 0; i < 64; ++i) {
            dst64[i] += 128 - 48;
        }
        CHECK(engine.Submit(src64.data(), dst64.data(), len64.data(), 64, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
        CHECK(fake_rt_last_window() == 7100000);       // on cache lines, 16 MiB each: the rate between
        CHECK(engine.DrainThread() == BM_OK);
    }
    l1 = (gib >> 3) - 1;                           // one byte below the limit of segments on cache lines: the ordinary form
    CHECK(engine.Submit(&s1, &d1, &l1, 1, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
    CHECK(fake_rt_last_window() == 0);
    l1 = gib >> 3;
    CHECK(engine.Submit(&s1, &d1, &l1, 1, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
    CHECK(fake_rt_last_window() == 7400000);
    {
        // between cache lines the same limit, at the general rate
        uint64_t so = s1 + 16;
        uint64_t dO = d1 + 48;
        uint64_t lo = (gib >> 3) - 1;
        CHECK(engine.Submit(&so, &dO, &lo, 1, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
        CHECK(fake_rt_last_window() == 0);
        lo = gib >> 3;
        CHECK(engine.Submit(&so, &dO, &lo, 1, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
        CHECK(fake_rt_last_window() == 6800000);
    }
    l1 = gib;
    CHECK(engine.Submit(&s1, &d1, &l1, 1, MF_ROUTE_HBM, stream, nullptr, 0, true) == BM_OK);
    CHECK(fake_rt_last_window() == 0);             // unordered launches overlap on purpose
    CHECK(mf_xcopy_windows(0) == BM_OK);
    CHECK(engine.Submit(&s1, &d1, &l1, 1, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
    CHECK(fake_rt_last_window() == 0);
    CHECK(mf_xcopy_windows(999) == BM_INVALID_PARAM && mf_xcopy_windows(6400000) == BM_OK);
    {
        std::atomic<int> phase{0};
        std::thread other([&] {
            (void)mf_xcopy_thread_stream();
            phase.store(1);
            while (phase.load() != 2) {
                std::this_thread::yield();
            }
        });
        while (phase.load() != 1) {
            std::this_thread::yield();
        }
        CHECK(engine.Submit(&s1, &d1, &l1, 1, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
        CHECK(fake_rt_last_window() == 0);         // a second submitter with a stream of its own
        phase.store(2);
        other.join();
    }
    CHECK(engine.Submit(&s1, &d1, &l1, 1, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
    CHECK(fake_rt_last_window() == 6400000);
    CHECK(mf_xcopy_windows(6800000) == BM_OK);
    CHECK(engine.DrainThread() == BM_OK);
    {
        // a table of long segments is cut into launches of 128 segments, each in windows: 300 x 4 MiB -> 128 + 128 + 44
        const uint32_t count = 300;
        const uint64_t seg = 4ull << 20;
        std::vector<uint64_t> src(count), dst(count), len(count, seg);
        for (uint32_t i = 0; i < count; ++i) {
            src[i] = s1 + (i % 200) * seg + 128 * i;     // not adjacent: no merging
            dst[i] = s1 + gib + ((i * 7) % 200) * seg + 256 * i;
        }
        const uint64_t before = mf_xcopy_launch_count();
        (void)fake_rt_last_window();
        uint64_t word = 0;
        CHECK(engine.Submit(src.data(), dst.data(), len.data(), count, MF_ROUTE_HBM, stream, &word, 32) == BM_OK);
        CHECK(mf_xcopy_launch_count() - before == 3);
        CHECK(fake_rt_last_window() == 6800000);   // all three slices in windows (512, 512 and 176 MiB of segments on cache lines)
        CHECK(word == 32);
        CHECK(engine.DrainThread() == BM_OK);
    }
    {
        // segments on cache lines are worth slicing from 1 MiB each (128 MiB a launch); between cache lines only from 4 MiB
        const uint32_t count = 300;
        const uint64_t seg = 1ull << 20;
        std::vector<uint64_t> src(count), dst(count), len(count, seg);
        for (uint32_t i = 0; i < count; ++i) {
            src[i] = s1 + (i % 200) * 2 * seg + 128 * i;
            dst[i] = s1 + gib + ((i * 7) % 300) * 2 * seg + 256 * i;        // 300 places of 2 MiB, none shared
        }
        uint64_t before = mf_xcopy_launch_count();
        (void)fake_rt_last_window();
        CHECK(engine.Submit(src.data(), dst.data(), len.data(), count, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
        CHECK(mf_xcopy_launch_count() - before == 3);      // 128 + 128 + 44 segments; the last launch (44 MiB) without windows
        CHECK(engine.DrainThread() == BM_OK);
        bool same = true;
        for (uint32_t i = 0; i < count && same; i += 7) {
            same = std::memcmp(reinterpret_cast<void *>(dst[i]), reinterpret_cast<void *>(src[i]), seg) == 0;
        }
        CHECK(same);
        for (uint32_t i = 0; i < count; ++i) {
            src[i] += 16;
            dst[i] += 48;
        }
        before = mf_xcopy_launch_count();
        (void)fake_rt_last_window();
        CHECK(engine.Submit(src.data(), dst.data(), len.data(), count, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
        CHECK(mf_xcopy_launch_count() - before <= 2 && fake_rt_last_window() == 0);     // one table launch (and its upload)
        CHECK(engine.DrainThread() == BM_OK);
    }
    CHECK(mf_xcopy_windows(MF_XCOPY_WINDOWS_OWN_CHOICE) == BM_OK);      // from the rate set by hand back to the library's three
    l1 = gib;
    CHECK(engine.Submit(&s1, &d1, &l1, 1, MF_ROUTE_HBM, stream, nullptr, 0) == BM_OK);
    CHECK(fake_rt_last_window() == XcopyTuning{}.windowLongMBps);
    CHECK(engine.DrainThread() == BM_OK);
    hybm_uninit();
}

int main()
{
    SetLogLevel(3);
    SetLogSink([](int, const char *) {});
    TestCompose();
    TestPlanners();
    TestHostCopy();
    TestSlotRing();
    TestCApi();                                  // device window: reserved address space, HBM mapped in
    setenv("MF_HIP_GVA_WINDOW", "malloc", 1);
    TestCApi();                                  // device window: one ordinary allocation
    unsetenv("MF_HIP_GVA_WINDOW");
    TestTrans();
    TestLeases();
    TestMappedWindow();
    TestPlugin();
    TestHeldStores();
    TestWindows();
    TestLongSegments();
    TestStreamDeck();
    TestWindowedRectangles();
    TestCalibration();
    TestUnorderedFanOut();
    TestHostLaunchCosts();
    TestWaitOfShortQueues();
    if (g_failed != 0) {
        std::printf("%d check(s) failed\n", g_failed);
        return 1;
    }
    // A caller that never tears down: a pool with memory, a transfer object with registered memory and
    // a used stream stay alive past main().  Static destructors must leave the runtime alone.
    smem_bm_config_t cfg;
    smem_bm_config_init(&cfg);
    CHECK(smem_bm_init("tcp://127.0.0.1:1", 1, 0, &cfg) == SM_OK);
    smem_bm_t left = smem_bm_create(5, 1, SMEMB_DATA_OP_SDMA, 4u << 20, 4u << 20, 0);
    CHECK(left != nullptr && smem_bm_join(left, 0) == SM_OK);
    smem_copy_params cp{smem_bm_ptr_by_mem_type(left, SMEM_MEM_TYPE_HOST, 0), smem_bm_ptr_by_mem_type(left, SMEM_MEM_TYPE_DEVICE, 0), 4096};
    CHECK(smem_bm_copy(left, &cp, SMEMB_COPY_G2G, ASYNC_COPY_FLAG) == SM_OK);
    smem_trans_config_t tc;
    smem_trans_config_init(&tc);
    tc.deviceId = 0;
    tc.role = SMEM_TRANS_BOTH;
    CHECK(smem_trans_init(&tc) == SM_OK);
    smem_trans_t leftTrans = smem_trans_create("tcp://127.0.0.1:5432", "127.0.0.1:5400", &tc);
    CHECK(leftTrans != nullptr && smem_trans_malloc(leftTrans, 100) != nullptr);
    if (g_failed != 0) {
        std::printf("%d check(s) failed\n", g_failed);
        return 1;
    }
    std::printf("host stack tests passed\n");
    std::fflush(stdout);
    fake_rt_seal();
    return 0;
}
