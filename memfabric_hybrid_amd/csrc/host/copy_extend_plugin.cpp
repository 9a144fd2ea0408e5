// The two symbols of libmf_hybm_copy_extend.so (declared in
// include/mf_hip_copy_extend.h).  They take over from the AscendC launchers at
// src/hybm/csrc/copy_extend/hybm_copy_kernel.cpp:80-83,121-124, so the
// reference's own HostDataOpSDMA can drive the HIP kernels through its
// COPY_EXTEND_FLAG path without a source change.
#include <stdint.h>

#include <atomic>
#include <vector>

#include "../../../include/mf_hip_copy_extend.h"
#include "../../../include/mf_xcopy_types.h"
#include "../rt/mf_rt.h"
#include "mf_log.h"
#include "xcopy_engine.h"

using namespace mf;

namespace {

// The host program selected its GPU long before it loaded the plugin; adopt it.
bool EngineReady()
{
    XcopyEngine &engine = XcopyEngine::Instance();
    if (engine.Started()) {
        return true;
    }
    int dev = mfrt_current_device();
    if (dev < 0) {
        MF_ERROR("copy plugin: no current GPU");
        return false;
    }
    return engine.Start(dev) == BM_OK;
}

// Neither entry point can return an error, so failures are counted (and logged) where a host
// program can ask for them.
std::atomic<uint64_t> g_failures{0};

void Failed(const char *what, int code, uint32_t count, const void *mask)
{
    g_failures.fetch_add(1, std::memory_order_relaxed);
    MF_ERROR("copy plugin: " << what << " failed with " << code << " (" << count << " segments, completion word at " << mask
             << " left untouched)");
}

int RouteFor(const void *src, const void *dst)
{
    if (mfrt_pointer_kind(dst) == MFRT_PTR_PINNED_HOST) {
        return MFRT_ROUTE_TO_HOST;
    }
    if (mfrt_pointer_kind(src) == MFRT_PTR_PINNED_HOST) {
        return MFRT_ROUTE_FROM_HOST;
    }
    return MFRT_ROUTE_HBM;
}

}  // namespace

extern "C" __attribute__((visibility("default"))) void hybm_copy_extend(void *src, void *dst, uint64_t len,
                                                                          uint32_t dim, void *stream)
{
    (void)dim;
    if (src == nullptr || dst == nullptr || len == 0 || !EngineReady()) {
        return;
    }
    const uint64_t s = reinterpret_cast<uint64_t>(src);
    const uint64_t d = reinterpret_cast<uint64_t>(dst);
    // NULL stream means the null stream to this ABI, which the engine cannot tell from "pick one":
    // the reference never passes NULL here (hybm_data_op_sdma.cpp:420), so the thread stream is fine.
    const int ret = XcopyEngine::Instance().Submit(&s, &d, &len, 1, RouteFor(src, dst), stream, nullptr, 0);
    if (ret != BM_OK) {
        Failed("hybm_copy_extend", ret, 1, nullptr);
    }
}

extern "C" __attribute__((visibility("default"))) uint64_t mf_copy_extend_failures(void)
{
    return g_failures.load(std::memory_order_relaxed);
}

extern "C" __attribute__((visibility("default"))) void hybm_batch_copy_extend(void *param, uint32_t count, void *mask,
                                                                                uint32_t dim, void *stream)
{
    if (param == nullptr || !EngineReady()) {
        Failed("hybm_batch_copy_extend (no table or no GPU)", BM_INVALID_PARAM, count, mask);
        return;
    }
    XcopyEngine &engine = XcopyEngine::Instance();
    if (mfrt_pointer_kind(param) != MFRT_PTR_DEVICE) {
        // Host-visible table (what the reference passes: a pinned, device-mapped parameter slot).
        // It is consumed right here, on the CPU: the descriptors travel on in the launch itself,
        // nothing on the GPU ever reads `param`.  The completion word is the caller's "this
        // parameter slot may be refilled" marker (TryGetOneParamSpace,
        // src/hybm/csrc/data_operation/host/hybm_data_op_sdma.cpp:485-502; completion of the
        // copy itself is awaited on the stream, :537-540), so when the CPU can write the word it
        // is stored here, after the launch went out, and no second launch is queued behind the copy.
        const uint64_t *t = static_cast<const uint64_t *>(param);
        thread_local std::vector<uint64_t> s;
        thread_local std::vector<uint64_t> d;
        thread_local std::vector<uint64_t> l;
        s.resize(count);
        d.resize(count);
        l.resize(count);
        for (uint32_t i = 0; i < count; ++i) {
            s[i] = t[3ull * i];
            d[i] = t[3ull * i + 1];
            l[i] = t[3ull * i + 2];
        }
        const int route = count == 0 ? MFRT_ROUTE_HBM
                                     : RouteFor(reinterpret_cast<const void *>(s[0]), reinterpret_cast<const void *>(d[0]));
        const bool hostWord = mask != nullptr && mfrt_pointer_kind(mask) != MFRT_PTR_DEVICE;
        const int ret = engine.Submit(s.data(), d.data(), l.data(), count, route, stream, hostWord ? nullptr : mask, dim);
        if (ret != BM_OK) {
            Failed("hybm_batch_copy_extend", ret, count, mask);
            return;
        }
        if (hostWord) {
            __atomic_store_n(static_cast<uint64_t *>(mask), static_cast<uint64_t>(dim), __ATOMIC_RELEASE);
        }
        return;
    }
    const int ret = engine.SubmitDeviceTable(param, count, MFRT_ROUTE_HBM, stream, mask, dim);
    if (ret != BM_OK) {
        Failed("hybm_batch_copy_extend (device-resident table)", ret, count, mask);
    }
}
