// HIP side of the thin runtime layer declared in mf_rt.h.
// On MI355X this replaces the reference's whole stream engine
// (src/hybm/csrc/ts_engine/hybm_stream.cpp:213-242,358-389: hand-built SQEs,
// one driver call per descriptor, usleep polling) and its dlopen shims for
// the vendor runtime (src/hybm/csrc/under_api/dl_acl_api.cpp:73-101): a HIP
// stream is the submission queue, an event is the completion record.
#include <hip/hip_runtime.h>

#include <chrono>

#include <atomic>
#include <cstring>
#include <mutex>

#include "mf_rt.h"

namespace {

std::mutex g_lock;
std::atomic<int> g_device{-1};
uint32_t g_cuCount = 0;

inline int Code(hipError_t e)
{
    return static_cast<int>(e);
}

}  // namespace

extern "C" int mfrt_init(int device)
{
    std::lock_guard<std::mutex> guard(g_lock);
    if (g_device.load() >= 0) {
        return g_device.load() == device ? 0 : Code(hipErrorInvalidDevice);
    }
    int count = 0;
    hipError_t err = hipGetDeviceCount(&count);
    if (err != hipSuccess) {
        return Code(err);
    }
    if (device < 0 || device >= count) {
        return Code(hipErrorInvalidDevice);
    }
    err = hipSetDevice(device);
    if (err != hipSuccess) {
        return Code(err);
    }
    hipDeviceProp_t prop;
    err = hipGetDeviceProperties(&prop, device);
    if (err != hipSuccess) {
        return Code(err);
    }
    g_cuCount = static_cast<uint32_t>(prop.multiProcessorCount);
    g_device.store(device);
    return 0;
}

extern "C" int mfrt_current_device(void)
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return -1;
    }
    return dev;
}

extern "C" int mfrt_bind_thread(void)
{
    const int dev = g_device.load();
    if (dev < 0) {
        return Code(hipErrorNotInitialized);
    }
    thread_local int bound = -1;
    if (bound == dev) {
        return 0;
    }
    hipError_t err = hipSetDevice(dev);
    if (err == hipSuccess) {
        bound = dev;
    }
    return Code(err);
}

extern "C" void mfrt_shutdown(void)
{
    std::lock_guard<std::mutex> guard(g_lock);
    if (g_device.load() >= 0) {
        (void)hipDeviceSynchronize();
        g_device.store(-1);
    }
}

extern "C" int mfrt_is_initialised(void)
{
    return g_device.load() >= 0 ? 1 : 0;
}

extern "C" int mfrt_device_id(void)
{
    return g_device.load();
}

extern "C" uint32_t mfrt_cu_count(void)
{
    return g_cuCount;
}

extern "C" const char *mfrt_error_string(int err)
{
    return hipGetErrorString(static_cast<hipError_t>(err));
}

extern "C" void *mfrt_alloc_device(uint64_t bytes)
{
    void *p = nullptr;
    if (hipMalloc(&p, bytes) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    return p;
}

extern "C" int mfrt_free_device(void *p)
{
    return Code(hipFree(p));
}

namespace {
hipMemAllocationProp WindowProp()
{
    hipMemAllocationProp prop{};
    prop.type = hipMemAllocationTypePinned;
    prop.location.type = hipMemLocationTypeDevice;
    prop.location.id = g_device.load();
    return prop;
}
}  // namespace

extern "C" uint64_t mfrt_window_granularity(void)
{
    const hipMemAllocationProp prop = WindowProp();
    size_t granularity = 0;
    if (hipMemGetAllocationGranularity(&granularity, &prop, hipMemAllocationGranularityRecommended) != hipSuccess ||
        granularity == 0) {
        (void)hipGetLastError();
        return 0;
    }
    return granularity;
}

extern "C" void *mfrt_window_reserve(uint64_t bytes)
{
    void *base = nullptr;
    if (hipMemAddressReserve(&base, bytes, 0, nullptr, 0) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    return base;
}

extern "C" int mfrt_window_release(void *base, uint64_t bytes)
{
    return Code(hipMemAddressFree(base, bytes));
}

namespace {
thread_local int t_windowError = 0;   // step * 10000 + hipError_t of the last failed window call
}  // namespace

extern "C" int mfrt_window_last_error(void)
{
    return t_windowError;
}

extern "C" void *mfrt_window_map(void *addr, uint64_t bytes, void *accessBase, uint64_t accessBytes)
{
    const hipMemAllocationProp prop = WindowProp();
    hipMemGenericAllocationHandle_t handle{};
    hipError_t err = hipMemCreate(&handle, bytes, &prop, 0);
    if (err != hipSuccess) {
        t_windowError = 10000 + static_cast<int>(err);
        (void)hipGetLastError();
        return nullptr;
    }
    err = hipMemMap(addr, bytes, 0, handle, 0);
    if (err != hipSuccess) {
        t_windowError = 20000 + static_cast<int>(err);
        (void)hipGetLastError();
        (void)hipMemRelease(handle);
        return nullptr;
    }
    hipMemAccessDesc access{};
    access.location = prop.location;
    access.flags = hipMemAccessFlagsProtReadWrite;
    // Access is granted on the caller's whole backed run, not on the new piece alone: on this
    // runtime a grant on a piece inside a reservation is refused (invalid value) unless the piece
    // has the size of the reservation's first mapping, while a grant that starts at the first
    // mapping and covers every mapped byte up to the new end is accepted.
    err = hipMemSetAccess(accessBase, accessBytes, &access, 1);
    if (err != hipSuccess) {
        t_windowError = 30000 + static_cast<int>(err);
        (void)hipGetLastError();
        (void)hipMemUnmap(addr, bytes);
        (void)hipMemRelease(handle);
        return nullptr;
    }
    static_assert(sizeof(handle) == sizeof(void *), "allocation handles travel as pointers");
    void *out = nullptr;
    std::memcpy(&out, &handle, sizeof(out));
    return out;
}

extern "C" int mfrt_window_unmap(void *addr, uint64_t bytes, void *handle)
{
    hipMemGenericAllocationHandle_t h{};
    std::memcpy(&h, &handle, sizeof(h));
    const int err = Code(hipMemUnmap(addr, bytes));
    const int rel = Code(hipMemRelease(h));
    return err != 0 ? err : rel;
}

extern "C" void *mfrt_alloc_host(uint64_t bytes)
{
    void *p = nullptr;
    // Coherent on purpose, whatever HIP_HOST_COHERENT says: kernels read descriptor tables out of this memory
    // that the CPU rewrites between launches, and the CPU reads staged data the moment an event has fired.
    if (hipHostMalloc(&p, bytes, hipHostMallocMapped | hipHostMallocPortable | hipHostMallocCoherent) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    return p;
}

extern "C" int mfrt_free_host(void *p)
{
    return Code(hipHostFree(p));
}

extern "C" int mfrt_pointer_kind(const void *p)
{
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError();  // unknown to the runtime: plain pageable memory
        return MFRT_PTR_PAGEABLE;
    }
    switch (attr.type) {
        case hipMemoryTypeDevice:
            return MFRT_PTR_DEVICE;
        case hipMemoryTypeHost:
            return MFRT_PTR_PINNED_HOST;
        case hipMemoryTypeManaged:
            return MFRT_PTR_DEVICE;
        default:
            return MFRT_PTR_PAGEABLE;
    }
}

extern "C" void *mfrt_stream_create(void)
{
    hipStream_t s = nullptr;
    if (hipStreamCreateWithFlags(&s, hipStreamNonBlocking) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    return s;
}

extern "C" int mfrt_stream_destroy(void *stream)
{
    return Code(hipStreamDestroy(static_cast<hipStream_t>(stream)));
}

extern "C" int mfrt_stream_sync(void *stream)
{
    return Code(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
}

extern "C" int mfrt_device_sync(void)
{
    return Code(hipDeviceSynchronize());
}

extern "C" void *mfrt_event_create(void)
{
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    return e;
}

extern "C" int mfrt_event_destroy(void *event)
{
    return Code(hipEventDestroy(static_cast<hipEvent_t>(event)));
}

extern "C" int mfrt_event_record(void *event, void *stream)
{
    return Code(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
}

extern "C" int mfrt_stream_wait_event(void *stream, void *event)
{
    return Code(hipStreamWaitEvent(static_cast<hipStream_t>(stream), static_cast<hipEvent_t>(event), 0));
}

extern "C" int mfrt_event_sync(void *event)
{
    return Code(hipEventSynchronize(static_cast<hipEvent_t>(event)));
}

extern "C" int mfrt_event_done(void *event)
{
    hipError_t err = hipEventQuery(static_cast<hipEvent_t>(event));
    if (err == hipSuccess) {
        return 1;
    }
    if (err == hipErrorNotReady) {
        (void)hipGetLastError();
        return 0;
    }
    return -Code(err);
}

extern "C" float mfrt_event_elapsed_ms(void *start, void *stop)
{
    float ms = -1.0f;
    if (hipEventElapsedTime(&ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)) != hipSuccess) {
        (void)hipGetLastError();
        return -1.0f;
    }
    return ms;
}

extern "C" int mfrt_memcpy(void *dst, const void *src, uint64_t bytes)
{
    return Code(hipMemcpy(dst, src, bytes, hipMemcpyDefault));
}

extern "C" int mfrt_memset(void *dst, int value, uint64_t bytes)
{
    hipError_t err = hipMemset(dst, value, bytes);
    if (err != hipSuccess) {
        return Code(err);
    }
    return Code(hipDeviceSynchronize());
}

extern "C" int mfrt_memcpy_async(void *dst, const void *src, uint64_t bytes, void *stream)
{
    return Code(hipMemcpyAsync(dst, src, bytes, hipMemcpyDefault, static_cast<hipStream_t>(stream)));
}

// Whether two streams share a hardware queue.  The runtime deals its streams out over a few hardware queues, and
// launches on streams that share one run one after the other however independent they are.  A single lane that waits
// 40 us by the clock is launched on `a`, an empty kernel on `b`; when the empty kernel has ended, either the wait
// still runs (different queues: 0) or it has ended too (the empty kernel had to queue behind it: 1).  -1: not known
// (no clock rate, or the host took so long between the two launches that the answer would mean nothing).  Both
// streams must be idle.  About 50 us.
namespace {
__global__ void DelayKernel(uint32_t ticks)
{
    const uint64_t t0 = wall_clock64();
    while (wall_clock64() - t0 < ticks) {
        __builtin_amdgcn_s_sleep(8);
    }
}

__global__ void NothingKernel() {}
}  // namespace

extern "C" int mfrt_streams_share_queue(void *a, void *b)
{
    int dev = 0;
    int khz = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess ||
        khz <= 0) {
        return -1;
    }
    hipEvent_t ea = nullptr;
    hipEvent_t eb = nullptr;
    if (hipEventCreateWithFlags(&ea, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&eb, hipEventDisableTiming) != hipSuccess) {
        if (ea != nullptr) {
            (void)hipEventDestroy(ea);
        }
        (void)hipGetLastError();
        return -1;
    }
    const uint32_t ticks = static_cast<uint32_t>(static_cast<uint64_t>(khz) * 40 / 1000);   // 40 us
    int answer = -1;
    for (int attempt = 0; attempt < 3 && answer < 0; ++attempt) {
        const auto t0 = std::chrono::steady_clock::now();
        hipLaunchKernelGGL(DelayKernel, dim3(1), dim3(1), 0, static_cast<hipStream_t>(a), ticks);
        (void)hipEventRecord(ea, static_cast<hipStream_t>(a));
        hipLaunchKernelGGL(NothingKernel, dim3(1), dim3(1), 0, static_cast<hipStream_t>(b));
        (void)hipEventRecord(eb, static_cast<hipStream_t>(b));
        const auto t1 = std::chrono::steady_clock::now();
        if (hipGetLastError() != hipSuccess || hipEventSynchronize(eb) != hipSuccess) {
            break;
        }
        const bool firstEnded = hipEventQuery(ea) == hipSuccess;
        (void)hipGetLastError();   // hipErrorNotReady is the other answer, not a failure
        if (hipEventSynchronize(ea) != hipSuccess) {
            break;
        }
        if (std::chrono::duration<double, std::micro>(t1 - t0).count() < 20.0) {
            answer = firstEnded ? 1 : 0;
        }
    }
    (void)hipEventDestroy(ea);
    (void)hipEventDestroy(eb);
    return answer;
}
