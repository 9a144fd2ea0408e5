// HIP side of the thin runtime layer declared in mf_rt.h.
// On MI355X this replaces the reference's whole stream engine
// (src/hybm/csrc/ts_engine/hybm_stream.cpp:213-242,358-389: hand-built SQEs,
// one driver call per descriptor, usleep polling) and its dlopen shims for
// the vendor runtime (src/hybm/csrc/under_api/dl_acl_api.cpp:73-101): a HIP
// stream is the submission queue, an event is the completion record.
#include <hip/hip_runtime.h>

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
