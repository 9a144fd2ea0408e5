// Batched discrete copy ("xcopy") for gfx950: one fused launch moves every
// segment of a batch, whatever mix of lengths it holds.
//
// Replaces the device side of the reference's copy plugin
// (src/hybm/csrc/copy_extend/hybm_copy_kernel.cpp:44-119: 32 blocks, whole
// segments per block, one 64 KiB staging tile, load and store serialised).
// Here a workgroup owns a chunk of bytes, not a segment; data goes
// register-to-register with four 128-bit loads in flight per lane, and
// the descriptor lookup costs two scalar loads from the kernel-argument
// block for batches of up to 128 segments.
//
// Bound: HBM bandwidth (2 bytes of traffic per payload byte) for device to
// device, the host link (1 byte per payload byte) when one side is pinned
// host memory.  No LDS, no MFMA: nothing here is reused or contracted.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "xcopy_plan.h"
#include "../rt/mf_rt.h"

namespace mf {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 u32x4_any __attribute__((aligned(1)));  // source side may sit at any byte address

#define MF_GLOBAL __attribute__((address_space(1)))
typedef const MF_GLOBAL u32x4_any *GSrcUnit;
typedef MF_GLOBAL u32x4 *GDstUnit;
typedef const MF_GLOBAL uint8_t *GSrcByte;
typedef MF_GLOBAL uint8_t *GDstByte;

// kRoute selects cache policy only; addressing is identical.
//   MFRT_ROUTE_HBM        both sides in HBM: streaming loads and stores
//   MFRT_ROUTE_TO_HOST    destination is pinned host DRAM: write-combining friendly nontemporal stores
//   MFRT_ROUTE_FROM_HOST  source is pinned host DRAM: plain stores into HBM
template <int kRoute>
__device__ __forceinline__ u32x4 LoadUnit(uint64_t addr)
{
    GSrcUnit p = reinterpret_cast<GSrcUnit>(addr);
    if (kRoute == MFRT_ROUTE_TO_HOST) {
        return *p;
    }
    return __builtin_nontemporal_load(p);
}

template <int kRoute>
__device__ __forceinline__ void StoreUnit(uint64_t addr, u32x4 v)
{
    GDstUnit p = reinterpret_cast<GDstUnit>(addr);
    if (kRoute == MFRT_ROUTE_FROM_HOST) {
        *p = v;
    } else {
        __builtin_nontemporal_store(v, p);
    }
}

__device__ __forceinline__ void CopyByte(uint64_t src, uint64_t dst)
{
    *reinterpret_cast<GDstByte>(dst) = *reinterpret_cast<GSrcByte>(src);
}

constexpr uint32_t kDepth = 4;                          // 128-bit loads in flight per lane
constexpr uint32_t kTile = kDepth * kXcopyThreads;      // units one workgroup moves per step

// Copy chunk k of one segment.  All arguments are wave-uniform.
template <int kRoute>
__device__ __forceinline__ void CopyChunk(uint64_t src, uint64_t dst, uint64_t len, uint64_t k, uint32_t units)
{
    const SegGeom g = SegmentGeometry(dst, len);
    const uint64_t u0 = k * units;
    const uint64_t left = g.body > u0 ? g.body - u0 : 0;
    const uint32_t n = left < units ? static_cast<uint32_t>(left) : units;
    const uint64_t s = src + g.head + u0 * kUnitBytes;
    const uint64_t d = dst + g.head + u0 * kUnitBytes;
    const uint32_t tid = threadIdx.x;

    uint32_t i = 0;
    for (; i + kTile <= n; i += kTile) {
        u32x4 v[kDepth];
#pragma unroll
        for (uint32_t j = 0; j < kDepth; ++j) {
            v[j] = LoadUnit<kRoute>(s + static_cast<uint64_t>(i + j * kXcopyThreads + tid) * kUnitBytes);
        }
#pragma unroll
        for (uint32_t j = 0; j < kDepth; ++j) {
            StoreUnit<kRoute>(d + static_cast<uint64_t>(i + j * kXcopyThreads + tid) * kUnitBytes, v[j]);
        }
    }
    if (i < n) {
        u32x4 v[kDepth];
#pragma unroll
        for (uint32_t j = 0; j < kDepth; ++j) {
            const uint32_t u = i + j * kXcopyThreads + tid;
            if (u < n) {
                v[j] = LoadUnit<kRoute>(s + static_cast<uint64_t>(u) * kUnitBytes);
            }
        }
#pragma unroll
        for (uint32_t j = 0; j < kDepth; ++j) {
            const uint32_t u = i + j * kXcopyThreads + tid;
            if (u < n) {
                StoreUnit<kRoute>(d + static_cast<uint64_t>(u) * kUnitBytes, v[j]);
            }
        }
    }
    if (k == 0 && tid < g.head) {
        CopyByte(src + tid, dst + tid);
    }
    if (u0 + units >= g.body && tid < g.tail) {
        const uint64_t off = g.head + g.body * kUnitBytes + tid;
        CopyByte(src + off, dst + off);
    }
}

// Completion word protocol of the plugin ABI: the last workgroup to finish
// stores `value` into *mask (system scope) after every workgroup's stores
// are visible; the per-launch counter returns to zero for its next user.
__device__ __forceinline__ void SignalDone(uint64_t *mask, uint32_t value, uint32_t *counter)
{
    __threadfence_system();
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t prev = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        if (prev + 1 == gridDim.x) {
            __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(mask, static_cast<uint64_t>(value), __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
        }
    }
}

template <int kRoute>
__global__ __launch_bounds__(kXcopyThreads) void XcopyInlineKernel(const InlinePlan p, uint64_t *mask, uint32_t maskValue,
                                                                   uint32_t *counter)
{
    for (uint32_t c = blockIdx.x; c < p.nchunk; c += gridDim.x) {
        // Two-level lookup of the segment that owns chunk c: largest s with first[s] <= c.
        uint32_t hi = 0;
#pragma unroll
        for (uint32_t i = 1; i < kInlineCoarse; ++i) {
            hi += (p.coarse[i] <= c) ? 1u : 0u;
        }
        const uint32_t base = hi * kInlineFan;
        uint32_t s = base;
#pragma unroll
        for (uint32_t j = 1; j < kInlineFan; ++j) {
            s += (p.first[base + j] <= c) ? 1u : 0u;
        }
        CopyChunk<kRoute>(p.src[s], p.dst[s], p.len[s], c - p.first[s], p.units);
    }
    if (mask != nullptr) {
        SignalDone(mask, maskValue, counter);
    }
}

template <int kRoute>
__global__ __launch_bounds__(kXcopyThreads) void XcopyTableKernel(const uint64_t *__restrict__ triples,
                                                                  const uint32_t *__restrict__ first,
                                                                  const uint32_t *__restrict__ nchunkDev, uint32_t nseg,
                                                                  uint32_t nchunkHost, uint32_t units, uint64_t *mask,
                                                                  uint32_t maskValue, uint32_t *counter)
{
    const uint32_t nchunk = nchunkDev != nullptr ? *nchunkDev : nchunkHost;
    for (uint32_t c = blockIdx.x; c < nchunk; c += gridDim.x) {
        // upper_bound(first, c) - 1 over nseg + 1 prefix entries
        uint32_t lo = 0;
        uint32_t hi = nseg;  // invariant: first[lo] <= c < first[hi]
        while (hi - lo > 1) {
            const uint32_t mid = (lo + hi) >> 1;
            if (first[mid] <= c) {
                lo = mid;
            } else {
                hi = mid;
            }
        }
        const uint64_t *t = triples + 3ull * lo;
        CopyChunk<kRoute>(t[0], t[1], t[2], c - first[lo], units);
    }
    if (mask != nullptr) {
        SignalDone(mask, maskValue, counter);
    }
}

// Device-side planner for a table the host cannot read: one workgroup turns
// the triples into the chunk prefix the table kernel searches.
constexpr uint32_t kPlanThreads = 1024;

__global__ __launch_bounds__(kPlanThreads) void XcopyPlanKernel(const uint64_t *__restrict__ triples, uint32_t nseg,
                                                                uint32_t units, uint32_t *__restrict__ first,
                                                                uint32_t *__restrict__ nchunk)
{
    __shared__ uint32_t partial[kPlanThreads];
    const uint32_t tid = threadIdx.x;
    const uint32_t per = (nseg + kPlanThreads - 1) / kPlanThreads;
    const uint32_t lo = tid * per;
    const uint32_t hi = lo + per < nseg ? lo + per : nseg;
    uint32_t sum = 0;
    for (uint32_t i = lo; i < hi; ++i) {
        sum += static_cast<uint32_t>(SegmentChunks(triples[3ull * i + 1], triples[3ull * i + 2], units));
    }
    partial[tid] = sum;
    __syncthreads();
    for (uint32_t step = 1; step < kPlanThreads; step <<= 1) {
        const uint32_t add = tid >= step ? partial[tid - step] : 0;
        __syncthreads();
        partial[tid] += add;
        __syncthreads();
    }
    uint32_t run = partial[tid] - sum;  // exclusive prefix of this lane's slice
    for (uint32_t i = lo; i < hi; ++i) {
        first[i] = run;
        run += static_cast<uint32_t>(SegmentChunks(triples[3ull * i + 1], triples[3ull * i + 2], units));
    }
    if (tid == kPlanThreads - 1) {
        first[nseg] = partial[tid];
        *nchunk = partial[tid];
    }
}

template <int kRoute>
int LaunchInline(const InlinePlan &plan, uint32_t grid, uint64_t *mask, uint32_t maskValue, uint32_t *counter,
                 hipStream_t stream)
{
    hipLaunchKernelGGL(XcopyInlineKernel<kRoute>, dim3(grid), dim3(kXcopyThreads), 0, stream, plan, mask, maskValue,
                       counter);
    return static_cast<int>(hipGetLastError());
}

template <int kRoute>
int LaunchTable(const TablePlan &plan, const uint32_t *nchunkDev, uint32_t grid, uint64_t *mask, uint32_t maskValue,
                uint32_t *counter, hipStream_t stream)
{
    hipLaunchKernelGGL(XcopyTableKernel<kRoute>, dim3(grid), dim3(kXcopyThreads), 0, stream, plan.triples, plan.first,
                       nchunkDev, plan.nseg, plan.nchunk, plan.units, mask, maskValue, counter);
    return static_cast<int>(hipGetLastError());
}

}  // namespace
}  // namespace mf

extern "C" int mfk_xcopy_inline(const void *inlinePlan, int route, uint32_t grid, void *mask, uint32_t maskValue,
                                void *counter, void *stream)
{
    const mf::InlinePlan &plan = *static_cast<const mf::InlinePlan *>(inlinePlan);
    if (plan.nchunk == 0 && mask == nullptr) {
        return 0;
    }
    if (grid == 0) {
        grid = 1;
    }
    uint64_t *m = static_cast<uint64_t *>(mask);
    uint32_t *c = static_cast<uint32_t *>(counter);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (route) {
        case MFRT_ROUTE_HBM:
            return mf::LaunchInline<MFRT_ROUTE_HBM>(plan, grid, m, maskValue, c, s);
        case MFRT_ROUTE_TO_HOST:
            return mf::LaunchInline<MFRT_ROUTE_TO_HOST>(plan, grid, m, maskValue, c, s);
        case MFRT_ROUTE_FROM_HOST:
            return mf::LaunchInline<MFRT_ROUTE_FROM_HOST>(plan, grid, m, maskValue, c, s);
        default:
            return -1;
    }
}

extern "C" int mfk_xcopy_table(const void *triples, const void *first, const void *nchunkDev, uint32_t nseg,
                               uint32_t nchunk, uint32_t units, int route, uint32_t grid, void *mask,
                               uint32_t maskValue, void *counter, void *stream)
{
    if (nseg == 0 || grid == 0) {
        return -1;
    }
    mf::TablePlan plan{static_cast<const uint64_t *>(triples), static_cast<const uint32_t *>(first), nseg, nchunk, units};
    const uint32_t *nd = static_cast<const uint32_t *>(nchunkDev);
    uint64_t *m = static_cast<uint64_t *>(mask);
    uint32_t *c = static_cast<uint32_t *>(counter);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (route) {
        case MFRT_ROUTE_HBM:
            return mf::LaunchTable<MFRT_ROUTE_HBM>(plan, nd, grid, m, maskValue, c, s);
        case MFRT_ROUTE_TO_HOST:
            return mf::LaunchTable<MFRT_ROUTE_TO_HOST>(plan, nd, grid, m, maskValue, c, s);
        case MFRT_ROUTE_FROM_HOST:
            return mf::LaunchTable<MFRT_ROUTE_FROM_HOST>(plan, nd, grid, m, maskValue, c, s);
        default:
            return -1;
    }
}

extern "C" int mfk_xcopy_plan(const void *triples, uint32_t nseg, uint32_t units, void *first, void *nchunk,
                              void *stream)
{
    if (nseg == 0) {
        return -1;
    }
    hipLaunchKernelGGL(mf::XcopyPlanKernel, dim3(1), dim3(mf::kPlanThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint64_t *>(triples), nseg, units, static_cast<uint32_t *>(first),
                       static_cast<uint32_t *>(nchunk));
    return static_cast<int>(hipGetLastError());
}
