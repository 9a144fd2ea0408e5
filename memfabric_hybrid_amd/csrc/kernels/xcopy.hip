// Batched discrete copy ("xcopy") for gfx950: one fused launch moves every
// segment of a batch, whatever mix of lengths it holds.
//
// Replaces the device side of the reference's copy plugin
// (src/hybm/csrc/copy_extend/hybm_copy_kernel.cpp:44-119: 32 blocks, whole
// segments per block, one 64 KiB staging tile, load and store serialised).
// Here a workgroup owns a chunk of bytes, not a segment; data goes
// register-to-register with four 128-bit loads in flight per lane, and
// the descriptor lookup costs one memory round trip (the table comes out of
// the kernel-argument block into registers, two rows per lane) for batches
// of up to 128 segments.
//
// Bound: HBM bandwidth (2 bytes of traffic per payload byte) for device to
// device, the host link (1 byte per payload byte) when one side is pinned
// host memory.  No LDS, no MFMA: nothing here is reused or contracted.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include <atomic>
#include <type_traits>

#include <cstdlib>

#include "xcopy_plan.h"
#include "window_clock.h"
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

// Cache policy of one launch.  Addressing is the same for all of them.
//   HBM to HBM          streaming loads and streaming stores (nothing is reused)
//   to pinned host      plain loads, stores written through at system scope as they are issued
//   from pinned host    streaming loads, plain stores into HBM
enum StoreMode : int { kStorePlain = 0, kStoreStream = 1, kStoreThrough = 2 };

struct Policy {
    bool ntLoad;
    int store;
};

template <bool kNtLoad>
__device__ __forceinline__ u32x4 LoadUnit(uint64_t addr)
{
    GSrcUnit p = reinterpret_cast<GSrcUnit>(addr);
    if (kNtLoad) {
        return __builtin_nontemporal_load(p);
    }
    return *p;
}

// kStoreStream: nontemporal hint, the line may still linger dirty in L2 until the end of the kernel.
// kStoreThrough: nontemporal and written through at system scope, so that the write-back of the
// destination overlaps the copy instead of trailing it.
template <int kStore>
__device__ __forceinline__ void StoreUnit(uint64_t addr, u32x4 v)
{
    GDstUnit p = reinterpret_cast<GDstUnit>(addr);
    if (kStore == kStoreThrough) {
        asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt" : : "v"(p), "v"(v) : "memory");
    } else if (kStore == kStoreStream) {
        __builtin_nontemporal_store(v, p);
    } else {
        *p = v;
    }
}

__device__ __forceinline__ void CopyByte(uint64_t src, uint64_t dst)
{
    *reinterpret_cast<GDstByte>(dst) = *reinterpret_cast<GSrcByte>(src);
}

constexpr uint32_t kDepth = 4;                          // 128-bit loads in flight per lane

// Wait until `ticks` of the constant-rate clock have passed since t0, after the loads have landed (so
// that the wait runs concurrently with the load latency instead of on top of it).
__device__ __forceinline__ void HoldStores(uint64_t t0, uint32_t ticks)
{
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    while (wall_clock64() - t0 < ticks) {
        __builtin_amdgcn_s_sleep(1);
    }
}

// Copy chunk k of one segment.  All arguments are wave-uniform.  kHold: the stores of the first step wait
// for HoldStores(t0, ticks).
template <bool kNtLoad, int kStore, bool kHold = false>
__device__ __forceinline__ void CopyChunk(uint64_t src, uint64_t dst, uint64_t len, uint64_t k, uint32_t units, uint64_t t0 = 0,
                                          uint32_t ticks = 0)
{
    const SegGeom g = SegmentGeometry(dst, len);
    const uint64_t u0 = k * units;
    const uint64_t left = g.body > u0 ? g.body - u0 : 0;
    const uint32_t n = left < units ? static_cast<uint32_t>(left) : units;
    const uint64_t s = src + g.head + u0 * kUnitBytes;
    const uint64_t d = dst + g.head + u0 * kUnitBytes;
    const uint32_t tid = threadIdx.x;
    const uint32_t lanes = blockDim.x;                  // 64, 128 or 256: the launcher's choice
    const uint32_t kTile = kDepth * lanes;              // units one workgroup moves per step

    uint32_t i = 0;
    for (; i + kTile <= n; i += kTile) {
        u32x4 v[kDepth];
#pragma unroll
        for (uint32_t j = 0; j < kDepth; ++j) {
            v[j] = LoadUnit<kNtLoad>(s + static_cast<uint64_t>(i + j * lanes + tid) * kUnitBytes);
        }
        if (kHold && i == 0) {
            HoldStores(t0, ticks);
        }
#pragma unroll
        for (uint32_t j = 0; j < kDepth; ++j) {
            StoreUnit<kStore>(d + static_cast<uint64_t>(i + j * lanes + tid) * kUnitBytes, v[j]);
        }
    }
    if (i < n) {
        u32x4 v[kDepth];
#pragma unroll
        for (uint32_t j = 0; j < kDepth; ++j) {
            const uint32_t u = i + j * lanes + tid;
            if (u < n) {
                v[j] = LoadUnit<kNtLoad>(s + static_cast<uint64_t>(u) * kUnitBytes);
            }
        }
        if (kHold && i == 0) {
            HoldStores(t0, ticks);
        }
#pragma unroll
        for (uint32_t j = 0; j < kDepth; ++j) {
            const uint32_t u = i + j * lanes + tid;
            if (u < n) {
                StoreUnit<kStore>(d + static_cast<uint64_t>(u) * kUnitBytes, v[j]);
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

__device__ __forceinline__ uint64_t ReadLane64(uint64_t v, uint32_t lane)
{
    const uint32_t lo = __builtin_amdgcn_readlane(static_cast<uint32_t>(v), lane);
    const uint32_t hi = __builtin_amdgcn_readlane(static_cast<uint32_t>(v >> 32), lane);
    return (static_cast<uint64_t>(hi) << 32) | lo;
}

// The plan sits in the kernel-argument block.  Every lane fetches "its" two
// table rows (rows lane and lane + 64) with loads that depend on nothing but
// the lane id, so the whole table is in registers after ONE memory round
// trip; the owner of a chunk is then found with two ballots and read out of
// the owning lane.  (A scalar search would chain three dependent loads, each
// a full L2 round trip, before the first byte of payload is requested.)
//
// kHold: every wave keeps its loaded data until `holdTicks` of the constant-rate clock after its own
// start, which separates the read burst of the launch from its write burst (HoldNanosFor has the
// measurements); such a launch has one chunk per workgroup.
template <bool kNtLoad, int kStore, bool kHold = false>
__global__ __launch_bounds__(kXcopyThreads) void XcopyInlineKernel(const InlinePlan p, uint32_t holdTicks)
{
    const uint64_t t0 = kHold ? wall_clock64() : 0;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t f0 = p.first[lane];
    const uint32_t f1 = p.first[lane + 64];
    const uint64_t s0 = p.src[lane];
    const uint64_t s1 = p.src[lane + 64];
    const uint64_t d0 = p.dst[lane];
    const uint64_t d1 = p.dst[lane + 64];
    const uint32_t l0 = p.len[lane];
    const uint32_t l1 = p.len[lane + 64];
    const uint32_t nchunk = p.nchunk;
    const uint32_t units = p.units;
    // The host launches at most nchunk workgroups (and never this kernel for an empty plan), so
    // the first chunk needs no bound check and the table loads above are not held behind one.
    uint32_t c = blockIdx.x;
    do {
        // rows are ordered by prefix: the owner is the last row whose prefix is <= c
        const uint32_t below = __popcll(__ballot(f0 <= c)) + __popcll(__ballot(f1 <= c));
        const uint32_t s = below - 1;
        const uint32_t row = s & 63u;
        uint64_t src;
        uint64_t dst;
        uint32_t len;
        uint32_t first;
        if (s < 64) {
            src = ReadLane64(s0, row);
            dst = ReadLane64(d0, row);
            len = __builtin_amdgcn_readlane(l0, row);
            first = __builtin_amdgcn_readlane(f0, row);
        } else {
            src = ReadLane64(s1, row);
            dst = ReadLane64(d1, row);
            len = __builtin_amdgcn_readlane(l1, row);
            first = __builtin_amdgcn_readlane(f1, row);
        }
        CopyChunk<kNtLoad, kStore, kHold>(src, dst, len, c - first, units, t0, holdTicks);
        c += gridDim.x;
    } while (c < nchunk);
}

// Read and write windows.  A copy that runs for hundreds of microseconds streams faster when the whole chip
// alternates between reading and writing than when every wave stores as soon as its loads have landed:
// HBM then sees long bursts of one direction instead of a mix.  The waves need no communication for
// that, only the constant-rate clock every wave can read: a period is cut into a read half and a write
// half, wave i of a launch of G waves issues the 16 loads per lane of its next 16 KiB chunk at
// offset i * (period / 2) / G into the read half, waits for them, and issues the stores at the same
// offset into the write half.  The period is the time the launch's 2 * G * 16 KiB per round need at a
// target rate; up to a target the part sustains, the copy simply runs at the pace the clock sets.
// Measured with a stand-alone kernel of this shape on 1 and 2 GiB (4096 waves: 64 MiB read and 64 MiB
// written per 18 to 20 us period): target 6.6 / 6.8 / 7.0 / 7.2 / 7.4 TB/s -> 6.39 / 6.59 / 6.7 / 6.97 / 7.15 TB/s
// achieved, against 6.1-6.2 TB/s for one wave per 4 KiB chunk that stores at once; at 7.6 TB/s the waves no
// longer keep up, the windows dissolve and the copy falls back to 5.8-6.1 TB/s.  This kernel, which also
// looks its chunk up in the plan, through smem_bm_copy_batch on a pool, target 6.8 against no windows:
// 512 MiB 6.65 / 6.34 TB/s, 1 GiB 6.73 / 6.23, 2 GiB 6.6-6.7 / 6.12, 100 segments of about 10 MB at odd addresses
// 6.28 / 5.84, 3 x 700 MB at odd addresses 6.05 / 5.73; at 6.6 it measures 6.47 / 6.54 / 6.57 / 6.09 / 6.1-6.2, at
// 7.0 the 2 GiB copy dissolves now and then (6.2-6.3), at 7.2 and above most launches do.  256 MiB gains nothing
// (the first and the last half period, in which the chip only reads or only writes, cost what the windows
// gain), 128 MiB loses.  Memory that has never been written copies erratically under windows (6.0 to 6.8 TB/s
// from one launch to the next); initialised memory does not.  2048 waves dissolve one step earlier than 4096;
// 4, 8 or 32 loads per lane and windows that are not spread over their half were slower or less stable.  A wave
// that is late proceeds at once: letting it skip to its slot in a later period made a dissolved launch slower
// (4.4 instead of 5.7 TB/s).
constexpr uint32_t kWindowDepth = 16;                       // 128-bit loads per lane and round
constexpr uint32_t kWindowUnits = 64 * kWindowDepth;        // 16 KiB chunks, one wave each
constexpr uint32_t kWindowWaves = 4096;                     // 16 per CU

// Copy chunk k (kWindowUnits units) of one segment: loads at `slot`, stores at `slot + half`.  A chunk that is
// not whole (the last one of a segment, or one with head or tail bytes) goes through CopyChunk in the
// write half: there are at most two such chunks per segment.
template <bool kNtLoad, int kStore>
__device__ __forceinline__ void CopyChunkWindowed(uint64_t src, uint64_t dst, uint64_t len, uint64_t k, uint64_t slot, uint32_t half)
{
    const SegGeom g = SegmentGeometry(dst, len);
    const uint64_t u0 = k * kWindowUnits;
    const bool whole = u0 + kWindowUnits <= g.body && (k != 0 || g.head == 0) && (u0 + kWindowUnits < g.body || g.tail == 0);
    WaitForClock(slot);
    if (!whole) {
        WaitForClock(slot + half);
        CopyChunk<kNtLoad, kStore>(src, dst, len, k, kWindowUnits);
        return;
    }
    const uint64_t s = src + g.head + u0 * kUnitBytes + threadIdx.x * kUnitBytes;
    const uint64_t d = dst + g.head + u0 * kUnitBytes + threadIdx.x * kUnitBytes;
    u32x4 v[kWindowDepth];
#pragma unroll
    for (uint32_t j = 0; j < kWindowDepth; ++j) {
        v[j] = LoadUnit<kNtLoad>(s + j * 64 * kUnitBytes);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    WaitForClock(slot + half);
#pragma unroll
    for (uint32_t j = 0; j < kWindowDepth; ++j) {
        StoreUnit<kStore>(d + j * 64 * kUnitBytes, v[j]);
    }
}

// The inline plan (chunks of kWindowUnits units) copied by gridDim.x single-wave workgroups that walk
// the chunks with stride gridDim.x, one chunk per period each.
template <bool kNtLoad, int kStore>
__global__ __launch_bounds__(64) void XcopyWindowKernel(const InlinePlan p, uint32_t period, uint32_t seq)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t f0 = p.first[lane];
    const uint32_t f1 = p.first[lane + 64];
    const uint64_t s0 = p.src[lane];
    const uint64_t s1 = p.src[lane + 64];
    const uint64_t d0 = p.dst[lane];
    const uint64_t d1 = p.dst[lane + 64];
    const uint32_t l0 = p.len[lane];
    const uint32_t l1 = p.len[lane + 64];
    const uint32_t nchunk = p.nchunk;
    const uint32_t half = period / 2;
    uint64_t slot = AgreedStart(seq) + static_cast<uint64_t>(blockIdx.x) * half / gridDim.x;
    for (uint32_t c = blockIdx.x; c < nchunk; c += gridDim.x) {
        const uint32_t below = __popcll(__ballot(f0 <= c)) + __popcll(__ballot(f1 <= c));
        const uint32_t s = below - 1;
        const uint32_t row = s & 63u;
        uint64_t src;
        uint64_t dst;
        uint32_t len;
        uint32_t first;
        if (s < 64) {
            src = ReadLane64(s0, row);
            dst = ReadLane64(d0, row);
            len = __builtin_amdgcn_readlane(l0, row);
            first = __builtin_amdgcn_readlane(f0, row);
        } else {
            src = ReadLane64(s1, row);
            dst = ReadLane64(d1, row);
            len = __builtin_amdgcn_readlane(l1, row);
            first = __builtin_amdgcn_readlane(f1, row);
        }
        CopyChunkWindowed<kNtLoad, kStore>(src, dst, len, c - first, slot, half);
        slot += period;
    }
}

// A single segment needs no table: its three words travel as plain kernel arguments (28 bytes
// instead of the 3080-byte plan), which is cheaper for the host to hand over and spares every
// wave the table fetch.  Measured against the table form on one box: an 8 MiB copy 13.7 us instead
// of 15.4 us per blocking call, back-to-back 32 MiB copies 10.8 us instead of 11.5 us each; from
// about 200 MiB on the table form is 1 % faster (512 MiB: 166.4 us against 168.8 us), hence the limit.
constexpr uint32_t kSingleMaxChunks = 49152;
template <bool kNtLoad, int kStore, bool kHold = false>
__global__ __launch_bounds__(kXcopyThreads) void XcopySingleKernel(uint64_t src, uint64_t dst, uint32_t len, uint32_t nchunk,
                                                                   uint32_t units, uint32_t holdTicks)
{
    const uint64_t t0 = kHold ? wall_clock64() : 0;
    uint32_t c = blockIdx.x;
    do {
        CopyChunk<kNtLoad, kStore, kHold>(src, dst, len, c, units, t0, holdTicks);
        c += gridDim.x;
    } while (c < nchunk);
}

// Completion word (of the plugin ABI for tables and words in device memory, and of blocking calls,
// whose host thread polls it).  It is written by a launch of its own right behind the copy
// launch on the same stream: the copy kernel's end-of-kernel release makes every store visible once
// for the whole grid.  (Signalling from inside the copy kernel needs a system-scope release in
// every workgroup before it may count itself done, an L2 write-back each: 77 us instead of 5.5 us
// for an 9 MB batch.)  An empty batch gets the word alone.
__global__ void XcopySignalKernel(uint64_t *mask, uint32_t maskValue)
{
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        __hip_atomic_store(mask, static_cast<uint64_t>(maskValue), __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
}

template <bool kNtLoad, int kStore>
__global__ __launch_bounds__(kXcopyThreads) void XcopyTableKernel(const uint64_t *__restrict__ triples,
                                                                  const uint32_t *__restrict__ first,
                                                                  const uint32_t *__restrict__ nchunkDev, uint32_t nseg,
                                                                  uint32_t nchunkHost, uint32_t units, const ChunkPattern pattern)
{
    const uint32_t nchunk = nchunkDev != nullptr ? *nchunkDev : nchunkHost;
    const uint32_t lane = threadIdx.x & 63u;
    for (uint32_t c = blockIdx.x; c < nchunk; c += gridDim.x) {
        if (pattern.period != 0) {
            // Chunk counts that repeat (pages of one size, K and V blocks in turn): the owner follows
            // from a division and a few comparisons on kernel arguments, and the only memory round
            // trip before the copy is the fetch of its descriptor.
            uint32_t seg;
            uint32_t k;
            PatternOwner(pattern, c, seg, k);
            const uint64_t *t = triples + 3ull * seg;
            CopyChunk<kNtLoad, kStore>(t[0], t[1], t[2], k, units);
            continue;
        }
        // 64-ary search for the last prefix entry <= c: every level is one load per lane and a
        // ballot, so 4096 segments resolve in two memory round trips (a binary search by one
        // lane would chain twelve).  Invariant: first[lo] <= c < first[hi].
        uint32_t lo = 0;
        uint32_t hi = nseg;
        while (hi - lo > 1) {
            const uint32_t span = hi - lo;
            const uint32_t step = (span + 63u) >> 6;            // entries per lane at this level
            const uint32_t probe = lo + (lane + 1) * step;      // lanes probe lo+step, lo+2*step, ...
            const bool inside = probe < hi;
            const uint32_t v = inside ? first[probe] : 0xFFFFFFFFu;
            const uint32_t hits = __popcll(__ballot(inside && v <= c));
            lo += hits * step;
            const uint32_t cap = lo + step;
            hi = cap < hi ? cap : hi;
        }
        const uint64_t *t = triples + 3ull * lo;
        CopyChunk<kNtLoad, kStore>(t[0], t[1], t[2], c - first[lo], units);
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

Policy PolicyOf(int route)
{
    switch (route) {
        case MFRT_ROUTE_TO_HOST:
            // measured over the host link with 122-segment batches: write-through 56.0 GB/s,
            // plain 54.4 GB/s, nontemporal-only 49 GB/s
            return Policy{false, kStoreThrough};
        case MFRT_ROUTE_FROM_HOST:
            return Policy{true, kStorePlain};
        default:
            // HBM to HBM, measured on the 9 MB batch: streaming loads and stores 5.2 us, plain 6.3 us,
            // stores written through 6.5 us (they are 4 % faster on a 1 GiB copy only)
            return Policy{true, kStoreStream};
    }
}

// Runs `launch` with the template instance matching a run-time policy.
template <class Launch>
int WithPolicy(const Policy &policy, Launch launch)
{
    if (policy.ntLoad) {
        switch (policy.store) {
            case kStoreThrough:
                return launch(std::true_type{}, std::integral_constant<int, kStoreThrough>{});
            case kStoreStream:
                return launch(std::true_type{}, std::integral_constant<int, kStoreStream>{});
            default:
                return launch(std::true_type{}, std::integral_constant<int, kStorePlain>{});
        }
    }
    switch (policy.store) {
        case kStoreThrough:
            return launch(std::false_type{}, std::integral_constant<int, kStoreThrough>{});
        case kStoreStream:
            return launch(std::false_type{}, std::integral_constant<int, kStoreStream>{});
        default:
            return launch(std::false_type{}, std::integral_constant<int, kStorePlain>{});
    }
}

// Lanes per workgroup: a workgroup moves its chunk in one step of kDepth accesses per lane, so the
// chunk size picks the workgroup size (4 KiB: one wave, 8 KiB: two, 16 KiB and more: four).
// Measured on a 9 MB batch and on 1 MiB ... 1 GiB copies: single-wave workgroups on 4 KiB chunks are
// the fastest shape at every size (KV batch 4.8 us against 5.5 us with four waves on 16 KiB).
uint32_t LanesFor(uint32_t units, int route)
{
    if (route == MFRT_ROUTE_TO_HOST || route == MFRT_ROUTE_FROM_HOST) {
        return kXcopyThreads;   // link routes were tuned with four-wave workgroups, one per CU
    }
    const uint32_t lanes = units / kDepth;
    return lanes <= 64 ? 64u : (lanes <= 128 ? 128u : kXcopyThreads);
}

// Ticks of the device's constant-rate clock (the one wall_clock64() reads) in `nanos`.
uint32_t HoldTicks(uint32_t nanos)
{
    static std::atomic<int> khzOf[64];
    int dev = 0;
    if (nanos == 0 || hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        return 0;
    }
    int khz = khzOf[dev].load(std::memory_order_relaxed);
    if (khz == 0) {
        if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess || khz <= 0) {
            khz = -1;   // unknown clock: no hold on this device
        }
        khzOf[dev].store(khz, std::memory_order_relaxed);
    }
    if (khz < 0) {
        return 0;
    }
    const uint64_t capped = nanos < 10000 ? nanos : 10000;   // no wave ever waits longer than 10 us
    return static_cast<uint32_t>(capped * static_cast<uint64_t>(khz) / 1000000u);
}

// anyOrder: the launch carries no barrier, so the command processor may start it while launches queued
// before it on the same stream still run (hipExtAnyOrderLaunch).  Measured on the 9 MB batch, one stream:
// 5.3 us per launch against 5.9 us with the barrier.
// holdNanos: the caller's HoldNanosFor(); the launch qualifies only if it still has one chunk per workgroup.
template <bool kNtLoad, int kStore>
int LaunchInline(const InlinePlan &plan, uint32_t grid, uint32_t lanes, hipStream_t stream, bool anyOrder, uint32_t holdNanos)
{
    const uint32_t flags = anyOrder ? hipExtAnyOrderLaunch : 0u;
    const uint32_t ticks = grid == plan.nchunk && lanes == 64 ? HoldTicks(holdNanos) : 0;
    if (plan.first[1] == kNoChunk && plan.nchunk <= kSingleMaxChunks) {
        if (anyOrder) {
            hipExtLaunchKernelGGL((XcopySingleKernel<kNtLoad, kStore>), dim3(grid), dim3(lanes), 0, stream, nullptr, nullptr, flags,
                                  plan.src[0], plan.dst[0], plan.len[0], plan.nchunk, plan.units, 0u);
        } else if (ticks != 0) {
            hipLaunchKernelGGL((XcopySingleKernel<kNtLoad, kStore, true>), dim3(grid), dim3(lanes), 0, stream, plan.src[0],
                               plan.dst[0], plan.len[0], plan.nchunk, plan.units, ticks);
        } else {
            hipLaunchKernelGGL((XcopySingleKernel<kNtLoad, kStore>), dim3(grid), dim3(lanes), 0, stream, plan.src[0], plan.dst[0],
                               plan.len[0], plan.nchunk, plan.units, 0u);
        }
        return static_cast<int>(hipGetLastError());
    }
    // The ordered launches go through hipLaunchKernel with an argument array: the triple-chevron form pushes and pops a
    // launch configuration around the same call, 0.15 us of host time per launch with this 3 KiB argument block.
    uint32_t holdTicks = ticks;
    void *args[] = {const_cast<InlinePlan *>(&plan), &holdTicks};
    if (ticks != 0) {
        if (anyOrder) {
            hipExtLaunchKernelGGL((XcopyInlineKernel<kNtLoad, kStore, true>), dim3(grid), dim3(lanes), 0, stream, nullptr, nullptr,
                                  flags, plan, ticks);
        } else {
            return static_cast<int>(hipLaunchKernel(reinterpret_cast<const void *>(&XcopyInlineKernel<kNtLoad, kStore, true>), dim3(grid),
                                                    dim3(lanes), args, 0, stream));
        }
    } else if (anyOrder) {
        hipExtLaunchKernelGGL((XcopyInlineKernel<kNtLoad, kStore>), dim3(grid), dim3(lanes), 0, stream, nullptr, nullptr, flags, plan,
                              0u);
    } else {
        return static_cast<int>(hipLaunchKernel(reinterpret_cast<const void *>(&XcopyInlineKernel<kNtLoad, kStore, false>), dim3(grid),
                                                dim3(lanes), args, 0, stream));
    }
    return static_cast<int>(hipGetLastError());
}

// windowMBps: the rate (MB/s of HBM traffic, read + written) the period of a windowed launch is cut for.
template <bool kNtLoad, int kStore>
int LaunchWindowed(const InlinePlan &plan, uint32_t grid, uint32_t windowMBps, hipStream_t stream)
{
    const uint32_t ticks = WindowPeriodTicks(2ull * grid * kWindowUnits * kUnitBytes, windowMBps);
    if (ticks == 0) {
        return static_cast<int>(hipErrorInvalidValue);
    }
    hipLaunchKernelGGL((XcopyWindowKernel<kNtLoad, kStore>), dim3(grid), dim3(64), 0, stream, plan, ticks, NextWindowSeq());
    return static_cast<int>(hipGetLastError());
}

template <bool kNtLoad, int kStore>
int LaunchTable(const TablePlan &plan, const uint32_t *nchunkDev, uint32_t grid, uint32_t lanes, hipStream_t stream)
{
    hipLaunchKernelGGL((XcopyTableKernel<kNtLoad, kStore>), dim3(grid), dim3(lanes), 0, stream, plan.triples,
                       plan.first, nchunkDev, plan.nseg, plan.nchunk, plan.units, plan.pattern);
    return static_cast<int>(hipGetLastError());
}

int Signal(void *mask, uint32_t maskValue, hipStream_t stream)
{
    if (mask == nullptr) {
        return 0;
    }
    hipLaunchKernelGGL(XcopySignalKernel, dim3(1), dim3(64), 0, stream, static_cast<uint64_t *>(mask), maskValue);
    return static_cast<int>(hipGetLastError());
}

}  // namespace
}  // namespace mf

extern "C" int mfk_xcopy_inline(const void *inlinePlan, int route, uint32_t grid, void *mask, uint32_t maskValue,
                                void *stream, int anyOrder, uint32_t holdNanos)
{
    const mf::InlinePlan &plan = *static_cast<const mf::InlinePlan *>(inlinePlan);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (plan.nchunk == 0) {
        return mf::Signal(mask, maskValue, s);
    }
    if (grid == 0 || grid > plan.nchunk) {
        grid = plan.nchunk;
    }
    if (grid > (1u << 24) - 1) {
        grid = (1u << 24) - 1;   // the grid size in lanes must stay below 2^32; workgroups loop over the rest
    }
    const int err = mf::WithPolicy(mf::PolicyOf(route), [&](auto ntLoad, auto store) {
        return mf::LaunchInline<decltype(ntLoad)::value, decltype(store)::value>(plan, grid, mf::LanesFor(plan.units, route), s,
                                                                                 anyOrder != 0, holdNanos);
    });
    return err != 0 ? err : mf::Signal(mask, maskValue, s);
}

extern "C" uint32_t mfk_xcopy_window_units(void)
{
    return mf::kWindowUnits;
}

extern "C" uint32_t mfk_xcopy_window_waves(void)
{
    return mf::kWindowWaves;
}

extern "C" int mfk_xcopy_windowed(const void *inlinePlan, uint32_t windowMBps, void *mask, uint32_t maskValue, void *stream)
{
    const mf::InlinePlan &plan = *static_cast<const mf::InlinePlan *>(inlinePlan);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (plan.units != mf::kWindowUnits || plan.nchunk == 0 || windowMBps == 0) {
        return -1;
    }
    const uint32_t grid = plan.nchunk < mf::kWindowWaves ? plan.nchunk : mf::kWindowWaves;
    const int err = mf::WithPolicy(mf::PolicyOf(MFRT_ROUTE_HBM), [&](auto ntLoad, auto store) {
        return mf::LaunchWindowed<decltype(ntLoad)::value, decltype(store)::value>(plan, grid, windowMBps, s);
    });
    return err != 0 ? err : mf::Signal(mask, maskValue, s);
}

extern "C" int mfk_xcopy_signal(void *word, uint32_t value, void *stream)
{
    return mf::Signal(word, value, static_cast<hipStream_t>(stream));
}

extern "C" int mfk_xcopy_table(const void *triples, const void *first, const void *nchunkDev, uint32_t nseg,
                               uint32_t nchunk, uint32_t units, const void *pattern, int route, uint32_t grid, void *mask,
                               uint32_t maskValue, void *stream)
{
    mf::ChunkPattern pat{};
    if (pattern != nullptr) {
        pat = *static_cast<const mf::ChunkPattern *>(pattern);
    }
    if (nseg == 0 || grid == 0 || (pat.period == 0 && first == nullptr)) {
        return -1;
    }
    if (pat.period != 0 && (pat.period > mf::kMaxPeriod || pat.chunksPerPeriod == 0 || nchunkDev != nullptr ||
                            pat.start[0] != 0 || pat.start[pat.period] != pat.chunksPerPeriod ||
                            mf::PatternChunks(pat, nseg) != nchunk)) {
        return -1;
    }
    mf::TablePlan plan{static_cast<const uint64_t *>(triples), static_cast<const uint32_t *>(first), nseg, nchunk, units, pat};
    const uint32_t *nd = static_cast<const uint32_t *>(nchunkDev);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int err = mf::WithPolicy(mf::PolicyOf(route), [&](auto ntLoad, auto store) {
        return mf::LaunchTable<decltype(ntLoad)::value, decltype(store)::value>(plan, nd, grid, mf::LanesFor(units, route), s);
    });
    return err != 0 ? err : mf::Signal(mask, maskValue, s);
}

#ifndef MF_RT_HIDDEN   // the plugin library has no entry point that needs it
// Scratch of the entry point that allocates nothing (mfk_xcopy_table_static): the chunk prefix
// first[0 .. nseg] and, behind it, the chunk count, both written by XcopyPlanKernel and read by
// XcopyTableKernel of the same call.  One copy per GPU, held until the process ends.  In host code
// the array's name is only a handle for hipGetSymbolAddress: kernels and copies get the address that
// call returned for the current device, never the name.
static __device__ __align__(256) uint32_t scratch[MFK_STATIC_TABLE_SEGMENTS + 64];

namespace {
constexpr int kMaxDevices = 64;
uint32_t *g_scratchOf[kMaxDevices] = {};   // device ordinal -> address of that device's copy of `scratch`
}  // namespace

extern "C" int mfk_xcopy_static_setup(void)
{
    int dev = -1;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess) {
        return static_cast<int>(err);
    }
    if (dev < 0 || dev >= kMaxDevices) {
        return static_cast<int>(hipErrorInvalidDevice);
    }
    void *ptr = nullptr;
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess) {
        return static_cast<int>(err);
    }
    g_scratchOf[dev] = static_cast<uint32_t *>(ptr);
    return 0;
}

extern "C" int mfk_xcopy_table_static(const void *triples, uint32_t nseg, uint32_t units, int route, uint32_t grid,
                                      void *stream)
{
    if (nseg == 0 || nseg > MFK_STATIC_TABLE_SEGMENTS || grid == 0) {
        return -1;
    }
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices || g_scratchOf[dev] == nullptr) {
        return -2;   // mfk_xcopy_static_setup has not run on this device
    }
    uint32_t *first = g_scratchOf[dev];
    uint32_t *nchunkDev = first + nseg + 1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // the plan kernel writes every word the table kernel reads: nothing has to start at zero
    hipLaunchKernelGGL(mf::XcopyPlanKernel, dim3(1), dim3(mf::kPlanThreads), 0, s, static_cast<const uint64_t *>(triples), nseg,
                       units, first, nchunkDev);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        return static_cast<int>(err);
    }
    mf::TablePlan plan{static_cast<const uint64_t *>(triples), first, nseg, 0, units, mf::ChunkPattern{}};
    return mf::WithPolicy(mf::PolicyOf(route), [&](auto ntLoad, auto store) {
        return mf::LaunchTable<decltype(ntLoad)::value, decltype(store)::value>(plan, nchunkDev, grid, mf::LanesFor(units, route), s);
    });
}
#endif  // MF_RT_HIDDEN

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
