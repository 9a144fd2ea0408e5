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
#include <mutex>
#include <type_traits>
#include <vector>

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
// rule); such a launch has one chunk per workgroup: of 4 KiB (kHoldShallow, four loads per lane) or, for
// batches whose 4 KiB chunks would outnumber the waves the chip holds at once, of 16 KiB (kHoldDeep).
enum HoldMode : int { kHoldNone = 0, kHoldShallow = 1, kHoldDeep = 2 };

template <bool kNtLoad, int kStore, int kHold>
__device__ __forceinline__ void CopyChunkHeld(uint64_t src, uint64_t dst, uint64_t len, uint64_t k, uint32_t units, uint64_t t0,
                                              uint32_t ticks);

template <bool kNtLoad, int kStore, int kHold = kHoldNone>
__global__ __launch_bounds__(kXcopyThreads) void XcopyInlineKernel(const InlinePlan p, uint32_t holdTicks)
{
    const uint64_t t0 = kHold != kHoldNone ? wall_clock64() : 0;
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
        CopyChunkHeld<kNtLoad, kStore, kHold>(src, dst, len, c - first, units, t0, holdTicks);
        c += gridDim.x;
    } while (c < nchunk);
}

// Read and write windows.  A copy that runs for hundreds of microseconds streams faster when the whole chip
// alternates between reading and writing than when every wave stores as soon as its loads have landed:
// HBM then sees long bursts of one direction instead of a mix (6.7 against 6.2 TB/s on 1 to 2 GiB).  The
// waves need no communication for that beyond the start, only the constant-rate clock every wave can read:
// a period is cut into a read half and a write half, wave i of a launch of G waves issues the 16 loads per
// lane of its next 16 KiB chunk at offset i * (period / 2) / G into the read half, waits for them, and
// issues the stores at the same offset into the write half.  The period is the time the launch's
// 2 * G * 16 KiB per round need at a target rate; up to a rate the part sustains, the copy runs at the pace
// the clock sets, beyond it the windows dissolve and the copy runs as it does without them.  A wave that
// is late proceeds at once (skipping to a later period made a dissolved launch slower).
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

// One chunk under a hold mode.  kHoldDeep: a chunk of up to kWindowUnits units is read by a single wave with up to
// 16 loads per lane in flight and stored when the wave's hold is over; units past the end of the segment's
// body are skipped lane by lane, head and tail bytes travel as in CopyChunk.
template <bool kNtLoad, int kStore, int kHold>
__device__ __forceinline__ void CopyChunkHeld(uint64_t src, uint64_t dst, uint64_t len, uint64_t k, uint32_t units, uint64_t t0,
                                              uint32_t ticks)
{
    if (kHold != kHoldDeep) {
        CopyChunk<kNtLoad, kStore, kHold == kHoldShallow>(src, dst, len, k, units, t0, ticks);
        return;
    }
    const SegGeom g = SegmentGeometry(dst, len);
    const uint64_t u0 = k * kWindowUnits;
    const uint64_t left = g.body > u0 ? g.body - u0 : 0;
    const uint32_t n = left < kWindowUnits ? static_cast<uint32_t>(left) : kWindowUnits;
    const uint32_t tid = threadIdx.x;                       // 64 lanes
    const uint64_t s = src + g.head + u0 * kUnitBytes + tid * kUnitBytes;
    const uint64_t d = dst + g.head + u0 * kUnitBytes + tid * kUnitBytes;
    u32x4 v[kWindowDepth];
    if (n == kWindowUnits) {    // the common case without a test per load: the sixteen loads leave back to back
#pragma unroll
        for (uint32_t j = 0; j < kWindowDepth; ++j) {
            v[j] = LoadUnit<kNtLoad>(s + j * 64 * kUnitBytes);
        }
        HoldStores(t0, ticks);
#pragma unroll
        for (uint32_t j = 0; j < kWindowDepth; ++j) {
            StoreUnit<kStore>(d + j * 64 * kUnitBytes, v[j]);
        }
    } else {
#pragma unroll
        for (uint32_t j = 0; j < kWindowDepth; ++j) {
            if (j * 64 + tid < n) {
                v[j] = LoadUnit<kNtLoad>(s + j * 64 * kUnitBytes);
            }
        }
        HoldStores(t0, ticks);
#pragma unroll
        for (uint32_t j = 0; j < kWindowDepth; ++j) {
            if (j * 64 + tid < n) {
                StoreUnit<kStore>(d + j * 64 * kUnitBytes, v[j]);
            }
        }
    }
    if (k == 0 && tid < g.head) {
        CopyByte(src + tid, dst + tid);
    }
    if (u0 + kWindowUnits >= g.body && tid < g.tail) {
        const uint64_t off = g.head + g.body * kUnitBytes + tid;
        CopyByte(src + off, dst + off);
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

// A single segment needs no table: its three words travel as plain kernel arguments (28 bytes instead of
// the 3080-byte plan), which is cheaper for the host to hand over and spares every wave the table fetch
// (an 8 MiB copy: 13.7 instead of 15.4 us per blocking call).  From about 200 MiB on the table form is
// 1 % faster, hence the limit.
constexpr uint32_t kSingleMaxChunks = 49152;
template <bool kNtLoad, int kStore, int kHold = kHoldNone>
__global__ __launch_bounds__(kXcopyThreads) void XcopySingleKernel(uint64_t src, uint64_t dst, uint32_t len, uint32_t nchunk,
                                                                   uint32_t units, uint32_t holdTicks)
{
    const uint64_t t0 = kHold != kHoldNone ? wall_clock64() : 0;
    uint32_t c = blockIdx.x;
    do {
        CopyChunkHeld<kNtLoad, kStore, kHold>(src, dst, len, c, units, t0, holdTicks);
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

// The table form: any number of segments, {src, dst, len} triples in memory.  A wave finds the owner of its
// chunk either by a division (chunk counts that repeat: pages of one size, K and V blocks in turn) or
// through the group map: two map entries bound the owner to a short range of segments, whose prefix
// entries AND triples the lanes then fetch side by side, one segment per lane, so that the descriptor is
// in registers two dependent loads after the wave started, whatever the size of the table.  (The form
// this replaces searched the whole prefix 64 ways per round: three rounds for 262 144 segments, then the
// prefix entry, then the triple.)  A wave that walks several chunks fetches what the next lookup starts
// from before it copies the current chunk.
struct ChunkRef {
    uint64_t src;
    uint64_t dst;
    uint64_t len;
    uint32_t k;
};

// Owner of chunk c, known to lie in segments [lo, hiEx): first[lo] <= c < first[hiEx].
__device__ __forceinline__ ChunkRef OwnerOf(const uint64_t *__restrict__ triples, const uint32_t *__restrict__ first, uint32_t lo,
                                            uint32_t hiEx, uint32_t c, uint32_t lane)
{
    // more than 64 candidates (a run of empty segments, or a map with coarse groups): narrow 64 ways per round
    while (hiEx - lo > 64) {
        const uint32_t span = hiEx - lo;
        const uint32_t step = (span + 63u) >> 6;
        const uint32_t probe = lo + (lane + 1) * step;
        const bool inside = probe < hiEx;
        const uint32_t v = inside ? first[probe] : 0xFFFFFFFFu;
        const uint32_t hits = __popcll(__ballot(inside && v <= c));
        lo += hits * step;
        const uint32_t cap = lo + step;
        hiEx = cap < hiEx ? cap : hiEx;
    }
    const uint32_t probe = lo + lane;
    const bool inside = probe < hiEx;
    uint32_t f = 0xFFFFFFFFu;
    uint64_t ts = 0;
    uint64_t td = 0;
    uint64_t tl = 0;
    if (inside) {
        f = first[probe];
        const uint64_t *t = triples + 3ull * probe;
        ts = t[0];
        td = t[1];
        tl = t[2];
    }
    const uint32_t row = __popcll(__ballot(inside && f <= c)) - 1;   // first[lo] <= c: at least one hit
    ChunkRef r;
    r.src = ReadLane64(ts, row);
    r.dst = ReadLane64(td, row);
    r.len = ReadLane64(tl, row);
    r.k = c - __builtin_amdgcn_readlane(f, row);
    return r;
}

// A value every lane holds alike, moved to a scalar register: what a wave loads from a uniform address after its
// first store lands in vector registers, and addresses and lengths computed from it would be computed per lane.
__device__ __forceinline__ uint32_t Uniform(uint32_t v)
{
    return __builtin_amdgcn_readfirstlane(v);
}

__device__ __forceinline__ uint64_t Uniform(uint64_t v)
{
    return (static_cast<uint64_t>(Uniform(static_cast<uint32_t>(v >> 32))) << 32) | Uniform(static_cast<uint32_t>(v));
}

// kHeader: chunk count, group shift and pattern come from the header the device-side planner left in
// device memory (the host knows none of them) instead of the kernel arguments.
// kHold: as for the inline kernel, for launches of one chunk per workgroup (the host knows the chunk count).
template <bool kNtLoad, int kStore, bool kHeader, int kHold = kHoldNone>
__global__ __launch_bounds__(kXcopyThreads) void XcopyTableKernel(const TablePlan plan, uint32_t holdTicks)
{
    const uint64_t t0 = kHold != kHoldNone ? wall_clock64() : 0;
    uint32_t nchunk = plan.nchunk;
    uint32_t shift = plan.groupShift;
    ChunkPattern pattern = plan.pattern;
    if (kHeader) {
        const TableHeader *__restrict__ header = plan.header;
        nchunk = Uniform(header->nchunk);
        shift = Uniform(header->groupShift);
        pattern.period = Uniform(header->pattern.period);
        pattern.chunksPerPeriod = Uniform(header->pattern.chunksPerPeriod);
#pragma unroll
        for (uint32_t i = 0; i <= kMaxPeriod; ++i) {
            pattern.start[i] = Uniform(header->pattern.start[i]);
        }
    }
    uint32_t c = blockIdx.x;
    if (c >= nchunk) {
        return;
    }
    const uint32_t units = plan.units;
    if (pattern.period != 0) {
        uint32_t seg;
        uint32_t k;
        PatternOwner(pattern, c, seg, k);
        const uint64_t *t = plan.triples + 3ull * seg;
        uint64_t src = t[0];
        uint64_t dst = t[1];
        uint64_t len = t[2];
        for (;;) {
            const uint32_t next = c + gridDim.x;
            const bool more = next < nchunk;
            uint64_t nsrc = 0;
            uint64_t ndst = 0;
            uint64_t nlen = 0;
            uint32_t nk = 0;
            if (more) {   // requested now, needed after the copy
                PatternOwner(pattern, next, seg, nk);
                t = plan.triples + 3ull * seg;
                nsrc = t[0];
                ndst = t[1];
                nlen = t[2];
            }
            CopyChunkHeld<kNtLoad, kStore, kHold>(src, dst, len, k, units, t0, holdTicks);
            if (!more) {
                return;
            }
            src = Uniform(nsrc);
            dst = Uniform(ndst);
            len = Uniform(nlen);
            k = nk;
            c = next;
        }
    }
    const uint32_t lane = threadIdx.x & 63u;
    // A workgroup that walks several chunks of a table it looks up through the map (the host did not know the chunk
    // count when it sized the grid) takes a run of consecutive chunks: their owners lie in the same few segments,
    // whose prefix entries and triples the lookup then finds in cache (16 384 ragged segments, four chunks per
    // workgroup: 907 against 963 us with the grid as the stride).  Under a pattern, where the lookup is a division,
    // the stride stays: all workgroups then write one contiguous span per round.
    uint32_t step = gridDim.x;
    uint32_t stop = nchunk;
    if (kHeader) {
        const uint32_t per = (nchunk + gridDim.x - 1) / gridDim.x;
        c = blockIdx.x * per;
        step = 1;
        stop = c + per < nchunk ? c + per : nchunk;
        if (c >= stop) {
            return;
        }
    }
    // even lanes fetch the map entry of the chunk's group, odd lanes the one behind it
    uint32_t bounds = plan.group[(c >> shift) + (lane & 1u)];
    for (;;) {
        const uint32_t lo = __builtin_amdgcn_readlane(bounds, 0);
        const uint32_t hiEx = __builtin_amdgcn_readlane(bounds, 1) + 1;
        const ChunkRef r = OwnerOf(plan.triples, plan.first, lo, hiEx, c, lane);
        const uint32_t next = c + step;
        const bool more = next < stop;
        if (more) {
            bounds = plan.group[(next >> shift) + (lane & 1u)];
        }
        CopyChunkHeld<kNtLoad, kStore, kHold>(r.src, r.dst, r.len, r.k, units, t0, holdTicks);
        if (!more) {
            return;
        }
        c = next;
    }
}

// Device-side planner for a table the host cannot read: chunk prefix, group map and, where the chunk
// counts repeat with a short period, the pattern that lets the table kernel do without both.
__device__ __forceinline__ uint32_t ChunksOf(const uint64_t *__restrict__ triples, uint32_t i, uint32_t units)
{
    return static_cast<uint32_t>(SegmentChunks(triples[3ull * i + 1], triples[3ull * i + 2], units));
}

__device__ __forceinline__ uint32_t WaveInclusiveSum(uint32_t v, uint32_t lane)
{
#pragma unroll
    for (uint32_t d = 1; d < 64; d <<= 1) {
        const uint32_t o = __shfl_up(v, d, 64);
        v += lane >= d ? o : 0u;
    }
    return v;
}

__device__ __forceinline__ uint32_t WaveSum(uint32_t v)
{
#pragma unroll
    for (uint32_t d = 32; d != 0; d >>= 1) {
        v += __shfl_xor(v, d, 64);
    }
    return v;
}

__device__ __forceinline__ uint32_t WaveAnd(uint32_t v)
{
#pragma unroll
    for (uint32_t d = 32; d != 0; d >>= 1) {
        v &= __shfl_xor(v, d, 64);
    }
    return v;
}

constexpr uint32_t kPlanWaves = kPlanThreads / 64;
constexpr uint32_t kAllPeriods = ((1u << kMaxPeriod) - 1) << 1;     // bit p: the counts repeat with period p

// First of two launches for tables beyond kPlanSingleBlockSegs segments: every workgroup sums the chunk
// counts of its kPlanThreads segments and notes which periods they contradict.
__global__ __launch_bounds__(kPlanThreads) void XcopyPlanSumsKernel(const uint64_t *__restrict__ triples, uint32_t nseg, uint32_t units,
                                                                    uint32_t *__restrict__ scratch, uint32_t groupCapacity)
{
    __shared__ uint32_t counts[kMaxPeriod + kPlanThreads];
    __shared__ uint32_t waveSum[kPlanWaves];
    __shared__ uint32_t waveAlive[kPlanWaves];
    const ScratchLayout at = ScratchLayoutFor(nseg, groupCapacity);
    const uint32_t tid = threadIdx.x;
    const uint32_t seg0 = blockIdx.x * kPlanThreads;
    const uint32_t i = seg0 + tid;
    const uint32_t mine = i < nseg ? ChunksOf(triples, i, units) : 0u;
    counts[kMaxPeriod + tid] = mine;
    if (tid < kMaxPeriod) {
        counts[tid] = seg0 + tid >= kMaxPeriod ? ChunksOf(triples, seg0 + tid - kMaxPeriod, units) : 0u;
    }
    __syncthreads();
    uint32_t alive = kAllPeriods;
    if (i < nseg) {
#pragma unroll
        for (uint32_t p = 1; p <= kMaxPeriod; ++p) {
            if (i >= p && counts[kMaxPeriod + tid - p] != mine) {
                alive &= ~(1u << p);
            }
        }
    }
    const uint32_t sum = WaveSum(mine);
    const uint32_t all = WaveAnd(alive);
    if ((tid & 63u) == 0) {
        waveSum[tid >> 6] = sum;
        waveAlive[tid >> 6] = all;
    }
    __syncthreads();
    if (tid == 0) {
        uint32_t s = 0;
        uint32_t a = kAllPeriods;
        for (uint32_t w = 0; w < kPlanWaves; ++w) {
            s += waveSum[w];
            a &= waveAlive[w];
        }
        scratch[at.blockSum + blockIdx.x] = s;
        scratch[at.blockAlive + blockIdx.x] = a;
    }
}

// The planner proper.  Thread t takes kEach consecutive segments.  One workgroup and one launch for up to
// kPlanSingleBlockSegs segments (kEach = 1, 2, 4 or 8); beyond, one workgroup per kPlanThreads segments
// (kEach = 1) behind XcopyPlanSumsKernel, which has left the sums and the periods of all workgroups.
template <uint32_t kEach>
__global__ __launch_bounds__(kPlanThreads) void XcopyPlanKernel(const uint64_t *__restrict__ triples, uint32_t nseg, uint32_t units,
                                                                uint32_t *__restrict__ scratch, uint32_t groupCapacity)
{
    __shared__ uint32_t counts[kMaxPeriod + kEach * kPlanThreads];
    __shared__ uint32_t waveTotal[kPlanWaves];      // inclusive sums of the waves, then their exclusive prefix
    __shared__ uint32_t reduced[2 * kPlanWaves + 4];
    const ScratchLayout at = ScratchLayoutFor(nseg, groupCapacity);
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = tid >> 6;
    const bool alone = gridDim.x == 1;
    const uint32_t i0 = (blockIdx.x * kPlanThreads + tid) * kEach;

    uint32_t mine[kEach];
    uint32_t sum = 0;
#pragma unroll
    for (uint32_t q = 0; q < kEach; ++q) {
        mine[q] = i0 + q < nseg ? ChunksOf(triples, i0 + q, units) : 0u;
        sum += mine[q];
        if (alone) {
            counts[kMaxPeriod + tid * kEach + q] = mine[q];
        }
    }
    if (alone && tid < kMaxPeriod) {
        counts[tid] = 0;
    }
    const uint32_t incl = WaveInclusiveSum(sum, lane);
    if (lane == 63) {
        waveTotal[wave] = incl;
    }
    __syncthreads();

    uint32_t aliveMine = kAllPeriods;
    if (alone) {
        // the eight counts in front of this thread's segments, then its own, checked against every period
        uint32_t window[kMaxPeriod + kEach];
#pragma unroll
        for (uint32_t w = 0; w < kMaxPeriod; ++w) {
            window[w] = counts[tid * kEach + w];
        }
#pragma unroll
        for (uint32_t q = 0; q < kEach; ++q) {
            window[kMaxPeriod + q] = mine[q];
        }
#pragma unroll
        for (uint32_t q = 0; q < kEach; ++q) {
#pragma unroll
            for (uint32_t p = 1; p <= kMaxPeriod; ++p) {
                if (i0 + q < nseg && i0 + q >= p && window[kMaxPeriod + q - p] != mine[q]) {
                    aliveMine &= ~(1u << p);
                }
            }
        }
    }
    const uint32_t aliveWave = WaveAnd(aliveMine);
    // wave 0: exclusive prefix over the wave totals and their sum
    if (wave == 0) {
        const uint32_t own = lane < kPlanWaves ? waveTotal[lane] : 0u;
        const uint32_t scan = WaveInclusiveSum(own, lane);
        if (lane < kPlanWaves) {
            waveTotal[lane] = scan - own;
        }
        if (lane == 63) {
            reduced[2 * kPlanWaves] = scan;          // chunks of this workgroup's segments
        }
    }
    if (lane == 0) {
        reduced[wave] = aliveWave;
    }
    __syncthreads();

    // chunks in front of this workgroup, chunks of the whole table, periods still alive
    uint32_t base = 0;
    uint32_t total = reduced[2 * kPlanWaves];
    uint32_t alive = kAllPeriods;
    if (alone) {
        for (uint32_t w = 0; w < kPlanWaves; ++w) {
            alive &= reduced[w];
        }
    } else {
        uint32_t front = 0;
        uint32_t whole = 0;
        uint32_t bits = kAllPeriods;
        for (uint32_t b = tid; b < gridDim.x; b += kPlanThreads) {
            const uint32_t blockSum = scratch[at.blockSum + b];
            whole += blockSum;
            front += b < blockIdx.x ? blockSum : 0u;
            bits &= scratch[at.blockAlive + b];
        }
        front = WaveSum(front);
        whole = WaveSum(whole);
        bits = WaveAnd(bits);
        __syncthreads();                               // every thread has read reduced[] above
        if (lane == 0) {
            reduced[wave] = front;
            reduced[kPlanWaves + wave] = whole;
            counts[wave] = bits;
        }
        __syncthreads();
        total = 0;
        for (uint32_t w = 0; w < kPlanWaves; ++w) {
            base += reduced[w];
            total += reduced[kPlanWaves + w];
            alive &= counts[w];
        }
    }

    const uint32_t shift = GroupShiftFor(total, at.groupCapacity);
    const uint32_t ngroups = GroupCount(total, shift);
    uint32_t *first = scratch + at.first;
    uint32_t *group = scratch + at.group;
    uint32_t f = base + waveTotal[wave] + incl - sum;
#pragma unroll
    for (uint32_t q = 0; q < kEach; ++q) {
        const uint32_t i = i0 + q;
        const bool live = i < nseg;
        if (live) {
            first[i] = f;
            if (i == nseg - 1) {
                first[nseg] = f + mine[q];
            }
        }
        // map entries of the groups whose first chunk this segment owns; the segment that owns the last chunk also closes the map
        uint32_t gLo = 1;
        uint32_t gHi = 0;
        if (live && mine[q] != 0) {
            gLo = static_cast<uint32_t>((static_cast<uint64_t>(f) + (1ull << shift) - 1) >> shift);
            gHi = (f + mine[q] - 1) >> shift;
            if (f + mine[q] == total) {
                group[ngroups] = i;
            }
        }
        const bool some = gLo <= gHi;
        const bool many = some && gHi - gLo >= 4;
        if (some && !many) {
            for (uint32_t g = gLo; g <= gHi; ++g) {
                group[g] = i;
            }
        }
        // a segment of many groups is written by its whole wave
        uint64_t todo = __ballot(many);
        while (todo != 0) {
            const uint32_t from = static_cast<uint32_t>(__builtin_ctzll(todo));
            todo &= todo - 1;
            const uint32_t lo = __builtin_amdgcn_readlane(gLo, from);
            const uint32_t hi = __builtin_amdgcn_readlane(gHi, from);
            const uint32_t owner = __builtin_amdgcn_readlane(i, from);
            for (uint64_t g = static_cast<uint64_t>(lo) + lane; g <= hi; g += 64) {
                group[g] = owner;
            }
        }
        f += mine[q];
    }

    if (blockIdx.x == 0 && tid == 0) {
        TableHeader *header = reinterpret_cast<TableHeader *>(scratch);
        header->nchunk = total;
        header->groupShift = shift;
        header->reserved[0] = 0;
        header->reserved[1] = 0;
        ChunkPattern pattern{};
        if (alive != 0 && total != 0) {
            // the shortest period never exceeds the segment count: period nseg is never contradicted
            const uint32_t period = static_cast<uint32_t>(__builtin_ctz(alive));
            uint32_t run = 0;
            for (uint32_t q = 0; q < period; ++q) {
                pattern.start[q] = run;
                run += ChunksOf(triples, q, units);
            }
            pattern.start[period] = run;
            if (run != 0) {
                pattern.period = period;
                pattern.chunksPerPeriod = run;
            } else {
                pattern = ChunkPattern{};
            }
        }
        header->pattern = pattern;
        header->pad = 0;
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
// before it on the same stream still run (hipExtAnyOrderLaunch; a 9 MB batch on one stream: 5.3 against 5.9 us).
// holdNanos: the caller's HoldNanosFor(); the launch qualifies only if it has one chunk per workgroup, of
// 4 KiB (stores of four loads per lane held) or of kWindowUnits units (of sixteen).
template <bool kNtLoad, int kStore>
int LaunchInline(const InlinePlan &plan, uint32_t grid, uint32_t lanes, hipStream_t stream, bool anyOrder, uint32_t holdNanos)
{
    const uint32_t flags = anyOrder ? hipExtAnyOrderLaunch : 0u;
    const bool deep = plan.units == kWindowUnits && grid == plan.nchunk && holdNanos != 0 && !anyOrder;
    if (deep) {
        lanes = 64;
    }
    const uint32_t ticks = grid == plan.nchunk && lanes == 64 ? HoldTicks(holdNanos) : 0;
    if (plan.first[1] == kNoChunk && plan.nchunk <= kSingleMaxChunks) {
        if (anyOrder) {
            hipExtLaunchKernelGGL((XcopySingleKernel<kNtLoad, kStore>), dim3(grid), dim3(lanes), 0, stream, nullptr, nullptr, flags,
                                  plan.src[0], plan.dst[0], plan.len[0], plan.nchunk, plan.units, 0u);
        } else if (ticks != 0 && deep) {
            hipLaunchKernelGGL((XcopySingleKernel<kNtLoad, kStore, kHoldDeep>), dim3(grid), dim3(lanes), 0, stream, plan.src[0],
                               plan.dst[0], plan.len[0], plan.nchunk, plan.units, ticks);
        } else if (ticks != 0) {
            hipLaunchKernelGGL((XcopySingleKernel<kNtLoad, kStore, kHoldShallow>), dim3(grid), dim3(lanes), 0, stream, plan.src[0],
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
    const void *kernel = reinterpret_cast<const void *>(&XcopyInlineKernel<kNtLoad, kStore, kHoldNone>);
    if (ticks != 0 && !anyOrder) {
        kernel = deep ? reinterpret_cast<const void *>(&XcopyInlineKernel<kNtLoad, kStore, kHoldDeep>)
                      : reinterpret_cast<const void *>(&XcopyInlineKernel<kNtLoad, kStore, kHoldShallow>);
    }
    if (anyOrder) {
        hipExtLaunchKernelGGL((XcopyInlineKernel<kNtLoad, kStore>), dim3(grid), dim3(lanes), 0, stream, nullptr, nullptr, flags, plan,
                              0u);
        return static_cast<int>(hipGetLastError());
    }
    return static_cast<int>(hipLaunchKernel(kernel, dim3(grid), dim3(lanes), args, 0, stream));
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
int LaunchTable(const TablePlan &plan, uint32_t grid, uint32_t lanes, hipStream_t stream, uint32_t holdNanos)
{
    if (plan.header != nullptr) {
        hipLaunchKernelGGL((XcopyTableKernel<kNtLoad, kStore, true>), dim3(grid), dim3(lanes), 0, stream, plan, 0u);
        return static_cast<int>(hipGetLastError());
    }
    const bool deep = plan.units == kWindowUnits && holdNanos != 0;
    if (deep) {
        lanes = 64;
    }
    const uint32_t ticks = grid == plan.nchunk && lanes == 64 ? HoldTicks(holdNanos) : 0;
    if (ticks != 0 && deep) {
        hipLaunchKernelGGL((XcopyTableKernel<kNtLoad, kStore, false, kHoldDeep>), dim3(grid), dim3(lanes), 0, stream, plan, ticks);
    } else if (ticks != 0) {
        hipLaunchKernelGGL((XcopyTableKernel<kNtLoad, kStore, false, kHoldShallow>), dim3(grid), dim3(lanes), 0, stream, plan, ticks);
    } else {
        hipLaunchKernelGGL((XcopyTableKernel<kNtLoad, kStore, false>), dim3(grid), dim3(lanes), 0, stream, plan, 0u);
    }
    return static_cast<int>(hipGetLastError());
}

// The planner's one or two launches for a table of nseg segments in device memory.
int LaunchPlanner(const uint64_t *triples, uint32_t nseg, uint32_t units, uint32_t *scratch, uint32_t groupCapacity,
                  hipStream_t stream)
{
    const uint32_t blocks = PlanBlocks(nseg);
    if (blocks > 1) {
        hipLaunchKernelGGL(XcopyPlanSumsKernel, dim3(blocks), dim3(kPlanThreads), 0, stream, triples, nseg, units, scratch,
                           groupCapacity);
        const hipError_t err = hipGetLastError();
        if (err != hipSuccess) {
            return static_cast<int>(err);
        }
    }
    const uint32_t tiles = blocks > 1 ? 1u : (nseg + kPlanThreads - 1) / kPlanThreads;   // segments per thread
    if (tiles <= 1) {
        hipLaunchKernelGGL(XcopyPlanKernel<1>, dim3(blocks), dim3(kPlanThreads), 0, stream, triples, nseg, units, scratch, groupCapacity);
    } else if (tiles <= 2) {
        hipLaunchKernelGGL(XcopyPlanKernel<2>, dim3(1), dim3(kPlanThreads), 0, stream, triples, nseg, units, scratch, groupCapacity);
    } else if (tiles <= 4) {
        hipLaunchKernelGGL(XcopyPlanKernel<4>, dim3(1), dim3(kPlanThreads), 0, stream, triples, nseg, units, scratch, groupCapacity);
    } else {
        hipLaunchKernelGGL(XcopyPlanKernel<kPlanTiles>, dim3(1), dim3(kPlanThreads), 0, stream, triples, nseg, units, scratch,
                           groupCapacity);
    }
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

// 1 when the period of a windowed launch can be computed on the current device (its constant-rate clock is known).
extern "C" int mfk_xcopy_windows_available(void)
{
    return mf::WindowPeriodTicks(2ull * mf::kWindowWaves * mf::kWindowUnits * mf::kUnitBytes, 6800000u) != 0 ? 1 : 0;
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
    const uint32_t grid = mf::WindowGrid(plan.nchunk, mf::kWindowWaves);
    const int err = mf::WithPolicy(mf::PolicyOf(MFRT_ROUTE_HBM), [&](auto ntLoad, auto store) {
        return mf::LaunchWindowed<decltype(ntLoad)::value, decltype(store)::value>(plan, grid, windowMBps, s);
    });
    return err != 0 ? err : mf::Signal(mask, maskValue, s);
}

extern "C" int mfk_xcopy_signal(void *word, uint32_t value, void *stream)
{
    return mf::Signal(word, value, static_cast<hipStream_t>(stream));
}

extern "C" int mfk_xcopy_table(const void *tablePlan, int route, uint32_t grid, void *mask, uint32_t maskValue, void *stream,
                               uint32_t holdNanos)
{
    const mf::TablePlan &plan = *static_cast<const mf::TablePlan *>(tablePlan);
    const mf::ChunkPattern &pat = plan.pattern;
    if (plan.nseg == 0 || grid == 0 || plan.triples == nullptr) {
        return -1;
    }
    if (plan.header == nullptr) {
        if (pat.period == 0 && (plan.first == nullptr || plan.group == nullptr || plan.groupShift < mf::kGroupShiftMin ||
                                plan.groupShift > 31)) {
            return -1;
        }
        if (pat.period != 0 && (pat.period > mf::kMaxPeriod || pat.chunksPerPeriod == 0 || pat.start[0] != 0 ||
                                pat.start[pat.period] != pat.chunksPerPeriod || mf::PatternChunks(pat, plan.nseg) != plan.nchunk)) {
            return -1;
        }
    } else if (plan.first == nullptr || plan.group == nullptr) {
        return -1;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int err = mf::WithPolicy(mf::PolicyOf(route), [&](auto ntLoad, auto store) {
        return mf::LaunchTable<decltype(ntLoad)::value, decltype(store)::value>(plan, grid, mf::LanesFor(plan.units, route), s,
                                                                                route == MFRT_ROUTE_HBM ? holdNanos : 0u);
    });
    return err != 0 ? err : mf::Signal(mask, maskValue, s);
}

extern "C" uint64_t mfk_xcopy_plan_scratch_words(uint32_t nseg, uint32_t groupCapacity)
{
    return mf::ScratchLayoutFor(nseg, groupCapacity).words;
}

// scratch: mfk_xcopy_plan_scratch_words(nseg, groupCapacity) words of device memory.  *tablePlan receives the plan for
// mfk_xcopy_table that reads what the planner leaves there.
extern "C" int mfk_xcopy_plan(const void *triples, uint32_t nseg, uint32_t units, void *scratch, uint32_t groupCapacity,
                              void *tablePlan, void *stream)
{
    if (nseg == 0 || scratch == nullptr || groupCapacity < 2 || tablePlan == nullptr) {
        return -1;
    }
    uint32_t *words = static_cast<uint32_t *>(scratch);
    const mf::ScratchLayout at = mf::ScratchLayoutFor(nseg, groupCapacity);
    mf::TablePlan &plan = *static_cast<mf::TablePlan *>(tablePlan);
    plan = mf::TablePlan{};
    plan.triples = static_cast<const uint64_t *>(triples);
    plan.first = words + at.first;
    plan.group = words + at.group;
    plan.header = reinterpret_cast<const mf::TableHeader *>(words);
    plan.nseg = nseg;
    plan.units = units;
    return mf::LaunchPlanner(plan.triples, nseg, units, words, groupCapacity, static_cast<hipStream_t>(stream));
}

// Every copy kernel once, on plans that hold nothing, so that a caller who captures a stream later finds the code of
// this file loaded and every kernel known to the runtime (a kernel's first launch is not capturable).
extern "C" int mfk_xcopy_prelaunch(void *stream)
{
    using namespace mf;
    hipStream_t s = static_cast<hipStream_t>(stream);
    InlinePlan empty{};
    for (uint32_t i = 0; i < kInlineSegs; ++i) {
        empty.first[i] = kNoChunk;
    }
    empty.units = kXcopyThreads;
    TablePlan none{};
    none.nseg = 1;
    none.units = kXcopyThreads;
    none.groupShift = kGroupShiftMin;
    for (int route = MFRT_ROUTE_HBM; route <= MFRT_ROUTE_FROM_HOST; ++route) {
        (void)WithPolicy(PolicyOf(route), [&](auto ntLoad, auto store) {
            constexpr bool kNt = decltype(ntLoad)::value;
            constexpr int kSt = decltype(store)::value;
            hipLaunchKernelGGL((XcopyInlineKernel<kNt, kSt, kHoldNone>), dim3(1), dim3(64), 0, s, empty, 0u);
            hipLaunchKernelGGL((XcopySingleKernel<kNt, kSt, kHoldNone>), dim3(1), dim3(64), 0, s, 0ull, 0ull, 0u, 0u, kXcopyThreads, 0u);
            hipLaunchKernelGGL((XcopyTableKernel<kNt, kSt, false, kHoldNone>), dim3(1), dim3(64), 0, s, none, 0u);
            if (route == MFRT_ROUTE_HBM) {
                hipLaunchKernelGGL((XcopyInlineKernel<kNt, kSt, kHoldShallow>), dim3(1), dim3(64), 0, s, empty, 1u);
                hipLaunchKernelGGL((XcopyInlineKernel<kNt, kSt, kHoldDeep>), dim3(1), dim3(64), 0, s, empty, 1u);
                hipLaunchKernelGGL((XcopySingleKernel<kNt, kSt, kHoldShallow>), dim3(1), dim3(64), 0, s, 0ull, 0ull, 0u, 0u, kXcopyThreads, 1u);
                hipLaunchKernelGGL((XcopySingleKernel<kNt, kSt, kHoldDeep>), dim3(1), dim3(64), 0, s, 0ull, 0ull, 0u, 0u, kWindowUnits, 1u);
                hipLaunchKernelGGL((XcopyTableKernel<kNt, kSt, false, kHoldShallow>), dim3(1), dim3(64), 0, s, none, 1u);
                hipLaunchKernelGGL((XcopyTableKernel<kNt, kSt, false, kHoldDeep>), dim3(1), dim3(64), 0, s, none, 1u);
                hipLaunchKernelGGL((XcopyWindowKernel<kNt, kSt>), dim3(1), dim3(64), 0, s, empty, 64u, NextWindowSeq());
            }
            return 0;
        });
    }
    return static_cast<int>(hipGetLastError());
}

// Calibration workloads, timed by events on `stream` (see XcopyEngine::Calibrate for what is chosen from them).
// out[0 .. 3]: microseconds per batch of 122 segments (61 x 128 KiB and 16 KiB in turn, 2196 chunks, 32 tables in turn
// inside 1 GiB of scratch) without a hold and held for holdNanos[0 .. 2]; out[4 .. 7]: microseconds per copy of 512 MiB by
// the kernel without windows and in windows cut for windowMBps[0 .. 2].  Batches: the fastest of three rounds of 128
// launches; copies: the fastest of six, each timed on its own.
extern "C" int mfk_xcopy_calibrate(void *stream, const uint32_t *holdNanos, const uint32_t *windowMBps, float *out)
{
    using namespace mf;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint64_t half = 512ull << 20;
    char *scratchMem = nullptr;
    hipError_t err = hipMalloc(&scratchMem, 2 * half);
    if (err != hipSuccess) {
        return static_cast<int>(err);
    }
    hipEvent_t e0 = nullptr;
    hipEvent_t e1 = nullptr;
    auto release = [&](hipError_t code) {
        (void)hipStreamSynchronize(s);
        if (e0 != nullptr) {
            (void)hipEventDestroy(e0);
        }
        if (e1 != nullptr) {
            (void)hipEventDestroy(e1);
        }
        (void)hipFree(scratchMem);
        return static_cast<int>(code);
    };
    if ((err = hipMemsetAsync(scratchMem, 0x5A, 2 * half, s)) != hipSuccess || (err = hipEventCreate(&e0)) != hipSuccess ||
        (err = hipEventCreate(&e1)) != hipSuccess) {
        return release(err);
    }
    // 32 tables of K and V blocks, every block in a 128 KiB slot of its own: sources in the lower half, destinations in
    // the upper; together they touch 576 MB, more than the last-level cache holds, as a caller's batches do
    constexpr uint32_t kTables = 32;
    constexpr uint32_t kSlotsPerHalf = 4096;
    std::vector<InlinePlan> plans(kTables);
    const uint64_t base = reinterpret_cast<uint64_t>(scratchMem);
    for (uint32_t t = 0; t < kTables; ++t) {
        InlinePlan &plan = plans[t];
        uint32_t run = 0;
        for (uint32_t i = 0; i < kInlineSegs; ++i) {
            if (i < 122) {
                const uint32_t len = (i & 1u) != 0 ? 16384u : 131072u;
                const uint32_t at = t * 122 + i;
                plan.src[i] = base + static_cast<uint64_t>((at * 1103u + 17u) % kSlotsPerHalf) * (128u << 10);
                plan.dst[i] = base + half + static_cast<uint64_t>((at * 757u + 5u) % kSlotsPerHalf) * (128u << 10);
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
        plan.units = kXcopyThreads;
    }
    InlinePlan big{};
    for (uint32_t i = 0; i < kInlineSegs; ++i) {
        big.first[i] = kNoChunk;
    }
    big.src[0] = base;
    big.dst[0] = base + half;
    big.len[0] = static_cast<uint32_t>(half);
    big.first[0] = 0;
    auto timed = [&](auto launch, int warm, int count, float &best) -> hipError_t {
        for (int i = 0; i < warm; ++i) {
            launch(i);
        }
        hipError_t code = hipEventRecord(e0, s);
        for (int i = 0; i < count && code == hipSuccess; ++i) {
            launch(i);
        }
        if (code == hipSuccess) {
            code = hipEventRecord(e1, s);
        }
        if (code == hipSuccess) {
            code = hipEventSynchronize(e1);
        }
        float ms = 0.0f;
        if (code == hipSuccess) {
            code = hipEventElapsedTime(&ms, e0, e1);
        }
        if (code == hipSuccess) {
            const float us = ms * 1000.0f / static_cast<float>(count);
            best = best == 0.0f || us < best ? us : best;
        }
        return code != hipSuccess ? code : hipGetLastError();
    };
    for (int i = 0; i < 8; ++i) {
        out[i] = 0.0f;
    }
    for (int round = 0; round < 3; ++round) {
        for (int v = 0; v < 4; ++v) {
            const uint32_t nanos = v == 0 ? 0u : holdNanos[v - 1];
            err = timed([&](int i) { (void)LaunchInline<true, kStoreStream>(plans[i % kTables], plans[0].nchunk, 64, s, false, nanos); }, 32, 128,
                        out[v]);
            if (err != hipSuccess) {
                return release(err);
            }
        }
    }
    // Every copy is timed on its own and the fastest of six counts: a windowed launch now and then loses its schedule part of
    // the way, at any rate, and the question here is whether this GPU holds the rate at all (two launches timed together,
    // three times, once gave 156.6 us for a rate whose launches otherwise take 148.4: one more such sample and the process
    // would have run at the lower rate for good).
    for (int round = 0; round < 6; ++round) {
        for (int v = 0; v < 4; ++v) {
            if (v == 0) {
                big.units = kXcopyThreads;
                big.nchunk = static_cast<uint32_t>(half / (kXcopyThreads * kUnitBytes));
                err = timed([&](int) { (void)LaunchInline<true, kStoreStream>(big, big.nchunk, 64, s, false, 0); }, round == 0 ? 1 : 0, 1, out[4]);
            } else {
                big.units = kWindowUnits;
                big.nchunk = static_cast<uint32_t>(half / (kWindowUnits * kUnitBytes));
                const uint32_t rate = windowMBps[v - 1];
                err = timed([&](int) { (void)LaunchWindowed<true, kStoreStream>(big, kWindowWaves, rate, s); }, round == 0 ? 1 : 0, 1,
                            out[4 + v]);
            }
            if (err != hipSuccess) {
                return release(err);
            }
        }
    }
    return release(hipSuccess);
}

#ifndef MF_RT_HIDDEN   // the plugin library has no entry point that needs it
// Scratch of the entry point that allocates nothing (mfk_xcopy_table_static): header, chunk prefix,
// the planner's partial sums and the group map, written by the planner and read by XcopyTableKernel of the
// same call.  One copy per GPU, held until the process ends.  In host code the array's name is only a
// handle for hipGetSymbolAddress: kernels get the address that call returned for the current device,
// never the name.
constexpr uint32_t kStaticGroupCapacity = MFK_STATIC_TABLE_SEGMENTS;
constexpr uint64_t kStaticScratchWords = mf::ScratchLayoutFor(MFK_STATIC_TABLE_SEGMENTS, kStaticGroupCapacity).words;
static __device__ __align__(256) uint32_t scratch[kStaticScratchWords];

namespace {
constexpr int kMaxDevices = 64;
uint32_t *g_scratchOf[kMaxDevices] = {};   // device ordinal -> address of that device's copy of `scratch`
// Calls on one GPU share the array.  The host side keeps them apart where it can without allocating: an event made at
// set-up is recorded behind every call, and a call that comes on another stream than the one before first makes its
// stream wait for that event.  Calls under stream capture are outside this (an event recorded there belongs to the graph).
hipEvent_t g_staticDone[kMaxDevices] = {};
hipStream_t g_staticLast[kMaxDevices] = {};
bool g_staticUsed[kMaxDevices] = {};
std::mutex g_staticLock;
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
    if (g_staticDone[dev] == nullptr && hipEventCreateWithFlags(&g_staticDone[dev], hipEventDisableTiming) != hipSuccess) {
        g_staticDone[dev] = nullptr;   // calls then go unguarded, as documented for callers that overlap them
        (void)hipGetLastError();
    }
    // The kernels of the device-table path once, on a table of no segments whose header lands in the array (what
    // mfk_xcopy_prelaunch cannot do without device memory): a caller may then capture its very first call.
    {
        using namespace mf;
        uint32_t *words = g_scratchOf[dev];
        const uint64_t *none = reinterpret_cast<const uint64_t *>(words);
        hipLaunchKernelGGL(XcopySignalKernel, dim3(1), dim3(64), 0, nullptr, reinterpret_cast<uint64_t *>(words + 2), 0u);   // the header's spare words
        hipLaunchKernelGGL(XcopyPlanSumsKernel, dim3(1), dim3(kPlanThreads), 0, nullptr, none, 0u, kXcopyThreads, words, kStaticGroupCapacity);
        hipLaunchKernelGGL(XcopyPlanKernel<1>, dim3(1), dim3(kPlanThreads), 0, nullptr, none, 0u, kXcopyThreads, words, kStaticGroupCapacity);
        hipLaunchKernelGGL(XcopyPlanKernel<2>, dim3(1), dim3(kPlanThreads), 0, nullptr, none, 0u, kXcopyThreads, words, kStaticGroupCapacity);
        hipLaunchKernelGGL(XcopyPlanKernel<4>, dim3(1), dim3(kPlanThreads), 0, nullptr, none, 0u, kXcopyThreads, words, kStaticGroupCapacity);
        hipLaunchKernelGGL(XcopyPlanKernel<8>, dim3(1), dim3(kPlanThreads), 0, nullptr, none, 0u, kXcopyThreads, words, kStaticGroupCapacity);
        const ScratchLayout at = ScratchLayoutFor(0, kStaticGroupCapacity);
        TablePlan plan{};
        plan.triples = none;
        plan.first = words + at.first;
        plan.group = words + at.group;
        plan.header = reinterpret_cast<const TableHeader *>(words);   // the planner launches above left nchunk = 0 there
        plan.units = kXcopyThreads;
        for (int route = MFRT_ROUTE_HBM; route <= MFRT_ROUTE_FROM_HOST; ++route) {
            (void)WithPolicy(PolicyOf(route), [&](auto ntLoad, auto store) {
                hipLaunchKernelGGL((XcopyTableKernel<decltype(ntLoad)::value, decltype(store)::value, true>), dim3(1), dim3(64), 0,
                                   nullptr, plan, 0u);
                return 0;
            });
        }
        err = hipGetLastError();
        if (err == hipSuccess) {
            err = hipStreamSynchronize(nullptr);
        }
        if (err != hipSuccess) {
            return static_cast<int>(err);
        }
    }
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
    std::lock_guard<std::mutex> guard(g_staticLock);
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    const bool capturing = hipStreamIsCapturing(s, &capture) == hipSuccess && capture != hipStreamCaptureStatusNone;
    const bool guarded = !capturing && g_staticDone[dev] != nullptr;
    if (guarded && g_staticUsed[dev] && g_staticLast[dev] != s && hipStreamWaitEvent(s, g_staticDone[dev], 0) != hipSuccess) {
        return static_cast<int>(hipGetLastError());
    }
    // the planner writes every word the table kernel reads: nothing has to start at zero
    mf::TablePlan plan;
    int err = mfk_xcopy_plan(triples, nseg, units, g_scratchOf[dev], kStaticGroupCapacity, &plan, stream);
    if (err == 0) {
        err = mfk_xcopy_table(&plan, route, grid, nullptr, 0, stream, 0);
    }
    if (guarded && hipEventRecord(g_staticDone[dev], s) == hipSuccess) {
        g_staticLast[dev] = s;
        g_staticUsed[dev] = true;
    }
    return err;
}
#endif  // MF_RT_HIDDEN
