// Work decomposition shared by the host planner and the xcopy kernels.
//
// A batch is a list of segments {src, dst, len} (the reference's uint64
// triples, src/hybm/csrc/data_operation/host/hybm_data_op_sdma.cpp:520-528).
// Each segment is cut into "chunks", the unit one workgroup copies in one
// loop iteration, so that work is proportional to bytes and not to segment
// count (the reference's kernel gives every core count/32 whole segments,
// src/hybm/csrc/copy_extend/hybm_copy_kernel.cpp:102-104).
//
// Geometry of one segment (all derived from dst, len and the chunk size):
//   head  = bytes until dst reaches a 16-byte boundary (capped at len)
//   body  = the following floor((len-head)/16) 16-byte units; stores are aligned
//   tail  = the remaining (len-head) % 16 bytes
//   chunk k covers body units [k*U, min((k+1)*U, body)); chunk 0 also copies
//   the head, the last chunk also copies the tail.  A segment of len > 0 has
//   max(1, ceil(body/U)) chunks, a segment of len 0 has none.
//
// This header is plain C++ (no HIP types) so the host planner and its CPU
// tests can include it.
#ifndef MF_XCOPY_PLAN_H
#define MF_XCOPY_PLAN_H

#include <stdint.h>

namespace mf {

constexpr uint32_t kXcopyThreads = 256;       // most lanes a copy workgroup has (4 wave64); 4 KiB chunks get one wave
constexpr uint32_t kUnitBytes = 16;           // one 128-bit access
constexpr uint32_t kInlineSegs = 128;         // segments that fit in the kernel-argument block: 2 table rows per lane of a wave64
constexpr uint32_t kNoChunk = 0xFFFFFFFFu;    // sentinel prefix for unused slots

#if defined(__HIPCC__)
#define MF_HD __host__ __device__
#else
#define MF_HD
#endif

struct SegGeom {
    uint32_t head;     // 0..15
    uint32_t tail;     // 0..15
    uint64_t body;     // 16-byte units
};

MF_HD inline SegGeom SegmentGeometry(uint64_t dst, uint64_t len)
{
    SegGeom g;
    uint64_t h = (0 - dst) & (kUnitBytes - 1);
    if (h > len) {
        h = len;
    }
    g.head = static_cast<uint32_t>(h);
    g.body = (len - h) / kUnitBytes;
    g.tail = static_cast<uint32_t>((len - h) % kUnitBytes);
    return g;
}

// Chunks of a segment for `units` 16-byte units per chunk.
MF_HD inline uint64_t SegmentChunks(uint64_t dst, uint64_t len, uint32_t units)
{
    if (len == 0) {
        return 0;
    }
    SegGeom g = SegmentGeometry(dst, len);
    uint64_t n = (g.body + units - 1) / units;
    return n == 0 ? 1 : n;
}

// Everything a launch of up to kInlineSegs segments needs, passed by value in
// the kernel-argument block (3080 bytes of the 4096 available): no table
// upload, no extra dependent memory round trip before the first data load.
struct InlinePlan {
    uint64_t src[kInlineSegs];
    uint64_t dst[kInlineSegs];
    uint32_t len[kInlineSegs];          // inline path carries segments < 4 GiB only
    uint32_t first[kInlineSegs];        // exclusive prefix of chunk counts, kNoChunk past the end
    uint32_t nchunk;
    uint32_t units;                     // 16-byte units per chunk, a multiple of 64
};

// Stores held back: how long after its start a wave of the inline kernel waits before it stores.
//
// A launch of a few thousand single-chunk waves has every load in flight within two microseconds and
// would store as the data trickle in, so HBM sees reads and writes mixed.  When every wave keeps its four
// loaded registers until the loads of the whole launch are out, the reads run as one burst and the
// writes as another: a 2196-chunk batch takes 4.5 instead of 5.3 us.  The wait is counted from the start
// of the wave, is the same for every wave, and grows with the number of waves the dispatcher has to start
// (a line fitted to sweeps over 976 ... 7076 chunks; it aims 50 to 100 ns long, because falling 200 ns short
// loses the gain while each 100 ns beyond costs 0.1 us).  It pays only while every wave of the launch is
// resident at once (up to 24 single-wave workgroups per CU) and only for launches that do not overlap
// others on purpose.  A single segment has no table to fetch and gets a line of its own.
constexpr uint32_t kHoldMinChunks = 960;        // table in the kernel arguments
constexpr uint32_t kHoldKneeChunks = 3904;
constexpr uint32_t kHoldMinChunksSingle = 1400; // one segment
constexpr uint32_t kHoldMaxChunks = 6144;
constexpr uint32_t kHoldSharedMaxChunks = 4096; // the limit while several threads submit on streams of their own
// Beyond kHoldMaxChunks chunks of 4 KiB the waves of a launch are no longer resident together.  Batches of up to
// kDeepMaxChunks chunks of kDeepUnits units (16 KiB, sixteen loads per lane in flight: 64 MiB in 4096 waves, 16 per CU)
// are, and hold their stores the same way.
constexpr uint32_t kDeepUnits = 1024;
constexpr uint32_t kDeepMaxChunks = 4096;
constexpr uint64_t kDeepMinBytes = static_cast<uint64_t>(kHoldMaxChunks) * kXcopyThreads * kUnitBytes;   // 24 MiB
constexpr uint64_t kDeepMaxBytes = static_cast<uint64_t>(kDeepMaxChunks) * kDeepUnits * kUnitBytes;      // 64 MiB
constexpr uint64_t kDeepMinSegmentBytes = 32768;   // on average: short segments make chunks that are not whole
inline uint32_t HoldNanosFor(uint32_t nchunk, uint32_t grid, uint32_t units, bool single)
{
    if (units == kDeepUnits && grid == nchunk && nchunk <= kDeepMaxChunks) {
        // fitted to sweeps over 1664 ... 4096 waves (26 to 64 MiB in 32 segments, one segment, 100 ragged ones): the best wait is
        // 600 ns and 2.15 ns per 16 KiB, a read rate of 7.6 TB/s; up to 10 % beyond costs 1 to 3 %, 10 % short loses half the gain
        return nchunk < kHoldMinChunks / 4 ? 0 : 600 + nchunk * 215 / 100;
    }
    if (units != kXcopyThreads || grid != nchunk || nchunk > kHoldMaxChunks) {
        return 0;   // only launches of one chunk per single-wave workgroup were measured
    }
    if (single) {
        return nchunk < kHoldMinChunksSingle ? 0 : 100 + nchunk * 57 / 100;
    }
    if (nchunk < kHoldMinChunks) {
        return 0;
    }
    if (nchunk <= kHoldKneeChunks) {
        return 640 + nchunk * 6 / 10;
    }
    return 640 + kHoldKneeChunks * 6 / 10 + (nchunk - kHoldKneeChunks) * 33 / 100;
}

// The start of a windowed launch's first period travels between its waves as the low kEpochClockBits bits of a
// clock value (2^40 ticks of 10 ns: three hours) under a sequence number; NearClock restores the full value: the
// one with those low bits that is nearest to `now`.
constexpr uint32_t kEpochClockBits = 40;
MF_HD inline uint64_t NearClock(uint64_t now, uint64_t low)
{
    const uint64_t mask = (1ull << kEpochClockBits) - 1;
    uint64_t t = (now & ~mask) | low;
    if (t > now && t - now > (mask >> 1)) {
        t -= mask + 1;
    } else if (t < now && now - t > (mask >> 1)) {
        t += mask + 1;
    }
    return t;
}

// Chunk counts that repeat with a short period: pages of one size (period 1), K and V blocks
// taking turns (period 2), ...  With such a pattern the owner of a chunk follows from a division
// and at most kMaxPeriod comparisons, and no chunk prefix is needed.
constexpr uint32_t kMaxPeriod = 8;

struct ChunkPattern {
    uint32_t period;                    // 0: no pattern, the chunk prefix is searched
    uint32_t chunksPerPeriod;
    uint32_t start[kMaxPeriod + 1];     // exclusive prefix of the counts inside one period; start[period] == chunksPerPeriod
};

// Segment and chunk-in-segment of global chunk c under a pattern.  Every start[] is read at a fixed index, so
// that a kernel keeps the pattern in scalar registers (the member that owns r is the last one whose start
// is <= r, and starts never decrease, so the hits form a prefix and the last hit's start is the owner's).
MF_HD inline void PatternOwner(const ChunkPattern &p, uint32_t c, uint32_t &seg, uint32_t &k)
{
    const uint32_t group = c / p.chunksPerPeriod;
    const uint32_t r = c - group * p.chunksPerPeriod;
    uint32_t j = 0;
    uint32_t base = 0;
    for (uint32_t i = 1; i < kMaxPeriod; ++i) {
        const bool hit = i < p.period && p.start[i] <= r;
        j += hit ? 1u : 0u;
        base = hit ? p.start[i] : base;
    }
    seg = group * p.period + j;
    k = r - base;
}

// Chunks of the first nseg segments under a pattern.
MF_HD inline uint64_t PatternChunks(const ChunkPattern &p, uint32_t nseg)
{
    return static_cast<uint64_t>(nseg / p.period) * p.chunksPerPeriod + p.start[nseg % p.period];
}

// Group map of a table without a pattern.  The chunks are taken in groups of 2^shift; group[g] is the
// segment that owns chunk g << shift, and one more entry names the segment that owns the last chunk.
// The owner of chunk c then lies in [group[g], group[g + 1]] with g = c >> shift, a range the 64 lanes
// of a wave probe in one round whenever it spans at most 64 segments: the lookup is two dependent loads
// instead of a search over the whole prefix.  A group of 2^shift chunks touches at most 2^shift + 1
// segments that are not empty, so groups of 32 chunks always resolve in that one round (groups of 64
// would need a second one for a run of 65 single-chunk segments).  The shift grows until the map fits
// the room there is for it.
constexpr uint32_t kGroupShiftMin = 5;

MF_HD constexpr inline uint32_t GroupCount(uint64_t nchunk, uint32_t shift)
{
    return static_cast<uint32_t>((nchunk + (1ull << shift) - 1) >> shift);
}

// Smallest shift from kGroupShiftMin on whose map (GroupCount + 1 entries) fits `capacity` entries.
MF_HD constexpr inline uint32_t GroupShiftFor(uint64_t nchunk, uint32_t capacity)
{
    uint32_t shift = kGroupShiftMin;
    while (shift < 32 && static_cast<uint64_t>(GroupCount(nchunk, shift)) + 1 > capacity) {
        ++shift;
    }
    return shift;
}

// Room the engine gives the map of a table of nseg segments: the finest groups for every table whose chunks
// number up to 32 times that (2 M chunks, 8 GiB in 4 KiB chunks, at the least), coarser ones beyond.
MF_HD constexpr inline uint32_t GroupCapacityFor(uint32_t nseg)
{
    return (nseg > 65536u ? nseg : 65536u) + 1u;
}

// Host-side build of the map from a finished prefix (first[0 .. nseg], first[nseg] == nchunk != 0); returns the shift.
// group: room for `capacity` entries.
inline uint32_t BuildGroupMap(const uint32_t *first, uint32_t nseg, uint32_t *group, uint32_t capacity)
{
    const uint32_t nchunk = first[nseg];
    const uint32_t shift = GroupShiftFor(nchunk, capacity);
    const uint32_t ngroups = GroupCount(nchunk, shift);
    uint32_t last = 0;
    for (uint32_t i = 0; i < nseg; ++i) {
        const uint32_t f = first[i];
        const uint32_t cnt = first[i + 1] - f;
        if (cnt == 0) {
            continue;
        }
        last = i;
        const uint32_t gLo = static_cast<uint32_t>((static_cast<uint64_t>(f) + (1ull << shift) - 1) >> shift);
        const uint32_t gHi = (f + cnt - 1) >> shift;
        for (uint64_t g = gLo; g <= gHi; ++g) {
            group[g] = i;
        }
    }
    group[ngroups] = last;
    return shift;
}

// What the device-side planner leaves for the table kernel of the same call (64 bytes).
struct TableHeader {
    uint32_t nchunk;
    uint32_t groupShift;
    uint32_t reserved[2];
    ChunkPattern pattern;               // period != 0: owner by division, prefix and group map are not read
    uint32_t pad;
};
static_assert(sizeof(TableHeader) == 64, "the planner's scratch layout counts on a 64-byte header");

// Segments one workgroup of the device-side planner takes, and its lanes.
constexpr uint32_t kPlanThreads = 1024;
constexpr uint32_t kPlanTiles = 8;                          // a workgroup walks up to this many tiles of kPlanThreads segments
constexpr uint32_t kPlanSingleBlockSegs = kPlanThreads * kPlanTiles;   // up to here one workgroup plans the whole table in one launch

// Words of device scratch the planner and the table kernel of a device-resident table share:
// header | first[nseg + 1] | blockSum[blocks] | blockAlive[blocks] | group[groupCapacity].
MF_HD constexpr inline uint32_t PlanBlocks(uint32_t nseg)
{
    return nseg <= kPlanSingleBlockSegs ? 1u : (nseg + kPlanThreads - 1) / kPlanThreads;
}
struct ScratchLayout {
    uint32_t first;                     // word offsets
    uint32_t blockSum;
    uint32_t blockAlive;
    uint32_t group;
    uint32_t groupCapacity;             // entries
    uint64_t words;
};
MF_HD constexpr inline ScratchLayout ScratchLayoutFor(uint32_t nseg, uint32_t groupCapacity)
{
    ScratchLayout l{};
    const uint32_t blocks = PlanBlocks(nseg);
    l.first = sizeof(TableHeader) / 4;
    l.blockSum = l.first + nseg + 1;
    l.blockAlive = l.blockSum + blocks;
    l.group = (l.blockAlive + blocks + 3u) & ~3u;
    l.groupCapacity = groupCapacity;
    l.words = static_cast<uint64_t>(l.group) + groupCapacity;
    return l;
}

// A table-driven launch: triples, prefix and group map live in device memory (under a pattern the
// triples may sit in pinned host memory and the other two are not read).
struct TablePlan {
    const uint64_t *triples;            // {src,dst,len} * nseg
    const uint32_t *first;              // nseg + 1 entries, first[nseg] == nchunk
    const uint32_t *group;              // GroupCount(nchunk, groupShift) + 1 entries
    const TableHeader *header;          // not NULL: nchunk, groupShift and pattern are read from there
    uint32_t nseg;
    uint32_t nchunk;
    uint32_t groupShift;
    uint32_t units;
    ChunkPattern pattern;
};

}  // namespace mf

#endif  // MF_XCOPY_PLAN_H
