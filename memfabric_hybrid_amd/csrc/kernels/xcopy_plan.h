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
// A launch of a few thousand single-chunk waves has every load in flight within the first two
// microseconds and would issue its stores as the data trickle in, so HBM sees reads and writes mixed
// for most of the kernel.  When every wave instead keeps its four loaded registers until the loads
// of the whole launch are out, the reads run as one burst and the writes as another, and the kernel
// is shorter.  Measured through smem_bm_copy_batch, batches back to back on one stream, K and V
// blocks in turn (61 of each, V blocks of 16 KiB), period per batch without the wait / at the best wait:
//    976 chunks 3.79 / 3.24 us (1300 ns)     2684 chunks 6.45 / 5.11 us (2200 ns)
//   1220 chunks 4.11 / 3.47 us (1400 ns)     3172 chunks 6.86 / 5.78 us (2600 ns)
//   1708 chunks 4.76 / 4.32 us (1500-1900)   3904 chunks 8.02 / 6.54 us (3000 ns)
//   2196 chunks 5.29 / 4.56 us (1900 ns)     5124 chunks 9.72 / 8.79 us (3400 ns)
// and for other mixes of about 2048 chunks: 64 x 128 KiB 5.05 / 4.64, 32 x 256 KiB 4.99 / 4.38,
// 128 x 64 KiB 5.07 / 4.61, 8 x 1 MiB + 100 x 20 KiB 6.12 / 5.07 us; 128 ragged segments of about
// 70000 bytes gain nothing and lose nothing (6.5 us either way).  The wait is counted from the start of
// the wave, which absorbs the spread of the table fetch (counted from the issue of the loads the same
// wait gains nothing), and it is the same for every wave: shortening it for waves that start later did
// not help.  The best wait grows with the number of waves the dispatcher has to start.  100 to 200 ns
// short of it the gain is lost (2196 chunks: 1700 ns 4.87 us, 1600 ns 5.09 us), each 100 ns beyond it
// costs 0.1 us, so the rule aims a little long: in steps of 50 ns, on four machines, 2196 chunks took 4.57 us at
// 1750 ns, 4.44 at 1800, 4.30 at 1850 to 1950, 4.35 at 2000 and 4.42 at 2050, and the rule gives 1957 ns; from 1220
// to 5124 chunks the rule is within 50 ns of the best step or level with it.  From about 7000 chunks on the gain is below 5 % and the
// best wait no longer follows the line: not every wave of such a launch is resident at once, and a wait
// only delays the ones behind (11956 chunks: 19.3 us without, 20.2 us with).  Below about
// 1000 chunks the period is the cost of a dependent launch and no wait changes it.
// Launches that overlap on purpose (no barrier between them) lose with a wait: 4.53 us without, 4.81 with.
//
// A single segment (its three words are plain kernel arguments, no table to fetch) has its loads out
// about 0.6 us earlier, and its best wait is shorter by as much; copies back to back on one stream,
// without / at the best wait:
//   1536 chunks (6 MiB) 3.64 / 3.39 us (1000 ns)     4096 chunks (16 MiB) 7.06 / 5.97 us (2300 ns)
//   2048 chunks (8 MiB) 4.08 / 3.83 us (1300 ns)     5120 chunks (20 MiB) 8.74 / 7.07 us (2900 ns)
//   3072 chunks (12 MiB) 5.71 / 4.90 us (1800 ns)    6144 chunks (24 MiB) 10.03 / 8.18 us (3400 ns)
// 1024 chunks gain nothing (3.1 us either way); 7168 chunks gain 5 %, 8192 and more 3 % and less: past
// 6144 single-wave workgroups (24 per CU) not every wave of the launch is resident at once.
constexpr uint32_t kHoldMinChunks = 960;        // table in the kernel arguments
constexpr uint32_t kHoldKneeChunks = 3904;
constexpr uint32_t kHoldMinChunksSingle = 1400; // one segment
constexpr uint32_t kHoldMaxChunks = 6144;
constexpr uint32_t kHoldSharedMaxChunks = 4096; // the limit while several threads submit on streams of their own
inline uint32_t HoldNanosFor(uint32_t nchunk, uint32_t grid, uint32_t units, bool single)
{
    if (units != kXcopyThreads || grid != nchunk || nchunk > kHoldMaxChunks) {
        return 0;   // only launches of one 4 KiB chunk per single-wave workgroup were measured
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

// Segment and chunk-in-segment of global chunk c under a pattern.
MF_HD inline void PatternOwner(const ChunkPattern &p, uint32_t c, uint32_t &seg, uint32_t &k)
{
    const uint32_t group = c / p.chunksPerPeriod;
    const uint32_t r = c - group * p.chunksPerPeriod;
    uint32_t j = 0;
    for (uint32_t i = 1; i < kMaxPeriod; ++i) {
        j += (i < p.period && p.start[i] <= r) ? 1u : 0u;
    }
    seg = group * p.period + j;
    k = r - p.start[j];
}

// Chunks of the first nseg segments under a pattern.
MF_HD inline uint64_t PatternChunks(const ChunkPattern &p, uint32_t nseg)
{
    return static_cast<uint64_t>(nseg / p.period) * p.chunksPerPeriod + p.start[nseg % p.period];
}

// A table-driven launch: triples and prefix live in device memory.
struct TablePlan {
    const uint64_t *triples;            // {src,dst,len} * nseg
    const uint32_t *first;              // nseg + 1 entries, first[nseg] == nchunk; not read under a pattern
    uint32_t nseg;
    uint32_t nchunk;
    uint32_t units;
    ChunkPattern pattern;
};

}  // namespace mf

#endif  // MF_XCOPY_PLAN_H
