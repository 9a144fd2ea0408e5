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
