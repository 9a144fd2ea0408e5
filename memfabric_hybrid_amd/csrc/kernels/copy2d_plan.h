// Strided 2-D copies ("height rows of width bytes, rows spitch / dpitch apart"),
// the shape a tensor-parallel re-layout reduces to.  The reference exposes no
// 2-D copy (aclrtMemcpy2d is loaded at src/hybm/csrc/under_api/dl_acl_api.cpp:87-88
// and never called); callers there would issue one segment per row.
// Plain C++ so the host planner can include it.
#ifndef MF_COPY2D_PLAN_H
#define MF_COPY2D_PLAN_H

#include <stdint.h>

namespace mf {

constexpr uint32_t kRectInline = 64;      // rectangles per launch: one table row per lane of a wave64
constexpr uint32_t kRectThreads = 256;

// Fast-path rectangle: every address, pitch and the width are multiples of 16.
struct RectPlan {
    uint64_t src[kRectInline];
    uint64_t dst[kRectInline];
    uint32_t spitchUnits[kRectInline];    // pitches and width in 16-byte units
    uint32_t dpitchUnits[kRectInline];
    uint32_t widthUnits[kRectInline];
    uint32_t height[kRectInline];
    uint32_t rowsPerChunk[kRectInline];
    uint32_t magic[kRectInline];          // floor(2^32 / widthUnits) + 1, see RectRowCol; unused when rowsPerChunk == 1
    uint32_t first[kRectInline];          // exclusive prefix of chunk counts, 0xFFFFFFFF past the end
    uint32_t mate[kRectInline];           // 0: alone; 1 / 2: first / second of two rectangles that lie side by side in the
                                          // destination (RectsSideBySide) and whose chunks are dealt out in turn
    uint32_t nchunk;
};

#if defined(__HIPCC__)
#define MF_RECT_HD __host__ __device__
#else
#define MF_RECT_HD
#endif

constexpr uint32_t kRectChunkBytes = 16384;   // a workgroup's share: this many bytes of whole rows, or one wider row

// Rows one workgroup takes for rows of `width` bytes (a multiple of 16).
MF_RECT_HD inline uint32_t RectRowsPerChunk(uint64_t width)
{
    const uint64_t rows = width == 0 ? 1 : kRectChunkBytes / width;
    return rows == 0 ? 1u : static_cast<uint32_t>(rows);
}

MF_RECT_HD inline uint32_t RectMagic(uint32_t widthUnits)
{
    return widthUnits <= 1 ? 0u : static_cast<uint32_t>((1ull << 32) / widthUnits) + 1u;
}

// Row (relative to the chunk's first row) and column, in 16-byte units, of unit u of a chunk.
// A chunk that holds a single row needs no division, whatever the width; a chunk of several rows
// has rows of at most kRectChunkBytes / 2 bytes, so u < 1024 and widthUnits <= 512, where the
// multiply-high by floor(2^32 / widthUnits) + 1 is exact (it is for all u, widthUnits < 65536).
MF_RECT_HD inline void RectRowCol(uint32_t u, uint32_t widthUnits, uint32_t rowsPerChunk, uint32_t magic, uint32_t &row,
                                  uint32_t &col)
{
    if (rowsPerChunk == 1) {
        row = 0;
        col = u;
        return;
    }
    row = widthUnits == 1 ? u : static_cast<uint32_t>((static_cast<uint64_t>(u) * magic) >> 32);
    col = u - row * widthUnits;
}

// The windowed form cuts a rectangle's payload, taken row-major, into chunks of kRectWindowUnits units
// regardless of row ends (16 loads per lane of a single wave).
constexpr uint32_t kRectWindowDepth = 16;
constexpr uint32_t kRectWindowUnits = 64 * kRectWindowDepth;
constexpr uint32_t kRectWindowWaves = 4096;   // 16 per CU

// Chunks of the windowed form, or 0 for a rectangle it cannot take (2^32 units and more).
MF_RECT_HD inline uint64_t RectWindowChunks(uint64_t widthUnits, uint64_t height)
{
    const uint64_t units = widthUnits * height;
    if (widthUnits == 0 || units / widthUnits != height || units > 0xFFFFFFFFull) {
        return 0;
    }
    return (units + kRectWindowUnits - 1) / kRectWindowUnits;
}

// Row (relative to the row the chunk starts in) and column of the unit x units past the start of that row,
// x < widthUnits + kRectWindowUnits: the quotient is 0 or 1 for rows of kRectWindowUnits units and more,
// and below that x < 2 * kRectWindowUnits, where the multiply-high of RectRowCol is exact.
MF_RECT_HD inline void RectWindowRowCol(uint32_t x, uint32_t widthUnits, uint32_t magic, uint32_t &row, uint32_t &col)
{
    if (widthUnits >= kRectWindowUnits) {
        row = x >= widthUnits ? 1u : 0u;
    } else {
        row = widthUnits == 1 ? x : static_cast<uint32_t>((static_cast<uint64_t>(x) * magic) >> 32);
    }
    col = x - row * widthUnits;
}

// Whether a rectangle can take the 2-D kernel: everything a multiple of 16 and, in 16-byte units
// (rows: in rows), within the 32-bit fields of the plan.
MF_RECT_HD inline bool RectFitsPlan(uint64_t src, uint64_t dst, uint64_t width, uint64_t height, uint64_t spitch,
                                    uint64_t dpitch)
{
    return ((src | dst | width | spitch | dpitch) & 15u) == 0 && width / 16 <= 0xFFFFFFFFull &&
           spitch / 16 <= 0xFFFFFFFFull && dpitch / 16 <= 0xFFFFFFFFull && height <= 0xFFFFFFFFull;
}

// Two rectangles of the same shape whose destination rows continue one another: b's rows start where a's end,
// in the same destination pitch (the two old column blocks of a row-parallel weight, side by side in the new shard).
MF_RECT_HD inline bool RectsSideBySide(uint64_t dstA, uint64_t dstB, uint64_t widthA, uint64_t widthB, uint64_t heightA,
                                       uint64_t heightB, uint64_t dpitchA, uint64_t dpitchB)
{
    return widthA == widthB && heightA == heightB && dpitchA == dpitchB && dstB == dstA + widthA && dpitchA >= 2 * widthA;
}

// Rectangle r and chunk k inside it that chunk c of a plan stands for; what Copy2dKernel works out with a ballot over
// `first` and lane reads, restated for host code.  Rectangles that are mates take the chunks of their common range in turn.
inline void RectOfChunk(const RectPlan &plan, uint32_t c, uint32_t &r, uint32_t &k)
{
    r = 0;
    while (r + 1 < kRectInline && plan.first[r + 1] <= c) {
        ++r;
    }
    k = c - plan.first[r];
    if (plan.mate[r] != 0) {
        const uint32_t r0 = r - (plan.mate[r] - 1);
        const uint32_t both = c - plan.first[r0];
        r = r0 + (both & 1u);
        k = both >> 1;
    }
}

}  // namespace mf

#endif  // MF_COPY2D_PLAN_H
