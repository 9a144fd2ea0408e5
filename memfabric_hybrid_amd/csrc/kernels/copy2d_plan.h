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
    uint32_t magic[kRectInline];          // floor(2^32 / widthUnits) + 1: row = (u * magic) >> 32
    uint32_t first[kRectInline];          // exclusive prefix of chunk counts, 0xFFFFFFFF past the end
    uint32_t nchunk;
};

}  // namespace mf

#endif  // MF_COPY2D_PLAN_H
