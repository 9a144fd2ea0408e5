// Batched strided 2-D copy for gfx950: up to 64 rectangles per launch, work cut
// into groups of rows of about 16 KiB so that narrow rows (a few hundred bytes)
// still fill every lane with 128-bit accesses.  HBM bound, 2 bytes of traffic
// per payload byte; no LDS, no MFMA.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../rt/mf_rt.h"
#include "copy2d_plan.h"

namespace mf {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#define MF_GLOBAL __attribute__((address_space(1)))

__device__ __forceinline__ uint64_t ReadLane64(uint64_t v, uint32_t lane)
{
    const uint32_t lo = __builtin_amdgcn_readlane(static_cast<uint32_t>(v), lane);
    const uint32_t hi = __builtin_amdgcn_readlane(static_cast<uint32_t>(v >> 32), lane);
    return (static_cast<uint64_t>(hi) << 32) | lo;
}

__global__ __launch_bounds__(kRectThreads) void Copy2dKernel(const RectPlan p)
{
    // the whole rectangle table in registers after one round trip, one row per lane
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t first = p.first[lane];
    const uint64_t src = p.src[lane];
    const uint64_t dst = p.dst[lane];
    const uint32_t sp = p.spitchUnits[lane];
    const uint32_t dp = p.dpitchUnits[lane];
    const uint32_t wu = p.widthUnits[lane];
    const uint32_t ht = p.height[lane];
    const uint32_t rpc = p.rowsPerChunk[lane];
    const uint32_t mg = p.magic[lane];
    const uint32_t mt = p.mate[lane];
    const uint32_t nchunk = p.nchunk;
    uint32_t c = blockIdx.x;
    do {
        // Two rectangles side by side in the destination take the chunks of their common range in turn, so that
        // workgroups launched together write both parts of the same destination rows.
        uint32_t r = __popcll(__ballot(first <= c)) - 1;
        uint32_t k = c - __builtin_amdgcn_readlane(first, r);
        const uint32_t m = __builtin_amdgcn_readlane(mt, r);
        if (m != 0) {
            const uint32_t r0 = r - (m - 1);
            const uint32_t both = c - __builtin_amdgcn_readlane(first, r0);
            r = r0 + (both & 1u);
            k = both >> 1;
        }
        const uint64_t rs = ReadLane64(src, r);
        const uint64_t rd = ReadLane64(dst, r);
        const uint32_t rsp = __builtin_amdgcn_readlane(sp, r);
        const uint32_t rdp = __builtin_amdgcn_readlane(dp, r);
        const uint32_t rwu = __builtin_amdgcn_readlane(wu, r);
        const uint32_t rht = __builtin_amdgcn_readlane(ht, r);
        const uint32_t rrpc = __builtin_amdgcn_readlane(rpc, r);
        const uint32_t rmg = __builtin_amdgcn_readlane(mg, r);
        const uint32_t row0 = k * rrpc;
        const uint32_t rows = rht - row0 < rrpc ? rht - row0 : rrpc;
        const uint32_t units = rows * rwu;
        const MF_GLOBAL u32x4 *s = reinterpret_cast<const MF_GLOBAL u32x4 *>(rs) + static_cast<uint64_t>(row0) * rsp;
        MF_GLOBAL u32x4 *d = reinterpret_cast<MF_GLOBAL u32x4 *>(rd) + static_cast<uint64_t>(row0) * rdp;
        for (uint32_t u0 = 0; u0 < units; u0 += 4 * kRectThreads) {
            u32x4 v[4];
            uint32_t row[4];
            uint32_t col[4];
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j) {
                const uint32_t u = u0 + j * kRectThreads + threadIdx.x;
                RectRowCol(u, rwu, rrpc, rmg, row[j], col[j]);
                if (u < units) {
                    v[j] = __builtin_nontemporal_load(s + static_cast<uint64_t>(row[j]) * rsp + col[j]);
                }
            }
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j) {
                const uint32_t u = u0 + j * kRectThreads + threadIdx.x;
                if (u < units) {
                    __builtin_nontemporal_store(v[j], d + static_cast<uint64_t>(row[j]) * rdp + col[j]);
                }
            }
        }
        c += gridDim.x;
    } while (c < nchunk);
}

}  // namespace
}  // namespace mf

extern "C" int mfk_copy2d(const void *rectPlan, uint32_t grid, void *stream)
{
    const mf::RectPlan &plan = *static_cast<const mf::RectPlan *>(rectPlan);
    if (plan.nchunk == 0) {
        return 0;
    }
    if (grid == 0 || grid > plan.nchunk) {
        grid = plan.nchunk;
    }
    if (grid > (1u << 24) - 1) {
        grid = (1u << 24) - 1;   // the grid size in lanes must stay below 2^32; workgroups loop over the rest
    }
    hipLaunchKernelGGL(mf::Copy2dKernel, dim3(grid), dim3(mf::kRectThreads), 0, static_cast<hipStream_t>(stream), plan);
    return static_cast<int>(hipGetLastError());
}
