// Batched strided 2-D copy for gfx950: up to 64 rectangles per launch, work cut
// into groups of rows of about 16 KiB so that narrow rows (a few hundred bytes)
// still fill every lane with 128-bit accesses.  HBM bound, 2 bytes of traffic
// per payload byte; no LDS, no MFMA.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../rt/mf_rt.h"
#include "copy2d_plan.h"
#include "window_clock.h"

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

// The same rectangles in read and write windows (the form XcopyWindowKernel gives long segments): single-wave
// workgroups walk chunks of kRectWindowUnits units of a rectangle's payload taken row-major, whatever the width,
// one chunk per period each; sixteen loads per lane at the wave's offset into the read half of the period, the
// stores at the same offset into the write half.  plan.first counts these chunks (RectWindowChunks), a
// rectangle holds fewer than 2^32 units, rowsPerChunk is not used.
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(5))) void Copy2dWindowKernel(const RectPlan p, uint32_t period, uint32_t seq)
{
    // Only what the search needs stays in vector registers; the rectangle a chunk belongs to is read from the
    // argument block by scalar loads once it is known (a period is microseconds long, their latency does not show).
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t first = p.first[lane];
    const uint32_t mt = p.mate[lane];
    const uint32_t nchunk = p.nchunk;
    const uint32_t half = period / 2;
    uint64_t slot = AgreedStart(seq) + static_cast<uint64_t>(blockIdx.x) * half / gridDim.x;
    for (uint32_t c = blockIdx.x; c < nchunk; c += gridDim.x) {
        uint32_t r = __popcll(__ballot(first <= c)) - 1;
        uint32_t k = c - __builtin_amdgcn_readlane(first, r);
        const uint32_t m = __builtin_amdgcn_readlane(mt, r);
        if (m != 0) {
            const uint32_t r0 = r - (m - 1);
            const uint32_t both = c - __builtin_amdgcn_readlane(first, r0);
            r = r0 + (both & 1u);
            k = both >> 1;
        }
        r &= kRectInline - 1;
        const uint64_t rs = p.src[r];
        const uint64_t rd = p.dst[r];
        const uint32_t rsp = p.spitchUnits[r];
        const uint32_t rdp = p.dpitchUnits[r];
        const uint32_t rwu = p.widthUnits[r];
        const uint32_t rht = p.height[r];
        const uint32_t rmg = p.magic[r];
        const uint32_t base = k * kRectWindowUnits;
        const uint32_t left = rht * rwu - base;
        const uint32_t n = left < kRectWindowUnits ? left : kRectWindowUnits;
        const uint32_t row0 = base / rwu;
        const uint32_t col0 = base - row0 * rwu;
        const MF_GLOBAL u32x4 *s = reinterpret_cast<const MF_GLOBAL u32x4 *>(rs) + static_cast<uint64_t>(row0) * rsp;
        MF_GLOBAL u32x4 *d = reinterpret_cast<MF_GLOBAL u32x4 *>(rd) + static_cast<uint64_t>(row0) * rdp;
        // Row and column of a unit are worked out where its address is needed, before the loads and again before the
        // stores, from a lane offset the compiler cannot see through: kept across the waits (or worked out ahead of them,
        // as it prefers) sixteen rows or thirty-two addresses beside the data take the kernel past the registers at which
        // all kRectWindowWaves waves are resident together with room to spare, which the schedule needs.
        uint32_t x0 = col0 + lane;
        auto unitOffset = [&](uint32_t j, uint32_t pitch) -> uint64_t {
            uint32_t row;
            uint32_t col;
            RectWindowRowCol(x0 + j * 64, rwu, rmg, row, col);
            return static_cast<uint64_t>(row) * pitch + col;
        };
        u32x4 v[kRectWindowDepth];
        WaitForClock(slot);
        asm volatile("" : "+v"(x0));
        if (n == kRectWindowUnits) {
#pragma unroll
            for (uint32_t j = 0; j < kRectWindowDepth; ++j) {
                v[j] = __builtin_nontemporal_load(s + unitOffset(j, rsp));
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            WaitForClock(slot + half);
            asm volatile("" : "+v"(x0));
#pragma unroll
            for (uint32_t j = 0; j < kRectWindowDepth; ++j) {
                __builtin_nontemporal_store(v[j], d + unitOffset(j, rdp));
            }
        } else {
#pragma unroll
            for (uint32_t j = 0; j < kRectWindowDepth; ++j) {
                if (j * 64 + lane < n) {
                    v[j] = __builtin_nontemporal_load(s + unitOffset(j, rsp));
                }
            }
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            WaitForClock(slot + half);
            asm volatile("" : "+v"(x0));
#pragma unroll
            for (uint32_t j = 0; j < kRectWindowDepth; ++j) {
                if (j * 64 + lane < n) {
                    __builtin_nontemporal_store(v[j], d + unitOffset(j, rdp));
                }
            }
        }
        slot += period;
    }
}

}  // namespace
}  // namespace mf

extern "C" int mfk_copy2d_windowed(const void *rectPlan, uint32_t windowMBps, void *stream)
{
    const mf::RectPlan &plan = *static_cast<const mf::RectPlan *>(rectPlan);
    if (plan.nchunk == 0) {
        return 0;
    }
    const uint32_t grid = mf::WindowGrid(plan.nchunk, mf::kRectWindowWaves);
    const uint32_t ticks = mf::WindowPeriodTicks(2ull * grid * mf::kRectWindowUnits * 16u, windowMBps);
    if (ticks == 0) {
        return static_cast<int>(hipErrorInvalidValue);
    }
    hipLaunchKernelGGL(mf::Copy2dWindowKernel, dim3(grid), dim3(64), 0, static_cast<hipStream_t>(stream), plan, ticks,
                       mf::NextWindowSeq());
    return static_cast<int>(hipGetLastError());
}

// Both kernels once on a plan that holds nothing: a kernel's first launch is not capturable.
extern "C" int mfk_copy2d_prelaunch(void *stream)
{
    mf::RectPlan empty{};
    for (uint32_t i = 0; i < mf::kRectInline; ++i) {
        empty.first[i] = 0xFFFFFFFFu;
        empty.rowsPerChunk[i] = 1;
    }
    hipLaunchKernelGGL(mf::Copy2dKernel, dim3(1), dim3(mf::kRectThreads), 0, static_cast<hipStream_t>(stream), empty);
    hipLaunchKernelGGL(mf::Copy2dWindowKernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), empty, 64u,
                       mf::NextWindowSeq());
    return static_cast<int>(hipGetLastError());
}

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
