// Clock windows of the kernel that alternates, chip-wide, between reading and writing (XcopyWindowKernel in
// xcopy.hip): waiting for a tick of the constant-rate clock, the word through which the waves of a launch
// agree on the start of their first period, and the host side's period and sequence numbers.  A
// translation unit that includes this header has its own copy of the word array and of the counter.
#ifndef MF_WINDOW_CLOCK_H
#define MF_WINDOW_CLOCK_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "xcopy_plan.h"

namespace mf {
namespace {

__device__ __forceinline__ void WaitForClock(uint64_t t)
{
    while (wall_clock64() < t) {
        __builtin_amdgcn_s_sleep(1);
    }
}

// Where the waves of a windowed launch agree on the start of their first period: workgroup 0, which the
// dispatcher starts first, publishes its clock under the launch's sequence number, the others read it.
// (Deriving the start from the clock alone, as the next multiple of the period, costs every launch half a
// period on average: 10 us, 3 % of a 1 GiB copy.  Letting whichever wave comes first publish with a
// compare-and-swap serialises 4096 same-address atomics across the XCDs: 1.2 ms.)  A wave that does not see
// a fresh value within its polls (workgroup 0 has not started yet, or started more than kEpochFreshTicks ago:
// other work holds part of the chip and the waves of this launch are not all resident together) gets 0, a
// start so long ago that every slot of its schedule has passed: it runs unpaced, as fast as it can, instead
// of holding a schedule cut for a chip it does not have.  One slot per launch in flight; a slot is reused
// after kEpochSlots launches.
constexpr uint32_t kEpochSlots = 64;
constexpr uint32_t kEpochPolls = 64;
constexpr uint32_t kEpochFreshTicks = 2000;                 // workgroup 0 starts at most 20 us before any other wave of its launch
__device__ unsigned long long g_windowEpoch[kEpochSlots];

__device__ __forceinline__ uint64_t AgreedStart(uint32_t seq)
{
    unsigned long long *slot = &g_windowEpoch[seq % kEpochSlots];
    const unsigned long long tag = static_cast<unsigned long long>(seq & 0xFFFFFFu) << kEpochClockBits;
    const unsigned long long mask = (1ull << kEpochClockBits) - 1;
    const uint64_t mine = wall_clock64() + 64;   // 0.6 us ahead: the first slots of the first waves do not lie in the past
    if (blockIdx.x == 0) {
        __hip_atomic_store(slot, tag | (mine & mask), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return mine;
    }
    for (uint32_t poll = 0; poll < kEpochPolls; ++poll) {
        const unsigned long long seen = __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if ((seen & ~mask) == tag) {
            // A start that lies long before this wave's own is not this launch's: a launch replayed from a HIP graph
            // carries the sequence number it was captured with and finds the start of the replay before.
            const uint64_t start = NearClock(mine, seen & mask);
            if (start + kEpochFreshTicks >= mine) {
                return start;
            }
        }
        __builtin_amdgcn_s_sleep(4);
    }
    return 0;
}

// Period (ticks of the constant-rate clock) in which `bytes` of HBM traffic, read + written, pass at windowMBps
// MB/s; 0 when the clock rate is unknown or the result is out of range.
inline uint32_t WindowPeriodTicks(uint64_t bytes, uint32_t windowMBps)
{
    int dev = 0;
    int khz = 0;
    if (windowMBps == 0 || hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess || khz <= 0) {
        return 0;
    }
    // bytes / (MB/s) = microseconds; ticks = microseconds * kHz / 1000
    const uint64_t ticks = bytes * static_cast<uint64_t>(khz) / (static_cast<uint64_t>(windowMBps) * 1000u);
    return ticks < 16 || ticks > 1000000 ? 0 : static_cast<uint32_t>(ticks);
}

// Waves of a windowed launch of nchunk chunks, at most maxWaves: the chunks are shared out evenly over the fewest
// periods that many waves need, so that the last period is as full as the others (the period is cut for the
// waves there are; 18.2 periods' worth of chunks on maxWaves waves would pay for 19).
inline uint32_t WindowGrid(uint32_t nchunk, uint32_t maxWaves)
{
    if (nchunk <= maxWaves) {
        return nchunk;
    }
    const uint32_t periods = (nchunk + maxWaves - 1) / maxWaves;
    return (nchunk + periods - 1) / periods;
}

// Sequence number of a windowed launch: the 24 bits the kernels compare are never 0, which is what an untouched slot holds.
inline uint32_t NextWindowSeq()
{
    static std::atomic<uint32_t> launches{0};
    uint32_t seq;
    do {
        seq = launches.fetch_add(1, std::memory_order_relaxed) + 1;
    } while ((seq & 0xFFFFFFu) == 0);
    return seq;
}

}  // namespace
}  // namespace mf

#endif  // MF_WINDOW_CLOCK_H
