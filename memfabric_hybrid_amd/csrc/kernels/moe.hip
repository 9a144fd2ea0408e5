// Local MoE token dispatch / combine for gfx950.
//
// The reference has no counterpart (its only device code is the copy plugin,
// src/hybm/csrc/copy_extend/hybm_copy_kernel.cpp); the arithmetic these kernels
// are held to is the specification in the test oracle:
//   dispatch  entry i = t*K + k goes to row offsets[e] + #{j < i : topk[j] == e}
//             (a stable counting sort of the flat (t,k) order by expert id)
//   combine   y[t][h] = bf16_rne(fma(w[t][K-1], v[K-1], ... fma(w[t][0], v[0], 0)))
//
// Three launches for dispatch (two when the entries fill at most eight rank blocks), one for combine:
//   MoeHistKernel    per-block expert histograms (wave ballots + LDS); not launched for a few blocks,
//                    which count one another's entries inside the rank kernel
//   MoeRankKernel    cross-block scan, stable rank of every entry -> rowOf/srcOf, counts, offsets,
//                    and for the tile permute the rows of every step of entries in ascending order
//   the permute, one of
//   MoePermuteTileKernel  rows of whole cache lines, enough work: the output walked in runs of
//                    consecutive rows, in 2 KiB tiles, one stream of steps per XCD, token rows
//                    re-read from that XCD's L2 (HBM bound: H*2*(1+K) bytes per token)
//   MoePermuteLoopKernel  other wide rows: waves that walk the tokens, a row read once into
//                    registers and stored to its K destination rows
//   MoePermuteKernel other narrow rows: one workgroup per token
//   MoeCombineKernel one workgroup per token: K rows gathered, fp32 FMA chain in slot
//                    order, one rounding to bf16 (HBM bound: H*2*(K+1) bytes per token)
//   MoeCombineWindowKernel  the same arithmetic for wide rows and many tokens, by waves that
//                    stay for the whole launch and, chip-wide and by the clock, read for
//                    most of a period and write at its end
// Ranks come from ballots and prefix sums, never from atomics on a shared
// cursor (the only atomics add up plain counts), so the permutation is the same on
// every run and equals the CPU sort.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../rt/mf_rt.h"
#include "window_clock.h"

namespace mf {
namespace {

constexpr uint32_t kRankThreads = 256;                 // 4 waves
constexpr uint32_t kRankRounds = 4;                    // entries per lane
constexpr uint32_t kRankBlock = kRankThreads * kRankRounds;  // 1024 entries per workgroup
constexpr uint32_t kRankSlices = kRankBlock / 64;      // 16 wave-sized slices, in entry order
constexpr uint32_t kMaxExperts = 512;
constexpr uint32_t kRowThreads = 256;
constexpr uint32_t kMaxTopK = 16;
constexpr uint32_t kCountingBlocks = 8;                 // launches of up to this many rank blocks need no histogram kernel
constexpr uint32_t kHistPad = 32;                      // rows of the [expert][block] table are padded to this many blocks

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#define MF_GLOBAL __attribute__((address_space(1)))

// Lanes of the wave whose expert id equals mine (among lanes with valid == true).
__device__ __forceinline__ uint64_t PeersOf(uint32_t expert, bool valid, uint32_t bits)
{
    uint64_t peers = __ballot(valid);
    for (uint32_t b = 0; b < bits; ++b) {
        const bool bit = (expert >> b) & 1u;
        const uint64_t vote = __ballot(bit);
        peers &= bit ? vote : ~vote;
    }
    return peers;
}

__device__ __forceinline__ uint32_t BitsFor(uint32_t experts)
{
    return 32u - __builtin_clz(experts > 1 ? experts - 1 : 1u);
}

// Slice s of a block holds entries [block*1024 + s*64, +64), lane = offset in the slice.
// Wave w of the workgroup handles slices w, w+4, w+8, w+12.
// hist[s][e] = number of entries of slice s routed to expert e.
__device__ __forceinline__ void SliceHistograms(const int32_t *__restrict__ topk, uint32_t total, uint32_t experts,
                                                uint32_t blockBase, uint32_t *hist /* [kRankSlices][experts] in LDS */,
                                                uint32_t *myExpert, uint32_t *myRank, uint32_t *bad)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t bits = BitsFor(experts);
    // all expert ids of this lane are requested before anything waits on them
    int32_t ids[kRankRounds];
#pragma unroll
    for (uint32_t r = 0; r < kRankRounds; ++r) {
        const uint32_t idx = blockBase + (wave + r * (kRankThreads / 64)) * 64 + lane;
        ids[r] = idx < total ? topk[idx] : -1;
    }
    for (uint32_t i = threadIdx.x; i < kRankSlices * experts; i += kRankThreads) {
        hist[i] = 0;
    }
    __syncthreads();
#pragma unroll
    for (uint32_t r = 0; r < kRankRounds; ++r) {
        const uint32_t slice = wave + r * (kRankThreads / 64);
        const uint32_t idx = blockBase + slice * 64 + lane;
        const int32_t e = ids[r];
        const bool valid = e >= 0 && static_cast<uint32_t>(e) < experts;
        if (idx < total && !valid) {
            *bad = 1;
        }
        const uint64_t peers = PeersOf(static_cast<uint32_t>(e), valid, bits);
        const uint64_t below = peers & ((1ull << lane) - 1ull);
        myExpert[r] = valid ? static_cast<uint32_t>(e) : 0xFFFFFFFFu;
        myRank[r] = __popcll(below);
        if (valid && below == 0) {  // first lane of each group publishes the group's size
            hist[slice * experts + static_cast<uint32_t>(e)] = __popcll(peers);
        }
    }
    __syncthreads();
}

__global__ __launch_bounds__(kRankThreads) void MoeHistKernel(const int32_t *__restrict__ topk, uint32_t total,
                                                              uint32_t experts, uint32_t *__restrict__ blockHist,
                                                              uint32_t histStride, uint32_t *__restrict__ blockBad)
{
    extern __shared__ uint32_t hist[];
    uint32_t e[kRankRounds];
    uint32_t r[kRankRounds];
    uint32_t bad = 0;
    SliceHistograms(topk, total, experts, blockIdx.x * kRankBlock, hist, e, r, &bad);
    for (uint32_t x = threadIdx.x; x < experts; x += kRankThreads) {
        uint32_t sum = 0;
        for (uint32_t s = 0; s < kRankSlices; ++s) {
            sum += hist[s * experts + x];
        }
        blockHist[static_cast<uint64_t>(x) * histStride + blockIdx.x] = sum;  // [expert][block], rows padded to kHistPad
        if (blockIdx.x == 0) {
            for (uint32_t pad = gridDim.x; pad < histStride; ++pad) {
                blockHist[static_cast<uint64_t>(x) * histStride + pad] = 0;
            }
        }
    }
    // every block reports, so the flags need no clearing between calls
    const uint32_t anyBad = __syncthreads_or(static_cast<int>(bad)) != 0 ? 1u : 0u;
    if (threadIdx.x == 0) {
        blockBad[blockIdx.x] = anyBad;
    }
}

__global__ __launch_bounds__(kRankThreads) void MoeRankKernel(const int32_t *__restrict__ topk, uint32_t total,
                                                              uint32_t experts, const uint32_t *__restrict__ blockHist,
                                                              uint32_t histStride, int32_t *__restrict__ counts, int32_t *__restrict__ offsets,
                                                              int32_t *__restrict__ rowOf, int32_t *__restrict__ srcOf,
                                                              const uint32_t *__restrict__ blockBad,
                                                              uint32_t *__restrict__ status, uint32_t topK,
                                                              int2 *__restrict__ runOrder, uint32_t stepSlices)
{
    extern __shared__ uint32_t lds[];
    uint32_t *hist = lds;                                 // [kRankSlices][experts]
    uint32_t *base = lds + kRankSlices * experts;         // [experts] first row of this block's entries per expert
    uint32_t *scan = base + experts;                      // [kRankThreads] scratch of the block scan
    uint32_t *stepValid = scan + kRankThreads;            // [kRankSlices] entries with a row in each step of the block
    uint32_t *cum = stepValid + kRankSlices;              // [steps][experts] entries of the step with a smaller expert id
    uint32_t myExpert[kRankRounds];
    uint32_t myRank[kRankRounds];
    uint32_t bad = 0;
    // blockHist == nullptr: no histogram kernel ran before this launch.  A single block has all it needs in its own
    // slice histograms and its own flag (a dispatch of up to 1024 entries: 128 tokens at top-8).  The blocks of a
    // launch of a few count the entries of the other blocks themselves, each for itself: per expert, the entries of
    // all other blocks and those of the blocks before it (plain counts, so LDS atomics give the same result every time).
    const bool tabled = blockHist != nullptr;
    const bool counting = !tabled && gridDim.x > 1;
    const uint32_t steps = runOrder != nullptr ? kRankSlices / stepSlices : 0;
    uint32_t *others = cum + steps * experts;             // [2][experts], counting only
    for (uint32_t i = threadIdx.x; counting && i < 2 * experts; i += kRankThreads) {
        others[i] = 0;
    }
    SliceHistograms(topk, total, experts, blockIdx.x * kRankBlock, hist, myExpert, myRank, &bad);
    if (counting) {
        const uint32_t blockBase = blockIdx.x * kRankBlock;
        for (uint32_t start = 0; start < total; start += kRankBlock) {
            if (start == blockBase) {
                continue;
            }
            int32_t id[kRankRounds];
#pragma unroll
            for (uint32_t q = 0; q < kRankRounds; ++q) {
                const uint32_t idx = start + q * kRankThreads + threadIdx.x;
                id[q] = idx < total ? topk[idx] : 0;
            }
#pragma unroll
            for (uint32_t q = 0; q < kRankRounds; ++q) {
                const uint32_t idx = start + q * kRankThreads + threadIdx.x;
                if (idx < total) {
                    if (id[q] >= 0 && static_cast<uint32_t>(id[q]) < experts) {
                        atomicAdd(&others[id[q]], 1u);
                        if (start < blockBase) {
                            atomicAdd(&others[experts + id[q]], 1u);
                        }
                    } else {
                        bad = 1;
                    }
                }
            }
        }
        __syncthreads();
    }
    if (blockIdx.x == 0) {
        uint32_t any = tabled ? 0 : bad;
        for (uint32_t blk = threadIdx.x; tabled && blk < gridDim.x; blk += kRankThreads) {
            any |= blockBad[blk];
        }
        any = __syncthreads_or(static_cast<int>(any)) != 0 ? 1u : 0u;
        if (threadIdx.x == 0) {
            status[0] = any;  // 1: some expert id was outside [0, experts); those entries got row -1
        }
    }
    // totals and "entries of earlier blocks" per expert
    uint32_t tot[kMaxExperts / kRankThreads];
    uint32_t before[kMaxExperts / kRankThreads];
    uint32_t mine = 0;
#pragma unroll
    for (uint32_t j = 0; j < kMaxExperts / kRankThreads; ++j) {
        // thread t owns the contiguous experts t*per .. t*per+per-1 so that a scan over threads is a scan over experts
        tot[j] = 0;
        before[j] = 0;
    }
    const uint32_t per = (experts + kRankThreads - 1) / kRankThreads;  // 1 or 2
    for (uint32_t j = 0; j < per; ++j) {
        const uint32_t x = threadIdx.x * per + j;
        if (x < experts) {
            // one contiguous row of the [expert][block] table per expert, fetched 16 bytes at a time
            const uint32_t *rowHist = blockHist + static_cast<uint64_t>(x) * histStride;
            uint32_t t = 0;
            uint32_t b = 0;
            for (uint32_t sl = 0; !tabled && sl < kRankSlices; ++sl) {
                t += hist[sl * experts + x];
            }
            if (counting) {
                t += others[x];
                b = others[experts + x];
            }
            // kHistPad blocks per step, all their loads requested before the first is used (with one load per step the
            // loop waited a round trip per four blocks)
            for (uint32_t blk = 0; tabled && blk < gridDim.x; blk += kHistPad) {
                u32x4 v[kHistPad / 4];
#pragma unroll
                for (uint32_t q = 0; q < kHistPad / 4; ++q) {
                    v[q] = *reinterpret_cast<const u32x4 *>(rowHist + blk + 4 * q);  // rows are padded with zeros up to histStride
                }
#pragma unroll
                for (uint32_t q = 0; q < kHistPad / 4; ++q) {
#pragma unroll
                    for (uint32_t i = 0; i < 4; ++i) {
                        t += v[q][i];
                        b += blk + 4 * q + i < blockIdx.x ? v[q][i] : 0u;
                    }
                }
            }
            tot[j] = t;
            before[j] = b;
            mine += t;
        }
    }
    // exclusive scan of `mine` over the 256 threads: shuffles inside each wave, LDS across the four waves
    uint32_t incl = mine;
#pragma unroll
    for (uint32_t step = 1; step < 64; step <<= 1) {
        const uint32_t up = __shfl_up(incl, step, 64);
        incl += (threadIdx.x & 63u) >= step ? up : 0u;
    }
    if ((threadIdx.x & 63u) == 63u) {
        scan[threadIdx.x >> 6] = incl;
    }
    __syncthreads();
    uint32_t waveBase = 0;
    for (uint32_t wv = 0; wv < (threadIdx.x >> 6); ++wv) {
        waveBase += scan[wv];
    }
    incl += waveBase;
    uint32_t run = incl - mine;
    for (uint32_t j = 0; j < per; ++j) {
        const uint32_t x = threadIdx.x * per + j;
        if (x < experts) {
            if (blockIdx.x == 0) {
                counts[x] = static_cast<int32_t>(tot[j]);
                offsets[x] = static_cast<int32_t>(run);
            }
            base[x] = run + before[j];
            run += tot[j];
        }
    }
    __syncthreads();
    // Turn slice histograms into exclusive prefixes over the slices of this block.  For the run-ordered list the
    // block is cut into steps of stepSlices slices (the tile permute works through one step at a time); the
    // entries per (step, expert) are what the prefix gains over a step.
    for (uint32_t x = threadIdx.x; x < experts; x += kRankThreads) {
        uint32_t acc = base[x];
        uint32_t stepStart = acc;
        for (uint32_t s = 0; s < kRankSlices; ++s) {
            const uint32_t v = hist[s * experts + x];
            hist[s * experts + x] = acc;
            acc += v;
            if (steps != 0 && (s + 1) % stepSlices == 0) {
                cum[(s / stepSlices) * experts + x] = acc - stepStart;
                stepStart = acc;
            }
        }
    }
    __syncthreads();
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    if (steps != 0) {
        // cum[j][x]: entries of step j routed to an expert below x, i.e. where the rows of expert x start in the list
        // of the step's rows in ascending order.  One wave per step; a lane scans experts/64 neighbours itself.
        const uint32_t perLane = (experts + 63) / 64;     // at most kMaxExperts / 64
        for (uint32_t j = wave; j < steps; j += kRankThreads / 64) {
            uint32_t mineOf[kMaxExperts / 64];
            uint32_t sum = 0;
#pragma unroll
            for (uint32_t i = 0; i < kMaxExperts / 64; ++i) {
                const uint32_t x = lane * perLane + i;
                mineOf[i] = i < perLane && x < experts ? cum[j * experts + x] : 0u;
                sum += mineOf[i];
            }
            uint32_t incl2 = sum;
#pragma unroll
            for (uint32_t step = 1; step < 64; step <<= 1) {
                const uint32_t up = __shfl_up(incl2, step, 64);
                incl2 += lane >= step ? up : 0u;
            }
            uint32_t at = incl2 - sum;
#pragma unroll
            for (uint32_t i = 0; i < kMaxExperts / 64; ++i) {
                const uint32_t x = lane * perLane + i;
                if (i < perLane && x < experts) {
                    cum[j * experts + x] = at;
                    at += mineOf[i];
                }
            }
            if (lane == 63) {
                stepValid[j] = incl2;
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (uint32_t r = 0; r < kRankRounds; ++r) {
        const uint32_t slice = wave + r * (kRankThreads / 64);
        const uint32_t idx = blockIdx.x * kRankBlock + slice * 64 + lane;
        if (idx < total) {
            int32_t row = -1;
            if (myExpert[r] != 0xFFFFFFFFu) {
                row = static_cast<int32_t>(hist[slice * experts + myExpert[r]] + myRank[r]);
                if (srcOf != nullptr) {
                    srcOf[row] = static_cast<int32_t>(idx);
                }
                if (runOrder != nullptr) {
                    const uint32_t j = slice / stepSlices;
                    const uint32_t firstOfStep = hist[j * stepSlices * experts + myExpert[r]];
                    const uint32_t at = cum[j * experts + myExpert[r]] + (static_cast<uint32_t>(row) - firstOfStep);
                    runOrder[static_cast<uint64_t>(blockIdx.x) * kRankBlock + j * stepSlices * 64 + at] =
                        make_int2(row, static_cast<int32_t>(idx / topK));
                }
            }
            rowOf[idx] = row;
        }
    }
    if (runOrder != nullptr) {
        // slots past a step's valid entries (ids out of range, the tail of the last block) name no row
        const uint32_t stepEntries = stepSlices * 64;
        for (uint32_t slot = threadIdx.x; slot < kRankBlock; slot += kRankThreads) {
            const uint32_t j = slot / stepEntries;
            if (slot - j * stepEntries >= stepValid[j]) {
                runOrder[static_cast<uint64_t>(blockIdx.x) * kRankBlock + slot] = make_int2(-1, 0);
            }
        }
    }
}

template <int kMode>
__device__ __forceinline__ void RowStore(MF_GLOBAL u32x4 *p, u32x4 v)
{
    if (kMode == 2) {
        asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt" : : "v"(p), "v"(v) : "memory");
    } else if (kMode == 1) {
        __builtin_nontemporal_store(v, p);
    } else {
        *p = v;
    }
}

// One workgroup per token.  unitsPerRow = H*2/16.  Each lane keeps up to kHold 128-bit pieces of
// the token's row in registers and stores them to the token's K destination rows.
template <uint32_t kThreads, uint32_t kHold, int kMode>
__global__ __launch_bounds__(kThreads) void MoePermuteKernel(const u32x4 *__restrict__ x,
                                                             const int32_t *__restrict__ rowOf, uint32_t topK,
                                                             uint32_t unitsPerRow, uint32_t parts, u32x4 *__restrict__ out)
{
    const uint32_t token = blockIdx.x / parts;
    const uint32_t part = blockIdx.x - token * parts;
    const uint32_t perPart = (unitsPerRow + parts - 1) / parts;
    const uint32_t begin = part * perPart;
    const uint32_t end = begin + perPart < unitsPerRow ? begin + perPart : unitsPerRow;
    const MF_GLOBAL u32x4 *src = reinterpret_cast<const MF_GLOBAL u32x4 *>(reinterpret_cast<uint64_t>(x)) +
                                 static_cast<uint64_t>(token) * unitsPerRow;
    int32_t rows[kMaxTopK];
#pragma unroll
    for (uint32_t k = 0; k < kMaxTopK; ++k) {
        rows[k] = k < topK ? rowOf[static_cast<uint64_t>(token) * topK + k] : -1;
    }
    for (uint32_t u0 = begin; u0 < end; u0 += kHold * kThreads) {
        u32x4 v[kHold];
#pragma unroll
        for (uint32_t j = 0; j < kHold; ++j) {
            const uint32_t u = u0 + j * kThreads + threadIdx.x;
            if (u < end) {
                v[j] = __builtin_nontemporal_load(src + u);
            }
        }
#pragma unroll
        for (uint32_t k = 0; k < kMaxTopK; ++k) {
            if (k < topK && rows[k] >= 0) {
                MF_GLOBAL u32x4 *dst = reinterpret_cast<MF_GLOBAL u32x4 *>(reinterpret_cast<uint64_t>(out)) +
                                       static_cast<uint64_t>(rows[k]) * unitsPerRow;
#pragma unroll
                for (uint32_t j = 0; j < kHold; ++j) {
                    const uint32_t u = u0 + j * kThreads + threadIdx.x;
                    if (u < end) {
                        RowStore<kMode>(dst + u, v[j]);
                    }
                }
            }
        }
    }
}

// Single-wave workgroups that walk items (token, part) with stride gridDim.x and fetch the next
// item's pieces before they store the current one's: after the first item of every wave, reads of
// x overlap the eight-fold stores instead of preceding them.
template <uint32_t kHold>
__global__ __launch_bounds__(64) void MoePermuteLoopKernel(const u32x4 *__restrict__ x, const int32_t *__restrict__ rowOf,
                                                           uint32_t topK, uint32_t unitsPerRow, uint32_t parts,
                                                           uint32_t items, u32x4 *__restrict__ out)
{
    const uint32_t perPart = (unitsPerRow + parts - 1) / parts;
    const MF_GLOBAL u32x4 *xg = reinterpret_cast<const MF_GLOBAL u32x4 *>(reinterpret_cast<uint64_t>(x));
    MF_GLOBAL u32x4 *og = reinterpret_cast<MF_GLOBAL u32x4 *>(reinterpret_cast<uint64_t>(out));
    auto fetch = [&](uint32_t item, u32x4(&v)[kHold], int32_t(&rows)[kMaxTopK]) {
        const uint32_t token = item / parts;
        const uint32_t begin = (item - token * parts) * perPart;
        const uint32_t end = begin + perPart < unitsPerRow ? begin + perPart : unitsPerRow;
#pragma unroll
        for (uint32_t k = 0; k < kMaxTopK; ++k) {
            rows[k] = k < topK ? rowOf[static_cast<uint64_t>(token) * topK + k] : -1;
        }
#pragma unroll
        for (uint32_t j = 0; j < kHold; ++j) {
            const uint32_t u = begin + j * 64 + threadIdx.x;
            if (u < end) {
                v[j] = __builtin_nontemporal_load(xg + static_cast<uint64_t>(token) * unitsPerRow + u);
            }
        }
    };
    auto spread = [&](uint32_t item, const u32x4(&v)[kHold], const int32_t(&rows)[kMaxTopK]) {
        const uint32_t token = item / parts;
        const uint32_t begin = (item - token * parts) * perPart;
        const uint32_t end = begin + perPart < unitsPerRow ? begin + perPart : unitsPerRow;
#pragma unroll
        for (uint32_t k = 0; k < kMaxTopK; ++k) {
            if (k < topK && rows[k] >= 0) {
                MF_GLOBAL u32x4 *dst = og + static_cast<uint64_t>(rows[k]) * unitsPerRow;
#pragma unroll
                for (uint32_t j = 0; j < kHold; ++j) {
                    const uint32_t u = begin + j * 64 + threadIdx.x;
                    if (u < end) {
                        dst[u] = v[j];
                    }
                }
            }
        }
    };
    // two register sets, a and b, alternate between "being fetched" and "being stored"
    uint32_t ia = blockIdx.x;
    if (ia >= items) {
        return;
    }
    u32x4 a[kHold];
    u32x4 b[kHold];
    int32_t ra[kMaxTopK];
    int32_t rb[kMaxTopK];
    fetch(ia, a, ra);
    while (true) {
        const uint32_t ib = ia + gridDim.x;
        const bool hasB = ib < items;
        if (hasB) {
            fetch(ib, b, rb);
        }
        spread(ia, a, ra);
        if (!hasB) {
            break;
        }
        ia = ib + gridDim.x;
        const bool hasA = ia < items;
        if (hasA) {
            fetch(ia, a, ra);
        }
        spread(ib, b, rb);
        if (!hasA) {
            break;
        }
    }
}

// The permute of wide rows when a block of kRankBlock entries holds no more of x than an XCD's L2 keeps:
// output-ordered, in tiles.  runOrder lists, step by step (a step is a block of kRankBlock entries or a power-of-two
// part of one, chosen so that the token rows of a step fit), the step's output rows in ascending
// order (runs of consecutive rows per expert) with the token each row is a copy of.  Workgroup i, a single
// wave, belongs to stream i % 8 (the dispatcher deals consecutive workgroups to the eight XCDs in turn);
// stream s takes the steps s, s + 8, ... one after the other and walks a step's rows in list order, a row in
// tiles of 128 units (2 KiB).  So an XCD writes runs of consecutive rows front to back, two stores per wave,
// the store pattern this part takes fastest, and the K reads of a token row all come from the same XCD within
// the time it spends on the block: the first from HBM, the others from its L2 (plain loads), which stores that
// are written through pass without evicting x.  8192 x 7168, top-8, 256 experts: 163-166 us against 192 us for
// the token-ordered loop kernel; streams that do not follow the XCDs 283 us.
constexpr uint32_t kTileUnits = 128;
constexpr uint32_t kTileStreams = 8;

__global__ __launch_bounds__(64) void MoePermuteTileKernel(const u32x4 *__restrict__ x, const int2 *__restrict__ runOrder,
                                                           uint32_t unitsPerRow, uint32_t tilesPerRow, uint32_t steps,
                                                           uint32_t stepEntries, u32x4 *__restrict__ out)
{
    const uint32_t stream = blockIdx.x % kTileStreams;
    const uint32_t q = blockIdx.x / kTileStreams;
    const uint32_t tilesPerStep = stepEntries * tilesPerRow;
    const uint32_t step = (q / tilesPerStep) * kTileStreams + stream;
    const uint32_t within = q % tilesPerStep;
    if (step >= steps) {
        return;
    }
    const int2 rowAndToken = runOrder[static_cast<uint64_t>(step) * stepEntries + within / tilesPerRow];
    if (rowAndToken.x < 0) {
        return;
    }
    const uint32_t begin = (within % tilesPerRow) * kTileUnits;
    const MF_GLOBAL u32x4 *src = reinterpret_cast<const MF_GLOBAL u32x4 *>(reinterpret_cast<uint64_t>(x)) +
                                 static_cast<uint64_t>(rowAndToken.y) * unitsPerRow;
    MF_GLOBAL u32x4 *dst = reinterpret_cast<MF_GLOBAL u32x4 *>(reinterpret_cast<uint64_t>(out)) +
                           static_cast<uint64_t>(rowAndToken.x) * unitsPerRow;
    u32x4 v[kTileUnits / 64];
#pragma unroll
    for (uint32_t j = 0; j < kTileUnits / 64; ++j) {
        const uint32_t u = begin + j * 64 + threadIdx.x;
        if (u < unitsPerRow) {
            v[j] = src[u];
        }
    }
#pragma unroll
    for (uint32_t j = 0; j < kTileUnits / 64; ++j) {
        const uint32_t u = begin + j * 64 + threadIdx.x;
        if (u < unitsPerRow) {
            RowStore<2>(dst + u, v[j]);
        }
    }
}

__device__ __forceinline__ float Bf16Lo(uint32_t w)
{
    return __uint_as_float(w << 16);
}

__device__ __forceinline__ float Bf16Hi(uint32_t w)
{
    return __uint_as_float(w & 0xFFFF0000u);
}

// round to nearest even; NaN stays a quiet NaN
__device__ __forceinline__ uint32_t ToBf16(float f)
{
    const uint32_t w = __float_as_uint(f);
    if ((w & 0x7FFFFFFFu) > 0x7F800000u) {
        return (w >> 16) | 0x0040u;
    }
    return (w + 0x7FFFu + ((w >> 16) & 1u)) >> 16;
}

template <uint32_t kTopK, uint32_t kThreads, bool kNtLoad, uint32_t kBatch = 1>
__global__ __launch_bounds__(kThreads) void MoeCombineKernel(const u32x4 *__restrict__ rowsIn,
                                                             const int32_t *__restrict__ rowOf,
                                                             const float *__restrict__ weights, uint32_t topK,
                                                             uint32_t unitsPerRow, uint32_t parts, u32x4 *__restrict__ y)
{
    const uint32_t token = blockIdx.x / parts;
    const uint32_t part = blockIdx.x - token * parts;
    const uint32_t perPart = (unitsPerRow + parts - 1) / parts;
    const uint32_t begin = part * perPart;
    const uint32_t end = begin + perPart < unitsPerRow ? begin + perPart : unitsPerRow;
    const uint32_t nk = kTopK != 0 ? kTopK : topK;
    constexpr uint32_t kSlots = kTopK != 0 ? kTopK : kMaxTopK;
    uint64_t rowBase[kSlots];
    float w[kSlots];
    // Slots without a row (an expert id that dispatch flagged) are skipped: neither loaded nor
    // multiplied, so whatever lies in row 0 (an infinity, a NaN) cannot reach y through 0 * x.
    // The mask is the same for every lane of the workgroup.
    uint32_t live = 0;
#pragma unroll
    for (uint32_t k = 0; k < kSlots; ++k) {
        if (k < nk) {
            const int32_t row = rowOf[static_cast<uint64_t>(token) * nk + k];
            rowBase[k] = static_cast<uint64_t>(row < 0 ? 0 : row) * unitsPerRow;
            w[k] = weights[static_cast<uint64_t>(token) * nk + k];
            live |= row < 0 ? 0u : 1u << k;
        } else {
            rowBase[k] = 0;
            w[k] = 0.0f;
        }
    }
    const MF_GLOBAL u32x4 *in = reinterpret_cast<const MF_GLOBAL u32x4 *>(reinterpret_cast<uint64_t>(rowsIn));
    MF_GLOBAL u32x4 *dst = reinterpret_cast<MF_GLOBAL u32x4 *>(reinterpret_cast<uint64_t>(y)) +
                           static_cast<uint64_t>(token) * unitsPerRow;
    // kBatch column positions per lane are requested together (kBatch * K loads in flight per lane)
    // before any of them is consumed.
    for (uint32_t u0 = begin + threadIdx.x; u0 < end; u0 += kBatch * kThreads) {
        u32x4 v[kBatch][kSlots];
#pragma unroll
        for (uint32_t b = 0; b < kBatch; ++b) {
            const uint32_t u = u0 + b * kThreads;
#pragma unroll
            for (uint32_t k = 0; k < kSlots; ++k) {
                if (((live >> k) & 1u) != 0 && u < end) {
                    v[b][k] = kNtLoad ? __builtin_nontemporal_load(in + rowBase[k] + u) : in[rowBase[k] + u];
                }
            }
        }
#pragma unroll
        for (uint32_t b = 0; b < kBatch; ++b) {
            const uint32_t u = u0 + b * kThreads;
            if (u >= end) {
                break;
            }
            float acc[8];
#pragma unroll
            for (uint32_t i = 0; i < 8; ++i) {
                acc[i] = 0.0f;
            }
#pragma unroll
            for (uint32_t k = 0; k < kSlots; ++k) {
                if (((live >> k) & 1u) != 0) {
#pragma unroll
                    for (uint32_t i = 0; i < 4; ++i) {
                        acc[2 * i] = __builtin_fmaf(w[k], Bf16Lo(v[b][k][i]), acc[2 * i]);
                        acc[2 * i + 1] = __builtin_fmaf(w[k], Bf16Hi(v[b][k][i]), acc[2 * i + 1]);
                    }
                }
            }
            u32x4 o;
#pragma unroll
            for (uint32_t i = 0; i < 4; ++i) {
                o[i] = ToBf16(acc[2 * i]) | (ToBf16(acc[2 * i + 1]) << 16);
            }
            __builtin_nontemporal_store(o, dst + u);
        }
    }
}

// The combine of wide rows when there are many tokens: gridDim.x single-wave workgroups, all
// resident at once, walk the items (token, 128-unit slice of the row) with stride gridDim.x.
// HBM streams reads at 7.0 TB/s and the combine's mix of eight reads to one write at 6.0, so
// the two are kept apart in time: a period is kItems read parts and one write part.  In read
// part j a wave requests the 16 pieces of its j-th item of the period (eight rows, two column
// positions per lane) at its own offset of the part, reduces them when they have arrived and
// keeps the result, 8 registers per item; in the write part it stores the kItems results at
// its own offset of that part (top-6: six rows, twelve pieces).  The start of the first period is agreed through
// AgreedStart(); after that every wave goes by the constant-rate clock alone.  8192 tokens of 7168
// elements at top-8: 164-168 us against 177-181 us for one workgroup per item; from about six items per
// wave on it is the faster form.  Read parts are paced at 6.8 TB/s, write parts at 6.2 (reads at 7.0
// make the waves fall behind now and then).
// Arithmetic and the rule for slots without a row are MoeCombineKernel's.
constexpr uint32_t kCombineItems = 4;                  // 32 result registers, 116 in all: sixteen waves per CU
constexpr uint32_t kCombineWavesPerCu = 16;
constexpr uint32_t kCombineSliceUnits = 128;           // two column positions per lane
constexpr uint32_t kCombineMinItemsPerWave = 6;

template <uint32_t kItems, uint32_t kSlots>
__global__ __launch_bounds__(64) void MoeCombineWindowKernel(const u32x4 *__restrict__ rowsIn,
                                                             const int32_t *__restrict__ rowOf,
                                                             const float *__restrict__ weights, uint32_t unitsPerRow,
                                                             uint32_t parts, uint32_t items, u32x4 *__restrict__ y,
                                                             uint32_t readTicks, uint32_t writeTicks, uint32_t seq)
{
    constexpr uint32_t kBatch = kCombineSliceUnits / 64;
    const uint64_t start = AgreedStart(seq);
    const uint32_t period = kItems * readTicks + writeTicks;
    const uint32_t readOffset = static_cast<uint32_t>(static_cast<uint64_t>(blockIdx.x) * readTicks / gridDim.x);
    const uint32_t writeOffset = static_cast<uint32_t>(static_cast<uint64_t>(blockIdx.x) * writeTicks / gridDim.x);
    const uint32_t perPart = (unitsPerRow + parts - 1) / parts;
    const MF_GLOBAL u32x4 *in = reinterpret_cast<const MF_GLOBAL u32x4 *>(reinterpret_cast<uint64_t>(rowsIn));
    MF_GLOBAL u32x4 *out = reinterpret_cast<MF_GLOBAL u32x4 *>(reinterpret_cast<uint64_t>(y));
    uint64_t t0 = start;
    for (uint32_t base = 0; base < items; base += kItems * gridDim.x, t0 += period) {
        if (base + blockIdx.x >= items) {
            break;                                     // nothing left for this wave
        }
        // The last period holds as many read parts as it has items per wave, and its last read part lasts as long
        // as the waves that still have an item need to request it (both the same for every wave).
        const uint32_t remaining = items - base;
        const uint32_t left = (remaining + gridDim.x - 1) / gridDim.x;
        const uint32_t readParts = left < kItems ? left : kItems;
        const uint32_t inLastPart = remaining - (readParts - 1) * gridDim.x;       // >= 1
        const uint32_t lastPartTicks = inLastPart >= gridDim.x ? readTicks
            : static_cast<uint32_t>(static_cast<uint64_t>(inLastPart) * readTicks / gridDim.x);
        const uint32_t readEnd = (readParts - 1) * readTicks + lastPartTicks;
        u32x4 o[kItems][kBatch];
#pragma unroll
        for (uint32_t j = 0; j < kItems; ++j) {
            const uint32_t item = base + j * gridDim.x + blockIdx.x;
            if (j < readParts && item < items) {
                const uint32_t token = item / parts;
                const uint32_t begin = (item - token * parts) * perPart;
                const uint32_t end = begin + perPart < unitsPerRow ? begin + perPart : unitsPerRow;
                // No branch on a slot without a row (rowOf < 0): its pieces are read from the token's own row
                // of y, which is memory this launch owns, masked to zero and multiplied by -0.0f, and
                // fma(-0.0f, 0.0f, acc) is acc for every acc, so the slot contributes nothing, as if skipped.
                const MF_GLOBAL u32x4 *rowPtr[kSlots];
                float w[kSlots];
                uint32_t keep[kSlots];
#pragma unroll
                for (uint32_t k = 0; k < kSlots; ++k) {
                    const int32_t row = rowOf[static_cast<uint64_t>(token) * kSlots + k];
                    const float weight = weights[static_cast<uint64_t>(token) * kSlots + k];
                    rowPtr[k] = row < 0 ? out + static_cast<uint64_t>(token) * unitsPerRow
                                        : in + static_cast<uint64_t>(row) * unitsPerRow;
                    w[k] = row < 0 ? -0.0f : weight;
                    keep[k] = row < 0 ? 0u : 0xFFFFFFFFu;
                }
                WaitForClock(t0 + j * readTicks + readOffset);
                u32x4 v[kBatch][kSlots];
#pragma unroll
                for (uint32_t b = 0; b < kBatch; ++b) {
                    const uint32_t u = begin + b * 64 + threadIdx.x;
                    if (u < end) {
#pragma unroll
                        for (uint32_t k = 0; k < kSlots; ++k) {
                            v[b][k] = __builtin_nontemporal_load(rowPtr[k] + u);
                        }
                    }
                }
#pragma unroll
                for (uint32_t b = 0; b < kBatch; ++b) {
                    float acc[8];
#pragma unroll
                    for (uint32_t i = 0; i < 8; ++i) {
                        acc[i] = 0.0f;
                    }
#pragma unroll
                    for (uint32_t k = 0; k < kSlots; ++k) {
#pragma unroll
                        for (uint32_t i = 0; i < 4; ++i) {
                            const uint32_t word = v[b][k][i] & keep[k];
                            acc[2 * i] = __builtin_fmaf(w[k], Bf16Lo(word), acc[2 * i]);
                            acc[2 * i + 1] = __builtin_fmaf(w[k], Bf16Hi(word), acc[2 * i + 1]);
                        }
                    }
#pragma unroll
                    for (uint32_t i = 0; i < 4; ++i) {
                        o[j][b][i] = ToBf16(acc[2 * i]) | (ToBf16(acc[2 * i + 1]) << 16);
                    }
                }
            }
        }
        WaitForClock(t0 + readEnd + writeOffset);
#pragma unroll
        for (uint32_t j = 0; j < kItems; ++j) {
            const uint32_t item = base + j * gridDim.x + blockIdx.x;
            if (j < readParts && item < items) {
                const uint32_t token = item / parts;
                const uint32_t begin = (item - token * parts) * perPart;
                const uint32_t end = begin + perPart < unitsPerRow ? begin + perPart : unitsPerRow;
#pragma unroll
                for (uint32_t b = 0; b < kBatch; ++b) {
                    const uint32_t u = begin + b * 64 + threadIdx.x;
                    if (u < end) {
                        __builtin_nontemporal_store(o[j][b], out + static_cast<uint64_t>(token) * unitsPerRow + u);
                    }
                }
            }
        }
    }
}

// Which XCD a wave runs on (XCC_ID, hardware register 20, bits 3:0), for mfk_moe_setup().
__global__ void XcdProbeKernel(uint32_t *__restrict__ ids)
{
    if (threadIdx.x == 0) {
        ids[blockIdx.x] = static_cast<uint32_t>(__builtin_amdgcn_s_getreg((3 << 11) | 20)) & 0xFu;
    }
}

// 1 once mfk_moe_setup() has seen consecutive workgroups go to kTileStreams different XCDs in turn, which is what the
// streams of MoePermuteTileKernel stand on; 0 (the loop kernel is used) before that and where the GPU deals them
// otherwise (a partition of one XCD, for instance).
std::atomic<int> g_xcdStreams{0};

// Pace of the windowed combine, MB/s of HBM traffic in the read parts and in the write parts; 0 = never windowed.
std::atomic<uint32_t> g_combineReadMBps{6800000};
std::atomic<uint32_t> g_combineWriteMBps{6200000};

}  // namespace
}  // namespace mf

extern "C" uint64_t mfk_moe_workspace_bytes(uint32_t tokens, uint32_t topK, uint32_t experts)
{
    const uint64_t total = static_cast<uint64_t>(tokens) * topK;
    const uint64_t blocks = (total + mf::kRankBlock - 1) / mf::kRankBlock;
    const uint64_t stride = (blocks + mf::kHistPad - 1) / mf::kHistPad * mf::kHistPad;
    // status words, per-block flags, the [expert][block] histogram, the run-ordered row list (8 bytes per entry slot)
    const uint64_t tables = 256 + stride * sizeof(uint32_t) + stride * experts * sizeof(uint32_t);
    return (tables + 15) / 16 * 16 + blocks * mf::kRankBlock * sizeof(int2);
}

extern "C" int mfk_moe_dispatch(const void *x, const void *topk, uint32_t tokens, uint32_t hidden, uint32_t topK,
                                uint32_t experts, void *out, void *counts, void *offsets, void *rowOf, void *srcOf,
                                void *workspace, void *stream)
{
    using namespace mf;
    const uint64_t total64 = static_cast<uint64_t>(tokens) * topK;
    if (total64 == 0 || total64 > 0x7FFFFFFFull || experts == 0 || experts > kMaxExperts || topK > kMaxTopK ||
        (static_cast<uint64_t>(hidden) * 2) % 16 != 0) {
        return -1;
    }
    const uint32_t total = static_cast<uint32_t>(total64);
    const uint32_t blocks = (total + kRankBlock - 1) / kRankBlock;
    hipStream_t s = static_cast<hipStream_t>(stream);
    uint32_t *status = static_cast<uint32_t *>(workspace);
    const uint32_t histStride = (blocks + kHistPad - 1) / kHistPad * kHistPad;   // rows of the [expert][block] table
    uint32_t *blockBad = status + 64;
    uint32_t *blockHist = blockBad + histStride;
    const size_t histLds = static_cast<size_t>(kRankSlices) * experts * sizeof(uint32_t);
    const uint32_t upr = hidden / 8;
    // The output-ordered tile permute needs the token rows of one step (a block of kRankBlock entries, or a half, a
    // quarter ... down to one slice of 64 entries: stepEntries / topK tokens) to stay in an XCD's 4 MiB L2 while the
    // step's rows are written, and enough steps for the eight streams.  It wins on every shape of whole cache lines
    // that was measured (8192 tokens, top-8, 256 experts, 7168 elements: 174 against 208 us with the loop kernel;
    // 1024 elements: 44 against 49 us with one workgroup per token).  Rows that are not whole cache lines
    // (10 000 elements) lose, whatever the step: every tile then begins and ends inside a line; they keep the loop kernel.
    uint32_t stepSlices = kRankSlices;
    while (stepSlices > 1 && static_cast<uint64_t>(stepSlices * 64 / topK + 1) * hidden * 2 > 2200000ull) {
        stepSlices /= 2;
    }
    // a small call is cut finer, so that every XCD gets steps to work on (256 / 512 tokens of 7168 elements at top-8:
    // 24 / 28 us per dispatch, 34 / 35 us with the loop kernel, whose single wave per token writes its 112 KiB alone)
    while (stepSlices > 1 && static_cast<uint64_t>(blocks) * (kRankSlices / stepSlices) < 2 * kTileStreams) {
        stepSlices /= 2;
    }
    const uint32_t stepEntries = stepSlices * 64;
    const uint32_t stepsPerBlock = kRankSlices / stepSlices;
    const uint64_t steps = static_cast<uint64_t>(blocks) * stepsPerBlock;
    const uint32_t tilesPerRow = (upr + kTileUnits - 1) / kTileUnits;
    const uint64_t tileGrid = (steps + kTileStreams - 1) / kTileStreams * kTileStreams * stepEntries * tilesPerRow;
    const bool tiles = g_xcdStreams.load(std::memory_order_relaxed) != 0 && x != nullptr && out != nullptr && upr >= kTileUnits &&
                       hidden % 64 == 0 && static_cast<uint64_t>(stepEntries / topK + 1) * hidden * 2 <= 2200000ull &&
                       stepsPerBlock * experts <= 4096 && tileGrid <= 0x7FFFFFFFull;
    // Up to kCountingBlocks blocks rank without a histogram launch in front of them: every block counts the entries
    // of the others itself.  129 / 256 / 512 / 1024 tokens of 7168 elements at top-8, 256 experts: 13.3 / 15.5 / 20.1 /
    // 29.5 us per dispatch against 22.0 / 24.1 / 27.7 / 35.1 with the launch; 640 tokens over 512 experts 26 against 38.
    // At sixteen blocks the two are level (50.5 us), at thirty-two the counting costs 10 us; over 8 or 16 experts,
    // where the counts of a wave land on few LDS words, eight blocks are level (23.9 against 23.4 us) and sixteen
    // lose 4 us.
    const bool counting = blocks > 1 && blocks <= kCountingBlocks;
    const size_t rankLds = histLds + (experts + kRankThreads + kRankSlices + (tiles ? stepsPerBlock * experts : 0) +
                                      (counting ? 2 * experts : 0)) * sizeof(uint32_t);
    const uint64_t tableBytes = 256 + histStride * sizeof(uint32_t) + static_cast<uint64_t>(histStride) * experts * sizeof(uint32_t);
    int2 *runOrder = tiles ? reinterpret_cast<int2 *>(static_cast<char *>(workspace) + (tableBytes + 15) / 16 * 16) : nullptr;
    if (blocks == 1 || counting) {
        blockHist = nullptr;   // one block ranks from its own histograms: no launch in front of it (16 / 64 / 128 tokens of
                               // 7168 elements at top-8: 12 / 12.5 / 14 us per dispatch; 22 / 23 / 24 us before, with the
                               // histogram launch and the token-ordered permute); a few blocks count for themselves
    } else {
        hipLaunchKernelGGL(MoeHistKernel, dim3(blocks), dim3(kRankThreads), histLds, s, static_cast<const int32_t *>(topk),
                           total, experts, blockHist, histStride, blockBad);
    }
    hipLaunchKernelGGL(MoeRankKernel, dim3(blocks), dim3(kRankThreads), rankLds, s, static_cast<const int32_t *>(topk),
                       total, experts, blockHist, histStride, static_cast<int32_t *>(counts), static_cast<int32_t *>(offsets),
                       static_cast<int32_t *>(rowOf), static_cast<int32_t *>(srcOf), blockBad, status, topK, runOrder, stepSlices);
    if (x != nullptr && out != nullptr && hidden != 0) {
        const u32x4 *xi = static_cast<const u32x4 *>(x);
        const int32_t *ro = static_cast<const int32_t *>(rowOf);
        u32x4 *oo = static_cast<u32x4 *>(out);
        if (tiles) {
            hipLaunchKernelGGL(MoePermuteTileKernel, dim3(static_cast<uint32_t>(tileGrid)), dim3(64), 0, s, xi, runOrder, upr,
                               tilesPerRow, static_cast<uint32_t>(steps), stepEntries, oo);
        } else if (upr >= 512) {
            // Wide rows: single-wave workgroups that hold up to 14 pieces per lane (a whole 7168-element
            // row) and write them with plain stores; sixteen waves per CU that each take several tokens and
            // fetch the next row while they store the current one (207 us for 8192 x 7168 at top-8; staging in
            // LDS, two waves per row, nontemporal stores and the destination-side form were all slower).
            // 123 vector registers per lane: four waves per SIMD, sixteen per CU, all resident at once
            const uint32_t wideParts = (upr + 64 * 14 - 1) / (64 * 14);
            const uint32_t items = tokens * wideParts;
            const uint32_t waves = static_cast<uint32_t>(mfrt_cu_count() > 0 ? mfrt_cu_count() : 256) * 16u;
            hipLaunchKernelGGL((MoePermuteLoopKernel<14>), dim3(items < waves ? items : waves), dim3(64), 0, s, xi, ro, topK, upr,
                               wideParts, items, oo);
        } else {
            // Narrow rows: one four-wave workgroup per token.
            hipLaunchKernelGGL((MoePermuteKernel<256, 4, 1>), dim3(tokens), dim3(256), 0, s, xi, ro, topK, upr, 1u, oo);
        }
    }
    return static_cast<int>(hipGetLastError());
}

extern "C" int mfk_moe_combine(const void *rows, const void *rowOf, const void *weights, uint32_t tokens,
                               uint32_t hidden, uint32_t topK, void *y, void *stream, int paced)
{
    using namespace mf;
    if (tokens == 0 || topK == 0 || topK > kMaxTopK || hidden == 0 || (static_cast<uint64_t>(hidden) * 2) % 16 != 0) {
        return -1;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const u32x4 *in = static_cast<const u32x4 *>(rows);
    const int32_t *ro = static_cast<const int32_t *>(rowOf);
    const float *w = static_cast<const float *>(weights);
    u32x4 *o = static_cast<u32x4 *>(y);
    const uint32_t upr = hidden / 8;
    if (upr >= 256 && (topK == 2 || topK == 4 || topK == 6 || topK == 8)) {
        // Wide rows: single-wave workgroups, each on a 128-unit slice of the row with two column positions per
        // lane in flight (2 x topK loads), the fastest shape measured on 7168-element rows at top-8 (178 us; one
        // four-wave workgroup per token 188 us; plain instead of nontemporal loads 194 us).  Compiled for the common
        // fan-ins, so that all of a lane's loads are in flight together: top-2 16 384 x 4096 65 against 74 us,
        // top-4 8192 x 7168 96 against 106 us, top-6 139 against 152 us (against the kernel that walks a run-time
        // number of slots).
        const uint32_t parts = (upr + kCombineSliceUnits - 1) / kCombineSliceUnits;
        const uint32_t perPart = (upr + parts - 1) / parts;
        const uint64_t items = static_cast<uint64_t>(tokens) * parts;
        const uint32_t waves = static_cast<uint32_t>(mfrt_cu_count() > 0 ? mfrt_cu_count() : 256) * kCombineWavesPerCu;
        // From six items per wave on, waves that stay and keep reads and writes apart in time; below that the
        // first read part and the last write part, in which the chip only reads or only writes for want of
        // work, cost what the separation gains (top-8, 16 800 items on 4096 waves: 51.4 against 50.5 us; 19 200: the
        // same; 25 200: 74.4 against 76.7 us).
        const uint32_t readTicks = WindowPeriodTicks(static_cast<uint64_t>(waves) * topK * perPart * 16,
                                                     g_combineReadMBps.load(std::memory_order_relaxed));
        const uint32_t writeTicks = WindowPeriodTicks(static_cast<uint64_t>(waves) * kCombineItems * perPart * 16,
                                                      g_combineWriteMBps.load(std::memory_order_relaxed));
        // Top-6 gains as top-8 does (8192 x 7168: 131-133 against 138-140 us); top-4 gains nothing (98 against 97 us)
        // and top-2 loses (16 384 x 4096: 79 against 66 us): their read parts are too short for the switch to pay.
        const bool windows = paced != 0 && topK >= 6 && items >= static_cast<uint64_t>(waves) * kCombineMinItemsPerWave &&
                             items < 0x40000000ull && readTicks != 0 && writeTicks != 0;
        const dim3 grid(windows ? waves : tokens * parts);
#define MF_COMBINE_SLICES(K)                                                                                           \
    hipLaunchKernelGGL((MoeCombineKernel<K, 64, true, 2>), grid, dim3(64), 0, s, in, ro, w, topK, upr, parts, o)
#define MF_COMBINE_WINDOWS(K)                                                                                          \
    hipLaunchKernelGGL((MoeCombineWindowKernel<kCombineItems, K>), grid, dim3(64), 0, s, in, ro, w, upr, parts,        \
                       static_cast<uint32_t>(items), o, readTicks, writeTicks, NextWindowSeq())
        if (topK == 2) {
            MF_COMBINE_SLICES(2);
        } else if (topK == 4) {
            MF_COMBINE_SLICES(4);
        } else if (topK == 6) {
            if (windows) {
                MF_COMBINE_WINDOWS(6);
            } else {
                MF_COMBINE_SLICES(6);
            }
        } else if (windows) {
            MF_COMBINE_WINDOWS(8);
        } else {
            MF_COMBINE_SLICES(8);
        }
#undef MF_COMBINE_SLICES
#undef MF_COMBINE_WINDOWS
    } else if (topK == 8) {
        hipLaunchKernelGGL((MoeCombineKernel<8, 256, true>), dim3(tokens), dim3(256), 0, s, in, ro, w, topK, upr, 1u, o);
    } else {
        hipLaunchKernelGGL((MoeCombineKernel<0, 256, true>), dim3(tokens), dim3(256), 0, s, in, ro, w, topK, upr, 1u, o);
    }
    return static_cast<int>(hipGetLastError());
}

extern "C" void mfk_moe_combine_windows(uint32_t readMBps, uint32_t writeMBps)
{
    mf::g_combineReadMBps.store(readMBps, std::memory_order_relaxed);
    mf::g_combineWriteMBps.store(writeMBps, std::memory_order_relaxed);
}

// Once per process, after the GPU has been bound and outside any stream capture (it waits for a small kernel):
// checks that workgroup i of a launch runs on XCD i mod 8.
extern "C" int mfk_moe_setup(void)
{
    constexpr uint32_t kProbe = 256;
    uint32_t *dev = nullptr;
    hipError_t err = hipMalloc(reinterpret_cast<void **>(&dev), kProbe * sizeof(uint32_t));
    if (err != hipSuccess) {
        return static_cast<int>(err);
    }
    uint32_t ids[kProbe];
    hipLaunchKernelGGL(mf::XcdProbeKernel, dim3(kProbe), dim3(64), 0, nullptr, dev);
    err = hipMemcpy(ids, dev, sizeof(ids), hipMemcpyDeviceToHost);
    (void)hipFree(dev);
    if (err != hipSuccess) {
        return static_cast<int>(err);
    }
    bool inTurn = true;
    for (uint32_t i = 0; i < kProbe; ++i) {
        inTurn = inTurn && ids[i] == ids[i % mf::kTileStreams];
    }
    for (uint32_t a = 0; a < mf::kTileStreams; ++a) {
        for (uint32_t b = a + 1; b < mf::kTileStreams; ++b) {
            inTurn = inTurn && ids[a] != ids[b];
        }
    }
    mf::g_xcdStreams.store(inTurn ? 1 : 0, std::memory_order_relaxed);
    return 0;
}

extern "C" int mfk_moe_xcd_streams(void)
{
    return mf::g_xcdStreams.load(std::memory_order_relaxed);
}
