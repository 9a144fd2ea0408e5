#include "hip_data_op.h"
#include "host_copy.h"

#include <cstring>
#include <vector>

#include "../../../include/mf_hip_dataplane.h"
#include "../rt/mf_rt.h"
#include "copy_direction.h"
#include "mf_log.h"
#include "xcopy_engine.h"

namespace mf {
namespace {

constexpr uint32_t kRounds = 16;                       // slots of the staging ring
constexpr uint64_t kRoundBytes = 2ull << 20;           // bytes per slot: ~70 us of CPU memcpy against ~40 us on the link
constexpr uint64_t kBounceBytes = kRounds * kRoundBytes;
constexpr uint32_t kAhead = 2;                        // launches queued beyond the slot being emptied (device to pageable memory)
static_assert(kRounds <= XcopyEngine::kBounceEvents, "one event per staging slot");

// Caller memory the GPU cannot address (ordinary pageable host memory) goes through a pinned
// staging area.  The reference allocates and frees a device buffer per segment for these
// directions (src/hybm/csrc/data_operation/host/hybm_data_op_sdma.cpp:171-221); here one pinned
// area per thread, owned by the engine, is filled by the CPU and scattered by one launch.

struct Piece {
    uint64_t src;
    uint64_t dst;
    uint64_t len;
};

bool AnyPageable(void *const *ptrs, uint32_t n)
{
    for (uint32_t i = 0; i < n; ++i) {
        if (mfrt_pointer_kind(ptrs[i]) == MFRT_PTR_PAGEABLE) {
            return true;
        }
    }
    return false;
}

int RouteOf(bool srcOnHost, bool dstOnHost)
{
    if (dstOnHost) {
        return MFRT_ROUTE_TO_HOST;
    }
    return srcOnHost ? MFRT_ROUTE_FROM_HOST : MFRT_ROUTE_HBM;
}

}  // namespace

HipDataOp::Result HipDataOp::Initialize() noexcept
{
    if (inited_) {
        return BM_OK;
    }
    if (!XcopyEngine::Instance().Started()) {
        MF_FAIL(BM_NOT_INITIALIZED, "GPU copy engine is not running; call hybm_init first");
    }
    inited_ = true;
    return BM_OK;
}

void HipDataOp::UnInitialize() noexcept
{
    inited_ = false;
}

HipDataOp::Result HipDataOp::Wait(int32_t) noexcept
{
    if (!inited_) {
        return BM_NOT_INITIALIZED;
    }
    return XcopyEngine::Instance().DrainThread();
}

void HipDataOp::CleanUp() noexcept
{
    (void)XcopyEngine::Instance().DrainThread();
    XcopyEngine::Instance().QuiesceSubmitters();   // batches of other threads that a submit thread has not launched yet
}

HipDataOp::Result HipDataOp::DataCopy(hybm_copy_params &params, hybm_data_copy_direction direction,
                                      const ExtOptions &options) noexcept
{
    void *src = params.src;
    void *dst = params.dest;
    uint64_t len = params.dataSize;
    return Run(&src, &dst, &len, 1, direction, options, (options.flags & ASYNC_COPY_FLAG) != 0);
}

HipDataOp::Result HipDataOp::DataCopyAsync(hybm_copy_params &params, hybm_data_copy_direction direction,
                                           const ExtOptions &options) noexcept
{
    void *src = params.src;
    void *dst = params.dest;
    uint64_t len = params.dataSize;
    return Run(&src, &dst, &len, 1, direction, options, true);
}

HipDataOp::Result HipDataOp::BatchDataCopy(hybm_batch_copy_params &params, hybm_data_copy_direction direction,
                                           const ExtOptions &options) noexcept
{
    return Run(params.sources, params.destinations, params.dataSizes, params.batchSize, direction, options,
               (options.flags & ASYNC_COPY_FLAG) != 0);
}

HipDataOp::Result HipDataOp::Run(void *const *src, void *const *dst, const uint64_t *len, uint32_t n,
                                 hybm_data_copy_direction direction, const ExtOptions &options, bool async) noexcept
{
    if (!inited_) {
        return BM_NOT_INITIALIZED;
    }
    if (!DirectionValid(direction)) {
        MF_FAIL(BM_INVALID_PARAM, "copy direction " << direction << " is not executable");
    }
    XcopyEngine &engine = XcopyEngine::Instance();
    const Endpoint se = SourceOf(direction);
    const Endpoint de = DestinationOf(direction);
    const bool srcOnHost = !se.device;
    const bool dstOnHost = !de.device;
    // Only caller-private host memory can be invisible to the GPU; pool memory is pinned by construction.
    const bool srcPageable = !se.pool && srcOnHost && AnyPageable(src, n);
    const bool dstPageable = !de.pool && dstOnHost && AnyPageable(dst, n);
    const bool unordered = async && (options.flags & MF_COPY_UNORDERED_FLAG) != 0;
    void *stream = options.stream;
    if (stream == nullptr && !(unordered && !srcPageable && !dstPageable)) {
        // (an unordered copy without a stream of the caller's leaves the choice to the engine, which may deal it to a side stream)
        stream = engine.ThreadStream();
        if (stream == nullptr) {
            MF_FAIL(BM_ERROR, "no stream available for the copy");
        }
    }

    if (!srcPageable && !dstPageable) {
        static_assert(sizeof(void *) == sizeof(uint64_t), "64-bit addresses expected");
        int ret = engine.Submit(reinterpret_cast<const uint64_t *>(src), reinterpret_cast<const uint64_t *>(dst), len, n,
                                RouteOf(srcOnHost, dstOnHost), stream, nullptr, 0, unordered);
        if (ret != BM_OK) {
            return ret;
        }
        if (!async) {
            uint64_t bytes = 0;
            if (n <= 4096) {   // a long table is not worth adding up: such a batch waits on the stream
                for (uint32_t i = 0; i < n; ++i) {
                    bytes += len[i];
                }
            }
            return engine.WaitStream(stream, bytes);
        }
        return BM_OK;
    }

    // Host DRAM to host DRAM with a pageable side: both buffers are only a CPU
    // store away from each other, no accelerator is involved.
    if (srcOnHost && dstOnHost) {
        int err = mfrt_stream_sync(stream);  // keep order with copies queued earlier
        if (err != 0) {
            MF_FAIL(BM_ERROR, "stream wait failed: " << mfrt_error_string(err));
        }
        // Elements whose own source and destination overlap are moved in place; the rest is shared
        // with the helper thread, one element at a time (elements may depend on one another only
        // if the caller broke the rule that destinations overlap nothing else in the batch).
        for (uint32_t i = 0; i < n; ++i) {
            const uint64_t s = reinterpret_cast<uint64_t>(src[i]);
            const uint64_t d = reinterpret_cast<uint64_t>(dst[i]);
            if (s < d + len[i] && d < s + len[i]) {
                std::memmove(dst[i], src[i], len[i]);
            } else {
                HostCopyHelper::Instance().Copy(dst[i], src[i], len[i]);
            }
        }
        return BM_OK;
    }

    uint8_t *bounce = static_cast<uint8_t *>(engine.ThreadBounce(kBounceBytes));
    if (bounce == nullptr) {
        MF_FAIL(BM_MALLOC_FAILED, "pinned staging allocation failed");
    }
    // The staging area is a ring of kRounds slots.  The CPU side (memcpy between caller memory and
    // a slot) and the GPU side (one fused launch per slot) overlap: towards the GPU the CPU fills
    // slot r+1 while the launch of slot r runs, away from it the CPU empties slot r-1 while the
    // launch that fills slot r runs.  An event per slot says when its launch has finished.
    // 512 KiB rounds were tried for small batches: slower (more launches).  Large transfers take
    // slots of twice the size: the launch and the event of a round cost the host about 10 us.
    uint64_t totalBytes = 0;
    for (uint32_t i = 0; i < n; ++i) {
        totalBytes += len[i];
    }
    const uint64_t roundBytes = totalBytes >= (64ull << 20) ? 2 * kRoundBytes : kRoundBytes;
    const uint32_t ringSlots = static_cast<uint32_t>(kBounceBytes / roundBytes);
    std::vector<Piece> pieces;
    pieces.reserve(n);
    for (uint32_t i = 0; i < n; ++i) {
        uint64_t s = reinterpret_cast<uint64_t>(src[i]);
        uint64_t d = reinterpret_cast<uint64_t>(dst[i]);
        uint64_t left = len[i];
        while (left > 0) {
            const uint64_t take = left > roundBytes ? roundBytes : left;
            pieces.push_back(Piece{s, d, take});
            s += take;
            d += take;
            left -= take;
        }
    }
    HostCopyHelper &copier = HostCopyHelper::Instance();   // large pieces are copied by two cores
    struct Round {
        size_t begin = 0;
        size_t end = 0;
        std::vector<uint64_t> staged;   // slot address of every piece of the round
    };
    Round rounds[kRounds];
    std::vector<uint64_t> a;
    std::vector<uint64_t> b;
    std::vector<uint64_t> l;
    std::vector<HostCopyHelper::Task> tasks;   // the CPU copies of one round
    auto drain = [&](Round &round, uint32_t slot) -> int {   // GPU -> caller: wait for the slot's launch, empty it
        if (round.begin == round.end) {
            return BM_OK;
        }
        int err = mfrt_event_sync(engine.ThreadBounceEvent(slot));
        if (err != 0) {
            MF_FAIL(BM_ERROR, "copy failed on the GPU: " << mfrt_error_string(err));
        }
        tasks.clear();
        for (size_t i = round.begin; i < round.end; ++i) {
            tasks.push_back(HostCopyHelper::Task{reinterpret_cast<void *>(pieces[i].dst),
                                                 reinterpret_cast<const void *>(round.staged[i - round.begin]), pieces[i].len});
        }
        copier.CopySet(tasks.data(), tasks.size());
        round.begin = round.end = 0;
        return BM_OK;
    };
    const int route = srcPageable ? MFRT_ROUTE_FROM_HOST : MFRT_ROUTE_TO_HOST;
    size_t at = 0;
    uint32_t r = 0;
    for (; at < pieces.size(); ++r) {
        const uint32_t slot = r % ringSlots;
        Round &round = rounds[slot];
        void *event = engine.ThreadBounceEvent(slot);
        if (event == nullptr) {
            MF_FAIL(BM_ERROR, "event creation failed");
        }
        if (r >= ringSlots) {   // the slot's previous launch must be over before the slot is reused
            if (dstPageable) {
                int ret = drain(round, slot);
                if (ret != BM_OK) {
                    return ret;
                }
            } else {
                int err = mfrt_event_sync(event);
                if (err != 0) {
                    MF_FAIL(BM_ERROR, "copy failed on the GPU: " << mfrt_error_string(err));
                }
            }
        }
        a.clear();
        b.clear();
        l.clear();
        tasks.clear();
        round.staged.clear();
        round.begin = at;
        uint64_t used = 0;
        const uint64_t base = reinterpret_cast<uint64_t>(bounce) + static_cast<uint64_t>(slot) * roundBytes;
        while (at < pieces.size()) {
            const uint64_t padded = (pieces[at].len + 63) & ~63ull;  // keep staged pieces 64-byte aligned
            if (used + padded > roundBytes) {
                break;
            }
            const uint64_t where = base + used;
            if (srcPageable) {
                tasks.push_back(HostCopyHelper::Task{reinterpret_cast<void *>(where), reinterpret_cast<const void *>(pieces[at].src),
                                                     pieces[at].len});
                a.push_back(where);
                b.push_back(pieces[at].dst);
            } else {
                a.push_back(pieces[at].src);
                b.push_back(where);
                round.staged.push_back(where);
            }
            l.push_back(pieces[at].len);
            used += padded;
            ++at;
        }
        round.end = at;
        if (srcPageable) {
            copier.CopySet(tasks.data(), tasks.size());
        }
        int ret = engine.Submit(a.data(), b.data(), l.data(), static_cast<uint32_t>(l.size()), route, stream, nullptr, 0);
        if (ret != BM_OK) {
            return ret;
        }
        int err = mfrt_event_record(event, stream);
        if (err != 0) {
            MF_FAIL(BM_ERROR, "event record failed: " << mfrt_error_string(err));
        }
        // Two launches stay queued while an older slot is emptied: with only one, the next launch is
        // submitted just as the running one ends, and any delay leaves the GPU idle.
        if (dstPageable && r >= kAhead) {
            ret = drain(rounds[(r - kAhead) % ringSlots], (r - kAhead) % ringSlots);
            if (ret != BM_OK) {
                return ret;
            }
        }
    }
    if (dstPageable) {
        for (uint32_t k = 0; k < ringSlots; ++k) {   // what is still staged, oldest first
            const uint32_t slot = (r + k) % ringSlots;
            int ret = drain(rounds[slot], slot);
            if (ret != BM_OK) {
                return ret;
            }
        }
    } else {
        int err = mfrt_stream_sync(stream);   // caller memory has been consumed; the copy itself is done as well
        if (err != 0) {
            MF_FAIL(BM_ERROR, "copy failed on the GPU: " << mfrt_error_string(err));
        }
    }
    return BM_OK;
}

}  // namespace mf
