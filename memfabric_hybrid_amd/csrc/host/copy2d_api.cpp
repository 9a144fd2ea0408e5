// Native C entry point of the batched strided 2-D copy (declared in
// include/mf_hip_dataplane.h).  Rectangles whose addresses, pitches and width
// are all multiples of 16 go to the 2-D kernel; anything else is expanded into
// one segment per row and takes the ordinary batch path.
#include <vector>

#include "../../../include/mf_hip_dataplane_internal.h"
#include "../../../include/mf_xcopy_types.h"
#include "../kernels/copy2d_plan.h"
#include "../rt/mf_rt.h"
#include "mf_log.h"
#include "xcopy_engine.h"

using namespace mf;

#define MF_EXPORT extern "C" __attribute__((visibility("default")))

namespace {

bool Aligned16(const mf_copy2d_desc &d)
{
    return RectFitsPlan(d.src, d.dst, d.width, d.height, d.spitch, d.dpitch);
}

}  // namespace

MF_EXPORT void mf_copy2d_describe(uint64_t width, uint32_t *rowsPerChunk, uint32_t *magic)
{
    *rowsPerChunk = RectRowsPerChunk(width);
    *magic = RectMagic(static_cast<uint32_t>(width / 16));
}

MF_EXPORT uint32_t mf_copy2d_rowcol_mismatches(uint32_t widthUnits, uint32_t rowsPerChunk, uint32_t magic, uint32_t unitsInChunk)
{
    uint32_t bad = 0;
    for (uint32_t u = 0; u < unitsInChunk; ++u) {
        uint32_t row = 0;
        uint32_t col = 0;
        RectRowCol(u, widthUnits, rowsPerChunk, magic, row, col);
        bad += (row != u / widthUnits || col != u % widthUnits) ? 1u : 0u;
    }
    return bad;
}

MF_EXPORT int32_t mf_xcopy_2d_batch(const mf_copy2d_desc *descs, uint32_t n, int32_t route, void *stream)
{
    if ((n != 0 && descs == nullptr) || route < 0 || route > MF_ROUTE_FROM_HOST) {
        MF_FAIL(BM_INVALID_PARAM, "mf_xcopy_2d_batch: null descriptors or unknown route");
    }
    XcopyEngine &engine = XcopyEngine::Instance();
    if (!engine.Started()) {
        MF_FAIL(BM_NOT_INITIALIZED, "GPU data plane is not running; call hybm_init first");
    }
    if (mfrt_bind_thread() != 0) {
        MF_FAIL(BM_ERROR, "cannot make the GPU current on this thread");
    }
    if (stream == nullptr) {
        stream = engine.ThreadStream();
    }
    engine.NoteQueued(stream, ~0ull);   // a wait behind these kernels sleeps on the stream
    for (uint32_t i = 0; i < n; ++i) {
        if (descs[i].width > descs[i].spitch && descs[i].height > 1) {
            MF_FAIL(BM_INVALID_PARAM, "rectangle " << i << ": width exceeds the source pitch");
        }
        if (descs[i].width > descs[i].dpitch && descs[i].height > 1) {
            MF_FAIL(BM_INVALID_PARAM, "rectangle " << i << ": width exceeds the destination pitch");
        }
    }
    const uint32_t cu = mfrt_cu_count() == 0 ? 256 : mfrt_cu_count();
    std::vector<uint64_t> rs;
    std::vector<uint64_t> rd;
    std::vector<uint64_t> rl;
    RectPlan plan;
    uint32_t used = 0;
    uint64_t run = 0;
    // the same launch in the chunks of the windowed form (RectWindowChunks), which a launch of kWindowRectMinBytes and
    // more between device addresses takes where the segment path would
    uint32_t firstWindowed[kRectInline];
    uint64_t runWindowed = 0;
    uint64_t bytes = 0;
    bool allWindowable = true;
    auto flush = [&]() -> int {
        if (used == 0) {
            return 0;
        }
        const bool windowed = allWindowable && runWindowed < 0xFFFFFFFFull && engine.WindowsApply(bytes, route);
        for (uint32_t i = used; i < kRectInline; ++i) {
            plan.src[i] = plan.dst[i] = 0;
            plan.spitchUnits[i] = plan.dpitchUnits[i] = plan.widthUnits[i] = plan.height[i] = 0;
            plan.rowsPerChunk[i] = 1;
            plan.magic[i] = 0;
            plan.first[i] = 0xFFFFFFFFu;
            plan.mate[i] = 0;
        }
        int err;
        if (windowed) {
            for (uint32_t i = 0; i < used; ++i) {
                plan.first[i] = firstWindowed[i];
            }
            plan.nchunk = static_cast<uint32_t>(runWindowed);
            err = mfk_copy2d_windowed(&plan, engine.Tuning().windowMBps, stream);
        } else {
            plan.nchunk = static_cast<uint32_t>(run);
            const uint32_t perCu = engine.Tuning().wgPerCu;   // 0: one workgroup per row group
            const uint64_t cap = perCu == 0 ? run : static_cast<uint64_t>(cu) * perCu;
            err = mfk_copy2d(&plan, static_cast<uint32_t>(run < cap ? run : cap), stream);
        }
        used = 0;
        run = 0;
        runWindowed = 0;
        bytes = 0;
        allWindowable = true;
        return err;
    };
    for (uint32_t i = 0; i < n; ++i) {
        const mf_copy2d_desc &d = descs[i];
        if (d.width == 0 || d.height == 0) {
            continue;
        }
        if (!Aligned16(d)) {
            for (uint64_t r = 0; r < d.height; ++r) {
                rs.push_back(d.src + r * d.spitch);
                rd.push_back(d.dst + r * d.dpitch);
                rl.push_back(d.width);
            }
            continue;
        }
        const uint32_t wu = static_cast<uint32_t>(d.width / 16);
        const uint32_t rpc = RectRowsPerChunk(d.width);
        const uint64_t chunks = (d.height + rpc - 1) / rpc;
        if (run + chunks >= 0xFFFFFFFFull || used == kRectInline) {
            int err = flush();
            if (err != 0) {
                MF_FAIL(BM_ERROR, "2-D copy launch failed: " << mfrt_error_string(err));
            }
        }
        plan.src[used] = d.src;
        plan.dst[used] = d.dst;
        plan.spitchUnits[used] = static_cast<uint32_t>(d.spitch / 16);
        plan.dpitchUnits[used] = static_cast<uint32_t>(d.dpitch / 16);
        plan.widthUnits[used] = wu;
        plan.height[used] = static_cast<uint32_t>(d.height);
        plan.rowsPerChunk[used] = rpc;
        plan.magic[used] = RectMagic(wu);
        plan.first[used] = static_cast<uint32_t>(run);
        plan.mate[used] = 0;
        const uint64_t windowChunks = RectWindowChunks(wu, d.height);
        firstWindowed[used] = static_cast<uint32_t>(runWindowed < 0xFFFFFFFFull ? runWindowed : 0xFFFFFFFFull);
        allWindowable = allWindowable && windowChunks != 0;
        runWindowed += windowChunks;
        bytes += d.width * d.height;
        if (used > 0 && plan.mate[used - 1] == 0 &&
            RectsSideBySide(plan.dst[used - 1], d.dst, static_cast<uint64_t>(plan.widthUnits[used - 1]) * 16, d.width,
                            plan.height[used - 1], d.height, static_cast<uint64_t>(plan.dpitchUnits[used - 1]) * 16, d.dpitch)) {
            plan.mate[used - 1] = 1;
            plan.mate[used] = 2;
        }
        run += chunks;
        ++used;
    }
    int err = flush();
    if (err != 0) {
        MF_FAIL(BM_ERROR, "2-D copy launch failed: " << mfrt_error_string(err));
    }
    if (!rs.empty()) {
        return engine.Submit(rs.data(), rd.data(), rl.data(), static_cast<uint32_t>(rs.size()), route, stream, nullptr, 0);
    }
    return BM_OK;
}
