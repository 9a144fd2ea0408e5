// Native C entry points of the local MoE dispatch / combine (declared in
// include/mf_hip_dataplane.h).
#include "../../../include/mf_hip_dataplane_internal.h"
#include "../../../include/mf_xcopy_types.h"
#include "../rt/mf_rt.h"
#include "mf_log.h"
#include "xcopy_engine.h"

using namespace mf;

#define MF_EXPORT extern "C" __attribute__((visibility("default")))

namespace {

int Prepare(void *&stream)
{
    XcopyEngine &engine = XcopyEngine::Instance();
    if (!engine.Started()) {
        MF_FAIL(BM_NOT_INITIALIZED, "GPU data plane is not running; call hybm_init first");
    }
    if (mfrt_bind_thread() != 0) {
        MF_FAIL(BM_ERROR, "cannot make the GPU current on this thread");
    }
    if (stream == nullptr) {
        stream = engine.ThreadStream();
        if (stream == nullptr) {
            MF_FAIL(BM_ERROR, "cannot create the thread's stream");
        }
    }
    engine.NoteQueued(stream, ~0ull);   // a wait behind these kernels sleeps on the stream
    return BM_OK;
}

}  // namespace

MF_EXPORT uint64_t mf_moe_workspace_bytes(uint32_t tokens, uint32_t topK, uint32_t experts)
{
    return mfk_moe_workspace_bytes(tokens, topK, experts);
}

MF_EXPORT int32_t mf_moe_dispatch(const void *x, const int32_t *topk, uint32_t tokens, uint32_t hidden, uint32_t topK,
                                  uint32_t experts, void *out, int32_t *counts, int32_t *offsets, int32_t *rowOf,
                                  int32_t *srcOf, void *workspace, uint64_t workspaceBytes, void *stream)
{
    if (topk == nullptr || counts == nullptr || offsets == nullptr || rowOf == nullptr || workspace == nullptr ||
        tokens == 0 || topK == 0 || experts == 0 || (x == nullptr) != (out == nullptr)) {
        MF_FAIL(BM_INVALID_PARAM, "mf_moe_dispatch: null argument or empty problem");
    }
    if (topK > 16 || experts > 512 || (out != nullptr && (hidden == 0 || hidden % 8 != 0))) {
        MF_FAIL(BM_INVALID_PARAM, "mf_moe_dispatch: needs topK <= 16, experts <= 512 and hidden a multiple of 8, got "
                                      << topK << ", " << experts << ", " << hidden);
    }
    if ((reinterpret_cast<uint64_t>(x) | reinterpret_cast<uint64_t>(out)) % 16 != 0) {
        MF_FAIL(BM_INVALID_PARAM, "mf_moe_dispatch: token buffers must be 16-byte aligned");
    }
    if (reinterpret_cast<uint64_t>(workspace) % 16 != 0) {
        MF_FAIL(BM_INVALID_PARAM, "mf_moe_dispatch: workspace must be 16-byte aligned");
    }
    if (workspaceBytes < mfk_moe_workspace_bytes(tokens, topK, experts)) {
        MF_FAIL(BM_INVALID_PARAM, "mf_moe_dispatch: workspace of " << workspaceBytes << " bytes is too small");
    }
    int ret = Prepare(stream);
    if (ret != BM_OK) {
        return ret;
    }
    int err = mfk_moe_dispatch(x, topk, tokens, hidden, topK, experts, out, counts, offsets, rowOf, srcOf, workspace,
                               stream);
    if (err != 0) {
        MF_FAIL(BM_ERROR, "mf_moe_dispatch: launch failed: " << (err > 0 ? mfrt_error_string(err) : "bad shape"));
    }
    return BM_OK;
}

MF_EXPORT int32_t mf_moe_combine(const void *rows, const int32_t *rowOf, const float *weights, uint32_t tokens,
                                 uint32_t hidden, uint32_t topK, void *y, void *stream)
{
    if (rows == nullptr || rowOf == nullptr || weights == nullptr || y == nullptr || tokens == 0 || topK == 0) {
        MF_FAIL(BM_INVALID_PARAM, "mf_moe_combine: null argument or empty problem");
    }
    if (topK > 16 || hidden == 0 || hidden % 8 != 0) {
        MF_FAIL(BM_INVALID_PARAM, "mf_moe_combine: needs topK <= 16 and hidden a multiple of 8");
    }
    if ((reinterpret_cast<uint64_t>(rows) | reinterpret_cast<uint64_t>(y)) % 16 != 0) {
        MF_FAIL(BM_INVALID_PARAM, "mf_moe_combine: row buffers must be 16-byte aligned");
    }
    int ret = Prepare(stream);
    if (ret != BM_OK) {
        return ret;
    }
    // A kernel that paces itself for the whole chip's rate is the wrong one while other threads submit work of their
    // own (beside a stream of 1 GiB copies the paced combine took 555 us, the other form 400 us), as for the copies.
    const int paced = XcopyEngine::Instance().SingleSubmitter() ? 1 : 0;
    int err = mfk_moe_combine(rows, rowOf, weights, tokens, hidden, topK, y, stream, paced);
    if (err != 0) {
        MF_FAIL(BM_ERROR, "mf_moe_combine: launch failed: " << (err > 0 ? mfrt_error_string(err) : "bad shape"));
    }
    return BM_OK;
}

MF_EXPORT int32_t mf_moe_combine_windows(uint32_t readMBps, uint32_t writeMBps)
{
    const bool off = readMBps == 0 && writeMBps == 0;
    const bool inRange = readMBps >= 1000000u && readMBps <= 16000000u && writeMBps >= 1000000u && writeMBps <= 16000000u;
    if (!off && !inRange) {
        MF_FAIL(BM_INVALID_PARAM, "mf_moe_combine_windows: rates are 0, 0 (off) or 1000000 ... 16000000 MB/s, got "
                                      << readMBps << ", " << writeMBps);
    }
    mfk_moe_combine_windows(readMBps, writeMBps);
    return BM_OK;
}

MF_EXPORT int32_t mf_moe_xcd_streams(void)
{
    return mfk_moe_xcd_streams();
}
