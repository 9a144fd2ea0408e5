// Copy-direction algebra.  The twelve hybm directions are a product of
// {local, pool} x {host, device} on each side with local->local excluded;
// this header derives them arithmetically instead of by table so that the
// literal tables of the reference
//   directMap            src/smem/csrc/smem_bm/smem_bm_entry.cpp:256-267
//   COPY_DIRECTION_TABLE src/hybm/csrc/mm/hybm_va_manager.h:252-261
//   g_checkMap           src/hybm/csrc/hybm_data_op_entry.cpp:24-30
// (restated verbatim in the test oracle) cross-check it exhaustively.
#ifndef MF_COPY_DIRECTION_H
#define MF_COPY_DIRECTION_H

#include "../../../include/mf_xcopy_types.h"

namespace mf {

struct Endpoint {
    bool pool;    // inside the pooled address space ("G") or caller-private ("L")
    bool device;  // HBM or host DRAM
};

inline hybm_data_copy_direction ComposeDirection(Endpoint src, Endpoint dst)
{
    if (!src.pool && !dst.pool) {
        return HYBM_DATA_COPY_DIRECTION_BUTT;
    }
    if (!src.pool) {
        return static_cast<hybm_data_copy_direction>((src.device ? 2 : 0) + (dst.device ? 1 : 0));
    }
    return static_cast<hybm_data_copy_direction>(4 + (src.device ? 4 : 0) + (dst.pool ? 0 : 2) + (dst.device ? 1 : 0));
}

inline bool DirectionValid(hybm_data_copy_direction d)
{
    return d >= HYBM_LOCAL_HOST_TO_GLOBAL_HOST && d <= HYBM_GLOBAL_DEVICE_TO_LOCAL_DEVICE;
}

inline Endpoint SourceOf(hybm_data_copy_direction d)
{
    const int v = static_cast<int>(d);
    if (v < 4) {
        return Endpoint{false, v >= 2};
    }
    return Endpoint{true, v >= 8};
}

inline Endpoint DestinationOf(hybm_data_copy_direction d)
{
    const int v = static_cast<int>(d);
    if (v < 4) {
        return Endpoint{true, (v & 1) != 0};
    }
    return Endpoint{(v & 2) == 0, (v & 1) != 0};
}

// Which sides must lie inside the entity's windows before a copy is accepted.
inline bool MustCheckSource(hybm_data_copy_direction d)
{
    return DirectionValid(d) && SourceOf(d).pool;
}

inline bool MustCheckDestination(hybm_data_copy_direction d)
{
    return DirectionValid(d) && DestinationOf(d).pool;
}

// smem layer: memory type of each side (as classified against the pool windows,
// SMEM_MEM_TYPE_BUTT when outside both) plus the caller's copy type.
inline hybm_data_copy_direction TranslateSmemCopy(smem_bm_copy_type t, smem_bm_mem_type srcInPool,
                                                  smem_bm_mem_type dstInPool)
{
    smem_bm_mem_type s = srcInPool;
    smem_bm_mem_type d = dstInPool;
    switch (t) {
        case SMEMB_COPY_L2G:
            s = SMEM_MEM_TYPE_LOCAL_DEVICE;
            break;
        case SMEMB_COPY_G2L:
            d = SMEM_MEM_TYPE_LOCAL_DEVICE;
            break;
        case SMEMB_COPY_G2H:
        case SMEMB_COPY_GH2H:
            d = SMEM_MEM_TYPE_LOCAL_HOST;
            break;
        case SMEMB_COPY_H2G:
        case SMEMB_COPY_H2GH:
            s = SMEM_MEM_TYPE_LOCAL_HOST;
            break;
        default:  // L2GH, GH2L, G2G keep what the windows said
            break;
    }
    if (s >= SMEM_MEM_TYPE_BUTT || d >= SMEM_MEM_TYPE_BUTT) {
        return HYBM_DATA_COPY_DIRECTION_BUTT;
    }
    const Endpoint se{s == SMEM_MEM_TYPE_DEVICE || s == SMEM_MEM_TYPE_HOST,
                      s == SMEM_MEM_TYPE_DEVICE || s == SMEM_MEM_TYPE_LOCAL_DEVICE};
    const Endpoint de{d == SMEM_MEM_TYPE_DEVICE || d == SMEM_MEM_TYPE_HOST,
                      d == SMEM_MEM_TYPE_DEVICE || d == SMEM_MEM_TYPE_LOCAL_DEVICE};
    return ComposeDirection(se, de);
}

}  // namespace mf

#endif  // MF_COPY_DIRECTION_H
