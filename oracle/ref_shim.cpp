// TEST INFRASTRUCTURE ONLY.  extern "C" doorway into pieces of the reference
// that compile from their own sources with g++ alone: the address registry
// (src/hybm/csrc/mm/hybm_va_manager.cpp), the host branch of
// DlHybridApi::Memcpy (src/hybm/csrc/under_api/dl_hybrid_api.h:150-169) and the
// loader of the copy plugin (src/hybm/csrc/under_api/dl_hybm_copy_extend.cpp).
// Built by oracle/Makefile into oracle/_ref/libmf_ref.so from the sources
// where they lie; nothing of the reference is copied into this repository.
// Used to validate oracle/mf_oracle.c and as the "reference" CPU baseline.
#include <cstdint>

#include "dl_hybrid_api.h"
#include "hybm_va_manager.h"

using namespace ock::mf;

extern "C" {

void ref_va_clear(void)
{
    HybmVaManager::GetInstance().ClearAll();
}

int32_t ref_va_add(uint64_t gva, uint64_t size, int32_t memType, uint64_t lva, uint32_t localRank)
{
    BaseAllocatedGvaInfo base{gva, size, static_cast<hybm_mem_type>(memType), lva};
    return HybmVaManager::GetInstance().AddVaInfo(base, localRank);
}

int32_t ref_va_add_external(uint64_t gva, uint64_t size, int32_t memType, uint64_t lva, uint32_t localRank,
                            uint32_t importedRank)
{
    BaseAllocatedGvaInfo base{gva, size, static_cast<hybm_mem_type>(memType), lva};
    return HybmVaManager::GetInstance().AddVaInfoFromExternal(base, localRank, importedRank);
}

void ref_va_remove(uint64_t va)
{
    HybmVaManager::GetInstance().RemoveOneVaInfo(va);
}

uint64_t ref_va_gva_of_lva(uint64_t lva)
{
    return HybmVaManager::GetInstance().GetGvaByLva(lva);
}

uint64_t ref_va_lva_of_gva(uint64_t gva)
{
    return HybmVaManager::GetInstance().GetLvaByGva(gva);
}

int32_t ref_va_is_gva(uint64_t va)
{
    return HybmVaManager::GetInstance().IsGva(va) ? 1 : 0;
}

int32_t ref_va_is_known(uint64_t va)
{
    return HybmVaManager::GetInstance().IsValidAddr(va) ? 1 : 0;
}

int32_t ref_va_mem_type(uint64_t va)
{
    return static_cast<int32_t>(HybmVaManager::GetInstance().GetMemType(va));
}

int64_t ref_va_rank(uint64_t gva)
{
    auto r = HybmVaManager::GetInstance().GetRank(gva);
    return r.second ? static_cast<int64_t>(r.first) : -1;
}

int32_t ref_va_infer_direction(uint64_t srcVa, uint64_t dstVa)
{
    return static_cast<int32_t>(HybmVaManager::GetInstance().InferCopyDirection(srcVa, dstVa));
}

uint64_t ref_va_reserve(uint32_t localRank, uint64_t size, int32_t memType)
{
    return HybmVaManager::GetInstance().AllocReserveGva(localRank, size, static_cast<hybm_mem_type>(memType)).start;
}

void ref_va_unreserve(uint64_t start)
{
    HybmVaManager::GetInstance().FreeReserveGva(start);
}

uint64_t ref_va_range_count(void)
{
    return HybmVaManager::GetInstance().GetAllocCount();
}

uint64_t ref_va_reserved_count(void)
{
    return HybmVaManager::GetInstance().GetReservedCount();
}

uint64_t ref_mask48(uint64_t address)
{
    return Valid48BitsAddress(address);
}

int32_t ref_memcpy(void *dst, uint64_t destMax, const void *src, uint64_t count, uint32_t kind)
{
    return DlHybridApi::Memcpy(dst, destMax, src, count, kind);
}

// The loop of HostDataOpRDMA::BatchCopyLH2LH
// (src/hybm/csrc/data_operation/host/hybm_data_op_host_rdma.cpp:697-709) around the reference's Memcpy.
int32_t ref_batch_copy(void *const *dsts, void *const *srcs, const uint64_t *counts, uint32_t batchSize)
{
    for (uint32_t i = 0; i < batchSize; ++i) {
        int32_t ret = DlHybridApi::Memcpy(dsts[i], counts[i], srcs[i], counts[i], ACL_MEMCPY_HOST_TO_HOST);
        if (ret != 0) {
            return ret;
        }
    }
    return 0;
}
}

// The reference's plugin loader as it is (src/hybm/csrc/under_api/dl_hybm_copy_extend.cpp:25-86:
// directory from MEMFABRIC_HYBRID_EXTEND_LIB_PATH, dlopen(RTLD_NOW | RTLD_NODELETE), both symbols
// or unload) and the thunks HostDataOpSDMA calls through (dl_hybm_copy_extend.h:29-51).
#include "dl_hybm_copy_extend.h"

extern "C" {

int32_t ref_extend_try_load(void)
{
    return DlHybmExtendApi::TryLoadLibrary();
}

void ref_extend_cleanup(void)
{
    DlHybmExtendApi::CleanupLibrary();
}

int32_t ref_extend_copy(const void *src, void *dst, uint64_t len, uint32_t concurrent, void *stream)
{
    return DlHybmExtendApi::HybmCopyExtend(src, dst, len, concurrent, stream);
}

int32_t ref_extend_batch_copy(void *param, uint32_t count, void *mask, uint32_t concurrent, void *stream)
{
    return DlHybmExtendApi::HybmBatchCopyExtend(param, count, mask, concurrent, stream);
}
}
