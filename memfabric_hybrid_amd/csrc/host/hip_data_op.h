// The MI355X copy engine behind the DataOperator contract: every direction of
// a copy or batch becomes one fused xcopy kernel launch on a HIP stream.
// It takes the place HostDataOpSDMA holds in the reference
// (src/hybm/csrc/data_operation/host/hybm_data_op_sdma.cpp:83-169,597-656).
#ifndef MF_HIP_DATA_OP_H
#define MF_HIP_DATA_OP_H

#include <atomic>

#ifdef MF_WITH_REFERENCE_HEADERS
#include "hybm_data_operator.h"   // the reference's own contract, from its include path
#else
#include "data_operator.h"
#endif

namespace mf {

class HipDataOp : public ock::mf::DataOperator {
public:
    using Result = ock::mf::Result;
    using ExtOptions = ock::mf::ExtOptions;

    Result Initialize() noexcept override;
    void UnInitialize() noexcept override;
    Result DataCopy(hybm_copy_params &params, hybm_data_copy_direction direction,
                    const ExtOptions &options) noexcept override;
    Result BatchDataCopy(hybm_batch_copy_params &params, hybm_data_copy_direction direction,
                         const ExtOptions &options) noexcept override;
    Result DataCopyAsync(hybm_copy_params &params, hybm_data_copy_direction direction,
                         const ExtOptions &options) noexcept override;
    Result Wait(int32_t waitId) noexcept override;
    void CleanUp() noexcept override;

private:
    Result Run(void *const *src, void *const *dst, const uint64_t *len, uint32_t n, hybm_data_copy_direction direction,
               const ExtOptions &options, bool async) noexcept;
    std::atomic<bool> inited_{false};   // operators are shared by all calling threads
};

}  // namespace mf

#endif  // MF_HIP_DATA_OP_H
