// Ordered set of copy engines with first-success-wins fallback, the role of
// HostComposeDataOp (src/hybm/csrc/data_operation/host/hybm_compose_data_op.cpp:25-241).
// Order of preference: intra-node engine (the HIP kernels here, SDMA in the
// reference) -> device RDMA -> host RDMA / URMA / TCP.  Only the first exists
// in this build; the others are slots a test or a later transport can fill
// through OperatorFactory.
#ifndef MF_COMPOSE_DATA_OP_H
#define MF_COMPOSE_DATA_OP_H

#include <functional>
#include <utility>
#include <vector>

#include "data_operator.h"

namespace mf {

struct OperatorFactory {
    std::function<ock::mf::DataOperatorPtr()> intraNode;   // HYBM_DOP_TYPE_SDMA slot
    std::function<ock::mf::DataOperatorPtr()> deviceRdma;  // HYBM_DOP_TYPE_DEVICE_RDMA slot
    std::function<ock::mf::DataOperatorPtr()> hostNet;     // HOST_RDMA | HOST_URMA | HOST_TCP slot
    static OperatorFactory Default();
};

class ComposeDataOp : public ock::mf::DataOperator {
public:
    using Result = ock::mf::Result;
    using ExtOptions = ock::mf::ExtOptions;
    // Engines in order of preference; raw pointers, the members below keep them alive.
    struct Ranked {
        std::pair<hybm_data_op_type, ock::mf::DataOperator *> item[5];
        uint32_t count = 0;
        bool empty() const
        {
            return count == 0;
        }
        const std::pair<hybm_data_op_type, ock::mf::DataOperator *> *begin() const
        {
            return item;
        }
        const std::pair<hybm_data_op_type, ock::mf::DataOperator *> *end() const
        {
            return item + count;
        }
        void emplace_back(hybm_data_op_type t, ock::mf::DataOperator *op)
        {
            item[count++] = {t, op};
        }
    };

    ComposeDataOp(const hybm_options &options, OperatorFactory factory);
    ~ComposeDataOp() override;

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
    Ranked Prioritised(const ExtOptions &options) const;

    hybm_options options_;
    OperatorFactory factory_;
    ock::mf::DataOperatorPtr intraNode_;
    ock::mf::DataOperatorPtr deviceRdma_;
    ock::mf::DataOperatorPtr hostNet_;
};

}  // namespace mf

#endif  // MF_COMPOSE_DATA_OP_H
