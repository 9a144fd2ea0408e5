#include "compose_data_op.h"

#include "hip_data_op.h"
#include "mf_log.h"

namespace mf {

using ock::mf::DataOperatorPtr;

OperatorFactory OperatorFactory::Default()
{
    OperatorFactory f;
    f.intraNode = []() -> DataOperatorPtr { return std::make_shared<HipDataOp>(); };
    return f;
}

ComposeDataOp::ComposeDataOp(const hybm_options &options, OperatorFactory factory)
    : options_(options), factory_(std::move(factory))
{}

ComposeDataOp::~ComposeDataOp()
{
    ComposeDataOp::UnInitialize();
}

ComposeDataOp::Result ComposeDataOp::Initialize() noexcept
{
    if (options_.bmType == HYBM_TYPE_AI_CORE_INITIATE) {
        return BM_OK;  // device-initiated pools carry no host copy engine
    }
    struct Slot {
        uint32_t bits;
        const std::function<DataOperatorPtr()> *make;
        DataOperatorPtr *into;
        const char *name;
    };
    const Slot slots[] = {
        {HYBM_DOP_TYPE_SDMA, &factory_.intraNode, &intraNode_, "intra-node"},
        {HYBM_DOP_TYPE_DEVICE_RDMA, &factory_.deviceRdma, &deviceRdma_, "device RDMA"},
        {HYBM_DOP_TYPE_HOST_RDMA | HYBM_DOP_TYPE_HOST_URMA | HYBM_DOP_TYPE_HOST_TCP, &factory_.hostNet, &hostNet_,
         "host network"},
    };
    for (const Slot &slot : slots) {
        if ((static_cast<uint32_t>(options_.bmDataOpType) & slot.bits) == 0) {
            continue;
        }
        if (!*slot.make) {
            MF_INFO(slot.name << " copy engine requested but not part of this build; skipped");
            continue;
        }
        DataOperatorPtr op = (*slot.make)();
        Result ret = op != nullptr ? op->Initialize() : BM_NEW_OBJECT_FAILED;
        if (ret != BM_OK) {
            MF_ERROR(slot.name << " copy engine failed to start: " << ret);
            // all-or-nothing: engines started earlier in this call are dropped again
            intraNode_ = nullptr;
            deviceRdma_ = nullptr;
            hostNet_ = nullptr;
            return ret;
        }
        *slot.into = op;
    }
    return BM_OK;
}

void ComposeDataOp::UnInitialize() noexcept
{
    for (DataOperatorPtr *op : {&hostNet_, &deviceRdma_, &intraNode_}) {
        if (*op != nullptr) {
            (*op)->UnInitialize();
            *op = nullptr;
        }
    }
}

ComposeDataOp::Ranked ComposeDataOp::Prioritised(const ExtOptions &) const
{
    // One rank, one node: every engine that exists reaches every address.
    const uint32_t reach = static_cast<uint32_t>(options_.bmDataOpType);
    Ranked out;
    if (intraNode_ != nullptr && (reach & HYBM_DOP_TYPE_SDMA) != 0) {
        out.emplace_back(HYBM_DOP_TYPE_SDMA, intraNode_.get());
    }
    if (deviceRdma_ != nullptr && (reach & HYBM_DOP_TYPE_DEVICE_RDMA) != 0) {
        out.emplace_back(HYBM_DOP_TYPE_DEVICE_RDMA, deviceRdma_.get());
    }
    for (hybm_data_op_type t : {HYBM_DOP_TYPE_HOST_RDMA, HYBM_DOP_TYPE_HOST_URMA, HYBM_DOP_TYPE_HOST_TCP}) {
        if (hostNet_ != nullptr && (reach & t) != 0) {
            out.emplace_back(t, hostNet_.get());
        }
    }
    return out;
}

ComposeDataOp::Result ComposeDataOp::DataCopy(hybm_copy_params &params, hybm_data_copy_direction direction,
                                              const ExtOptions &options) noexcept
{
    Ranked ops = Prioritised(options);
    if (ops.empty()) {
        MF_FAIL(BM_INVALID_PARAM, "no copy engine reaches rank " << options.srcRankId << " -> " << options.destRankId);
    }
    Result result = BM_ERROR;
    for (auto &op : ops) {
        result = op.second->DataCopy(params, direction, options);
        if (result == BM_OK) {
            break;
        }
        MF_WARN("copy engine " << op.first << " failed with " << result << ", trying the next one");
    }
    return result;
}

ComposeDataOp::Result ComposeDataOp::BatchDataCopy(hybm_batch_copy_params &params, hybm_data_copy_direction direction,
                                                   const ExtOptions &options) noexcept
{
    Ranked ops = Prioritised(options);
    if (ops.empty()) {
        MF_FAIL(BM_INVALID_PARAM, "no copy engine available for the batch");
    }
    Result result = BM_ERROR;
    for (auto &op : ops) {
        if (op.first == HYBM_DOP_TYPE_SDMA) {
            // The intra-node engine addresses every rank directly: one call, whole batch.
            result = op.second->BatchDataCopy(params, direction, options);
            if (result == BM_OK) {
                return result;
            }
            MF_WARN("intra-node batch copy failed with " << result << ", trying the next engine");
            continue;
        }
        // Network engines work per (source rank, destination rank) pair.  A
        // caller that did no grouping means "all of it, between the two ranks named".
        decltype(options.groupMap) whole;
        if (options.groupMap.empty()) {
            std::vector<uint32_t> &all = whole[{options.srcRankId, options.destRankId}];
            all.resize(params.batchSize);
            for (uint32_t i = 0; i < params.batchSize; ++i) {
                all[i] = i;
            }
        }
        for (const auto &group : options.groupMap.empty() ? whole : options.groupMap) {
            const std::vector<uint32_t> &index = group.second;
            std::vector<void *> s(index.size());
            std::vector<void *> d(index.size());
            std::vector<uint64_t> l(index.size());
            for (size_t j = 0; j < index.size(); ++j) {
                s[j] = params.sources[index[j]];
                d[j] = params.destinations[index[j]];
                l[j] = params.dataSizes[index[j]];
            }
            hybm_batch_copy_params sub = {s.data(), d.data(), l.data(), static_cast<uint32_t>(index.size())};
            ExtOptions subOptions{};
            subOptions.srcRankId = group.first.first;
            subOptions.destRankId = group.first.second;
            subOptions.stream = options.stream;
            subOptions.flags = options.flags;
            result = op.second->BatchDataCopy(sub, direction, subOptions);
            if (result != BM_OK) {
                break;
            }
        }
        if (result == BM_OK) {
            return result;
        }
    }
    return result;
}

ComposeDataOp::Result ComposeDataOp::DataCopyAsync(hybm_copy_params &params, hybm_data_copy_direction direction,
                                                   const ExtOptions &options) noexcept
{
    Ranked ops = Prioritised(options);
    if (ops.empty()) {
        MF_FAIL(BM_INVALID_PARAM, "no copy engine reaches rank " << options.srcRankId << " -> " << options.destRankId);
    }
    Result result = BM_ERROR;
    for (auto &op : ops) {
        result = op.second->DataCopyAsync(params, direction, options);
        if (result == BM_OK) {
            break;
        }
    }
    return result;
}

ComposeDataOp::Result ComposeDataOp::Wait(int32_t waitId) noexcept
{
    // Only the intra-node engine queues work asynchronously.
    if (intraNode_ == nullptr) {
        MF_FAIL(BM_ERROR, "wait requested but no asynchronous copy engine exists");
    }
    return intraNode_->Wait(waitId);
}

void ComposeDataOp::CleanUp() noexcept
{
    for (const DataOperatorPtr &op : {intraNode_, deviceRdma_, hostNet_}) {
        if (op != nullptr) {
            op->CleanUp();
        }
    }
}

}  // namespace mf
