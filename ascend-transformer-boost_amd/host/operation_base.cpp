#include "operation_base.h"
#include <exception>
#include "atb/utils.h"
#include "context_impl.h"
#include "log.h"

namespace atb {
namespace {
constexpr uint64_t MAX_TENSOR_BYTES = 256ULL * 1024ULL * 1024ULL * 1024ULL;

// Reference src/atb/utils/tensor_check.cpp:25-62.
Status CheckOneShape(const TensorDesc &desc, bool mayBeEmpty = false)
{
    if (desc.shape.dimNum == 0 || desc.shape.dimNum > MAX_DIM) {
        ATB_LOG(ERROR) << "tensor dimNum " << desc.shape.dimNum << " is invalid, should be in (0, 8]";
        return ERROR_INVALID_TENSOR_DIM;
    }
    const uint64_t bytes = Utils::GetTensorSize(desc);
    if (bytes == 0 && mayBeEmpty) {
        return NO_ERROR;
    }
    if (bytes == 0 || bytes > MAX_TENSOR_BYTES) {
        ATB_LOG(ERROR) << "tensor size " << bytes << " is invalid, should be in (0, 256 GiB]";
        return ERROR_INVALID_TENSOR_SIZE;
    }
    return NO_ERROR;
}

void DescsOf(const SVector<Tensor> &tensors, SVector<TensorDesc> &descs)
{
    descs.reserve(tensors.size());
    descs.resize(tensors.size());
    for (size_t i = 0; i < tensors.size(); ++i) {
        descs.at(i) = tensors.at(i).desc;
    }
}
} // namespace

Status OperationBase::CheckShapes(const SVector<Tensor> &tensors, const char *what, bool inputs) const
{
    for (size_t i = 0; i < tensors.size(); ++i) {
        Status st = CheckOneShape(tensors.at(i).desc, inputs && InputMayBeEmpty(i));
        if (st != NO_ERROR) {
            ATB_LOG(ERROR) << name_ << " " << what << "[" << i << "] shape check failed: " << st;
            return st;
        }
    }
    return NO_ERROR;
}

bool OperationBase::IrMatch(const SVector<TensorDesc> &inDescs, const SVector<TensorDesc> *outDescs) const
{
    if (!ir_) {
        return true;
    }
    for (const IrCombo &c : *ir_) {
        if (c.inDtypes.size() != inDescs.size()) {
            continue;
        }
        bool ok = true;
        for (size_t i = 0; ok && i < inDescs.size(); ++i) {
            if (InputMayBeEmpty(i) && Utils::GetTensorSize(inDescs.at(i)) == 0) {
                continue; // an optional operand that is left out
            }
            ok = inDescs.at(i).dtype == c.inDtypes[i] && inDescs.at(i).format == c.inFormats[i];
        }
        if (ok && outDescs && outDescs->size() != 0) {
            ok = outDescs->size() == c.outDtypes.size();
            for (size_t i = 0; ok && i < outDescs->size(); ++i) {
                ok = outDescs->at(i).dtype == c.outDtypes[i] && outDescs->at(i).format == c.outFormats[i];
            }
        }
        if (ok) {
            return true;
        }
    }
    return false;
}

Status OperationBase::InferShape(const SVector<TensorDesc> &inTensorDescs, SVector<TensorDesc> &outTensorDescs) const
{
    try {
        if (inTensorDescs.size() != GetInputNum()) {
            ATB_LOG(ERROR) << name_ << " InferShape: " << inTensorDescs.size() << " inputs given, " << GetInputNum()
                           << " expected";
            return ERROR_INVALID_IN_TENSOR_NUM;
        }
        for (size_t i = 0; i < inTensorDescs.size(); ++i) {
            Status st = CheckOneShape(inTensorDescs.at(i), InputMayBeEmpty(i));
            if (st != NO_ERROR) {
                return st;
            }
        }
        if (!IrMatch(inTensorDescs, nullptr)) {
            ATB_LOG(ERROR) << name_ << " InferShape: input dtype/format combination is not supported";
            return ERROR_INVALID_TENSOR_INI_MATCH;
        }
        Status st = InferShapeCheckImpl(inTensorDescs);
        if (st != NO_ERROR) {
            return st;
        }
        outTensorDescs.reserve(GetOutputNum());
        outTensorDescs.resize(GetOutputNum());
        return InferShapeImpl(inTensorDescs, outTensorDescs);
    } catch (const std::exception &e) {
        ATB_LOG(ERROR) << name_ << " InferShape threw: " << e.what();
        return ERROR_OUT_OF_HOST_MEMORY;
    }
}

Status OperationBase::Setup(const VariantPack &variantPack, uint64_t &workspaceSize, Context *context)
{
    setupOk_ = false;
    preLaunched_ = false;
    if (!context) {
        ATB_LOG(ERROR) << name_ << " Setup: context is null";
        return ERROR_INVALID_PARAM;
    }
    try {
        if (variantPack.inTensors.size() != GetInputNum() || variantPack.outTensors.size() != GetOutputNum()) {
            ATB_LOG(ERROR) << name_ << " Setup: pack has " << variantPack.inTensors.size() << " inputs / "
                           << variantPack.outTensors.size() << " outputs, expected " << GetInputNum() << " / "
                           << GetOutputNum();
            return ERROR_INVALID_IN_TENSOR_NUM;
        }
        Status st = CheckShapes(variantPack.inTensors, "inTensor", true);
        if (st != NO_ERROR) {
            return st;
        }
        st = CheckShapes(variantPack.outTensors, "outTensor", false);
        if (st != NO_ERROR) {
            return st;
        }
        SVector<TensorDesc> inDescs;
        SVector<TensorDesc> outDescs;
        DescsOf(variantPack.inTensors, inDescs);
        DescsOf(variantPack.outTensors, outDescs);
        if (!IrMatch(inDescs, &outDescs)) {
            ATB_LOG(ERROR) << name_ << " Setup: tensor dtype/format combination is not supported";
            return ERROR_INVALID_TENSOR_INI_MATCH;
        }
        st = SetupCheckImpl(variantPack.inTensors, variantPack.outTensors);
        if (st != NO_ERROR) {
            return st;
        }
        ContextImpl *impl = dynamic_cast<ContextImpl *>(context);
        if (!impl) {
            ATB_LOG(ERROR) << name_ << " Setup: context was not made by atb::CreateContext";
            return ERROR_INVALID_PARAM;
        }
        uint64_t ws = 0;
        st = PlanImpl(variantPack, ws);
        if (st != NO_ERROR) {
            ATB_LOG(ERROR) << name_ << " Setup: planning failed: " << st;
            return st;
        }
        context_ = impl;
        workspaceSize_ = ws;
        workspaceSize = ws;
        setupPack_ = variantPack;
        setupInSizes_.clear();
        setupOutSizes_.clear();
        for (size_t i = 0; i < variantPack.inTensors.size(); ++i) {
            setupInSizes_.push_back(Utils::GetTensorSize(variantPack.inTensors.at(i).desc));
        }
        for (size_t i = 0; i < variantPack.outTensors.size(); ++i) {
            setupOutSizes_.push_back(Utils::GetTensorSize(variantPack.outTensors.at(i).desc));
        }
    } catch (const std::exception &e) {
        ATB_LOG(ERROR) << name_ << " Setup threw: " << e.what();
        return ERROR_OUT_OF_HOST_MEMORY;
    }
    setupOk_ = true;
    return NO_ERROR;
}

aclrtStream OperationBase::ExecuteStream() const
{
    const std::vector<aclrtStream> streams = context_->GetExecuteStreams();
    if (streams.size() < static_cast<size_t>(streamId_) + 1) {
        ATB_LOG(ERROR) << name_ << ": stream id " << streamId_ << ", the context holds " << streams.size() << " streams";
        return nullptr;
    }
    return streams.at(streamId_);
}

Status OperationBase::PreLaunch(const VariantPack &variantPack, uint8_t *workspace, uint64_t workspaceSize,
                                Context *context)
{
    if (!setupOk_) {
        ATB_LOG(ERROR) << name_ << " Execute: no successful Setup before Execute";
        return ERROR_INVALID_PARAM;
    }
    if (ExecuteStream() == nullptr) {
        ATB_LOG(ERROR) << name_ << " Execute: execute stream is null";
        return ERROR_INVALID_PARAM;
    }
    if (context != context_) {
        ATB_LOG(ERROR) << name_ << " Execute: context differs from the Setup context";
        return ERROR_INVALID_PARAM;
    }
    if (workspaceSize < workspaceSize_) {
        ATB_LOG(ERROR) << name_ << " Execute: workspaceSize " << workspaceSize << " < " << workspaceSize_;
        return ERROR_INVALID_PARAM;
    }
    if (workspaceSize_ != 0 && workspace == nullptr) {
        ATB_LOG(ERROR) << name_ << " Execute: workspace is null but " << workspaceSize_ << " bytes are needed";
        return ERROR_INVALID_PARAM;
    }
    if (variantPack.inTensors.size() != setupInSizes_.size() ||
        variantPack.outTensors.size() != setupOutSizes_.size()) {
        ATB_LOG(ERROR) << name_ << " Execute: tensor counts differ from Setup";
        return ERROR_INVALID_PARAM;
    }
    for (size_t i = 0; i < variantPack.inTensors.size(); ++i) {
        const Tensor &t = variantPack.inTensors.at(i);
        if (t.dataSize != setupInSizes_[i]) {
            ATB_LOG(ERROR) << name_ << " Execute: inTensors(" << i << ").dataSize differs from the Setup size";
            return ERROR_INVALID_PARAM;
        }
        if (!t.deviceData && !t.hostData && !(t.dataSize == 0 && InputMayBeEmpty(i))) {
            ATB_LOG(ERROR) << name_ << " Execute: inTensors(" << i << ") has no data pointer";
            return ERROR_INVALID_PARAM;
        }
    }
    for (size_t i = 0; i < variantPack.outTensors.size(); ++i) {
        const Tensor &t = variantPack.outTensors.at(i);
        if (t.dataSize != setupOutSizes_[i]) {
            ATB_LOG(ERROR) << name_ << " Execute: outTensors(" << i << ").dataSize differs from the Setup size";
            return ERROR_INVALID_PARAM;
        }
        if (!t.deviceData && !t.hostData) {
            ATB_LOG(ERROR) << name_ << " Execute: outTensors(" << i << ") has no data pointer";
            return ERROR_INVALID_PARAM;
        }
    }
    return NO_ERROR;
}

Status OperationBase::Execute(const VariantPack &variantPack, uint8_t *workspace, uint64_t workspaceSize,
                              Context *context)
{
    if (!context) {
        ATB_LOG(ERROR) << name_ << " Execute: context is null";
        return ERROR_INVALID_PARAM;
    }
    const ExecuteType type = context->GetExecuteType();
    // A pack without tensors stands for the one Setup was given: the two-call C wrappers
    // (AtbMLAGetWorkspaceSize + AtbMLA, reference src/ops/ops_infer/multi_latent_attention/
    // atb_acl_mla.cpp:118-124) run Execute that way.
    if (variantPack.inTensors.size() == 0 && variantPack.outTensors.size() == 0 && setupOk_ &&
        (type == EXECUTE_NORMAL || type == EXECUTE_PRELAUNCH)) {
        const VariantPack kept = setupPack_;
        return Execute(kept, workspace, workspaceSize, context);
    }
    try {
        if (type == EXECUTE_NORMAL || type == EXECUTE_PRELAUNCH) {
            Status st = PreLaunch(variantPack, workspace, workspaceSize, context);
            if (st != NO_ERROR) {
                return st;
            }
            if (type == EXECUTE_PRELAUNCH) {
                launchPack_ = variantPack;
                launchWorkspace_ = workspace;
                launchWorkspaceSize_ = workspaceSize;
                preLaunched_ = true;
                return NO_ERROR;
            }
            return LaunchImpl(variantPack, workspace, workspaceSize, ExecuteStream());
        }
        // EXECUTE_LAUNCH: second half of a split execute.
        if (!setupOk_ || !preLaunched_ || context != context_) {
            ATB_LOG(ERROR) << name_ << " Execute(LAUNCH) without a matching pre-launch";
            return ERROR_INVALID_PARAM;
        }
        preLaunched_ = false;
        return LaunchImpl(launchPack_, launchWorkspace_, launchWorkspaceSize_, ExecuteStream());
    } catch (const std::exception &e) {
        ATB_LOG(ERROR) << name_ << " Execute threw: " << e.what();
        return ERROR_RT_FAIL;
    }
}

Status DestroyOperation(Operation *operation)
{
    delete operation;
    return NO_ERROR;
}

// Reference src/atb/operation/operation.cpp:24-55.
Status SetExecuteStreamId(Operation *operation, uint32_t streamId)
{
    OperationBase *base = dynamic_cast<OperationBase *>(operation);
    if (base == nullptr) {
        return ERROR_INVALID_PARAM;
    }
    base->SetExecuteStreamId(streamId);
    return NO_ERROR;
}

uint32_t GetExecuteStreamId(Operation *operation)
{
    OperationBase *base = dynamic_cast<OperationBase *>(operation);
    if (base == nullptr) {
        ATB_LOG(ERROR) << "GetExecuteStreamId: not an operation of this library";
        return 0;
    }
    return base->GetExecuteStreamId();
}
} // namespace atb
