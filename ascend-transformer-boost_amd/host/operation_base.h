// Common Setup / Execute state machine of the operators, restating the
// observable behaviour of the reference OperationBase
// (reference src/atb/operation/operation_base.cpp:180-449 checks,
// :600-668 Setup, :752-862 execute checks, :898-940 pre-launch, :1095-1133 Execute):
//   InferShape : input count -> shapes -> dtype/format table -> op dim checks
//   Setup      : pack counts -> shapes -> dtype/format table -> op dim checks
//                -> context -> op planning (host only) -> workspace size
//   Execute    : needs a successful Setup with the same context, a non-null
//                stream, a large-enough workspace and unchanged tensor sizes;
//                then launches asynchronously.
#ifndef ATB_MI_OPERATION_BASE_H
#define ATB_MI_OPERATION_BASE_H
#include <string>
#include <vector>
#include "atb/operation.h"

namespace atb {
class ContextImpl;

// One row of an operator's dtype/format table: the i-th entry applies to the
// i-th input (then the outputs). The tables restate the sections of the
// reference ops_configs/atb_ops_info.ini that the supported params select.
struct IrCombo {
    std::vector<aclDataType> inDtypes;
    std::vector<aclFormat> inFormats;
    std::vector<aclDataType> outDtypes;
    std::vector<aclFormat> outFormats;
};
using OpIr = std::vector<IrCombo>;

class OperationBase : public Operation {
public:
    explicit OperationBase(const std::string &name) : name_(name) {}
    ~OperationBase() override = default;

    std::string GetName() const override { return name_; }
    Status InferShape(const SVector<TensorDesc> &inTensorDescs, SVector<TensorDesc> &outTensorDescs) const final;
    Status Setup(const VariantPack &variantPack, uint64_t &workspaceSize, Context *context) final;
    Status Execute(const VariantPack &variantPack, uint8_t *workspace, uint64_t workspaceSize,
                   Context *context) final;
    // Which of the context's execute streams the launches go to (reference operation_base.cpp:1356-1379).
    void SetExecuteStreamId(uint32_t streamId) { streamId_ = streamId; }
    uint32_t GetExecuteStreamId() const { return streamId_; }

protected:
    // Operator-specific hooks.
    virtual Status InferShapeCheckImpl(const SVector<TensorDesc> &inTensorDescs) const { (void)inTensorDescs; return NO_ERROR; }
    virtual Status InferShapeImpl(const SVector<TensorDesc> &inTensorDescs,
                                  SVector<TensorDesc> &outTensorDescs) const = 0;
    virtual Status SetupCheckImpl(const SVector<Tensor> &inTensors, const SVector<Tensor> &outTensors) const
    {
        (void)inTensors;
        (void)outTensors;
        return NO_ERROR;
    }
    // Host-only planning; reports the device workspace the launch needs.
    virtual Status PlanImpl(const VariantPack &variantPack, uint64_t &workspaceSize) = 0;
    // Enqueues the kernels on `stream`; must not wait for them.
    virtual Status LaunchImpl(const VariantPack &variantPack, uint8_t *workspace, uint64_t workspaceSize,
                              aclrtStream stream) = 0;

    const OpIr *ir_ = nullptr;

private:
    // Inputs an operation accepts as empty tensors (a dimension of 0): optional operands such as a
    // quantiser's offset (reference Operation::GetEmptyInTensorPermissions).
    virtual bool InputMayBeEmpty(size_t index) const { (void)index; return false; }
    Status CheckShapes(const SVector<Tensor> &tensors, const char *what, bool inputs) const;
    bool IrMatch(const SVector<TensorDesc> &inDescs, const SVector<TensorDesc> *outDescs) const;
    Status PreLaunch(const VariantPack &variantPack, uint8_t *workspace, uint64_t workspaceSize, Context *context);
    // Stream number streamId_ of the Setup context, null when the context holds fewer streams.
    aclrtStream ExecuteStream() const;

    std::string name_;
    uint32_t streamId_ = 0;
    bool setupOk_ = false;
    ContextImpl *context_ = nullptr;
    uint64_t workspaceSize_ = 0;
    VariantPack setupPack_;
    std::vector<uint64_t> setupInSizes_;
    std::vector<uint64_t> setupOutSizes_;
    // Captured by a pre-launch for the launch half.
    VariantPack launchPack_;
    uint8_t *launchWorkspace_ = nullptr;
    uint64_t launchWorkspaceSize_ = 0;
    bool preLaunched_ = false;
};

// True when every byte of the param's reserved area is zero
// (reference src/atb/operation/op_param_funcs.h:72-80).
template <typename Param> bool ReservedIsZero(const Param &p)
{
    for (uint8_t b : p.rsv) {
        if (b != 0) {
            return false;
        }
    }
    return true;
}
} // namespace atb
#endif
