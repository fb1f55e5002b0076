// atb::Operation - the abstract operator interface, and the factory
// functions that create and destroy operators from their parameter structs.
// Mirrors reference include/atb/operation.h:34-99 (virtuals), :109 (create),
// :120 (destroy).
#ifndef ATB_OPERATION_H
#define ATB_OPERATION_H
#include <cstdint>
#include <string>
#include "atb/types.h"
#include "atb/svector.h"
#include "atb/context.h"

namespace atb {
class Operation {
public:
    Operation() = default;
    virtual ~Operation() = default;

    virtual std::string GetName() const = 0;

    // Output tensor descriptions for the given input descriptions.
    virtual Status InferShape(const SVector<TensorDesc> &inTensorDescs, SVector<TensorDesc> &outTensorDescs) const = 0;

    virtual uint32_t GetInputNum() const = 0;
    virtual uint32_t GetOutputNum() const = 0;

    // Validates the pack, plans the launch (host only, no device work) and
    // reports the device workspace Execute will need.
    virtual Status Setup(const VariantPack &variantPack, uint64_t &workspaceSize, Context *context) = 0;

    // Enqueues the kernels on the context's execute stream and returns
    // without waiting for them.
    virtual Status Execute(const VariantPack &variantPack, uint8_t *workspace, uint64_t workspaceSize,
                           Context *context) = 0;
};

// Specialised for infer::PagedAttentionParam, ReshapeAndCacheParam, ReshapeAndCacheWithStrideParam,
// ReshapeAndCacheOmniParam, RopeParam, ElewiseParam, NormRopeReshapeParam, MultiLatentAttentionParam, BlockCopyParam and PagedCacheLoadParam.
template <typename OpParam> Status CreateOperation(const OpParam &opParam, Operation **operation);

Status DestroyOperation(Operation *operation);

// Chooses which of the context's execute streams (Context::SetExecuteStreams) an operation's launches go to; the
// default is stream 0. Execute fails with ERROR_INVALID_PARAM when the context holds fewer streams
// (reference include/atb/operation.h:150,159).
Status SetExecuteStreamId(Operation *operation, uint32_t streamId);
uint32_t GetExecuteStreamId(Operation *operation);

// Copies the param an operation was created with / replaces it (no-op when equal). Specialised for
// infer::ReshapeAndCacheOmniParam, the one operation of this library whose reference counterpart exports them
// (reference include/atb/operation.h:130,140; src/atb/operation/op_param_funcs.h:36-70). An operation of another type
// gives ERROR_INVALID_PARAM.
template <typename OpParam> Status CloneOperationParam(const Operation *operation, OpParam &opParam);
template <typename OpParam> Status UpdateOperationParam(Operation *operation, const OpParam &opParam);
} // namespace atb
#endif
