// ReshapeAndCacheOmniOperation on MI355X: the KV-cache write for caches that keep, per (sequence, head)
// pair, everything but one window of tokens. Eight inputs (key, value, keyCache, valueCache,
// slotMapping, wins, seqLen, offsetIndex), the caches again as outputs
// (reference src/ops/ops_infer/reshape_and_cache_omni/reshape_and_cache_omni_operation.cpp:20-29,43 create,
// :53-64 tensor counts, :77-83 InferShape, :85-152 dim checks, :154-171 Setup checks; dtype table
// ops_configs/atb_ops_info.ini:6637-6650).
//
// The reference creates the operation on its 910B products only; here it is always available.
#include <new>
#include "atb/infer_op_params.h"
#include "atb/utils.h"
#include "atbmi_kernels.h"
#include "log.h"
#include "operation_base.h"

namespace atb {
namespace {
using Param = infer::ReshapeAndCacheOmniParam;
constexpr int64_t MAX_PAIRS = 500; // batch * heads stays below this (reference :146-149)

OpIr MakeIr()
{
    OpIr ir;
    for (aclDataType t : {ACL_FLOAT16, ACL_BF16}) {
        IrCombo c;
        c.inDtypes = {t, t, t, t, ACL_INT32, ACL_INT32, ACL_INT32, ACL_INT32};
        c.outDtypes = {t, t};
        c.inFormats.assign(c.inDtypes.size(), ACL_FORMAT_ND);
        c.outFormats.assign(c.outDtypes.size(), ACL_FORMAT_ND);
        ir.push_back(c);
    }
    return ir;
}

bool SameDesc(const TensorDesc &a, const TensorDesc &b)
{
    if (a.dtype != b.dtype || a.format != b.format || a.shape.dimNum != b.shape.dimNum) {
        return false;
    }
    for (uint64_t i = 0; i < a.shape.dimNum; ++i) {
        if (a.shape.dims[i] != b.shape.dims[i]) {
            return false;
        }
    }
    return true;
}

class ReshapeAndCacheOmniOperation : public OperationBase {
public:
    explicit ReshapeAndCacheOmniOperation(const Param &param)
        : OperationBase("ReshapeAndCacheOmniOperation"), param_(param)
    {
        static const OpIr table = MakeIr();
        ir_ = &table;
    }

    uint32_t GetInputNum() const override { return 8; }
    uint32_t GetOutputNum() const override { return 2; }
    const Param &GetParam() const { return param_; }
    void SetParam(const Param &param) { param_ = param; }

protected:
    Status InferShapeImpl(const SVector<TensorDesc> &in, SVector<TensorDesc> &out) const override
    {
        out.at(0) = in.at(2);
        out.at(1) = in.at(3);
        return NO_ERROR;
    }

    Status InferShapeCheckImpl(const SVector<TensorDesc> &in) const override
    {
        static const uint64_t dimNums[8] = {3, 3, 4, 4, 1, 1, 1, 1};
        for (size_t i = 0; i < 8; ++i) {
            if (in.at(i).shape.dimNum != dimNums[i]) {
                ATB_LOG(ERROR) << "ReshapeAndCacheOmni: expected dims 3/3/4/4/1/1/1/1";
                return ERROR_INVALID_TENSOR_DIM_NUM;
            }
        }
        return DimCheck(in);
    }

    // The reference's Setup repeats the dim check without the dim counts; they are checked here as
    // well, since the launch reads dims by position.
    Status SetupCheckImpl(const SVector<Tensor> &inTensors, const SVector<Tensor> &outTensors) const override
    {
        SVector<TensorDesc> in;
        for (size_t i = 0; i < inTensors.size(); ++i) {
            in.push_back(inTensors.at(i).desc);
        }
        Status st = InferShapeCheckImpl(in);
        if (st != NO_ERROR) {
            return st;
        }
        if (!SameDesc(in.at(2), outTensors.at(0).desc) || !SameDesc(in.at(3), outTensors.at(1).desc)) {
            ATB_LOG(ERROR) << "ReshapeAndCacheOmni: output descs must equal the cache input descs";
            return ERROR_INVALID_TENSOR_DIM;
        }
        return NO_ERROR;
    }

    Status PlanImpl(const VariantPack &, uint64_t &workspaceSize) override
    {
        workspaceSize = 0;
        return NO_ERROR;
    }

    Status LaunchImpl(const VariantPack &pack, uint8_t *, uint64_t, aclrtStream stream) override
    {
        const Tensor &key = pack.inTensors.at(0);
        const Tensor &keyCacheIn = pack.inTensors.at(2);
        for (size_t i : {size_t(0), size_t(1), size_t(4), size_t(5), size_t(6), size_t(7)}) {
            if (!pack.inTensors.at(i).deviceData) {
                ATB_LOG(ERROR) << "ReshapeAndCacheOmni: device pointer of input " << i << " is null";
                return ERROR_INVALID_PARAM;
            }
        }
        if (!pack.outTensors.at(0).deviceData || !pack.outTensors.at(1).deviceData) {
            ATB_LOG(ERROR) << "ReshapeAndCacheOmni: cache device pointer is null";
            return ERROR_INVALID_PARAM;
        }
        int rc = atbmi_reshape_and_cache_omni(
            key.deviceData, pack.inTensors.at(1).deviceData, pack.outTensors.at(0).deviceData,
            pack.outTensors.at(1).deviceData, static_cast<const int32_t *>(pack.inTensors.at(4).deviceData),
            static_cast<const int32_t *>(pack.inTensors.at(5).deviceData),
            static_cast<const int32_t *>(pack.inTensors.at(6).deviceData),
            static_cast<const int32_t *>(pack.inTensors.at(7).deviceData), pack.inTensors.at(6).desc.shape.dims[0],
            key.desc.shape.dims[1], key.desc.shape.dims[2], key.desc.shape.dims[0],
            keyCacheIn.desc.shape.dims[0] * keyCacheIn.desc.shape.dims[1],
            key.desc.dtype == ACL_BF16 ? ATBMI_BF16 : ATBMI_F16, stream);
        if (rc != 0) {
            ATB_LOG(ERROR) << "ReshapeAndCacheOmni launch failed: " << atbmi_last_error();
        }
        return rc;
    }

private:
    // Reference reshape_and_cache_omni_operation.cpp:101-152.
    Status DimCheck(const SVector<TensorDesc> &in) const
    {
        const Dims &k = in.at(0).shape;
        const Dims &v = in.at(1).shape;
        const Dims &kc = in.at(2).shape;
        const Dims &vc = in.at(3).shape;
        const int64_t heads = k.dims[1];
        const int64_t headSize = k.dims[2];
        const int64_t batch = in.at(6).shape.dims[0];
        if (headSize % 32 != 0) {
            ATB_LOG(ERROR) << "ReshapeAndCacheOmni: headSize must be a multiple of 32";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (k.dims[0] != v.dims[0]) {
            ATB_LOG(ERROR) << "ReshapeAndCacheOmni: key and value must agree on tokens";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (heads != v.dims[1] || heads * batch != in.at(4).shape.dims[0] || heads * batch != in.at(5).shape.dims[0] ||
            heads * batch != in.at(7).shape.dims[0]) {
            ATB_LOG(ERROR) << "ReshapeAndCacheOmni: slotMapping, wins and offsetIndex hold batch * heads entries";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (headSize != v.dims[2] || headSize != kc.dims[3] || headSize != vc.dims[3]) {
            ATB_LOG(ERROR) << "ReshapeAndCacheOmni: key, value and the caches must agree on headSize";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (kc.dims[0] != vc.dims[0] || kc.dims[1] != vc.dims[1]) {
            ATB_LOG(ERROR) << "ReshapeAndCacheOmni: caches must agree on numBlocks and blockSize";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (kc.dims[2] != 1 || vc.dims[2] != 1) {
            ATB_LOG(ERROR) << "ReshapeAndCacheOmni: dim 2 of keyCache and valueCache must be 1";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (batch * heads >= MAX_PAIRS) {
            ATB_LOG(ERROR) << "ReshapeAndCacheOmni: batch * heads must stay below " << MAX_PAIRS;
            return ERROR_INVALID_TENSOR_DIM;
        }
        return NO_ERROR;
    }

    Param param_;
};
} // namespace

// Reference reshape_and_cache_omni_operation.cpp:43 (OPERATION_PARAM_FUNCS: reserved bytes, then ParamCheck :20-29).
template <> Status CreateOperation(const infer::ReshapeAndCacheOmniParam &opParam, Operation **operation)
{
    if (operation == nullptr) {
        return ERROR_INVALID_PARAM;
    }
    if (!ReservedIsZero(opParam)) {
        ATB_LOG(ERROR) << "ReshapeAndCacheOmniParam rsv has a non-zero byte";
        return ERROR_INVALID_PARAM;
    }
    *operation = new (std::nothrow) ReshapeAndCacheOmniOperation(opParam);
    if (*operation == nullptr) {
        return ERROR_OUT_OF_HOST_MEMORY;
    }
    return NO_ERROR;
}

// Reference src/atb/operation/op_param_funcs.h:36-48.
template <> Status CloneOperationParam(const Operation *operation, infer::ReshapeAndCacheOmniParam &opParam)
{
    const auto *op = dynamic_cast<const ReshapeAndCacheOmniOperation *>(operation);
    if (op == nullptr) {
        ATB_LOG(ERROR) << "CloneOperationParam: not a ReshapeAndCacheOmniOperation";
        return ERROR_INVALID_PARAM;
    }
    opParam = op->GetParam();
    return NO_ERROR;
}

// Reference src/atb/operation/op_param_funcs.h:50-70 (the param holds reserved bytes only, so every legal
// param equals the current one: reshape_and_cache_omni_ops_runner.h:29-34).
template <> Status UpdateOperationParam(Operation *operation, const infer::ReshapeAndCacheOmniParam &opParam)
{
    auto *op = dynamic_cast<ReshapeAndCacheOmniOperation *>(operation);
    if (op == nullptr) {
        ATB_LOG(ERROR) << "UpdateOperationParam: not a ReshapeAndCacheOmniOperation";
        return ERROR_INVALID_PARAM;
    }
    op->SetParam(opParam);
    return NO_ERROR;
}
} // namespace atb
