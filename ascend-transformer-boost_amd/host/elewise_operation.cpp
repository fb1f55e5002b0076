// ElewiseOperation on MI355X, the two per-channel forms that sit beside the int8 KV cache:
// ELEWISE_QUANT_PER_CHANNEL (x fp16 / bf16, scale of the same type, int8 offset -> int8) and
// ELEWISE_DEQUANT_PER_CHANNEL (int8 x, fp16 scale, int8 offset -> fp16)
// (reference src/ops/ops_infer/elewise/elewise_operation.cpp:40-99 create, :158-192 tensor counts,
// :195-230 InferShape, :451-472 the two forms, :474-486 the offset may be an empty tensor;
// dtype tables ops_configs/atb_ops_info.ini:2410-2437).
//
// The scale and the offset cover the trailing dimensions of x, or hold a single value; the output
// has x's shape. Every other elewiseType is rejected when the operation is created: they are general
// tensor arithmetic with no part in the decode path this library serves.
#include <new>
#include "atb/infer_op_params.h"
#include "atb/utils.h"
#include "atbmi_kernels.h"
#include "log.h"
#include "operation_base.h"

namespace atb {
namespace {
using Param = infer::ElewiseParam;

OpIr MakeIr(bool dequant)
{
    OpIr ir;
    if (dequant) {
        IrCombo c;
        c.inDtypes = {ACL_INT8, ACL_FLOAT16, ACL_INT8};
        c.outDtypes = {ACL_FLOAT16};
        ir.push_back(c);
    } else {
        for (aclDataType t : {ACL_FLOAT16, ACL_BF16}) {
            IrCombo c;
            c.inDtypes = {t, t, ACL_INT8};
            c.outDtypes = {ACL_INT8};
            ir.push_back(c);
        }
    }
    for (IrCombo &c : ir) {
        c.inFormats.assign(3, ACL_FORMAT_ND);
        c.outFormats.assign(1, ACL_FORMAT_ND);
    }
    return ir;
}

int64_t Numel(const Dims &d)
{
    int64_t n = 1;
    for (uint64_t i = 0; i < d.dimNum; ++i) {
        n *= d.dims[i];
    }
    return d.dimNum == 0 ? 0 : n;
}

class ElewiseOperation : public OperationBase {
public:
    explicit ElewiseOperation(const Param &param)
        : OperationBase("ElewiseOperation"), dequant_(param.elewiseType == Param::ELEWISE_DEQUANT_PER_CHANNEL)
    {
        static const OpIr quant = MakeIr(false);
        static const OpIr dequant = MakeIr(true);
        ir_ = dequant_ ? &dequant : &quant;
    }

    uint32_t GetInputNum() const override { return 3; }
    uint32_t GetOutputNum() const override { return 1; }
    bool InputMayBeEmpty(size_t index) const override { return index == 2; } // the offset is optional

protected:
    Status InferShapeImpl(const SVector<TensorDesc> &in, SVector<TensorDesc> &out) const override
    {
        out.at(0) = in.at(0);
        out.at(0).dtype = dequant_ ? ACL_FLOAT16 : ACL_INT8;
        return NO_ERROR;
    }

    Status InferShapeCheckImpl(const SVector<TensorDesc> &) const override { return NO_ERROR; }

    Status SetupCheckImpl(const SVector<Tensor> &, const SVector<Tensor> &) const override { return NO_ERROR; }

    // What the kernel needs beyond the reference's checks: the scale (and the offset, when there is
    // one) must tile x exactly, and the output must have x's element count.
    Status PlanImpl(const VariantPack &pack, uint64_t &workspaceSize) override
    {
        const int64_t total = Numel(pack.inTensors.at(0).desc.shape);
        const int64_t channels = Numel(pack.inTensors.at(1).desc.shape);
        const int64_t offsets = Numel(pack.inTensors.at(2).desc.shape);
        if (channels <= 0 || total % channels != 0 || (offsets != 0 && offsets != channels) ||
            Numel(pack.outTensors.at(0).desc.shape) != total) {
            ATB_LOG(ERROR) << "Elewise: scale / offset must cover the trailing dimensions of x, the output x's shape";
            return ERROR_INVALID_TENSOR_DIM;
        }
        workspaceSize = 0;
        return NO_ERROR;
    }

    Status LaunchImpl(const VariantPack &pack, uint8_t *, uint64_t, aclrtStream stream) override
    {
        const Tensor &x = pack.inTensors.at(0);
        const Tensor &scale = pack.inTensors.at(1);
        const Tensor &offset = pack.inTensors.at(2);
        const int64_t total = Numel(x.desc.shape);
        const int64_t channels = Numel(scale.desc.shape);
        const int8_t *off = Numel(offset.desc.shape) == 0 ? nullptr : static_cast<const int8_t *>(offset.deviceData);
        if (!x.deviceData || !scale.deviceData || !pack.outTensors.at(0).deviceData ||
            (Numel(offset.desc.shape) != 0 && off == nullptr)) {
            ATB_LOG(ERROR) << "Elewise: a device pointer is null";
            return ERROR_INVALID_PARAM;
        }
        int rc;
        if (dequant_) {
            rc = atbmi_elewise_dequant_per_channel(static_cast<const int8_t *>(x.deviceData), scale.deviceData, off,
                                                   pack.outTensors.at(0).deviceData, total, channels, stream);
        } else {
            rc = atbmi_elewise_quant_per_channel(x.deviceData, scale.deviceData, off,
                                                 static_cast<int8_t *>(pack.outTensors.at(0).deviceData), total, channels,
                                                 x.desc.dtype == ACL_BF16 ? ATBMI_BF16 : ATBMI_F16, stream);
        }
        if (rc != 0) {
            ATB_LOG(ERROR) << "Elewise launch failed: " << atbmi_last_error();
        }
        return rc;
    }

private:
    bool dequant_;
};
} // namespace

// Reference elewise_operation.cpp:40-99.
template <> Status CreateOperation(const infer::ElewiseParam &opParam, Operation **operation)
{
    if (operation == nullptr) {
        return ERROR_INVALID_PARAM;
    }
    if (!ReservedIsZero(opParam) || !ReservedIsZero(opParam.mulsParam) || !ReservedIsZero(opParam.quantParam)) {
        ATB_LOG(ERROR) << "ElewiseParam rsv has a non-zero byte";
        return ERROR_INVALID_PARAM;
    }
    if (opParam.elewiseType <= Param::ELEWISE_UNDEFINED || opParam.elewiseType >= Param::ELEWISE_TYPE_MAX) {
        ATB_LOG(ERROR) << "ElewiseParam: elewiseType out of range";
        return ERROR_INVALID_PARAM;
    }
    if (opParam.elewiseType != Param::ELEWISE_QUANT_PER_CHANNEL && opParam.elewiseType != Param::ELEWISE_DEQUANT_PER_CHANNEL) {
        ATB_LOG(ERROR) << "ElewiseParam: only the per-channel quantiser and dequantiser are implemented on MI355X";
        return ERROR_INVALID_PARAM;
    }
    *operation = new (std::nothrow) ElewiseOperation(opParam);
    if (*operation == nullptr) {
        return ERROR_OUT_OF_HOST_MEMORY;
    }
    return NO_ERROR;
}
} // namespace atb
