// RopeOperation on MI355X: rotary position embedding of the query and key rows, the step that
// precedes the KV-cache write and the attention (reference src/ops/ops_infer/rope/rope_operation.cpp:33-56
// create, :68-84 tensor counts / InferShape, :86-134 checks, :136-225 dim checks;
// rope_ops_runner.cpp:22-32: 4-dim q / k are viewed as [dim0 * dim1, dim2 * dim3]).
//
// Inputs: q and k ([tokens, hidden] or [batch, seq, heads, headSize]), cos and sin [rows, headDim],
// seqLen [batch] (int32 / uint32, on the device); outputs shaped like q and k. Both table layouts
// (cosFormat 0: a row per token, 1: a row per position) and every rotaryCoeff the reference takes
// (2, 4, headDim) run on the same kernel.
#include <new>
#include "atb/infer_op_params.h"
#include "atb/utils.h"
#include "atbmi_kernels.h"
#include "log.h"
#include "operation_base.h"

namespace atb {
namespace {
using Param = infer::RopeParam;
constexpr int64_t MAX_HEAD_SIZE = 4096;
constexpr int64_t MIN_HEAD_SIZE = 16;

// Reference ops_configs/atb_ops_info.ini:1060-1081.
OpIr MakeIr()
{
    OpIr ir;
    struct Row { aclDataType x, table, len; };
    for (Row r : {Row{ACL_FLOAT16, ACL_FLOAT16, ACL_INT32}, Row{ACL_FLOAT16, ACL_FLOAT16, ACL_UINT32},
                  Row{ACL_FLOAT16, ACL_FLOAT, ACL_INT32}, Row{ACL_FLOAT16, ACL_FLOAT, ACL_UINT32},
                  Row{ACL_BF16, ACL_BF16, ACL_INT32}, Row{ACL_BF16, ACL_BF16, ACL_UINT32}}) {
        IrCombo c;
        c.inDtypes = {r.x, r.x, r.table, r.table, r.len};
        c.outDtypes = {r.x, r.x};
        c.inFormats.assign(5, ACL_FORMAT_ND);
        c.outFormats.assign(2, ACL_FORMAT_ND);
        ir.push_back(c);
    }
    return ir;
}

int64_t Rows(const Dims &d)
{
    return d.dimNum == 2 ? d.dims[0] : d.dims[0] * d.dims[1];
}

int64_t Hidden(const Dims &d)
{
    return d.dimNum == 4 ? d.dims[2] * d.dims[3] : d.dims[1];
}

class RopeOperation : public OperationBase {
public:
    explicit RopeOperation(const Param &param) : OperationBase("RopeOperation"), param_(param)
    {
        static const OpIr ir = MakeIr();
        ir_ = &ir;
    }

    uint32_t GetInputNum() const override { return 5; }
    uint32_t GetOutputNum() const override { return 2; }

protected:
    Status InferShapeImpl(const SVector<TensorDesc> &in, SVector<TensorDesc> &out) const override
    {
        out.at(0) = in.at(0);
        out.at(1) = in.at(1);
        return NO_ERROR;
    }

    Status InferShapeCheckImpl(const SVector<TensorDesc> &in) const override
    {
        Status st = DimCheck(in);
        return st != NO_ERROR ? st : ParamCheck(in);
    }

    Status SetupCheckImpl(const SVector<Tensor> &inTensors, const SVector<Tensor> &) const override
    {
        SVector<TensorDesc> in;
        for (size_t i = 0; i < inTensors.size(); ++i) {
            in.push_back(inTensors.at(i).desc);
        }
        return InferShapeCheckImpl(in);
    }

    Status PlanImpl(const VariantPack &, uint64_t &workspaceSize) override
    {
        workspaceSize = 0;
        return NO_ERROR;
    }

    Status LaunchImpl(const VariantPack &pack, uint8_t *, uint64_t, aclrtStream stream) override
    {
        const Tensor &q = pack.inTensors.at(0);
        const Tensor &k = pack.inTensors.at(1);
        const Tensor &cos = pack.inTensors.at(2);
        const Tensor &sin = pack.inTensors.at(3);
        const Tensor &lens = pack.inTensors.at(4);
        for (size_t i = 0; i < 5; ++i) {
            if (pack.inTensors.at(i).deviceData == nullptr) {
                ATB_LOG(ERROR) << "Rope: device pointer of input " << i << " is null";
                return ERROR_INVALID_PARAM;
            }
        }
        if (pack.outTensors.at(0).deviceData == nullptr || pack.outTensors.at(1).deviceData == nullptr) {
            ATB_LOG(ERROR) << "Rope: device pointer of an output is null";
            return ERROR_INVALID_PARAM;
        }
        int rc = atbmi_rope(q.deviceData, k.deviceData, cos.deviceData, sin.deviceData,
                            static_cast<const int32_t *>(lens.deviceData), pack.outTensors.at(0).deviceData,
                            pack.outTensors.at(1).deviceData, Rows(q.desc.shape), Hidden(q.desc.shape),
                            Hidden(k.desc.shape), cos.desc.shape.dims[1], cos.desc.shape.dims[0],
                            lens.desc.shape.dims[0], param_.rotaryCoeff, param_.cosFormat,
                            q.desc.dtype == ACL_BF16 ? ATBMI_BF16 : ATBMI_F16, cos.desc.dtype == ACL_FLOAT ? 1 : 0,
                            stream);
        if (rc != 0) {
            ATB_LOG(ERROR) << "Rope launch failed: " << atbmi_last_error();
        }
        return rc;
    }

private:
    // Reference rope_operation.cpp:114-134.
    Status ParamCheck(const SVector<TensorDesc> &in) const
    {
        const int64_t cosDim = in.at(2).shape.dims[1];
        const int64_t sinDim = in.at(3).shape.dims[1];
        if (param_.rotaryCoeff != 2 && param_.rotaryCoeff != 4 && param_.rotaryCoeff != cosDim) {
            ATB_LOG(ERROR) << "Rope: rotaryCoeff must be 2, 4 or the table row size, got " << param_.rotaryCoeff;
            return ERROR_INVALID_PARAM;
        }
        if (cosDim % param_.rotaryCoeff != 0 || sinDim % param_.rotaryCoeff != 0) {
            ATB_LOG(ERROR) << "Rope: rotaryCoeff " << param_.rotaryCoeff << " does not divide the table row size";
            return ERROR_INVALID_PARAM;
        }
        if (param_.cosFormat != 0 && param_.cosFormat != 1) {
            ATB_LOG(ERROR) << "Rope: cosFormat must be 0 or 1, got " << param_.cosFormat;
            return ERROR_INVALID_PARAM;
        }
        return NO_ERROR;
    }

    // Reference rope_operation.cpp:136-190 (DimCheck) and :192-225 (HiddenSizeCheck).
    Status DimCheck(const SVector<TensorDesc> &in) const
    {
        const Dims &q = in.at(0).shape;
        const Dims &k = in.at(1).shape;
        const Dims &cos = in.at(2).shape;
        const Dims &sin = in.at(3).shape;
        if ((q.dimNum != 2 && q.dimNum != 4) || (k.dimNum != 2 && k.dimNum != 4) || cos.dimNum != 2 ||
            sin.dimNum != 2 || in.at(4).shape.dimNum != 1) {
            ATB_LOG(ERROR) << "Rope: q / k take 2 or 4 dims, cos / sin 2, seqLen 1";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (Rows(k) != Rows(q)) {
            ATB_LOG(ERROR) << "Rope: q and k must hold the same number of tokens";
            return ERROR_INVALID_TENSOR_SIZE;
        }
        if (cos.dims[1] > MAX_HEAD_SIZE || sin.dims[1] > MAX_HEAD_SIZE || cos.dims[1] < MIN_HEAD_SIZE ||
            sin.dims[1] < MIN_HEAD_SIZE) {
            ATB_LOG(ERROR) << "Rope: the table row size must lie in [16, 4096]";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (cos.dims[0] != sin.dims[0] || cos.dims[1] != sin.dims[1]) {
            ATB_LOG(ERROR) << "Rope: cos and sin must have the same shape";
            return ERROR_INVALID_TENSOR_SIZE;
        }
        const int64_t hiddenQ = Hidden(q);
        const int64_t hiddenK = Hidden(k);
        if (hiddenK == 0 || hiddenQ % hiddenK != 0) {
            ATB_LOG(ERROR) << "Rope: the row size of q must be a multiple of that of k";
            return ERROR_INVALID_TENSOR_SIZE;
        }
        if (hiddenK % cos.dims[1] != 0) {
            ATB_LOG(ERROR) << "Rope: the row size of k must be a multiple of the table row size";
            return ERROR_INVALID_TENSOR_DIM;
        }
        return NO_ERROR;
    }

    Param param_;
};
} // namespace

// Reference rope_operation.cpp:33-56.
template <> Status CreateOperation(const infer::RopeParam &opParam, Operation **operation)
{
    if (operation == nullptr) {
        return ERROR_INVALID_PARAM;
    }
    if (!ReservedIsZero(opParam)) {
        ATB_LOG(ERROR) << "RopeParam rsv has a non-zero byte";
        return ERROR_INVALID_PARAM;
    }
    *operation = new (std::nothrow) RopeOperation(opParam);
    if (*operation == nullptr) {
        return ERROR_OUT_OF_HOST_MEMORY;
    }
    return NO_ERROR;
}
} // namespace atb
