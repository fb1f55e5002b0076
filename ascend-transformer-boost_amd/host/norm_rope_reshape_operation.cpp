// NormRopeReshapeOperation on MI355X: RMSNorm of the latent row, rotary embedding of the rotary
// row and the write of both into the token's slot of a single cache, in one kernel: the producer of
// the combined (MLA) cache that PagedAttention / MultiLatentAttention read
// (reference src/ops/ops_infer/norm_rope_reshape/norm_rope_reshape_operation.cpp:35-55 create,
// :65-103 tensor counts / InferShape / checks, :113-176 dim checks, :178-201 output check;
// kernel-level checks src/kernels/mixkernels/rms_norm_and_rope_and_reshape_and_cache/
// rms_norm_and_rope_and_reshape_and_cache_operation.cpp:63-117).
//
// Inputs: x [T, 1, normDim], gamma [normDim], keyRope [T, ropeDim], cos [T, ropeDim],
// sin [T, ropeDim], slotMapping [T] int32, keyCache [blocks, blockSize, 1, normDim + ropeDim];
// output: the cache. fp16 only, as in the reference's dtype table (ops_configs/atb_ops_info.ini:5870-5894).
//
// Left out: the reference's bound on the row sizes (11 * normDim * 2 + cacheDim * 2 < 196352, the
// size of an Ascend core's buffer; rows of any size work here) and rotaryCoeff values other than 2,
// for which the reference's goldens define no result.
#include <cmath>
#include <limits>
#include <new>
#include "atb/infer_op_params.h"
#include "atb/utils.h"
#include "atbmi_kernels.h"
#include "log.h"
#include "operation_base.h"

namespace atb {
namespace {
using Param = infer::NormRopeReshapeParam;

OpIr MakeIr()
{
    IrCombo c;
    c.inDtypes = {ACL_FLOAT16, ACL_FLOAT16, ACL_FLOAT16, ACL_FLOAT16, ACL_FLOAT16, ACL_INT32, ACL_FLOAT16};
    c.outDtypes = {ACL_FLOAT16};
    c.inFormats.assign(c.inDtypes.size(), ACL_FORMAT_ND);
    c.outFormats.assign(c.outDtypes.size(), ACL_FORMAT_ND);
    return OpIr{c};
}

class NormRopeReshapeOperation : public OperationBase {
public:
    explicit NormRopeReshapeOperation(const Param &param) : OperationBase("NormRopeReshapeOperation"), param_(param)
    {
        static const OpIr ir = MakeIr();
        ir_ = &ir;
    }

    uint32_t GetInputNum() const override { return 7; }
    uint32_t GetOutputNum() const override { return 1; }

protected:
    Status InferShapeImpl(const SVector<TensorDesc> &in, SVector<TensorDesc> &out) const override
    {
        out.at(0) = in.at(6);
        return NO_ERROR;
    }

    // Reference norm_rope_reshape_operation.cpp:77-92 (without the Ascend buffer-size bound).
    Status InferShapeCheckImpl(const SVector<TensorDesc> &in) const override
    {
        static const uint64_t dimNums[7] = {3, 1, 2, 2, 2, 1, 4};
        for (size_t i = 0; i < 7; ++i) {
            if (in.at(i).shape.dimNum != dimNums[i]) {
                ATB_LOG(ERROR) << "NormRopeReshape: expected dims 3/1/2/2/2/1/4";
                return ERROR_INVALID_TENSOR_DIM_NUM;
            }
        }
        return DimCheck(in) ? NO_ERROR : ERROR_INVALID_TENSOR_DIM;
    }

    // Reference norm_rope_reshape_operation.cpp:94-106: the output against the cache input first
    // (dtype, format, rank, dims: four different codes), then the input checks.
    Status SetupCheckImpl(const SVector<Tensor> &inTensors, const SVector<Tensor> &outTensors) const override
    {
        SVector<TensorDesc> in;
        for (size_t i = 0; i < inTensors.size(); ++i) {
            in.push_back(inTensors.at(i).desc);
        }
        const TensorDesc &cache = in.at(6);
        const TensorDesc &out = outTensors.at(0).desc;
        if (cache.dtype != out.dtype) {
            ATB_LOG(ERROR) << "NormRopeReshape: output dtype differs from the cache's";
            return ERROR_INVALID_TENSOR_DTYPE;
        }
        if (cache.format != out.format) {
            ATB_LOG(ERROR) << "NormRopeReshape: output format differs from the cache's";
            return ERROR_INVALID_TENSOR_FORMAT;
        }
        if (cache.shape.dimNum != out.shape.dimNum) {
            ATB_LOG(ERROR) << "NormRopeReshape: output rank differs from the cache's";
            return ERROR_INVALID_TENSOR_SIZE;
        }
        for (uint64_t i = 0; i < cache.shape.dimNum; ++i) {
            if (cache.shape.dims[i] != out.shape.dims[i]) {
                ATB_LOG(ERROR) << "NormRopeReshape: output dims differ from the cache's";
                return ERROR_INVALID_TENSOR_DIM;
            }
        }
        return InferShapeCheckImpl(in);
    }

    // The checks the reference's kernel library makes when the runner is set up
    // (rms_norm_and_rope_and_reshape_and_cache_operation.cpp:63-117): one head, every row count
    // equal (slotMapping included), row sizes multiples of 16.
    Status PlanImpl(const VariantPack &pack, uint64_t &workspaceSize) override
    {
        const Dims &x = pack.inTensors.at(0).desc.shape;
        const Dims &rope = pack.inTensors.at(2).desc.shape;
        const Dims &sin = pack.inTensors.at(4).desc.shape;
        const Dims &slots = pack.inTensors.at(5).desc.shape;
        const Dims &cache = pack.inTensors.at(6).desc.shape;
        if (x.dims[1] != 1 || cache.dims[2] != 1) {
            ATB_LOG(ERROR) << "NormRopeReshape: x and the cache hold one head";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (sin.dims[0] != x.dims[0] || slots.dims[0] != x.dims[0]) {
            ATB_LOG(ERROR) << "NormRopeReshape: x, keyRope, cos, sin and slotMapping must have the same rows";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (x.dims[0] == 0 || x.dims[2] == 0 || rope.dims[1] == 0) {
            ATB_LOG(ERROR) << "NormRopeReshape: no dimension of an input may be 0";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (rope.dims[1] % 16 != 0 || cache.dims[3] % 16 != 0) {
            ATB_LOG(ERROR) << "NormRopeReshape: row sizes must be multiples of 16";
            return ERROR_INVALID_TENSOR_DIM;
        }
        workspaceSize = 0;
        return NO_ERROR;
    }

    Status LaunchImpl(const VariantPack &pack, uint8_t *, uint64_t, aclrtStream stream) override
    {
        const Tensor &x = pack.inTensors.at(0);
        const Tensor &cacheIn = pack.inTensors.at(6);
        // the output is the cache itself; the reference kernel never reads the cache input either
        void *cache = pack.outTensors.at(0).deviceData;
        for (size_t i = 0; i < 6; ++i) {
            if (pack.inTensors.at(i).deviceData == nullptr) {
                ATB_LOG(ERROR) << "NormRopeReshape: device pointer of input " << i << " is null";
                return ERROR_INVALID_PARAM;
            }
        }
        if (cache == nullptr) {
            ATB_LOG(ERROR) << "NormRopeReshape: device pointer of the cache is null";
            return ERROR_INVALID_PARAM;
        }
        const int64_t numSlots = cacheIn.desc.shape.dims[0] * cacheIn.desc.shape.dims[1];
        int rc = atbmi_norm_rope_reshape_and_cache(
            x.deviceData, pack.inTensors.at(1).deviceData, pack.inTensors.at(2).deviceData,
            pack.inTensors.at(3).deviceData, pack.inTensors.at(4).deviceData,
            static_cast<const int32_t *>(pack.inTensors.at(5).deviceData), cache, x.desc.shape.dims[0],
            x.desc.shape.dims[2], pack.inTensors.at(2).desc.shape.dims[1], numSlots, ATBMI_F16, param_.epsilon, stream);
        if (rc != 0) {
            ATB_LOG(ERROR) << "NormRopeReshape launch failed: " << atbmi_last_error();
        }
        return rc;
    }

private:
    // Reference norm_rope_reshape_operation.cpp:130-176 (NormRopeReshapeCheckImpl910B).
    bool DimCheck(const SVector<TensorDesc> &in) const
    {
        const TensorDesc &x = in.at(0);
        const TensorDesc &gamma = in.at(1);
        const Dims &rope = in.at(2).shape;
        const Dims &cos = in.at(3).shape;
        const Dims &sin = in.at(4).shape;
        const Dims &cache = in.at(6).shape;
        if (x.dtype != gamma.dtype || x.format != gamma.format || gamma.shape.dims[0] != x.shape.dims[2]) {
            ATB_LOG(ERROR) << "NormRopeReshape: gamma must have x's dtype, format and last dim";
            return false;
        }
        if (x.shape.dims[0] != rope.dims[0] || x.shape.dims[0] != cos.dims[0]) {
            ATB_LOG(ERROR) << "NormRopeReshape: x, keyRope and cos must have the same rows";
            return false;
        }
        if (rope.dims[1] != cos.dims[1] || rope.dims[1] != sin.dims[1]) {
            ATB_LOG(ERROR) << "NormRopeReshape: keyRope, cos and sin must have the same row size";
            return false;
        }
        if (cache.dims[3] != x.shape.dims[2] + rope.dims[1]) {
            ATB_LOG(ERROR) << "NormRopeReshape: the cache row must hold x's row and keyRope's row";
            return false;
        }
        if (x.shape.dims[2] % 16 != 0 || gamma.shape.dims[0] % 16 != 0) {
            ATB_LOG(ERROR) << "NormRopeReshape: the last dim of x and gamma must be a multiple of 16";
            return false;
        }
        return true;
    }

    Param param_;
};
} // namespace

// Reference norm_rope_reshape_operation.cpp:35-55.
template <> Status CreateOperation(const infer::NormRopeReshapeParam &opParam, Operation **operation)
{
    if (operation == nullptr) {
        return ERROR_INVALID_PARAM;
    }
    if (!ReservedIsZero(opParam)) {
        ATB_LOG(ERROR) << "NormRopeReshapeParam rsv has a non-zero byte";
        return ERROR_INVALID_PARAM;
    }
    if (std::fabs(opParam.epsilon) < std::numeric_limits<float>::min()) {
        ATB_LOG(ERROR) << "NormRopeReshapeParam: epsilon must not be (nearly) zero";
        return ERROR_INVALID_PARAM;
    }
    if (opParam.rotaryCoeff != 2) {
        ATB_LOG(ERROR) << "NormRopeReshapeParam: only rotaryCoeff 2 (rotate halves) is implemented on MI355X";
        return ERROR_INVALID_PARAM;
    }
    *operation = new (std::nothrow) NormRopeReshapeOperation(opParam);
    if (*operation == nullptr) {
        return ERROR_OUT_OF_HOST_MEMORY;
    }
    return NO_ERROR;
}
} // namespace atb
