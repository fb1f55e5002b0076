// ReshapeAndCacheWithStrideOperation on MI355X: ReshapeAndCache for key / value inputs that are
// strided views of larger buffers (a slice of a fused QKV projection, for instance). The element
// strides [3] and the element offset [1] of each view arrive as host int64 tensors
// (reference src/ops/ops_infer/reshape_and_cache_with_stride/reshape_and_cache_with_stride_operation.cpp:51-88
// create, :116-148 tensor counts / InferShape, :163-299 dim checks;
// reshape_and_cache_with_stride_ops_runner.cpp:78-104 and ..._ops_runner_SISO.cpp: strides and offset
// are read from hostData at every Setup).
//
// Supported: COMPRESS_TYPE_UNDEFINED with K_CACHE_V_CACHE or K_CACHE_V_BYPASS. Head compression is
// Ascend-specific and rejected at creation.
#include <new>
#include "atb/infer_op_params.h"
#include "atb/utils.h"
#include "atbmi_kernels.h"
#include "log.h"
#include "operation_base.h"

namespace atb {
namespace {
using Param = infer::ReshapeAndCacheWithStrideParam;

// Reference ops_configs/atb_ops_info.ini:923-956 and :1040-1058.
OpIr MakeIr(bool siso)
{
    OpIr ir;
    for (aclDataType t : {ACL_FLOAT16, ACL_BF16}) {
        IrCombo c;
        if (siso) {
            c.inDtypes = {t, t, ACL_INT32, ACL_INT64, ACL_INT64};
            c.outDtypes = {t};
        } else {
            c.inDtypes = {t, t, t, t, ACL_INT32, ACL_INT64, ACL_INT64, ACL_INT64, ACL_INT64};
            c.outDtypes = {t, t};
        }
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

class ReshapeAndCacheWithStrideOperation : public OperationBase {
public:
    explicit ReshapeAndCacheWithStrideOperation(const Param &param)
        : OperationBase("ReshapeAndCacheWithStrideOperation"), siso_(param.kvCacheCfg == Param::K_CACHE_V_BYPASS)
    {
        static const OpIr normal = MakeIr(false);
        static const OpIr single = MakeIr(true);
        ir_ = siso_ ? &single : &normal;
    }

    uint32_t GetInputNum() const override { return siso_ ? 5 : 9; }
    uint32_t GetOutputNum() const override { return siso_ ? 1 : 2; }

protected:
    Status InferShapeImpl(const SVector<TensorDesc> &in, SVector<TensorDesc> &out) const override
    {
        if (siso_) {
            out.at(0) = in.at(1);
        } else {
            out.at(0) = in.at(2);
            out.at(1) = in.at(3);
        }
        return NO_ERROR;
    }

    Status InferShapeCheckImpl(const SVector<TensorDesc> &in) const override
    {
        return siso_ ? DimCheckSiso(in) : DimCheck(in);
    }

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
        if (!SameDesc(in.at(siso_ ? 1 : 2), outTensors.at(0).desc) ||
            (!siso_ && !SameDesc(in.at(3), outTensors.at(1).desc))) {
            ATB_LOG(ERROR) << "ReshapeAndCacheWithStride: output descs must equal the cache input descs";
            return ERROR_INVALID_TENSOR_DIM;
        }
        return NO_ERROR;
    }

    // The strides and offsets are host data, read at every Setup as the reference's runners do.
    // The reference takes whatever the host tensors hold; here a view has exactly three strides and
    // one offset, and the host pointers must be there.
    Status PlanImpl(const VariantPack &pack, uint64_t &workspaceSize) override
    {
        const size_t kStrideIdx = siso_ ? 3 : 5;
        const size_t kOffsetIdx = siso_ ? 4 : 7;
        Status st = ReadView(pack.inTensors.at(kStrideIdx), pack.inTensors.at(kOffsetIdx), kStrides_, kOffset_);
        if (st != NO_ERROR) {
            return st;
        }
        if (!siso_) {
            st = ReadView(pack.inTensors.at(6), pack.inTensors.at(8), vStrides_, vOffset_);
            if (st != NO_ERROR) {
                return st;
            }
        }
        workspaceSize = 0;
        return NO_ERROR;
    }

    Status LaunchImpl(const VariantPack &pack, uint8_t *, uint64_t, aclrtStream stream) override
    {
        const Tensor &key = pack.inTensors.at(0);
        const Tensor &keyCacheIn = pack.inTensors.at(siso_ ? 1 : 2);
        const Tensor &slots = pack.inTensors.at(siso_ ? 2 : 4);
        const Tensor &keyCacheOut = pack.outTensors.at(0);
        const int64_t tokens = key.desc.shape.dims[0];
        const int64_t heads = key.desc.shape.dims[1];
        const int64_t dk = key.desc.shape.dims[2];
        const int64_t numSlots = keyCacheIn.desc.shape.dims[0] * keyCacheIn.desc.shape.dims[1];
        const void *value = nullptr;
        void *valueCache = nullptr;
        int64_t dv = 0;
        if (!siso_) {
            value = pack.inTensors.at(1).deviceData;
            valueCache = pack.outTensors.at(1).deviceData;
            dv = pack.inTensors.at(1).desc.shape.dims[2];
            if (!value || !valueCache) {
                ATB_LOG(ERROR) << "ReshapeAndCacheWithStride: value / valueCache device pointer is null";
                return ERROR_INVALID_PARAM;
            }
        }
        if (!key.deviceData || !keyCacheOut.deviceData || !slots.deviceData) {
            ATB_LOG(ERROR) << "ReshapeAndCacheWithStride: key / keyCache / slotMapping device pointer is null";
            return ERROR_INVALID_PARAM;
        }
        // the slot tensor bounds the rows written (the SISO form requires it to match the token count)
        const int64_t rows = tokens < slots.desc.shape.dims[0] ? tokens : slots.desc.shape.dims[0];
        int rc = atbmi_reshape_and_cache_strided(key.deviceData, value, keyCacheOut.deviceData, valueCache,
                                                 static_cast<const int32_t *>(slots.deviceData), rows, heads, dk, dv,
                                                 numSlots, 2, kStrides_, kOffset_, siso_ ? nullptr : vStrides_,
                                                 vOffset_, stream);
        if (rc != 0) {
            ATB_LOG(ERROR) << "ReshapeAndCacheWithStride launch failed: " << atbmi_last_error();
        }
        return rc;
    }

private:
    static Status ReadView(const Tensor &strides, const Tensor &offset, int64_t *outStrides, int64_t &outOffset)
    {
        if (strides.hostData == nullptr || offset.hostData == nullptr) {
            ATB_LOG(ERROR) << "ReshapeAndCacheWithStride: strides and offset are host tensors, hostData is null";
            return ERROR_INVALID_PARAM;
        }
        if (strides.desc.shape.dims[0] != 3 || offset.desc.shape.dims[0] < 1) {
            ATB_LOG(ERROR) << "ReshapeAndCacheWithStride: a view has 3 strides and 1 offset";
            return ERROR_INVALID_TENSOR_DIM;
        }
        for (int i = 0; i < 3; ++i) {
            outStrides[i] = static_cast<const int64_t *>(strides.hostData)[i];
        }
        outOffset = static_cast<const int64_t *>(offset.hostData)[0];
        return NO_ERROR;
    }

    // Reference reshape_and_cache_with_stride_operation.cpp:189-226 (DimCheck) and :255-299
    // (KVCacheDimCheck910B, the part without head compression).
    Status DimCheck(const SVector<TensorDesc> &in) const
    {
        if (in.at(0).shape.dimNum != 3 || in.at(1).shape.dimNum != 3 || in.at(2).shape.dimNum != 4 ||
            in.at(3).shape.dimNum != 4) {
            ATB_LOG(ERROR) << "ReshapeAndCacheWithStride: expected dims 3/3/4/4/1/1/1/1/1";
            return ERROR_INVALID_TENSOR_DIM_NUM;
        }
        for (size_t i = 4; i < 9; ++i) {
            if (in.at(i).shape.dimNum != 1) {
                ATB_LOG(ERROR) << "ReshapeAndCacheWithStride: expected dims 3/3/4/4/1/1/1/1/1";
                return ERROR_INVALID_TENSOR_DIM_NUM;
            }
        }
        const Dims &k = in.at(0).shape;
        const Dims &v = in.at(1).shape;
        const Dims &kc = in.at(2).shape;
        const Dims &vc = in.at(3).shape;
        if (k.dims[0] != v.dims[0] || k.dims[1] != v.dims[1]) {
            ATB_LOG(ERROR) << "ReshapeAndCacheWithStride: key and value must agree on tokens and heads";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (kc.dims[0] != vc.dims[0] || kc.dims[1] != vc.dims[1]) {
            ATB_LOG(ERROR) << "ReshapeAndCacheWithStride: caches must agree on numBlocks and blockSize";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (k.dims[1] != kc.dims[2] || v.dims[1] != vc.dims[2]) {
            ATB_LOG(ERROR) << "ReshapeAndCacheWithStride: head count of key/value must equal that of the caches";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (k.dims[2] != kc.dims[3] || v.dims[2] != vc.dims[3]) {
            ATB_LOG(ERROR) << "ReshapeAndCacheWithStride: head size of key/value must equal that of the caches";
            return ERROR_INVALID_TENSOR_DIM;
        }
        return NO_ERROR;
    }

    // Reference reshape_and_cache_with_stride_operation.cpp:228-253 (DimCheckSISO).
    Status DimCheckSiso(const SVector<TensorDesc> &in) const
    {
        if (in.at(0).shape.dimNum != 3 || in.at(1).shape.dimNum != 4 || in.at(2).shape.dimNum != 1 ||
            in.at(3).shape.dimNum != 1 || in.at(4).shape.dimNum != 1) {
            ATB_LOG(ERROR) << "ReshapeAndCacheWithStride: expected dims 3/4/1/1/1";
            return ERROR_INVALID_TENSOR_DIM_NUM;
        }
        const Dims &k = in.at(0).shape;
        const Dims &kc = in.at(1).shape;
        if (k.dims[0] != in.at(2).shape.dims[0] || k.dims[1] != kc.dims[2] || k.dims[2] != kc.dims[3]) {
            ATB_LOG(ERROR) << "ReshapeAndCacheWithStride: key does not match keyCache / slotMapping";
            return ERROR_INVALID_TENSOR_DIM;
        }
        return NO_ERROR;
    }

    bool siso_;
    int64_t kStrides_[3] = {0, 0, 0};
    int64_t vStrides_[3] = {0, 0, 0};
    int64_t kOffset_ = 0;
    int64_t vOffset_ = 0;
};
} // namespace

// Reference reshape_and_cache_with_stride_operation.cpp:51-88. The reference refuses K_CACHE_V_BYPASS
// and head compression outside its 910B products; here the single-cache form is available and head
// compression is not.
template <> Status CreateOperation(const infer::ReshapeAndCacheWithStrideParam &opParam, Operation **operation)
{
    if (operation == nullptr) {
        return ERROR_INVALID_PARAM;
    }
    if (!ReservedIsZero(opParam)) {
        ATB_LOG(ERROR) << "ReshapeAndCacheWithStrideParam rsv has a non-zero byte";
        return ERROR_INVALID_PARAM;
    }
    if (opParam.compressType < Param::COMPRESS_TYPE_UNDEFINED || opParam.compressType > Param::COMPRESS_TYPE_KVHEAD_ROPE ||
        opParam.kvCacheCfg < Param::K_CACHE_V_CACHE || opParam.kvCacheCfg > Param::K_CACHE_V_BYPASS) {
        ATB_LOG(ERROR) << "ReshapeAndCacheWithStrideParam enum value out of range";
        return ERROR_INVALID_PARAM;
    }
    if (opParam.compressType != Param::COMPRESS_TYPE_UNDEFINED) {
        ATB_LOG(ERROR) << "ReshapeAndCacheWithStrideParam: head compression is not implemented on MI355X";
        return ERROR_INVALID_PARAM;
    }
    *operation = new (std::nothrow) ReshapeAndCacheWithStrideOperation(opParam);
    if (*operation == nullptr) {
        return ERROR_OUT_OF_HOST_MEMORY;
    }
    return NO_ERROR;
}
} // namespace atb
