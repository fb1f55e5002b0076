// BlockCopyOperation on MI355X: copies blocks of the key and value caches onto
// other blocks of the same caches (the cache side of beam search / prefix
// sharing). Checks as in the reference operator for its Atlas 800I A2 feature
// set (reference src/ops/ops_infer/block_copy/block_copy_operation.cpp:30-47
// create, :57-67 counts, :69-99 InferShape checks, :109-156 Setup checks; dtype
// table ops_configs/atb_ops_info.ini:134-155 without its fractal-NZ column).
// Inputs: keyCache, valueCache [blocks, blockSize, heads, headSize], srcBlocks
// [n], dstBlocks [m], cumSum [n]; no outputs, the caches are updated in place.
#include <new>
#include "atb/infer_op_params.h"
#include "atb/utils.h"
#include "atbmi_kernels.h"
#include "log.h"
#include "operation_base.h"

namespace atb {
namespace {
using Param = infer::BlockCopyParam;
constexpr size_t KEY_CACHE = 0, VALUE_CACHE = 1, SRC_BLOCKS = 2, DST_BLOCKS = 3, CUM_SUM = 4;

OpIr MakeIr()
{
    OpIr ir;
    for (aclDataType t : {ACL_FLOAT16, ACL_BF16, ACL_INT8}) {
        IrCombo c;
        c.inDtypes = {t, t, ACL_INT32, ACL_INT32, ACL_INT32};
        c.inFormats.assign(c.inDtypes.size(), ACL_FORMAT_ND);
        ir.push_back(c);
    }
    return ir;
}

bool SameShape(const Dims &a, const Dims &b)
{
    if (a.dimNum != b.dimNum) {
        return false;
    }
    for (uint64_t i = 0; i < a.dimNum; ++i) {
        if (a.dims[i] != b.dims[i]) {
            return false;
        }
    }
    return true;
}

class BlockCopyOperation : public OperationBase {
public:
    explicit BlockCopyOperation(const Param &param) : OperationBase("BlockCopyOperation"), param_(param)
    {
        static const OpIr table = MakeIr();
        ir_ = &table;
    }

    uint32_t GetInputNum() const override { return 5; }
    uint32_t GetOutputNum() const override { return 0; }

protected:
    Status InferShapeImpl(const SVector<TensorDesc> &in, SVector<TensorDesc> &out) const override
    {
        (void)in;
        (void)out;
        return NO_ERROR;
    }

    // Reference :69-99.
    Status InferShapeCheckImpl(const SVector<TensorDesc> &in) const override
    {
        const int64_t blockCount = in.at(KEY_CACHE).shape.dims[0];
        if (!SameShape(in.at(KEY_CACHE).shape, in.at(VALUE_CACHE).shape)) {
            ATB_LOG(ERROR) << "keyCache and valueCache should have the same shape";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (in.at(KEY_CACHE).shape.dimNum != 4) {
            ATB_LOG(ERROR) << "the caches should have 4 dims";
            return ERROR_INVALID_TENSOR_DIM_NUM;
        }
        if (in.at(SRC_BLOCKS).shape.dimNum != 1 || in.at(DST_BLOCKS).shape.dimNum != 1) {
            ATB_LOG(ERROR) << "the block index vectors should have 1 dim";
            return ERROR_INVALID_TENSOR_DIM_NUM;
        }
        if (!SameShape(in.at(CUM_SUM).shape, in.at(SRC_BLOCKS).shape)) {
            ATB_LOG(ERROR) << "cumSum should have the shape of srcBlocks";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (in.at(SRC_BLOCKS).shape.dims[0] > blockCount || in.at(DST_BLOCKS).shape.dims[0] > blockCount) {
            ATB_LOG(ERROR) << "more block indices than the caches have blocks";
            return ERROR_INVALID_TENSOR_DIM;
        }
        return NO_ERROR;
    }

    Status SetupCheckImpl(const SVector<Tensor> &inTensors, const SVector<Tensor> &outTensors) const override
    {
        (void)outTensors;
        SVector<TensorDesc> in;
        for (size_t i = 0; i < inTensors.size(); ++i) {
            in.push_back(inTensors.at(i).desc);
        }
        return InferShapeCheckImpl(in);
    }

    Status PlanImpl(const VariantPack &pack, uint64_t &workspaceSize) override
    {
        (void)pack;
        workspaceSize = 0;
        return NO_ERROR;
    }

    Status LaunchImpl(const VariantPack &pack, uint8_t *workspace, uint64_t workspaceSize, aclrtStream stream) override
    {
        (void)workspace;
        (void)workspaceSize;
        const Tensor &kc = pack.inTensors.at(KEY_CACHE);
        const Dims &s = kc.desc.shape;
        const int64_t elem = kc.desc.dtype == ACL_INT8 ? 1 : 2;
        const int64_t blockBytes = s.dims[1] * s.dims[2] * s.dims[3] * elem;
        int rc = atbmi_block_copy(kc.deviceData, pack.inTensors.at(VALUE_CACHE).deviceData,
                                  static_cast<const int32_t *>(pack.inTensors.at(SRC_BLOCKS).deviceData),
                                  static_cast<const int32_t *>(pack.inTensors.at(DST_BLOCKS).deviceData),
                                  static_cast<const int32_t *>(pack.inTensors.at(CUM_SUM).deviceData),
                                  pack.inTensors.at(SRC_BLOCKS).desc.shape.dims[0],
                                  pack.inTensors.at(DST_BLOCKS).desc.shape.dims[0], s.dims[0], blockBytes, blockBytes,
                                  stream);
        if (rc != 0) {
            ATB_LOG(ERROR) << "BlockCopy launch failed: " << atbmi_last_error();
        }
        return rc;
    }

private:
    Param param_;
};
} // namespace

template <> Status CreateOperation(const infer::BlockCopyParam &opParam, Operation **operation)
{
    if (operation == nullptr) {
        return ERROR_INVALID_PARAM;
    }
    if (!ReservedIsZero(opParam)) {
        ATB_LOG(ERROR) << "BlockCopyParam rsv has a non-zero byte";
        return ERROR_INVALID_PARAM;
    }
    *operation = new (std::nothrow) BlockCopyOperation(opParam);
    if (*operation == nullptr) {
        return ERROR_OUT_OF_HOST_MEMORY;
    }
    return NO_ERROR;
}
} // namespace atb
