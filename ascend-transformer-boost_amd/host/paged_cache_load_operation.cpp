// PagedCacheLoadOperation on MI355X: gathers the cached K and V rows of every
// sequence into contiguous tensors, the reverse of ReshapeAndCache. Checks as in
// the reference operator (reference src/ops/ops_infer/paged_cache_load/
// paged_cache_load_operation.cpp:51-78 create, :95-115 counts and InferShape,
// :117-148 Setup checks, :150-206 DimCheck, :261-297 ND cache rules; dtype table
// ops_configs/atb_ops_info.ini section PagedCacheLoadOperationND).
// Inputs: keyCache [blocks, blockSize, heads, headSizeK], valueCache [.., headSizeV],
// blockTables [batch, maxBlocks], seqLens [batch] (or running sums [batch + 1]),
// key [tokens, heads, headSizeK], value [tokens, heads, headSizeV], seqStarts [batch];
// outputs alias key and value. The lengths stay on the device.
//
// Implemented: kvCacheCfg K_CACHE_V_CACHE_ND. The fractal-NZ cache layout is
// Ascend-specific and rejected at creation.
#include <algorithm>
#include <new>
#include "atb/infer_op_params.h"
#include "atb/utils.h"
#include "atbmi_kernels.h"
#include "log.h"
#include "operation_base.h"

namespace atb {
namespace {
using Param = infer::PagedCacheLoadParam;
constexpr size_t KEY_CACHE = 0, VALUE_CACHE = 1, BLOCK_TABLES = 2, SEQ_LENS = 3, KEY = 4, VALUE = 5, SEQ_STARTS = 6;

OpIr MakeIr()
{
    OpIr ir;
    for (aclDataType t : {ACL_FLOAT16, ACL_INT8, ACL_BF16}) {
        IrCombo c;
        c.inDtypes = {t, t, ACL_INT32, ACL_INT32, t, t, ACL_INT32};
        c.inFormats.assign(c.inDtypes.size(), ACL_FORMAT_ND);
        c.outDtypes = {t, t};
        c.outFormats = {ACL_FORMAT_ND, ACL_FORMAT_ND};
        ir.push_back(c);
    }
    return ir;
}

class PagedCacheLoadOperation : public OperationBase {
public:
    explicit PagedCacheLoadOperation(const Param &param) : OperationBase("PagedCacheLoadOperation"), param_(param)
    {
        static const OpIr table = MakeIr();
        ir_ = &table;
    }

    uint32_t GetInputNum() const override { return 7; }
    uint32_t GetOutputNum() const override { return 2; }

protected:
    Status InferShapeImpl(const SVector<TensorDesc> &in, SVector<TensorDesc> &out) const override
    {
        out.at(0) = in.at(KEY);
        out.at(1) = in.at(VALUE);
        return NO_ERROR;
    }

    Status InferShapeCheckImpl(const SVector<TensorDesc> &in) const override { return DimCheck(in); }

    // Reference :117-148.
    Status SetupCheckImpl(const SVector<Tensor> &inTensors, const SVector<Tensor> &outTensors) const override
    {
        SVector<TensorDesc> in;
        for (size_t i = 0; i < inTensors.size(); ++i) {
            in.push_back(inTensors.at(i).desc);
        }
        const Dims &ok = outTensors.at(0).desc.shape;
        const Dims &ov = outTensors.at(1).desc.shape;
        if (ok.dims[1] != in.at(KEY_CACHE).shape.dims[2] || ok.dims[2] != in.at(KEY_CACHE).shape.dims[3] ||
            ov.dims[1] != in.at(VALUE_CACHE).shape.dims[2] || ov.dims[2] != in.at(VALUE_CACHE).shape.dims[3]) {
            ATB_LOG(ERROR) << "the outputs should have the heads and head sizes of the caches";
            return ERROR_INVALID_TENSOR_DIM;
        }
        return DimCheck(in);
    }

    Status PlanImpl(const VariantPack &pack, uint64_t &workspaceSize) override
    {
        const Dims &k = pack.inTensors.at(KEY).desc.shape;
        const Dims &v = pack.inTensors.at(VALUE).desc.shape;
        const Dims &kc = pack.inTensors.at(KEY_CACHE).desc.shape;
        const Dims &vc = pack.inTensors.at(VALUE_CACHE).desc.shape;
        if (k.dims[1] != kc.dims[2] || k.dims[2] != kc.dims[3] || v.dims[1] != vc.dims[2] || v.dims[2] != vc.dims[3]) {
            ATB_LOG(ERROR) << "key and value should have the heads and head sizes of the caches";
            return ERROR_INVALID_PARAM;
        }
        if (pack.outTensors.at(0).deviceData != pack.inTensors.at(KEY).deviceData ||
            pack.outTensors.at(1).deviceData != pack.inTensors.at(VALUE).deviceData) {
            ATB_LOG(ERROR) << "the outputs are the key and value inputs, updated in place";
            return ERROR_INVALID_PARAM;
        }
        workspaceSize = 0;
        return NO_ERROR;
    }

    Status LaunchImpl(const VariantPack &pack, uint8_t *workspace, uint64_t workspaceSize, aclrtStream stream) override
    {
        (void)workspace;
        (void)workspaceSize;
        const Tensor &kc = pack.inTensors.at(KEY_CACHE);
        const Tensor &vc = pack.inTensors.at(VALUE_CACHE);
        const Tensor &tables = pack.inTensors.at(BLOCK_TABLES);
        const int64_t elem = kc.desc.dtype == ACL_INT8 ? 1 : 2;
        const int64_t blockSize = kc.desc.shape.dims[1];
        const int64_t outRows = pack.inTensors.at(KEY).desc.shape.dims[0];
        // no sequence is longer than its block-table row reaches or than the output holds
        const int64_t maxSeqLen = std::min(outRows, tables.desc.shape.dims[1] * blockSize);
        int rc = atbmi_paged_cache_load(
            kc.deviceData, vc.deviceData, static_cast<const int32_t *>(tables.deviceData),
            static_cast<const int32_t *>(pack.inTensors.at(SEQ_LENS).deviceData),
            param_.hasSeqStarts ? static_cast<const int32_t *>(pack.inTensors.at(SEQ_STARTS).deviceData) : nullptr,
            pack.inTensors.at(KEY).deviceData, pack.inTensors.at(VALUE).deviceData, tables.desc.shape.dims[0],
            tables.desc.shape.dims[1], blockSize, kc.desc.shape.dims[0],
            kc.desc.shape.dims[2] * kc.desc.shape.dims[3] * elem, vc.desc.shape.dims[2] * vc.desc.shape.dims[3] * elem,
            outRows, maxSeqLen, param_.isSeqLensCumsumMode ? 1 : 0, stream);
        if (rc != 0) {
            ATB_LOG(ERROR) << "PagedCacheLoad launch failed: " << atbmi_last_error();
        }
        return rc;
    }

private:
    // Reference :150-206 with :261-297.
    Status DimCheck(const SVector<TensorDesc> &in) const
    {
        if (in.at(KEY_CACHE).shape.dims[0] != in.at(VALUE_CACHE).shape.dims[0]) {
            ATB_LOG(ERROR) << "numBlocks of the caches should be the same";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (in.at(KEY).shape.dims[0] != in.at(VALUE).shape.dims[0]) {
            ATB_LOG(ERROR) << "key and value should hold the same number of tokens";
            return ERROR_INVALID_TENSOR_DIM;
        }
        const int64_t blockSize = in.at(KEY_CACHE).shape.dims[1];
        const int64_t heads = in.at(KEY_CACHE).shape.dims[2];
        if (blockSize != in.at(VALUE_CACHE).shape.dims[1]) {
            ATB_LOG(ERROR) << "blockSize of the caches should be the same";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (heads != in.at(VALUE_CACHE).shape.dims[2]) {
            ATB_LOG(ERROR) << "numHeads of the caches should be the same";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (blockSize == 0) {
            ATB_LOG(ERROR) << "blockSize cannot be zero";
            return ERROR_INVALID_TENSOR_DIM;
        }
        const int64_t batch = in.at(BLOCK_TABLES).shape.dims[0];
        if (batch != in.at(SEQ_LENS).shape.dims[0] - (param_.isSeqLensCumsumMode ? 1 : 0)) {
            ATB_LOG(ERROR) << "seqLens should have one entry per row of blockTables (one more in cumsum mode)";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (in.at(KEY_CACHE).shape.dimNum != 4 || in.at(VALUE_CACHE).shape.dimNum != 4 ||
            in.at(BLOCK_TABLES).shape.dimNum != 2 || in.at(SEQ_LENS).shape.dimNum != 1 || in.at(KEY).shape.dimNum != 3 ||
            in.at(VALUE).shape.dimNum != 3 || in.at(SEQ_STARTS).shape.dimNum != 1) {
            ATB_LOG(ERROR) << "expected dims: caches 4, blockTables 2, seqLens 1, key 3, value 3, seqStarts 1";
            return ERROR_INVALID_TENSOR_DIM_NUM;
        }
        const int64_t align = in.at(KEY_CACHE).dtype == ACL_INT8 ? 32 : 16;
        if (heads * in.at(KEY_CACHE).shape.dims[3] % align != 0 || heads * in.at(VALUE_CACHE).shape.dims[3] % align != 0) {
            ATB_LOG(ERROR) << "numHeads * headSize should be a multiple of " << align;
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (param_.hasSeqStarts && in.at(SEQ_STARTS).shape.dims[0] != batch) {
            ATB_LOG(ERROR) << "seqStarts should have one entry per sequence";
            return ERROR_INVALID_TENSOR_DIM;
        }
        return NO_ERROR;
    }

    Param param_;
};
} // namespace

template <> Status CreateOperation(const infer::PagedCacheLoadParam &opParam, Operation **operation)
{
    if (operation == nullptr) {
        return ERROR_INVALID_PARAM;
    }
    if (!ReservedIsZero(opParam)) {
        ATB_LOG(ERROR) << "PagedCacheLoadParam rsv has a non-zero byte";
        return ERROR_INVALID_PARAM;
    }
    if (opParam.kvCacheCfg < Param::K_CACHE_V_CACHE_NZ || opParam.kvCacheCfg > Param::K_CACHE_V_CACHE_ND) {
        ATB_LOG(ERROR) << "wrong kvCacheCfg";
        return ERROR_INVALID_PARAM;
    }
    if (opParam.kvCacheCfg == Param::K_CACHE_V_CACHE_NZ && (opParam.hasSeqStarts || opParam.isSeqLensCumsumMode)) {
        ATB_LOG(ERROR) << "the NZ format takes neither hasSeqStarts nor isSeqLensCumsumMode";
        return ERROR_INVALID_PARAM;
    }
    if (opParam.kvCacheCfg == Param::K_CACHE_V_CACHE_NZ) {
        ATB_LOG(ERROR) << "PagedCacheLoad: fractal-NZ caches not implemented on MI355X";
        return ERROR_INVALID_PARAM;
    }
    *operation = new (std::nothrow) PagedCacheLoadOperation(opParam);
    if (*operation == nullptr) {
        return ERROR_OUT_OF_HOST_MEMORY;
    }
    return NO_ERROR;
}
} // namespace atb
