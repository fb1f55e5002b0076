// PagedCacheLoadOperation on MI355X: gathers the cached K and V rows of every
// sequence into contiguous tensors, the reverse of ReshapeAndCache. Checks as in
// the reference operator (reference src/ops/ops_infer/paged_cache_load/
// paged_cache_load_operation.cpp:51-78 create, :95-115 counts and InferShape,
// :117-148 Setup checks, :150-206 DimCheck, :208-259 NZ cache rules, :261-297 ND cache
// rules; dtype tables ops_configs/atb_ops_info.ini sections PagedCacheLoadOperation and
// PagedCacheLoadOperationND).
// K_CACHE_V_CACHE_ND inputs: keyCache [blocks, blockSize, heads, headSizeK], valueCache
// [.., headSizeV], blockTables [batch, maxBlocks], seqLens [batch] (or running sums
// [batch + 1]), key [tokens, heads, headSizeK], value [tokens, heads, headSizeV],
// seqStarts [batch]. K_CACHE_V_CACHE_NZ (the param's default) inputs: keyCache
// [blocks, heads * headSizeK / L, blockSize, L] and valueCache likewise in the fractal-NZ
// format (L = 32 for int8, 16 for 16-bit elements), blockTables, seqLens [batch],
// key [tokens, heads * headSizeK], value [tokens, heads * headSizeV]. The outputs alias
// key and value. The lengths stay on the device.
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

// reference ops_configs/atb_ops_info.ini:7155-7179: equal 16-bit or int8 caches, or an int8 key cache with a
// 16-bit value cache
OpIr MakeNzIr()
{
    OpIr ir;
    const aclDataType pairs[5][2] = {{ACL_FLOAT16, ACL_FLOAT16}, {ACL_INT8, ACL_INT8}, {ACL_BF16, ACL_BF16},
                                     {ACL_INT8, ACL_FLOAT16},    {ACL_INT8, ACL_BF16}};
    for (const auto &p : pairs) {
        IrCombo c;
        c.inDtypes = {p[0], p[1], ACL_INT32, ACL_INT32, p[0], p[1]};
        c.inFormats = {ACL_FORMAT_FRACTAL_NZ, ACL_FORMAT_FRACTAL_NZ, ACL_FORMAT_ND, ACL_FORMAT_ND, ACL_FORMAT_ND,
                       ACL_FORMAT_ND};
        c.outDtypes = {p[0], p[1]};
        c.outFormats = {ACL_FORMAT_ND, ACL_FORMAT_ND};
        ir.push_back(c);
    }
    return ir;
}

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
    explicit PagedCacheLoadOperation(const Param &param)
        : OperationBase("PagedCacheLoadOperation"), param_(param), nz_(param.kvCacheCfg == Param::K_CACHE_V_CACHE_NZ)
    {
        static const OpIr table = MakeIr();
        static const OpIr fractal = MakeNzIr();
        ir_ = nz_ ? &fractal : &table;
    }

    uint32_t GetInputNum() const override { return nz_ ? 6 : 7; }
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
        if (nz_) {
            if (ok.dims[1] != in.at(KEY_CACHE).shape.dims[1] * in.at(KEY_CACHE).shape.dims[3] ||
                ov.dims[1] != in.at(VALUE_CACHE).shape.dims[1] * in.at(VALUE_CACHE).shape.dims[3]) {
                ATB_LOG(ERROR) << "the rows of the outputs should have dims 1 x 3 of the caches as their length";
                return ERROR_INVALID_TENSOR_DIM;
            }
            return DimCheck(in);
        }
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
        if (nz_ && (k.dims[1] != kc.dims[1] * kc.dims[3] || v.dims[1] != vc.dims[1] * vc.dims[3])) {
            ATB_LOG(ERROR) << "key and value rows should be as long as dims 1 x 3 of the caches";
            return ERROR_INVALID_PARAM;
        }
        if (!nz_ && (k.dims[1] != kc.dims[2] || k.dims[2] != kc.dims[3] || v.dims[1] != vc.dims[2] || v.dims[2] != vc.dims[3])) {
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
        const int64_t blockSize = kc.desc.shape.dims[nz_ ? 2 : 1];
        const int64_t outRows = pack.inTensors.at(KEY).desc.shape.dims[0];
        // no sequence is longer than its block-table row reaches or than the output holds
        const int64_t maxSeqLen = std::min(outRows, tables.desc.shape.dims[1] * blockSize);
        if (nz_) {
            const int64_t velem = vc.desc.dtype == ACL_INT8 ? 1 : 2;
            int rc = atbmi_paged_cache_load_nz(
                kc.deviceData, vc.deviceData, static_cast<const int32_t *>(tables.deviceData),
                static_cast<const int32_t *>(pack.inTensors.at(SEQ_LENS).deviceData), pack.inTensors.at(KEY).deviceData,
                pack.inTensors.at(VALUE).deviceData, tables.desc.shape.dims[0], tables.desc.shape.dims[1], blockSize,
                kc.desc.shape.dims[0], kc.desc.shape.dims[1] * kc.desc.shape.dims[3] * elem,
                vc.desc.shape.dims[1] * vc.desc.shape.dims[3] * velem, kc.desc.shape.dims[3] * elem,
                vc.desc.shape.dims[3] * velem, outRows, maxSeqLen, stream);
            if (rc != 0) {
                ATB_LOG(ERROR) << "PagedCacheLoad launch failed: " << atbmi_last_error();
            }
            return rc;
        }
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
        if (nz_) {
            return DimCheckNz(in);
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

    // Reference :179-199 (the NZ branch of DimCheck) and :208-259 (KVCacheDimCheck910BNZ), in that order.
    Status DimCheckNz(const SVector<TensorDesc> &in) const
    {
        const int64_t blockSize = in.at(KEY_CACHE).shape.dims[2];
        if (blockSize != in.at(VALUE_CACHE).shape.dims[2]) {
            ATB_LOG(ERROR) << "blockSize of the caches should be the same";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (blockSize == 0 || blockSize % 16 != 0) {
            ATB_LOG(ERROR) << "blockSize should be a non-zero multiple of 16";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (in.at(BLOCK_TABLES).shape.dims[0] != in.at(SEQ_LENS).shape.dims[0]) {
            ATB_LOG(ERROR) << "seqLens should have one entry per row of blockTables";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (in.at(KEY_CACHE).shape.dimNum != 4 || in.at(VALUE_CACHE).shape.dimNum != 4 ||
            in.at(BLOCK_TABLES).shape.dimNum != 2 || in.at(SEQ_LENS).shape.dimNum != 1 || in.at(KEY).shape.dimNum != 2 ||
            in.at(VALUE).shape.dimNum != 2) {
            ATB_LOG(ERROR) << "expected dims: caches 4, blockTables 2, seqLens 1, key 2, value 2";
            return ERROR_INVALID_TENSOR_DIM_NUM;
        }
        const int64_t keyLast = in.at(KEY_CACHE).dtype == ACL_INT8 ? 32 : 16;
        const int64_t valueLast = in.at(VALUE_CACHE).dtype == ACL_INT8 ? 32 : 16;
        if (in.at(KEY_CACHE).shape.dims[3] != keyLast || in.at(VALUE_CACHE).shape.dims[3] != valueLast) {
            ATB_LOG(ERROR) << "the last dim of an NZ cache should be 32 for int8 and 16 for 16-bit elements";
            return ERROR_INVALID_TENSOR_DIM;
        }
        // the reference's bound on a row, as it writes it (dim 1 times 32 for every dtype)
        constexpr int64_t MAX_ROW = 147456;
        if (in.at(KEY_CACHE).shape.dims[1] * 32 > MAX_ROW || in.at(VALUE_CACHE).shape.dims[1] * 32 > MAX_ROW) {
            ATB_LOG(ERROR) << "numHeads * headSize of the caches should stay within " << MAX_ROW;
            return ERROR_INVALID_TENSOR_DIM;
        }
        return NO_ERROR;
    }

    Param param_;
    bool nz_;
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
    *operation = new (std::nothrow) PagedCacheLoadOperation(opParam);
    if (*operation == nullptr) {
        return ERROR_OUT_OF_HOST_MEMORY;
    }
    return NO_ERROR;
}
} // namespace atb
