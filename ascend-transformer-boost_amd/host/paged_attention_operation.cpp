// PagedAttentionOperation on MI355X: the decode-attention operator of ATB.
//
// Creation-time parameter checks, tensor counts, InferShape and the dim
// checks follow the reference operator for its Atlas 800I A2 (910B) feature
// set (reference src/ops/ops_infer/paged_attention/paged_attention_operation.cpp:
// 53-70 common, 92-143 create, 145-365 per-feature checks, 408-472 counts and
// InferShape, 561-632 cache dim rules, 663-695 and 926-963 setup dim checks);
// the second validation layer of the reference kernel library is restated in
// PlanImpl (src/kernels/mixkernels/pagedattention/paged_attention_operation.cpp:159-210,
// 284-340, 446-495 and tiling/paged_attention_tiling.cpp:156-192,357-358).
// Context lengths are read from contextLens.hostData during Setup, as the
// reference runner does (src/ops/ops_infer/paged_attention/param.cpp:16-62).
//
// Implemented feature set: fp16/bf16 caches; int8 caches with fp32 per-channel
// descales, plain or uint64-packed, (+ int32 offsets); the MLA combined cache
// (mlaVHeadSize > 0); additive NORM and ALIBI masks; the dynamic-batch status
// input; per-sequence LogN scaling; several query tokens per sequence
// (CALC_TYPE_SPEC) with the SPEC or the square NORM mask; head-major (BNSD)
// caches; head compression with its per-slot score offsets.
// int8 queries over int8 caches (quantType QKV online / offline) run on a kernel of their own
// (csrc/pa_int8q.hip); combined with the MLA cache they are legal in the reference but not implemented
// here; such params are rejected at creation with ERROR_INVALID_PARAM.
// MASK_TYPE_MASK_FREE can be created and fails InferShape / Setup with
// ERROR_INVALID_TENSOR_DIM, as the reference does off Atlas 300I Duo.
#include <vector>
#include <cmath>
#include <new>
#include "atb/infer_op_params.h"
#include "atb/utils.h"
#include "atbmi_kernels.h"
#include "log.h"
#include "operation_base.h"

namespace atb {
namespace {
using Param = infer::PagedAttentionParam;

constexpr int64_t MAX_HEAD_SIZE = 576;
constexpr int64_t MLA_THRESHOLD = 256;
constexpr int64_t BLOCK_LIMIT = 128 * 128;
constexpr int64_t MAX_MLA_BATCH = 8192;

// Reference paged_attention_operation.cpp:53-70.
bool CommonParamCheck(const Param &p)
{
    if (p.headNum <= 0) {
        ATB_LOG(ERROR) << "PagedAttentionParam: headNum = " << p.headNum << ", a positive head count is required";
        return false;
    }
    if (p.kvHeadNum < 0) {
        ATB_LOG(ERROR) << "PagedAttentionParam: kvHeadNum = " << p.kvHeadNum << " is negative (0 means one KV head per query head)";
        return false;
    }
    if (p.kvHeadNum != 0 && p.headNum % p.kvHeadNum != 0) {
        ATB_LOG(ERROR) << "PagedAttentionParam: " << p.headNum << " query heads do not divide into " << p.kvHeadNum << " KV heads";
        return false;
    }
    return true;
}

// The cross-feature rules of the reference (:145-365), in its order.
bool FeatureParamCheck(const Param &p)
{
    if (p.maskType == Param::MASK_TYPE_NORM_COMPRESS) {
        ATB_LOG(ERROR) << "MASK_TYPE_NORM_COMPRESS is an Atlas 300I Duo feature";
        return false;
    }
    if (p.compressType >= Param::COMPRESS_TYPE_MAX || p.compressType < Param::COMPRESS_TYPE_UNDEFINED) {
        ATB_LOG(ERROR) << "compressType out of range";
        return false;
    }
    if (p.compressType == Param::COMPRESS_TYPE_KVHEAD_ROPE &&
        (p.maskType != Param::UNDEFINED || p.batchRunStatusEnable)) {
        ATB_LOG(ERROR) << "COMPRESS_TYPE_KVHEAD_ROPE needs maskType UNDEFINED and no dynamic batch";
        return false;
    }
    if (p.calcType != Param::CALC_TYPE_UNDEFINED) {
        if (p.batchRunStatusEnable || p.compressType != Param::COMPRESS_TYPE_UNDEFINED) {
            ATB_LOG(ERROR) << "SPEC does not support dynamic batch or head compression";
            return false;
        }
        if (p.mlaVHeadSize == 0 && p.maskType != Param::MASK_TYPE_NORM && p.maskType != Param::MASK_TYPE_SPEC) {
            ATB_LOG(ERROR) << "SPEC only supports norm mask and spec mask";
            return false;
        }
    }
    if (p.quantType == Param::TYPE_DEQUANT_FUSION && p.calcType != Param::CALC_TYPE_UNDEFINED) {
        ATB_LOG(ERROR) << "dequant fusion needs calcType CALC_TYPE_UNDEFINED";
        return false;
    }
    if (p.quantType == Param::TYPE_QUANT_QKV_OFFLINE || p.quantType == Param::TYPE_QUANT_QKV_ONLINE) {
        if ((p.outDataType != ACL_FLOAT16 && p.outDataType != ACL_BF16) || p.hasQuantOffset ||
            p.compressType != Param::COMPRESS_TYPE_UNDEFINED || p.calcType != Param::CALC_TYPE_UNDEFINED) {
            ATB_LOG(ERROR) << "QKV quant: outDataType fp16/bf16, no offset, no compress, no SPEC";
            return false;
        }
    }
    if (p.scaleType >= Param::SCALE_TYPE_MAX || p.scaleType < Param::SCALE_TYPE_TOR) {
        ATB_LOG(ERROR) << "scaleType out of range";
        return false;
    }
    if (p.scaleType == Param::SCALE_TYPE_LOGN &&
        (p.quantType != Param::TYPE_QUANT_UNQUANT || p.calcType != Param::CALC_TYPE_UNDEFINED ||
         p.compressType != Param::COMPRESS_TYPE_UNDEFINED)) {
        ATB_LOG(ERROR) << "logN does not combine with quant, SPEC or head compression";
        return false;
    }
    if (p.inputLayout == infer::TYPE_BNSD &&
        (p.calcType == Param::CALC_TYPE_SPEC || p.compressType != Param::COMPRESS_TYPE_UNDEFINED ||
         p.quantType != Param::TYPE_QUANT_UNQUANT || p.scaleType != Param::SCALE_TYPE_TOR)) {
        ATB_LOG(ERROR) << "BNSD does not combine with SPEC, compress, quant or logN";
        return false;
    }
    if (p.mlaVHeadSize > 0) {
        if (p.maskType == Param::MASK_TYPE_ALIBI) {
            ATB_LOG(ERROR) << "mla mode does not support alibi mask";
            return false;
        }
        if (p.calcType == Param::CALC_TYPE_SPEC &&
            (p.maskType == Param::MASK_TYPE_NORM || p.quantType != Param::TYPE_QUANT_UNQUANT ||
             p.batchRunStatusEnable)) {
            ATB_LOG(ERROR) << "mla SPEC does not support norm mask, quant or dynamic batch";
            return false;
        }
        if (p.compressType != Param::COMPRESS_TYPE_UNDEFINED || p.quantType == Param::TYPE_DEQUANT_FUSION ||
            p.scaleType != Param::SCALE_TYPE_TOR || p.inputLayout != infer::TYPE_BSND) {
            ATB_LOG(ERROR) << "mla mode does not support compress, dequant fusion, logN or BNSD";
            return false;
        }
        if (p.kvHeadNum != 1) {
            ATB_LOG(ERROR) << "kvHeadNum should be 1, mla mode only supports MQA";
            return false;
        }
        if (p.mlaVHeadSize > MAX_HEAD_SIZE) {
            ATB_LOG(ERROR) << "mlaVHeadSize should be no greater than 576";
            return false;
        }
    }
    return true;
}

// Features that are legal in the reference but have no MI355X kernel yet.
bool ImplementedCheck(const Param &p)
{
    const char *what = nullptr;
    if ((p.quantType == Param::TYPE_QUANT_QKV_OFFLINE || p.quantType == Param::TYPE_QUANT_QKV_ONLINE) &&
        p.mlaVHeadSize > 0) {
        what = "int8 query quantisation over the MLA cache";
    } else if (p.quantType < Param::TYPE_QUANT_UNQUANT || p.quantType > Param::TYPE_QUANT_QKV_ONLINE) {
        what = "this quantType";
    }
    if (what) {
        ATB_LOG(ERROR) << "PagedAttention: " << what << " not implemented on MI355X";
        return false;
    }
    return true;
}

// One row of the dtype table: query dtype q, and for an int8 cache the dtype of
// its descales, fp32 or uint64-packed fp32 (Utils::QuantParamConvert). Optional
// inputs follow in the reference's order (:408-444).
IrCombo MakeCombo(const Param &p, aclDataType q, aclDataType descale)
{
    IrCombo c;
    const bool dequant = p.quantType == Param::TYPE_DEQUANT_FUSION;
    if (p.mlaVHeadSize > 0) {
        c.inDtypes = {q, q, ACL_INT32, ACL_INT32};
    } else if (dequant) {
        c.inDtypes = {q, ACL_INT8, ACL_INT8, ACL_INT32, ACL_INT32};
    } else {
        c.inDtypes = {q, q, q, ACL_INT32, ACL_INT32};
    }
    if (p.maskType != Param::UNDEFINED) {
        c.inDtypes.push_back(q);
    }
    if (p.batchRunStatusEnable) {
        c.inDtypes.push_back(ACL_INT32);
    }
    if (p.calcType == Param::CALC_TYPE_SPEC) {
        c.inDtypes.push_back(ACL_INT32); // qSeqLens; never together with the descales below
    }
    if (dequant) {
        c.inDtypes.push_back(descale);
        if (p.hasQuantOffset) {
            c.inDtypes.push_back(ACL_INT32);
        }
        c.inDtypes.push_back(descale);
        if (p.hasQuantOffset) {
            c.inDtypes.push_back(ACL_INT32);
        }
    }
    if (p.compressType == Param::COMPRESS_TYPE_KVHEAD_ROPE) {
        c.inDtypes.push_back(ACL_FLOAT); // razorOffset (reference paged_attention_ops_runner.cpp:126-128)
    }
    if (p.scaleType == Param::SCALE_TYPE_LOGN) {
        c.inDtypes.push_back(ACL_FLOAT);
    }
    c.inFormats.assign(c.inDtypes.size(), ACL_FORMAT_ND);
    c.outDtypes = {q};
    c.outFormats = {ACL_FORMAT_ND};
    return c;
}

// int8 query, keys and values; the mask and the output in outDataType; one fp32 descale per query head for the
// scores and one for the values, offline also the factor of the weights (reference ops_configs/atb_ops_info.ini,
// sections PagedAttentionOperationQKVQuantOnline.. / ..Offline.., their int8 columns; inputs :429-436).
IrCombo MakeQkvCombo(const Param &p, aclDataType o)
{
    IrCombo c;
    c.inDtypes = {ACL_INT8, ACL_INT8, ACL_INT8, ACL_INT32, ACL_INT32};
    if (p.maskType != Param::UNDEFINED) {
        c.inDtypes.push_back(o);
    }
    if (p.batchRunStatusEnable) {
        c.inDtypes.push_back(ACL_INT32);
    }
    c.inDtypes.push_back(ACL_FLOAT);
    c.inDtypes.push_back(ACL_FLOAT);
    if (p.quantType == Param::TYPE_QUANT_QKV_OFFLINE) {
        c.inDtypes.push_back(ACL_FLOAT);
    }
    c.inFormats.assign(c.inDtypes.size(), ACL_FORMAT_ND);
    c.outDtypes = {o};
    c.outFormats = {ACL_FORMAT_ND};
    return c;
}

OpIr MakeIr(const Param &p)
{
    OpIr ir;
    if (p.quantType == Param::TYPE_QUANT_QKV_OFFLINE || p.quantType == Param::TYPE_QUANT_QKV_ONLINE) {
        ir.push_back(MakeQkvCombo(p, p.outDataType));
        return ir;
    }
    for (aclDataType q : {ACL_FLOAT16, ACL_BF16}) {
        ir.push_back(MakeCombo(p, q, ACL_FLOAT));
        if (p.quantType == Param::TYPE_DEQUANT_FUSION) {
            ir.push_back(MakeCombo(p, q, ACL_INT64));
        }
    }
    return ir;
}

class PagedAttentionOperation : public OperationBase {
public:
    explicit PagedAttentionOperation(const Param &param)
        : OperationBase("PagedAttentionOperation"), param_(param), mla_(param.mlaVHeadSize > 0),
          dequant_(param.quantType == Param::TYPE_DEQUANT_FUSION), bnsd_(param.inputLayout == infer::TYPE_BNSD),
          compress_(param.compressType != Param::COMPRESS_TYPE_UNDEFINED),
          qkv_(param.quantType == Param::TYPE_QUANT_QKV_OFFLINE || param.quantType == Param::TYPE_QUANT_QKV_ONLINE),
          irTable_(MakeIr(param))
    {
        ir_ = &irTable_;
        tablesIdx_ = mla_ ? 2 : 3;
        lensIdx_ = mla_ ? 3 : 4;
        size_t next = lensIdx_ + 1;
        if (param.maskType != Param::UNDEFINED) {
            maskIdx_ = next++;
        }
        if (param.batchRunStatusEnable) {
            statusIdx_ = next++;
        }
        if (param.calcType == Param::CALC_TYPE_SPEC) {
            qLensIdx_ = next++;
        }
        if (dequant_) {
            kScaleIdx_ = next++;
            if (param.hasQuantOffset) {
                kOffsetIdx_ = next++;
            }
            vScaleIdx_ = next++;
            if (param.hasQuantOffset) {
                vOffsetIdx_ = next++;
            }
        }
        if (qkv_) {
            // reference paged_attention_ops_runner.cpp:118-131: kDescale, vDescale, then (offline) pScale
            kScaleIdx_ = next++;
            vScaleIdx_ = next++;
        }
        if (param.compressType == Param::COMPRESS_TYPE_KVHEAD_ROPE) {
            razorIdx_ = next++;
        }
        if (param.quantType == Param::TYPE_QUANT_QKV_OFFLINE) {
            pScaleIdx_ = next++;
        }
        if (param.scaleType == Param::SCALE_TYPE_LOGN) {
            logNIdx_ = next++;
        }
        inputNum_ = static_cast<uint32_t>(next);
    }

    ~PagedAttentionOperation() override
    {
        if (plan_) {
            atbmi_pa_plan_destroy(plan_);
        }
    }

    uint32_t GetInputNum() const override { return inputNum_; }
    uint32_t GetOutputNum() const override { return 1; }

protected:
    Status InferShapeImpl(const SVector<TensorDesc> &in, SVector<TensorDesc> &out) const override
    {
        out.at(0) = in.at(0);
        if (qkv_) {
            out.at(0).dtype = param_.outDataType; // reference :455-459
        }
        const int64_t dv = mla_ ? static_cast<int64_t>(param_.mlaVHeadSize)
                                : in.at(2).shape.dims[in.at(2).shape.dimNum - 1];
        out.at(0).shape.dims[out.at(0).shape.dimNum - 1] = dv;
        return NO_ERROR;
    }

    // Reference :697-726 (InferShapeDimCheck) + :634-661 (KVCacheDimCheck).
    Status InferShapeCheckImpl(const SVector<TensorDesc> &in) const override
    {
        const Status st = bnsd_ ? BnsdDimCheck(in) : ShapeDimCheck(in);
        if (st != NO_ERROR) {
            return st;
        }
        if (param_.maskType == Param::MASK_TYPE_MASK_FREE) {
            // reference :769-791: the operation can be created anywhere, its shapes pass on Atlas 300I Duo only
            ATB_LOG(ERROR) << "Only Atlas 300I Duo inference products support mask free";
            return ERROR_INVALID_TENSOR_DIM;
        }
        return NO_ERROR;
    }

    Status ShapeDimCheck(const SVector<TensorDesc> &in) const
    {
        if (!mla_ && in.at(2).shape.dimNum != 4) {
            ATB_LOG(ERROR) << "valueCache should have 4 dims";
            return ERROR_INVALID_TENSOR_DIM_NUM;
        }
        if (in.at(0).shape.dimNum != 3 || in.at(1).shape.dimNum != 4 || in.at(tablesIdx_).shape.dimNum != 2 ||
            in.at(lensIdx_).shape.dimNum != 1) {
            ATB_LOG(ERROR) << "expected dims: query 3, keyCache 4, blockTables 2, contextLens 1";
            return ERROR_INVALID_TENSOR_DIM_NUM;
        }
        if (param_.batchRunStatusEnable) {
            // reference :679-688: with a dynamic batch the query may hold fewer rows than the tables
            const int64_t numTokens = in.at(0).shape.dims[0];
            if (numTokens > in.at(tablesIdx_).shape.dims[0] || numTokens > in.at(lensIdx_).shape.dims[0]) {
                ATB_LOG(ERROR) << "numTokens in q should be no greater than blockTables and contextLens";
                return ERROR_INVALID_TENSOR_DIM;
            }
        }
        const Dims &kc = in.at(1).shape;
        if (!mla_) {
            const Dims &vc = in.at(2).shape;
            if (kc.dims[0] != vc.dims[0] || kc.dims[1] != vc.dims[1] || kc.dims[2] != vc.dims[2]) {
                ATB_LOG(ERROR) << "keyCache and valueCache must agree on numBlocks, blockSize and heads";
                return ERROR_INVALID_TENSOR_DIM;
            }
        }
        return CacheDimCheck(in);
    }

    // Reference :492-525 (SetupCheckImpl) + :926-963 (SetupDimCheck) + :856-877 (BlockDimCheck).
    Status SetupCheckImpl(const SVector<Tensor> &inTensors, const SVector<Tensor> &outTensors) const override
    {
        if (inTensors.at(1).desc.shape.dimNum != 4) {
            ATB_LOG(ERROR) << "keyCache should have 4 dims";
            return ERROR_INVALID_TENSOR_DIM_NUM;
        }
        SVector<TensorDesc> in;
        for (size_t i = 0; i < inTensors.size(); ++i) {
            in.push_back(inTensors.at(i).desc);
        }
        Status st = InferShapeCheckImpl(in);
        if (st != NO_ERROR) {
            return st;
        }
        const Dims &out = outTensors.at(0).desc.shape;
        const int64_t dv = mla_ ? static_cast<int64_t>(param_.mlaVHeadSize) : in.at(2).shape.dims[3];
        if (out.dimNum < 3 || out.dims[2] != dv) {
            ATB_LOG(ERROR) << "head size of the output should be " << dv;
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (bnsd_) {
            return NO_ERROR; // reference :965-994 (SetupDimCheckBNSD910B) stops here
        }
        if (in.at(0).shape.dims[1] != out.dims[1]) {
            ATB_LOG(ERROR) << "query and output must have the same head count";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (param_.batchRunStatusEnable && in.at(0).shape.dims[0] != out.dims[0]) {
            ATB_LOG(ERROR) << "numTokens of the output should be the same as q";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (razorIdx_ != NONE) {
            // reference :877-898 (RazorDimCheck): one score offset per cache slot
            const Dims &razor = in.at(razorIdx_).shape;
            if (razor.dimNum != 2 || razor.dims[0] != in.at(1).shape.dims[0] || razor.dims[1] != in.at(1).shape.dims[1]) {
                ATB_LOG(ERROR) << "razorOffset should be [numBlocks, blockSize] of keyCache";
                return ERROR_INVALID_TENSOR_DIM;
            }
        }
        if (logNIdx_ != NONE) {
            // reference :900-924 (LogNDimCheck)
            const Dims &logN = in.at(logNIdx_).shape;
            if (logN.dimNum != 1) {
                ATB_LOG(ERROR) << "logN should have 1 dim";
                return ERROR_INVALID_TENSOR_DIM;
            }
            if (in.at(lensIdx_).shape.dims[0] != logN.dims[0]) {
                ATB_LOG(ERROR) << "contextLens and logN have different batch sizes";
                return ERROR_INVALID_TENSOR_DIM;
            }
            if (statusIdx_ != NONE && in.at(statusIdx_).shape.dims[0] != logN.dims[0]) {
                ATB_LOG(ERROR) << "batchRunStatus and logN have different batch sizes";
                return ERROR_INVALID_TENSOR_DIM;
            }
        }
        return NO_ERROR;
    }

    Status PlanImpl(const VariantPack &pack, uint64_t &workspaceSize) override
    {
        const Tensor &q = pack.inTensors.at(0);
        const Tensor &kc = pack.inTensors.at(1);
        const Tensor &tables = pack.inTensors.at(tablesIdx_);
        const Tensor &lens = pack.inTensors.at(lensIdx_);
        const Tensor &out = pack.outTensors.at(0);
        if (!lens.hostData) {
            ATB_LOG(ERROR) << "contextLens.hostData is null; the lengths are read on the host during Setup";
            return ERROR_INVALID_PARAM;
        }
        const int64_t kvHeads = param_.kvHeadNum > 0 ? param_.kvHeadNum : param_.headNum;
        const int64_t d = kc.desc.shape.dims[3];
        const int64_t dv = mla_ ? static_cast<int64_t>(param_.mlaVHeadSize) : pack.inTensors.at(2).desc.shape.dims[3];
        const int64_t blockSize = kc.desc.shape.dims[bnsd_ ? 2 : 1];
        // Kernel-library level checks of the reference.
        if (q.desc.shape.dims[1] != param_.headNum) {
            ATB_LOG(ERROR) << "query head count " << q.desc.shape.dims[1] << " != headNum " << param_.headNum;
            return ERROR_INVALID_PARAM;
        }
        const int64_t cacheHeads = kc.desc.shape.dims[bnsd_ ? 1 : 2];
        if (compress_) {
            // reference kernel library paged_attention_operation.cpp:316-325,342-354: the caches hold one head
            // per block and contextLens / blockTables one row per (sequence, KV head)
            if (cacheHeads != 1 || pack.inTensors.at(2).desc.shape.dims[2] != 1) {
                ATB_LOG(ERROR) << "head compression: the caches should have one head, [numBlocks, blockSize, 1, headSize]";
                return ERROR_INVALID_PARAM;
            }
            if (q.desc.shape.dims[0] * kvHeads != lens.desc.shape.dims[0]) {
                ATB_LOG(ERROR) << "head compression: contextLens should have numTokens * kvHeadNum entries";
                return ERROR_INVALID_PARAM;
            }
            if (dequant_ && q.desc.dtype != ACL_FLOAT16) {
                ATB_LOG(ERROR) << "head compression with an int8 cache needs an fp16 query";
                return ERROR_INVALID_PARAM;
            }
        } else if (cacheHeads != kvHeads || (bnsd_ && pack.inTensors.at(2).desc.shape.dims[1] != kvHeads)) {
            ATB_LOG(ERROR) << "cache head count " << cacheHeads << " != kvHeadNum " << kvHeads;
            return ERROR_INVALID_PARAM;
        }
        if (blockSize % 16 != 0) {
            ATB_LOG(ERROR) << "blockSize must be a multiple of 16";
            return ERROR_INVALID_PARAM;
        }
        if (d > MLA_THRESHOLD || dv > MLA_THRESHOLD) {
            if (blockSize > 128) {
                ATB_LOG(ERROR) << "blockSize should not exceed 128 when a head size exceeds 256";
                return ERROR_INVALID_PARAM;
            }
        } else if (d == MLA_THRESHOLD && dv == MLA_THRESHOLD && blockSize >= 128) {
            if (blockSize % 128 != 0) {
                ATB_LOG(ERROR) << "head size 256 needs a 128-aligned blockSize";
                return ERROR_INVALID_PARAM;
            }
        } else if (d == dv && d * blockSize > BLOCK_LIMIT) {
            ATB_LOG(ERROR) << "headSize * blockSize should not exceed 128 * 128";
            return ERROR_INVALID_PARAM;
        }
        if (tables.desc.shape.dims[0] < lens.desc.shape.dims[0]) {
            ATB_LOG(ERROR) << "blockTables has fewer rows than contextLens";
            return ERROR_INVALID_PARAM;
        }
        if (out.desc.shape.dims[0] != q.desc.shape.dims[0] || out.desc.shape.dims[1] != q.desc.shape.dims[1]) {
            ATB_LOG(ERROR) << "output and query must have the same token and head counts";
            return ERROR_INVALID_PARAM;
        }
        if (dequant_) {
            const int64_t kLen = kvHeads * d;
            const int64_t vLen = kvHeads * dv;
            if (pack.inTensors.at(kScaleIdx_).desc.shape.dims[0] != kLen ||
                pack.inTensors.at(vScaleIdx_).desc.shape.dims[0] != vLen) {
                ATB_LOG(ERROR) << "descale vectors must have kvHeadNum * headSize elements";
                return ERROR_INVALID_PARAM;
            }
            if (param_.hasQuantOffset && (pack.inTensors.at(kOffsetIdx_).desc.shape.dims[0] != kLen ||
                                          pack.inTensors.at(vOffsetIdx_).desc.shape.dims[0] != vLen)) {
                ATB_LOG(ERROR) << "offset vectors must have kvHeadNum * headSize elements";
                return ERROR_INVALID_PARAM;
            }
        }
        if (statusIdx_ != NONE && !pack.inTensors.at(statusIdx_).hostData) {
            // reference src/ops/ops_infer/paged_attention/param.cpp:39-49: the status vector is read on the
            // host; its values do not reach the kernel, which skips a sequence by its zero context length
            ATB_LOG(ERROR) << "batchRunStatus.hostData is null";
            return ERROR_INVALID_PARAM;
        }
        if (logNIdx_ != NONE && pack.inTensors.at(logNIdx_).desc.shape.dims[0] < q.desc.shape.dims[0]) {
            // reference kernel library paged_attention_operation.cpp:199-203
            ATB_LOG(ERROR) << "logN has fewer elements than the query has rows";
            return ERROR_INVALID_PARAM;
        }
        int64_t maskBatchStride = 0;
        int64_t maskHeadStride = 0;
        int64_t maskLen = 0;
        int32_t maskRowBy = ATBMI_PA_MASK_ROW_SEQUENCE;
        int32_t maskSeqDiv = 0;
        int32_t maskSeqMod = 0;
        if (maskIdx_ != NONE) {
            Status st = MaskLayout(pack.inTensors.at(maskIdx_).desc.shape, lens, q.desc.shape.dims[0], maskBatchStride,
                                   maskHeadStride, maskLen, maskRowBy, maskSeqDiv, maskSeqMod);
            if (st != NO_ERROR) {
                return st;
            }
        }
        if (qkv_) {
            return PlanQkv(pack, maskBatchStride, maskHeadStride, maskLen, maskRowBy, workspaceSize);
        }
        const int32_t *queryLens = nullptr;
        if (qLensIdx_ != NONE) {
            // reference param.cpp:96-110: the query lengths are read on the host, one per sequence
            const Tensor &ql = pack.inTensors.at(qLensIdx_);
            if (!ql.hostData) {
                ATB_LOG(ERROR) << "qSeqLens.hostData is null";
                return ERROR_INVALID_PARAM;
            }
            if (ql.desc.shape.dimNum != 1 || ql.desc.shape.dims[0] != lens.desc.shape.dims[0]) {
                ATB_LOG(ERROR) << "qSeqLens should have one entry per sequence of contextLens";
                return ERROR_INVALID_PARAM;
            }
            queryLens = static_cast<const int32_t *>(ql.hostData);
        }

        AtbmiPaShape shape{};
        shape.qDtype = q.desc.dtype == ACL_BF16 ? ATBMI_BF16 : ATBMI_F16;
        shape.kvDtype = kc.desc.dtype == ACL_INT8 ? ATBMI_INT8 : shape.qDtype;
        // head compression: the kernels see one sequence per (sequence, KV head) pair, each with the query heads of
        // that KV head; [tokens, heads, D] is the same memory as [tokens * kvHeads, heads / kvHeads, D]
        // (reference tiling/paged_attention_tiling.cpp:217-226)
        shape.numHeads = compress_ ? static_cast<int32_t>(param_.headNum / kvHeads) : param_.headNum;
        shape.numKvHeads = compress_ ? 1 : static_cast<int32_t>(kvHeads);
        shape.descaleHeads = (compress_ && dequant_) ? static_cast<int32_t>(kvHeads) : 0;
        shape.maskSeqDiv = maskSeqDiv;
        shape.maskSeqMod = maskSeqMod;
        shape.hasRazorOffset = razorIdx_ != NONE ? 1 : 0;
        shape.headDimK = static_cast<int32_t>(d);
        shape.headDimV = static_cast<int32_t>(dv);
        shape.blockSize = static_cast<int32_t>(blockSize);
        shape.numBlocks = static_cast<int32_t>(kc.desc.shape.dims[0]);
        shape.maxBlocksPerSeq = static_cast<int32_t>(tables.desc.shape.dims[1]);
        shape.numQueryRows = static_cast<int32_t>(q.desc.shape.dims[0] * (compress_ ? kvHeads : 1));
        shape.mlaCombined = mla_ ? 1 : 0;
        shape.hasOffset = (dequant_ && param_.hasQuantOffset) ? 1 : 0;
        shape.kernel = ATBMI_PA_KERNEL_AUTO;
        shape.qkScale = param_.qkScale;
        shape.qScale = param_.qScale;
        shape.hasMask = maskIdx_ != NONE ? 1 : 0;
        shape.maskBatchStride = maskBatchStride;
        shape.maskHeadStride = maskHeadStride;
        shape.maskLen = static_cast<int32_t>(maskLen);
        shape.maskRowBy = maskRowBy;
        shape.hasLogN = logNIdx_ != NONE ? 1 : 0;
        shape.kvLayout = bnsd_ ? ATBMI_PA_KV_HEAD_MAJOR : ATBMI_PA_KV_TOKEN_MAJOR;
        shape.descalePacked = (dequant_ && pack.inTensors.at(kScaleIdx_).desc.dtype == ACL_INT64) ? 1 : 0;
        if (!plan_ || !SameShape(shape, planShape_)) {
            if (plan_) {
                atbmi_pa_plan_destroy(plan_);
                plan_ = nullptr;
            }
            int rc = atbmi_pa_plan_create(&shape, &plan_);
            if (rc != 0) {
                ATB_LOG(ERROR) << "PagedAttention plan: " << atbmi_last_error();
                return rc;
            }
            planShape_ = shape;
        }
        // Lengths are re-read on every Setup, like the reference runner does.
        int rc = atbmi_pa_plan_update_multi(plan_, static_cast<const int32_t *>(lens.hostData), queryLens,
                                            static_cast<int32_t>(lens.desc.shape.dims[0]));
        if (rc != 0) {
            ATB_LOG(ERROR) << "PagedAttention plan: " << atbmi_last_error();
            return rc;
        }
        workspaceSize = atbmi_pa_plan_workspace_size(plan_);
        return NO_ERROR;
    }

    Status LaunchImpl(const VariantPack &pack, uint8_t *workspace, uint64_t workspaceSize,
                      aclrtStream stream) override
    {
        if (qkv_) {
            AtbmiPaInt8QCall call = MakeQkvCall(pack);
            int rc = atbmi_pa_int8q_decode(&call, workspace, workspaceSize, stream);
            if (rc != 0) {
                ATB_LOG(ERROR) << "PagedAttention launch failed: " << atbmi_last_error();
            }
            return rc;
        }
        AtbmiPaTensors t{};
        t.query = pack.inTensors.at(0).deviceData;
        t.keyCache = pack.inTensors.at(1).deviceData;
        t.valueCache = mla_ ? nullptr : pack.inTensors.at(2).deviceData;
        t.blockTables = static_cast<const int32_t *>(pack.inTensors.at(tablesIdx_).deviceData);
        if (dequant_) {
            t.kScale = static_cast<const float *>(pack.inTensors.at(kScaleIdx_).deviceData);
            t.vScale = static_cast<const float *>(pack.inTensors.at(vScaleIdx_).deviceData);
            if (param_.hasQuantOffset) {
                t.kOffset = static_cast<const int32_t *>(pack.inTensors.at(kOffsetIdx_).deviceData);
                t.vOffset = static_cast<const int32_t *>(pack.inTensors.at(vOffsetIdx_).deviceData);
            }
        }
        if (maskIdx_ != NONE) {
            t.mask = pack.inTensors.at(maskIdx_).deviceData;
        }
        if (logNIdx_ != NONE) {
            t.logN = static_cast<const float *>(pack.inTensors.at(logNIdx_).deviceData);
        }
        if (razorIdx_ != NONE) {
            t.razorOffset = static_cast<const float *>(pack.inTensors.at(razorIdx_).deviceData);
        }
        t.out = pack.outTensors.at(0).deviceData;
        int rc = atbmi_pa_decode(plan_, &t, workspace, workspaceSize, stream);
        if (rc != 0) {
            ATB_LOG(ERROR) << "PagedAttention launch failed: " << atbmi_last_error();
        }
        return rc;
    }

private:
    // int8 queries: the kernel-library checks of the reference (src/kernels/mixkernels/pagedattention/
    // paged_attention_operation.cpp:357-403: one descale per query head, fp32) and the call of the kernel layer.
    Status PlanQkv(const VariantPack &pack, int64_t maskSeqStride, int64_t maskHeadStride, int64_t maskLen,
                   int32_t maskRowBy, uint64_t &workspaceSize)
    {
        if (maskRowBy == ATBMI_PA_MASK_ROW_POSITION) {
            ATB_LOG(ERROR) << "int8 queries: a mask whose rows go by position belongs to several query tokens";
            return ERROR_INVALID_PARAM;
        }
        const int64_t d = pack.inTensors.at(1).desc.shape.dims[3];
        if (d != 64 && d != 128 && d != 256) {
            ATB_LOG(ERROR) << "int8 queries: head size " << d << " (64, 128 and 256 are built)";
            return ERROR_INVALID_PARAM;
        }
        for (size_t idx : {kScaleIdx_, vScaleIdx_, pScaleIdx_}) {
            if (idx == NONE) {
                continue;
            }
            const Dims &shape = pack.inTensors.at(idx).desc.shape;
            if (shape.dimNum != 1 || shape.dims[0] != param_.headNum) {
                ATB_LOG(ERROR) << "int8 queries: kDescale, vDescale and pScale should be [headNum]";
                return ERROR_INVALID_PARAM;
            }
        }
        qkvMaskSeqStride_ = maskSeqStride;
        qkvMaskHeadStride_ = maskHeadStride;
        qkvMaskLen_ = maskLen;
        qkvMaskRowByQuery_ = maskRowBy == ATBMI_PA_MASK_ROW_QUERY;
        // the lengths as they are now: Execute works from this copy, like the other paths (the reference reads
        // hostData during Setup only, src/ops/ops_infer/paged_attention/param.cpp:16-62)
        const Tensor &lens = pack.inTensors.at(lensIdx_);
        const int32_t *hostLens = static_cast<const int32_t *>(lens.hostData);
        try {
            qkvLens_.assign(hostLens, hostLens + lens.desc.shape.dims[0]);
        } catch (const std::bad_alloc &) {
            return ERROR_OUT_OF_HOST_MEMORY;
        }
        AtbmiPaInt8QCall call = MakeQkvCall(pack);
        int rc = atbmi_pa_int8q_workspace_size(&call, &workspaceSize);
        if (rc != 0) {
            ATB_LOG(ERROR) << "PagedAttention plan: " << atbmi_last_error();
        }
        return rc;
    }

    AtbmiPaInt8QCall MakeQkvCall(const VariantPack &pack) const
    {
        const Tensor &q = pack.inTensors.at(0);
        const Tensor &kc = pack.inTensors.at(1);
        const Tensor &tables = pack.inTensors.at(tablesIdx_);
        const Tensor &lens = pack.inTensors.at(lensIdx_);
        AtbmiPaInt8QCall c{};
        c.outDtype = param_.outDataType == ACL_BF16 ? ATBMI_BF16 : ATBMI_F16;
        c.numHeads = param_.headNum;
        c.numKvHeads = param_.kvHeadNum > 0 ? param_.kvHeadNum : param_.headNum;
        c.headDim = static_cast<int32_t>(kc.desc.shape.dims[3]);
        c.blockSize = static_cast<int32_t>(kc.desc.shape.dims[1]);
        c.numBlocks = static_cast<int32_t>(kc.desc.shape.dims[0]);
        c.maxBlocksPerSeq = static_cast<int32_t>(tables.desc.shape.dims[1]);
        c.batch = static_cast<int32_t>(lens.desc.shape.dims[0]);
        c.numQueryRows = static_cast<int32_t>(q.desc.shape.dims[0]);
        c.offline = param_.quantType == Param::TYPE_QUANT_QKV_OFFLINE ? 1 : 0;
        c.hasMask = maskIdx_ != NONE ? 1 : 0;
        c.maskLen = static_cast<int32_t>(qkvMaskLen_);
        c.qkScale = param_.qkScale;
        c.maskSeqStride = qkvMaskSeqStride_;
        c.maskHeadStride = qkvMaskHeadStride_;
        c.hostContextLens = qkvLens_.data();
        c.maskRowByQuery = qkvMaskRowByQuery_ ? 1 : 0;
        c.query = q.deviceData;
        c.keyCache = kc.deviceData;
        c.valueCache = pack.inTensors.at(2).deviceData;
        c.blockTables = static_cast<const int32_t *>(tables.deviceData);
        c.kDescale = static_cast<const float *>(pack.inTensors.at(kScaleIdx_).deviceData);
        c.vDescale = static_cast<const float *>(pack.inTensors.at(vScaleIdx_).deviceData);
        c.pScale = pScaleIdx_ != NONE ? static_cast<const float *>(pack.inTensors.at(pScaleIdx_).deviceData) : nullptr;
        c.mask = maskIdx_ != NONE ? pack.inTensors.at(maskIdx_).deviceData : nullptr;
        c.out = pack.outTensors.at(0).deviceData;
        return c;
    }

    static bool SameShape(const AtbmiPaShape &a, const AtbmiPaShape &b)
    {
        return a.qDtype == b.qDtype && a.kvDtype == b.kvDtype && a.numHeads == b.numHeads &&
               a.numKvHeads == b.numKvHeads && a.headDimK == b.headDimK && a.headDimV == b.headDimV &&
               a.blockSize == b.blockSize && a.numBlocks == b.numBlocks && a.maxBlocksPerSeq == b.maxBlocksPerSeq &&
               a.numQueryRows == b.numQueryRows && a.mlaCombined == b.mlaCombined && a.hasOffset == b.hasOffset &&
               a.qkScale == b.qkScale && a.qScale == b.qScale && a.hasMask == b.hasMask &&
               a.maskBatchStride == b.maskBatchStride && a.maskHeadStride == b.maskHeadStride &&
               a.maskLen == b.maskLen && a.hasLogN == b.hasLogN && a.descalePacked == b.descalePacked &&
               a.maskRowBy == b.maskRowBy && a.kvLayout == b.kvLayout && a.maskSeqDiv == b.maskSeqDiv &&
               a.maskSeqMod == b.maskSeqMod && a.descaleHeads == b.descaleHeads && a.hasRazorOffset == b.hasRazorOffset;
    }

    // Element strides of the additive mask, as the reference derives them from
    // its shape (src/kernels/mixkernels/pagedattention/tiling/paged_attention_tiling.cpp:36-74),
    // with the shapes its kernel library accepts for one query token per sequence
    // (src/kernels/mixkernels/pagedattention/paged_attention_operation.cpp:728-763):
    //   NORM  (1, maxS): one row for every sequence and head; (batch, 1, maxS): one row per sequence;
    //   ALIBI (heads, 1, maxS): one row per head; (batch, 1 | heads, 1, maxS): per sequence (and head).
    // maxS has to cover the longest context. The reference's shape check also lets
    // through shapes with more than one query row, which its stride rules then
    // ignore, and a 4-dim NORM mask, for which it derives no strides at all; those
    // are refused here rather than read with strides that do not fit them.
    //
    // With several query tokens per sequence (CALC_TYPE_SPEC; reference
    // tiling/paged_attention_tiling_dependency.cpp:557-569): MASK_TYPE_SPEC is
    // (query rows, maxS), one row per query token; MASK_TYPE_NORM is the square
    // causal (maxS, maxS), of which the i-th query token of a sequence uses row
    // contextLen - queryLen + i. Other NORM shapes are refused under
    // CALC_TYPE_SPEC: the reference would step from a sequence's row into its
    // neighbour's for the second query token.
    //
    // Under head compression the kernels' sequences are (sequence, KV head) pairs and their heads the
    // query heads of one KV head (reference tiling :36-80, kernel library :754-758): a mask with one
    // row per model sequence is indexed by pair / kvHeads, the ALIBI (heads, 1, maxS) mask by pair %
    // kvHeads with a row group of heads / kvHeads rows, and (batch, heads, 1, maxS) reads as
    // (pairs, heads / kvHeads, 1, maxS) as it lies.
    Status MaskLayout(const Dims &m, const Tensor &lens, int64_t queryRows, int64_t &batchStride,
                      int64_t &headStride, int64_t &maskLen, int32_t &rowBy, int32_t &seqDiv, int32_t &seqMod) const
    {
        const int64_t kvHeads = param_.kvHeadNum > 0 ? param_.kvHeadNum : param_.headNum;
        const int64_t pairs = compress_ ? kvHeads : 1; // kernel sequences per model sequence
        const int64_t batch = lens.desc.shape.dims[0] / pairs;
        const int64_t heads = param_.headNum;
        seqDiv = 0;
        seqMod = 0;
        const bool alibi = param_.maskType == Param::MASK_TYPE_ALIBI;
        const bool multi = param_.calcType == Param::CALC_TYPE_SPEC;
        bool ok = false;
        rowBy = ATBMI_PA_MASK_ROW_SEQUENCE;
        if (multi || param_.maskType == Param::MASK_TYPE_SPEC) {
            // (MASK_TYPE_SPEC without CALC_TYPE_SPEC: one query token per sequence, still one mask row per query row)
            if (m.dimNum == 2 && param_.maskType == Param::MASK_TYPE_SPEC) {
                ok = m.dims[0] == queryRows && !compress_; // (under head compression the rows are pairs, not tokens)
                rowBy = ATBMI_PA_MASK_ROW_QUERY;
            } else if (m.dimNum == 2 && param_.maskType == Param::MASK_TYPE_NORM) {
                ok = m.dims[0] == m.dims[1];
                rowBy = ATBMI_PA_MASK_ROW_POSITION;
            }
            batchStride = m.dimNum == 2 ? m.dims[1] : 0;
            headStride = 0;
        } else if (!alibi && m.dimNum == 2) {
            ok = m.dims[0] == 1;
            batchStride = 0;
            headStride = 0;
        } else if (!alibi && m.dimNum == 3) {
            ok = m.dims[0] == batch && m.dims[1] == 1;
            batchStride = m.dims[2];
            headStride = 0;
            seqDiv = static_cast<int32_t>(pairs);
        } else if (!alibi && m.dimNum == 4) {
            // The reference lets (batch, 1 | heads, 1, maxS) through for every mask type (kernel library
            // paged_attention_operation.cpp:760) but its tiling derives strides for the 2- and 3-dim NORM
            // shapes only (tiling/paged_attention_tiling.cpp:62-74): both strides stay 0, and every sequence
            // and head reads the first row of the tensor. The same here.
            ok = m.dims[0] == batch && (m.dims[1] == 1 || m.dims[1] == heads) && m.dims[2] == 1 && !compress_;
            batchStride = 0;
            headStride = 0;
        } else if (alibi && m.dimNum == 3) {
            ok = m.dims[0] == heads && m.dims[1] == 1;
            batchStride = compress_ ? heads / kvHeads * m.dims[2] : 0;
            headStride = m.dims[2];
            seqMod = compress_ ? static_cast<int32_t>(kvHeads) : 0;
        } else if (alibi && m.dimNum == 4) {
            ok = m.dims[0] == batch && (m.dims[1] == 1 || m.dims[1] == heads) && m.dims[2] == 1;
            batchStride = m.dims[1] / (m.dims[1] == 1 ? 1 : pairs) * m.dims[3];
            headStride = m.dims[1] == 1 ? 0 : m.dims[3];
            seqDiv = m.dims[1] == 1 ? static_cast<int32_t>(pairs) : 0;
        }
        if (!ok) {
            ATB_LOG(ERROR) << "mask shape is not one of NORM (1,maxS) / (batch,1,maxS) / (batch,1|heads,1,maxS), "
                              "ALIBI (heads,1,maxS) / (batch,1|heads,1,maxS), or with CALC_TYPE_SPEC "
                              "SPEC (query rows,maxS) / NORM (maxS,maxS)";
            return ERROR_INVALID_PARAM;
        }
        maskLen = m.dims[m.dimNum - 1];
        const int32_t *ctx = static_cast<const int32_t *>(lens.hostData);
        for (int64_t i = 0; i < lens.desc.shape.dims[0]; ++i) {
            if (ctx[i] > maskLen) {
                ATB_LOG(ERROR) << "mask covers " << maskLen << " positions but contextLens[" << i << "] is " << ctx[i];
                return ERROR_INVALID_PARAM;
            }
        }
        return NO_ERROR;
    }

    // Reference :697-726 (InferShapeDimCheckBNSD910B): caches [numBlocks, kvHeads, blockSize, headSize].
    Status BnsdDimCheck(const SVector<TensorDesc> &in) const
    {
        if (in.at(0).shape.dimNum != 3 || in.at(1).shape.dimNum != 4 || in.at(2).shape.dimNum != 4 ||
            in.at(3).shape.dimNum != 2 || in.at(4).shape.dimNum != 1) {
            ATB_LOG(ERROR) << "expected dims: query 3, keyCache 4, valueCache 4, blockTables 2, contextLens 1";
            return ERROR_INVALID_TENSOR_DIM_NUM;
        }
        const int64_t headSize = in.at(0).shape.dims[2];
        if (headSize != in.at(1).shape.dims[3] || headSize != in.at(2).shape.dims[3]) {
            ATB_LOG(ERROR) << "headSize of query, keyCache and valueCache should be same";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (in.at(1).shape.dims[0] != in.at(2).shape.dims[0]) {
            ATB_LOG(ERROR) << "numBlocks of keyCache and valueCache should be same";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (in.at(1).shape.dims[2] != in.at(2).shape.dims[2]) {
            ATB_LOG(ERROR) << "blockSize of keyCache and valueCache should be same";
            return ERROR_INVALID_TENSOR_DIM;
        }
        return NO_ERROR;
    }

    // Reference :585-632 (KVCacheDimCheck910B) with :561-572 (IsInMLAIncompatible).
    Status CacheDimCheck(const SVector<TensorDesc> &in) const
    {
        const int64_t d = in.at(1).shape.dims[3];
        if (d != in.at(0).shape.dims[2]) {
            ATB_LOG(ERROR) << "headSize of keyCache and query should be same";
            return ERROR_INVALID_TENSOR_DIM;
        }
        const int64_t blockSize = in.at(1).shape.dims[1];
        const bool strict = dequant_ || qkv_ || (param_.calcType == Param::CALC_TYPE_SPEC && !mla_) ||
                            param_.scaleType == Param::SCALE_TYPE_LOGN || compress_;
        if (strict) {
            // strict regime (reference :561-572): features that predate the split K/V head sizes
            if (d != in.at(2).shape.dims[3]) {
                ATB_LOG(ERROR) << "headSize of keyCache and valueCache should be same";
                return ERROR_INVALID_TENSOR_DIM;
            }
            if (d > 256 || d * blockSize > BLOCK_LIMIT) {
                ATB_LOG(ERROR) << "headSize should be <= 256 and blockSize * headSize <= 128 * 128";
                return ERROR_INVALID_TENSOR_DIM;
            }
            return NO_ERROR;
        }
        if (static_cast<int64_t>(param_.mlaVHeadSize) > d) {
            ATB_LOG(ERROR) << "mlaVHeadSize should be no greater than headSizeK";
            return ERROR_INVALID_TENSOR_DIM;
        }
        const int64_t dv = mla_ ? static_cast<int64_t>(param_.mlaVHeadSize) : in.at(2).shape.dims[3];
        if (d > MAX_HEAD_SIZE || dv > MAX_HEAD_SIZE) {
            ATB_LOG(ERROR) << "head sizes should be no greater than 576";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (mla_ && in.at(lensIdx_).shape.dims[0] > MAX_MLA_BATCH) {
            ATB_LOG(ERROR) << "batch should be <= 8192 in mla mode";
            return ERROR_INVALID_TENSOR_DIM;
        }
        const bool blockSize256 = mla_ && blockSize == 256 && param_.kvHeadNum == 1 &&
                                  (param_.headNum == 16 || param_.headNum == 32) && d == 576 && dv == 512 &&
                                  param_.calcType != Param::CALC_TYPE_SPEC;
        if (blockSize256) {
            return NO_ERROR;
        }
        if ((d > 256 || dv > 256) && blockSize > 128) {
            ATB_LOG(ERROR) << "blockSize should be no greater than 128 if a head size exceeds 256";
            return ERROR_INVALID_TENSOR_DIM;
        }
        return NO_ERROR;
    }

    Param param_;
    bool mla_;
    bool dequant_;
    bool bnsd_;
    bool compress_; // every (sequence, KV head) pair comes with its own context length and block-table row
    bool qkv_;      // int8 queries over int8 caches (quantType QKV online / offline)
    OpIr irTable_;
    static constexpr size_t NONE = ~static_cast<size_t>(0);
    size_t razorIdx_ = NONE;
    size_t tablesIdx_ = 3;
    size_t lensIdx_ = 4;
    size_t maskIdx_ = NONE;
    size_t statusIdx_ = NONE;
    size_t kScaleIdx_ = NONE;
    size_t kOffsetIdx_ = NONE;
    size_t vScaleIdx_ = NONE;
    size_t vOffsetIdx_ = NONE;
    size_t logNIdx_ = NONE;
    size_t qLensIdx_ = NONE;
    size_t pScaleIdx_ = NONE;
    int64_t qkvMaskSeqStride_ = 0;
    int64_t qkvMaskHeadStride_ = 0;
    int64_t qkvMaskLen_ = 0;
    bool qkvMaskRowByQuery_ = false;
    std::vector<int32_t> qkvLens_; // contextLens as read at Setup
    uint32_t inputNum_ = 5;
    AtbmiPaPlan *plan_ = nullptr;
    AtbmiPaShape planShape_{};
};
} // namespace

template <> Status CreateOperation(const infer::PagedAttentionParam &opParam, Operation **operation)
{
    if (operation == nullptr) {
        return ERROR_INVALID_PARAM;
    }
    if (!ReservedIsZero(opParam)) {
        ATB_LOG(ERROR) << "PagedAttentionParam rsv has a non-zero byte";
        return ERROR_INVALID_PARAM;
    }
    if (!CommonParamCheck(opParam) || !FeatureParamCheck(opParam) || !ImplementedCheck(opParam)) {
        return ERROR_INVALID_PARAM;
    }
    *operation = new (std::nothrow) PagedAttentionOperation(opParam);
    if (*operation == nullptr) {
        return ERROR_OUT_OF_HOST_MEMORY;
    }
    return NO_ERROR;
}
} // namespace atb
