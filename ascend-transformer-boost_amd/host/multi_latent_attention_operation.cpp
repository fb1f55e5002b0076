// MultiLatentAttentionOperation on MI355X: decode attention over the split
// latent cache (512 latent + 64 rotary channels per token, one KV head).
//
// Creation-time checks, tensor counts, InferShape and the dim checks follow the
// reference operator (reference src/ops/ops_infer/multi_latent_attention/
// multi_latent_attention_operation.cpp: 58-89 create, 91-148 decode param rules,
// 150-173 ranges, 175-206 prefill rules, 245-293 counts and InferShape, 350-392
// QKVDimCheck, 478-490 qSeqlen, 558-620 DimCheck). Context and query lengths are
// read from hostData during Setup, as the reference runner does
// (src/ops/ops_infer/multi_latent_attention/param.cpp).
//
// Implemented: cacheMode KROPE_CTKV and NZCACHE (the same 16-bit caches in the
// fractal-NZ layout, [blocks, 512 / 16, 128, 16] and [blocks, 64 / 16, 128, 16];
// reference :394-425 QKVDimCheckNz) with fp16/bf16 tensors; calcType UNDEFINED,
// SPEC (qSeqlen, optionally with the MASK_TYPE_SPEC mask), RING and
// SPEC_AND_RING (second output: log-sum-exp). cacheMode INT8_NZCACHE (int8 query and
// latent cache [blocks, 512 / 32, 128, 32] with a descale per head for the scores and
// one for the values, the rotary parts 16-bit; reference :427-476, :493-511, :513-541)
// runs on a kernel of its own (csrc/mla_int8.hip); its log-sum-exp output is fp32.
// calcType PREFILL is an operation class of its own
// (multi_latent_attention_prefill_operation.cpp).
//
// Several query tokens per sequence (SPEC, SPEC_AND_RING). The reference's tiling runs one
// job per query token, each over the context up to that token, when headNum is 128 or
// the cache is int8 with more than one query token, and drops the mask type in that
// case (src/kernels/mixkernels/multi_latent_attention/tiling/mla_tiling.cpp:139-144,
// mla_tiling_dependency.cpp:292-316): the t-th of n query rows sees the first
// contextLens - n + t + 1 tokens whatever mask tensor came with the call, and a
// sequence whose maskUseStatus entry is 0 keeps the whole context for every row. The
// same rule applies here (kernel layer: causal rows). With fewer heads the
// MASK_TYPE_SPEC mask [numTokens, maxS] is added to the scores as given;
// MASK_TYPE_CAUSAL_MASK (no mask tensor) is causal rows for any head count.
// MASK_TYPE_MASK_FREE with fewer heads: the [125 + 2 q, 128] template (or one per
// sequence), which the reference's other kernel path indexes by the last two 128-token
// tiles (op_kernel/mla.cce:3719-3750), is expanded on the device into one mask row per
// query token (atbmi_mla_mask_free_expand, in the workspace) and added like a SPEC mask.
//
// The kernels are those of PagedAttention's combined-cache variant reading
// each query and key row from two tensors.
#include <algorithm>
#include <new>
#include <vector>
#include "atb/infer_op_params.h"
#include "atb/utils.h"
#include "atbmi_kernels.h"
#include "log.h"
#include "operation_base.h"

namespace atb {
namespace {
using Param = infer::MultiLatentAttentionParam;

constexpr size_t QUERY = 0, QUERY_ROPE = 1, KV_CACHE = 2, KV_CACHE_ROPE = 3, BLOCK_TABLES = 4, CONTEXT_LENS = 5;
constexpr int64_t LATENT_DIM = 512;
constexpr int64_t ROPE_DIM = 64;
constexpr int64_t DECODER_BLOCK_SIZE = 128;
constexpr int64_t MAX_BATCH = 8192;
constexpr int64_t NZ_CHANNELS = 16; // channels of one fractal-NZ slab row (16-bit elements)
constexpr int64_t NZ_CHANNELS_INT8 = 32;
constexpr int32_t JOB_PER_TOKEN_HEADS = 128; // reference tiling/mla_tiling_dependency.h:31 (M_LIMIT)

bool IsSpec(const Param &p)
{
    return p.calcType == Param::CALC_TYPE_SPEC || p.calcType == Param::CALC_TYPE_SPEC_AND_RING;
}

bool IsRing(const Param &p)
{
    return p.calcType == Param::CALC_TYPE_RING || p.calcType == Param::CALC_TYPE_SPEC_AND_RING;
}

bool HasMaskInput(const Param &p)
{
    return p.maskType != Param::UNDEFINED && p.maskType != Param::MASK_TYPE_CAUSAL_MASK;
}

// Reference :150-173.
bool ParamRangeCheck(const Param &p)
{
    if (p.qkScale <= 0 || p.qkScale > 1) {
        ATB_LOG(ERROR) << "qkScale should be > 0 and <= 1";
        return false;
    }
    if (p.maskType < Param::UNDEFINED || p.maskType > Param::MASK_TYPE_SWA_NORM) {
        ATB_LOG(ERROR) << "invalid maskType";
        return false;
    }
    if (p.calcType < Param::CALC_TYPE_UNDEFINED || p.calcType > Param::CALC_TYPE_PREFILL) {
        ATB_LOG(ERROR) << "invalid calcType";
        return false;
    }
    if (p.cacheMode > Param::NZCACHE) {
        ATB_LOG(ERROR) << "invalid cacheMode";
        return false;
    }
    return true;
}

// Reference :91-148 (decode).
bool ParamCheck(const Param &p)
{
    if (p.headNum != 8 && p.headNum != 16 && p.headNum != 32 && p.headNum != 64 && p.headNum != 128) {
        ATB_LOG(ERROR) << "headNum should be one of 8, 16, 32, 64, 128";
        return false;
    }
    if (p.kvHeadNum != 1) {
        ATB_LOG(ERROR) << "kvHeadNum should be 1, only MQA is supported";
        return false;
    }
    if (p.cacheMode == Param::KVCACHE) {
        ATB_LOG(ERROR) << "cacheMode KVCACHE is not supported";
        return false;
    }
    if (!IsSpec(p) && p.maskType != Param::UNDEFINED) {
        ATB_LOG(ERROR) << "only CALC_TYPE_SPEC takes a mask";
        return false;
    }
    if (IsSpec(p) && p.maskType == Param::MASK_TYPE_SWA_NORM) {
        ATB_LOG(ERROR) << "decode with CALC_TYPE_SPEC does not take the SWA_NORM mask";
        return false;
    }
    if (p.cacheMode == Param::INT8_NZCACHE && IsRing(p) && p.maskType != Param::UNDEFINED) {
        ATB_LOG(ERROR) << "int8 NZ cache with log-sum-exp output does not take a mask";
        return false;
    }
    if (p.maskUseStatusType < Param::MASK_USE_STATUS_TYPE_UNDEFINED ||
        p.maskUseStatusType >= Param::MASK_USE_STATUS_TYPE_MAX) {
        ATB_LOG(ERROR) << "invalid maskUseStatusType";
        return false;
    }
    if (p.maskUseStatusType == Param::MASK_USE_STATUS_TYPE_BATCH_MASK && p.calcType != Param::CALC_TYPE_SPEC_AND_RING) {
        ATB_LOG(ERROR) << "maskUseStatus needs CALC_TYPE_SPEC_AND_RING";
        return false;
    }
    if (p.maskType == Param::MASK_TYPE_SWA_NORM && p.windowSize <= 0) {
        ATB_LOG(ERROR) << "windowSize in swa mode should be greater than 0";
        return false;
    }
    return true;
}

// Reference :175-206 (prefill).
bool ParamPrefillCheck(const Param &p)
{
    if (p.headNum < 1 || p.headNum > 128) {
        ATB_LOG(ERROR) << "headNum should be >= 1 and <= 128";
        return false;
    }
    if (p.maskType != Param::MASK_TYPE_CAUSAL_MASK && p.headNum != p.kvHeadNum) {
        ATB_LOG(ERROR) << "prefill: headNum should equal kvHeadNum";
        return false;
    }
    if (p.maskType != Param::UNDEFINED && p.maskType != Param::MASK_TYPE_MASK_FREE &&
        p.maskType != Param::MASK_TYPE_CAUSAL_MASK && p.maskType != Param::MASK_TYPE_SWA_NORM) {
        ATB_LOG(ERROR) << "prefill: maskType should be UNDEFINED, MASK_FREE, CAUSAL_MASK or SWA_NORM";
        return false;
    }
    if (p.cacheMode != Param::KROPE_CTKV) {
        ATB_LOG(ERROR) << "prefill: cacheMode should be KROPE_CTKV";
        return false;
    }
    if (p.maskType == Param::MASK_TYPE_SWA_NORM && p.windowSize <= 0) {
        ATB_LOG(ERROR) << "prefill: windowSize in swa mode should be greater than 0";
        return false;
    }
    return true;
}

bool HasMaskUseStatus(const Param &p)
{
    return p.maskUseStatusType == Param::MASK_USE_STATUS_TYPE_BATCH_MASK;
}

// The dtype table of the implemented sections of the reference
// ops_configs/atb_ops_info.ini (:6669-6690 base, :6691-6715 Mask, :6716-6740 IsRing,
// :6772-6824 Qlens / QlensIsRing, :6859-6917 MaskQlens / MaskQlensIsRing, :6946-6967 Nz).
// The reference builds the section name from the param (:208-240); NZCACHE together with a mask,
// qSeqlen or the log-sum-exp output names a section that does not exist, and an operation without
// a table skips the check (reference operation_base.cpp:229-233): HasIr() says which.
bool HasIr(const Param &p)
{
    if (HasMaskUseStatus(p)) {
        // (always SPEC_AND_RING) sections MaskQlensIsRingMaskUseStatus and QlensIsRingInt8NzMaskUseStatus
        // (:7021-7055, :7091-7126)
        return p.cacheMode == Param::INT8_NZCACHE ? !HasMaskInput(p) : p.cacheMode == Param::KROPE_CTKV && HasMaskInput(p);
    }
    if (p.cacheMode == Param::INT8_NZCACHE) {
        // sections Int8Nz, IsRingInt8Nz and QlensIsRingInt8Nz (:6918-6945, :6741-6771, :6825-6858)
        return !HasMaskInput(p) && (!IsSpec(p) || IsRing(p));
    }
    return p.cacheMode != Param::NZCACHE || (!HasMaskInput(p) && !IsSpec(p) && !IsRing(p));
}

OpIr MakeIr(const Param &p)
{
    OpIr ir;
    const bool int8 = p.cacheMode == Param::INT8_NZCACHE;
    const aclFormat cacheFormat = p.cacheMode == Param::KROPE_CTKV ? ACL_FORMAT_ND : ACL_FORMAT_FRACTAL_NZ;
    for (aclDataType q : {ACL_FLOAT16, ACL_BF16}) {
        IrCombo c;
        c.inDtypes = {int8 ? ACL_INT8 : q, q, int8 ? ACL_INT8 : q, q, ACL_INT32, ACL_INT32};
        if (HasMaskInput(p)) {
            c.inDtypes.push_back(q);
        }
        if (IsSpec(p)) {
            c.inDtypes.push_back(ACL_INT32);
        }
        if (int8) {
            c.inDtypes.push_back(ACL_FLOAT);
            c.inDtypes.push_back(ACL_FLOAT);
        }
        if (HasMaskUseStatus(p)) {
            c.inDtypes.push_back(ACL_INT32);
        }
        c.inFormats.assign(c.inDtypes.size(), ACL_FORMAT_ND);
        c.inFormats[KV_CACHE] = cacheFormat;
        c.inFormats[KV_CACHE_ROPE] = cacheFormat;
        c.outDtypes = {q};
        if (IsRing(p)) {
            c.outDtypes.push_back(int8 ? ACL_FLOAT : q);
        }
        c.outFormats.assign(c.outDtypes.size(), ACL_FORMAT_ND);
        ir.push_back(c);
    }
    return ir;
}

} // namespace

Operation *NewMultiLatentAttentionPrefillOperation(const infer::MultiLatentAttentionParam &param);

namespace {
class MultiLatentAttentionOperation : public OperationBase {
public:
    explicit MultiLatentAttentionOperation(const Param &param)
        : OperationBase("MultiLatentAttentionOperation"), param_(param), irTable_(MakeIr(param))
    {
        ir_ = HasIr(param) ? &irTable_ : nullptr;
        size_t next = CONTEXT_LENS + 1;
        if (HasMaskInput(param)) {
            maskIdx_ = next++;
        }
        if (IsSpec(param)) {
            qLensIdx_ = next++;
        }
        if (param.cacheMode == Param::INT8_NZCACHE) {
            descaleIdx_ = next;
            next += 2; // qkDescale, pvDescale
        }
        if (HasMaskUseStatus(param)) {
            maskUseIdx_ = next++;
        }
        inputNum_ = static_cast<uint32_t>(next);
    }

    ~MultiLatentAttentionOperation() override
    {
        if (plan_) {
            atbmi_pa_plan_destroy(plan_);
        }
    }

    uint32_t GetInputNum() const override { return inputNum_; }
    uint32_t GetOutputNum() const override { return IsRing(param_) ? 2 : 1; }
    bool InputMayBeEmpty(size_t index) const override { return index == maskUseIdx_; } // reference ini: optional

protected:
    // Reference :268-283.
    Status InferShapeImpl(const SVector<TensorDesc> &in, SVector<TensorDesc> &out) const override
    {
        out.at(0) = in.at(QUERY);
        out.at(0).dtype = in.at(QUERY_ROPE).dtype;
        if (IsRing(param_)) {
            out.at(1) = out.at(0);
            if (param_.cacheMode == Param::INT8_NZCACHE) {
                out.at(1).dtype = ACL_FLOAT;
            }
            out.at(1).shape.dims[2] = 1;
        }
        return NO_ERROR;
    }

    Status InferShapeCheckImpl(const SVector<TensorDesc> &in) const override { return DimCheck(in); }

    Status SetupCheckImpl(const SVector<Tensor> &inTensors, const SVector<Tensor> &outTensors) const override
    {
        SVector<TensorDesc> in;
        for (size_t i = 0; i < inTensors.size(); ++i) {
            in.push_back(inTensors.at(i).desc);
        }
        Status st = DimCheck(in);
        if (st != NO_ERROR) {
            return st;
        }
        if (IsRing(param_) && param_.maskType == Param::UNDEFINED && param_.cacheMode == Param::INT8_NZCACHE) {
            // reference :513-541
            const Dims &q = inTensors.at(QUERY).desc.shape;
            for (size_t i = 0; i < 2; ++i) {
                const Dims &o = outTensors.at(i).desc.shape;
                if (o.dimNum != q.dimNum) {
                    ATB_LOG(ERROR) << "outputs should have as many dims as query";
                    return ERROR_INVALID_TENSOR_DIM_NUM;
                }
                if (o.dims[0] != q.dims[0] || o.dims[1] != q.dims[1] || o.dims[2] != (i == 0 ? q.dims[2] : 1)) {
                    ATB_LOG(ERROR) << "attenOut should be shaped like query, lse like query with a last dim of 1";
                    return ERROR_INVALID_TENSOR_DIM;
                }
            }
        }
        return NO_ERROR;
    }

    Status PlanImpl(const VariantPack &pack, uint64_t &workspaceSize) override
    {
        const Tensor &q = pack.inTensors.at(QUERY);
        const Tensor &kv = pack.inTensors.at(KV_CACHE);
        const Tensor &tables = pack.inTensors.at(BLOCK_TABLES);
        const Tensor &lens = pack.inTensors.at(CONTEXT_LENS);
        const Tensor &out = pack.outTensors.at(0);
        if (!lens.hostData) {
            ATB_LOG(ERROR) << "contextLens.hostData is null; the lengths are read on the host during Setup";
            return ERROR_INVALID_PARAM;
        }
        const int32_t batch = static_cast<int32_t>(lens.desc.shape.dims[0]);
        const int32_t *queryLens = nullptr;
        if (qLensIdx_ != NONE) {
            const Tensor &ql = pack.inTensors.at(qLensIdx_);
            if (!ql.hostData) {
                ATB_LOG(ERROR) << "qSeqlen.hostData is null; the lengths are read on the host during Setup";
                return ERROR_INVALID_PARAM;
            }
            queryLens = static_cast<const int32_t *>(ql.hostData);
        }
        // One job per query token, each over the context up to its token, and no mask: the reference's tiling
        // for 128 heads and for an int8 cache with several query tokens (mla_tiling.cpp:139-144,
        // mla_tiling_dependency.cpp:292-316); MASK_TYPE_CAUSAL_MASK asks for the same.
        const bool int8 = param_.cacheMode == Param::INT8_NZCACHE;
        int32_t maxQuery = 1;
        for (int32_t i = 0; queryLens && i < batch; ++i) {
            maxQuery = std::max(maxQuery, queryLens[i]);
        }
        const bool jobPerToken = param_.headNum == JOB_PER_TOKEN_HEADS || (int8 && maxQuery > 1);
        const bool causalRows = IsSpec(param_) && (jobPerToken || param_.maskType == Param::MASK_TYPE_CAUSAL_MASK);
        useMask_ = maskIdx_ != NONE && !jobPerToken && !int8; // (the int8 kernels of the reference never read it)
        maskFree_ = useMask_ && param_.maskType == Param::MASK_TYPE_MASK_FREE;
        causalUse_.clear();
        if (causalRows && maskUseIdx_ != NONE && Utils::GetTensorSize(pack.inTensors.at(maskUseIdx_).desc) != 0) {
            const Tensor &use = pack.inTensors.at(maskUseIdx_);
            if (!use.hostData) {
                ATB_LOG(ERROR) << "maskUseStatus.hostData is null; the flags are read on the host during Setup";
                return ERROR_INVALID_PARAM;
            }
            if (use.desc.shape.dimNum != 1 || use.desc.shape.dims[0] != batch) {
                ATB_LOG(ERROR) << "maskUseStatus should be [batch]";
                return ERROR_INVALID_PARAM;
            }
            causalUse_.assign(static_cast<const int32_t *>(use.hostData), static_cast<const int32_t *>(use.hostData) + batch);
        }
        const Dims &o = out.desc.shape;
        if (o.dimNum != 3 || o.dims[0] != q.desc.shape.dims[0] || o.dims[1] != param_.headNum ||
            o.dims[2] != LATENT_DIM) {
            ATB_LOG(ERROR) << "the output should be [numTokens, headNum, 512]";
            return ERROR_INVALID_PARAM;
        }
        if (IsRing(param_)) {
            const Dims &l = pack.outTensors.at(1).desc.shape;
            if (l.dimNum != 3 || l.dims[0] != o.dims[0] || l.dims[1] != o.dims[1] || l.dims[2] != 1) {
                ATB_LOG(ERROR) << "the log-sum-exp output should be [numTokens, headNum, 1]";
                return ERROR_INVALID_PARAM;
            }
        }
        int64_t maskLen = 0;
        uint64_t maskFreeTableBytes = 0;
        if (maskFree_) {
            // the template [rows, 128] or [batch, rows, 128] (reference tiling/mla_tiling.cpp:156-166) becomes a
            // mask of one row per query token in the workspace
            const Dims &m = pack.inTensors.at(maskIdx_).desc.shape;
            if ((m.dimNum != 2 && m.dimNum != 3) || m.dims[m.dimNum - 1] != DECODER_BLOCK_SIZE ||
                (m.dimNum == 3 && m.dims[0] != batch)) {
                ATB_LOG(ERROR) << "the MASK_FREE mask should be [rows, 128] or [batch, rows, 128]";
                return ERROR_INVALID_PARAM;
            }
            const int32_t *ctx = static_cast<const int32_t *>(lens.hostData);
            lens_.assign(ctx, ctx + batch);
            qLens_.assign(queryLens, queryLens + batch);
            for (int32_t i = 0; i < batch; ++i) {
                maskLen = std::max<int64_t>(maskLen, ctx[i]);
            }
            // (in whole cache blocks: the plan is rebuilt when this changes, which should not be every few decode steps)
            maskLen = std::max<int64_t>(DECODER_BLOCK_SIZE, (maskLen + DECODER_BLOCK_SIZE - 1) / DECODER_BLOCK_SIZE * DECODER_BLOCK_SIZE);
            maskFreeRows_ = static_cast<int32_t>(m.dims[m.dimNum - 2]);
            maskFreeBatch_ = m.dimNum == 3 ? batch : 0;
            maskLen_ = maskLen;
            AtbmiMlaMaskFreeCall call = MakeMaskFreeCall(pack, nullptr);
            int rc = atbmi_mla_mask_free_workspace_size(&call, &maskFreeTableBytes);
            if (rc != 0) {
                ATB_LOG(ERROR) << "MultiLatentAttention mask-free plan: " << atbmi_last_error();
                return rc;
            }
        } else if (useMask_) {
            // one mask row per query token (reference tests/apitest/opstest/python/operations/
            // multi_latent_attention/test_multi_latent_attention_mtp.py:262-274)
            const Dims &m = pack.inTensors.at(maskIdx_).desc.shape;
            if (m.dimNum != 2 || m.dims[0] != q.desc.shape.dims[0]) {
                ATB_LOG(ERROR) << "the mask should be [numTokens, maxS]";
                return ERROR_INVALID_PARAM;
            }
            maskLen = m.dims[1];
            const int32_t *ctx = static_cast<const int32_t *>(lens.hostData);
            for (int32_t i = 0; i < batch; ++i) {
                if (ctx[i] > maskLen) {
                    ATB_LOG(ERROR) << "mask covers " << maskLen << " positions but contextLens[" << i << "] is " << ctx[i];
                    return ERROR_INVALID_PARAM;
                }
            }
        }

        if (param_.cacheMode == Param::INT8_NZCACHE) {
            for (size_t i = descaleIdx_; i < descaleIdx_ + 2; ++i) {
                const Dims &d = pack.inTensors.at(i).desc.shape;
                if (d.dimNum != 1 || d.dims[0] != param_.headNum) {
                    ATB_LOG(ERROR) << "qkDescale and pvDescale should be [headNum]";
                    return ERROR_INVALID_PARAM;
                }
            }
            lens_.assign(static_cast<const int32_t *>(lens.hostData), static_cast<const int32_t *>(lens.hostData) + batch);
            qLens_.clear();
            if (queryLens) {
                qLens_.assign(queryLens, queryLens + batch);
            }
            causalRows_ = causalRows;
            AtbmiMlaInt8Call call = MakeInt8Call(pack);
            int rc = atbmi_mla_int8_workspace_size(&call, &workspaceSize);
            if (rc != 0) {
                ATB_LOG(ERROR) << "MultiLatentAttention int8 plan: " << atbmi_last_error();
                return rc;
            }
            return NO_ERROR;
        }
        AtbmiPaShape shape{};
        shape.qDtype = q.desc.dtype == ACL_BF16 ? ATBMI_BF16 : ATBMI_F16;
        shape.kvDtype = shape.qDtype;
        shape.numHeads = param_.headNum;
        shape.numKvHeads = 1;
        shape.headDimK = static_cast<int32_t>(LATENT_DIM + ROPE_DIM);
        shape.headDimV = static_cast<int32_t>(LATENT_DIM);
        const bool nz = param_.cacheMode == Param::NZCACHE;
        shape.blockSize = static_cast<int32_t>(kv.desc.shape.dims[nz ? 2 : 1]);
        shape.kvLayout = nz ? ATBMI_PA_KV_FRACTAL_NZ : ATBMI_PA_KV_TOKEN_MAJOR;
        shape.numBlocks = static_cast<int32_t>(kv.desc.shape.dims[0]);
        shape.maxBlocksPerSeq = static_cast<int32_t>(tables.desc.shape.dims[1]);
        shape.numQueryRows = static_cast<int32_t>(q.desc.shape.dims[0]);
        shape.mlaCombined = 1;
        shape.kernel = ATBMI_PA_KERNEL_AUTO;
        shape.qkScale = param_.qkScale;
        shape.ropeDim = static_cast<int32_t>(ROPE_DIM);
        shape.hasMask = useMask_ ? 1 : 0;
        shape.maskBatchStride = maskLen;
        shape.maskLen = static_cast<int32_t>(maskLen);
        shape.maskRowBy = useMask_ ? ATBMI_PA_MASK_ROW_QUERY : ATBMI_PA_MASK_ROW_SEQUENCE;
        if (!plan_ || !SameShape(shape, planShape_)) {
            if (plan_) {
                atbmi_pa_plan_destroy(plan_);
                plan_ = nullptr;
            }
            int rc = atbmi_pa_plan_create(&shape, &plan_);
            if (rc != 0) {
                ATB_LOG(ERROR) << "MultiLatentAttention plan: " << atbmi_last_error();
                return rc;
            }
            planShape_ = shape;
        }
        int rc = atbmi_pa_plan_set_causal_rows(plan_, causalRows ? 1 : 0, causalUse_.empty() ? nullptr : causalUse_.data(),
                                               static_cast<int32_t>(causalUse_.size()));
        if (rc == 0) {
            // a sequence without context keeps its query rows (reference tiling/mla_tiling.cpp:146-149)
            rc = atbmi_pa_plan_set_empty_keep_rows(plan_, 1);
        }
        if (rc == 0) {
            rc = atbmi_pa_plan_update_multi(plan_, static_cast<const int32_t *>(lens.hostData), queryLens, batch);
        }
        if (rc != 0) {
            ATB_LOG(ERROR) << "MultiLatentAttention plan: " << atbmi_last_error();
            return rc;
        }
        workspaceSize = atbmi_pa_plan_workspace_size(plan_);
        if (maskFree_) {
            planBytes_ = workspaceSize;
            maskFreeTableOff_ = (workspaceSize + 255) / 256 * 256;
            maskFreeTableBytes_ = maskFreeTableBytes;
            maskFreeMaskOff_ = (maskFreeTableOff_ + maskFreeTableBytes + 255) / 256 * 256;
            workspaceSize = maskFreeMaskOff_ + static_cast<uint64_t>(q.desc.shape.dims[0]) * static_cast<uint64_t>(maskLen) * 2;
            maskFreeBytes_ = workspaceSize;
        }
        return NO_ERROR;
    }

    Status LaunchImpl(const VariantPack &pack, uint8_t *workspace, uint64_t workspaceSize,
                      aclrtStream stream) override
    {
        if (param_.cacheMode == Param::INT8_NZCACHE) {
            AtbmiMlaInt8Call call = MakeInt8Call(pack);
            int rc = atbmi_mla_int8_decode(&call, workspace, workspaceSize, stream);
            if (rc != 0) {
                ATB_LOG(ERROR) << "MultiLatentAttention int8 launch failed: " << atbmi_last_error();
            }
            return rc;
        }
        AtbmiPaTensors t{};
        t.query = pack.inTensors.at(QUERY).deviceData;
        t.queryRope = pack.inTensors.at(QUERY_ROPE).deviceData;
        t.keyCache = pack.inTensors.at(KV_CACHE).deviceData;
        t.keyRopeCache = pack.inTensors.at(KV_CACHE_ROPE).deviceData;
        t.blockTables = static_cast<const int32_t *>(pack.inTensors.at(BLOCK_TABLES).deviceData);
        uint64_t planBytes = workspaceSize;
        if (maskFree_) {
            if (!workspace || workspaceSize < maskFreeBytes_) {
                ATB_LOG(ERROR) << "MultiLatentAttention: the workspace is smaller than Setup asked for";
                return ERROR_INVALID_PARAM;
            }
            AtbmiMlaMaskFreeCall call = MakeMaskFreeCall(pack, workspace + maskFreeMaskOff_);
            int rc = atbmi_mla_mask_free_expand(&call, workspace + maskFreeTableOff_, maskFreeTableBytes_, stream);
            if (rc != 0) {
                ATB_LOG(ERROR) << "MultiLatentAttention mask-free launch failed: " << atbmi_last_error();
                return rc;
            }
            t.mask = workspace + maskFreeMaskOff_;
            planBytes = planBytes_;
        } else if (useMask_) {
            t.mask = pack.inTensors.at(maskIdx_).deviceData;
        }
        t.out = pack.outTensors.at(0).deviceData;
        if (IsRing(param_)) {
            t.lse = pack.outTensors.at(1).deviceData;
        }
        int rc = atbmi_pa_decode(plan_, &t, workspace, planBytes, stream);
        if (rc != 0) {
            ATB_LOG(ERROR) << "MultiLatentAttention launch failed: " << atbmi_last_error();
        }
        return rc;
    }

private:
    static constexpr size_t NONE = ~static_cast<size_t>(0);

    AtbmiMlaInt8Call MakeInt8Call(const VariantPack &pack) const
    {
        const Tensor &kv = pack.inTensors.at(KV_CACHE);
        AtbmiMlaInt8Call c{};
        c.outDtype = pack.inTensors.at(QUERY_ROPE).desc.dtype == ACL_BF16 ? ATBMI_BF16 : ATBMI_F16;
        c.numHeads = param_.headNum;
        c.blockSize = static_cast<int32_t>(kv.desc.shape.dims[2]);
        c.numBlocks = static_cast<int32_t>(kv.desc.shape.dims[0]);
        c.maxBlocksPerSeq = static_cast<int32_t>(pack.inTensors.at(BLOCK_TABLES).desc.shape.dims[1]);
        c.batch = static_cast<int32_t>(lens_.size());
        c.numQueryRows = static_cast<int32_t>(pack.inTensors.at(QUERY).desc.shape.dims[0]);
        c.hasMask = 0; // (the reference's int8 kernels never read the mask: mla_tiling.cpp:142-144)
        c.maskLen = 0;
        c.causalRows = causalRows_ ? 1 : 0;
        c.hostCausalUse = causalUse_.empty() ? nullptr : causalUse_.data();
        c.qkScale = param_.qkScale;
        c.hostContextLens = lens_.data();
        c.hostQueryLens = qLens_.empty() ? nullptr : qLens_.data();
        c.query = pack.inTensors.at(QUERY).deviceData;
        c.queryRope = pack.inTensors.at(QUERY_ROPE).deviceData;
        c.kvCache = kv.deviceData;
        c.kRopeCache = pack.inTensors.at(KV_CACHE_ROPE).deviceData;
        c.blockTables = static_cast<const int32_t *>(pack.inTensors.at(BLOCK_TABLES).deviceData);
        c.qkDescale = static_cast<const float *>(pack.inTensors.at(descaleIdx_).deviceData);
        c.pvDescale = static_cast<const float *>(pack.inTensors.at(descaleIdx_ + 1).deviceData);
        c.mask = nullptr;
        c.out = pack.outTensors.at(0).deviceData;
        c.lse = IsRing(param_) ? static_cast<float *>(pack.outTensors.at(1).deviceData) : nullptr;
        return c;
    }

    AtbmiMlaMaskFreeCall MakeMaskFreeCall(const VariantPack &pack, void *outMask) const
    {
        AtbmiMlaMaskFreeCall c{};
        c.batch = static_cast<int32_t>(lens_.size());
        c.numQueryRows = static_cast<int32_t>(pack.inTensors.at(QUERY).desc.shape.dims[0]);
        c.templateBatch = maskFreeBatch_;
        c.templateRows = maskFreeRows_;
        c.maskLen = static_cast<int32_t>(maskLen_);
        c.hostContextLens = lens_.data();
        c.hostQueryLens = qLens_.data();
        c.maskTemplate = pack.inTensors.at(maskIdx_).deviceData;
        c.outMask = outMask;
        return c;
    }

    static bool SameShape(const AtbmiPaShape &a, const AtbmiPaShape &b)
    {
        return a.qDtype == b.qDtype && a.numHeads == b.numHeads && a.blockSize == b.blockSize &&
               a.numBlocks == b.numBlocks && a.maxBlocksPerSeq == b.maxBlocksPerSeq &&
               a.numQueryRows == b.numQueryRows && a.qkScale == b.qkScale && a.hasMask == b.hasMask &&
               a.maskBatchStride == b.maskBatchStride && a.maskLen == b.maskLen && a.kvLayout == b.kvLayout;
    }

    // Reference :558-620 (DimCheck) with :350-392 (QKVDimCheck) and :478-490 (DimCheckSpec).
    Status DimCheck(const SVector<TensorDesc> &in) const
    {
        if (in.at(QUERY).shape.dimNum != 3 || in.at(QUERY_ROPE).shape.dimNum != 3 || in.at(KV_CACHE).shape.dimNum != 4 ||
            in.at(KV_CACHE_ROPE).shape.dimNum != 4 || in.at(BLOCK_TABLES).shape.dimNum != 2 ||
            in.at(CONTEXT_LENS).shape.dimNum != 1) {
            ATB_LOG(ERROR) << "expected dims: query 3, queryRope 3, kvCache 4, kvCacheRope 4, blockTables 2, contextLens 1";
            return ERROR_INVALID_TENSOR_DIM_NUM;
        }
        const int64_t numTokens = in.at(QUERY).shape.dims[0];
        const int64_t batch = in.at(BLOCK_TABLES).shape.dims[0];
        if (batch > MAX_BATCH) {
            ATB_LOG(ERROR) << "batch should be <= " << MAX_BATCH;
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (param_.calcType == Param::CALC_TYPE_UNDEFINED && numTokens != batch) {
            ATB_LOG(ERROR) << "numTokens and batch should be the same in the decode stage";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (in.at(CONTEXT_LENS).shape.dims[0] != batch) {
            ATB_LOG(ERROR) << "dim 0 of blockTables and contextLens should be the same";
            return ERROR_INVALID_TENSOR_DIM;
        }
        const Dims &kv = in.at(KV_CACHE).shape;
        const Dims &kr = in.at(KV_CACHE_ROPE).shape;
        // token-major caches [blocks, blockSize, kvHeads, channels] (reference :350-392) or fractal-NZ
        // caches [blocks, channels / 16, blockSize, 16] (reference :394-425)
        const bool int8 = param_.cacheMode == Param::INT8_NZCACHE;
        const bool nz = param_.cacheMode == Param::NZCACHE || int8;
        const int64_t nzLatent = int8 ? NZ_CHANNELS_INT8 : NZ_CHANNELS; // slab width of the latent cache
        const int blockDim = nz ? 2 : 1;
        if (kv.dims[blockDim] != DECODER_BLOCK_SIZE) {
            ATB_LOG(ERROR) << "decoder blockSize should be " << DECODER_BLOCK_SIZE << ", got " << kv.dims[blockDim];
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (in.at(QUERY_ROPE).shape.dims[0] != numTokens) {
            ATB_LOG(ERROR) << "dim 0 of query and queryRope should be the same";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (kr.dims[0] != kv.dims[0] || kr.dims[blockDim] != kv.dims[blockDim]) {
            ATB_LOG(ERROR) << "block count and block size of kvCache and kvCacheRope should be the same";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (nz) {
            if (kv.dims[3] != nzLatent || kr.dims[3] != NZ_CHANNELS) {
                ATB_LOG(ERROR) << "dim 3 of kvCache should be " << nzLatent << ", of kvCacheRope " << NZ_CHANNELS;
                return ERROR_INVALID_TENSOR_DIM;
            }
        } else if (kv.dims[2] != param_.kvHeadNum || kr.dims[2] != param_.kvHeadNum) {
            ATB_LOG(ERROR) << "dim 2 of kvCache and kvCacheRope should equal kvHeadNum";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (in.at(QUERY).shape.dims[1] != param_.headNum || in.at(QUERY_ROPE).shape.dims[1] != param_.headNum) {
            ATB_LOG(ERROR) << "dim 1 of query and queryRope should equal headNum";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (in.at(QUERY).shape.dims[2] != LATENT_DIM || (nz ? kv.dims[1] * nzLatent : kv.dims[3]) != LATENT_DIM) {
            ATB_LOG(ERROR) << "head size of query and kvCache should be 512";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (in.at(QUERY_ROPE).shape.dims[2] != ROPE_DIM || (nz ? kr.dims[1] * NZ_CHANNELS : kr.dims[3]) != ROPE_DIM) {
            ATB_LOG(ERROR) << "head size of queryRope and kvCacheRope should be 64";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (qLensIdx_ != NONE) {
            const Dims &ql = in.at(qLensIdx_).shape;
            if (ql.dimNum != 1) {
                ATB_LOG(ERROR) << "qSeqlen should have 1 dim";
                return ERROR_INVALID_TENSOR_DIM_NUM;
            }
            if (ql.dims[0] != batch) {
                ATB_LOG(ERROR) << "dim 0 of qSeqlen should equal dim 0 of contextLens";
                return ERROR_INVALID_TENSOR_DIM;
            }
        }
        if (IsSpec(param_) && maskUseIdx_ != NONE && (param_.headNum == JOB_PER_TOKEN_HEADS || int8)) {
            // reference :536-551 with :569-575
            const Dims &u = in.at(maskUseIdx_).shape;
            if (u.dimNum != 0 && Utils::GetTensorSize(in.at(maskUseIdx_)) != 0) { // (an empty tensor: left out)
                if (u.dimNum != 1) {
                    ATB_LOG(ERROR) << "maskUseStatus should have 1 dim";
                    return ERROR_INVALID_TENSOR_DIM_NUM;
                }
                if (u.dims[0] != batch) {
                    ATB_LOG(ERROR) << "dim 0 of maskUseStatus should equal dim 0 of contextLens";
                    return ERROR_INVALID_TENSOR_DIM;
                }
            }
        }
        if (int8 && IsRing(param_) && param_.maskType == Param::UNDEFINED) {
            // reference :493-511 (only this combination checks the descales there)
            const Dims &d0 = in.at(descaleIdx_).shape;
            const Dims &d1 = in.at(descaleIdx_ + 1).shape;
            if (d0.dimNum != 1 || d1.dimNum != 1) {
                ATB_LOG(ERROR) << "qkDescale and pvDescale should have 1 dim";
                return ERROR_INVALID_TENSOR_DIM_NUM;
            }
            if (d0.dims[0] != param_.headNum || d1.dims[0] != param_.headNum) {
                ATB_LOG(ERROR) << "qkDescale and pvDescale should be [headNum]";
                return ERROR_INVALID_TENSOR_DIM;
            }
        }
        return NO_ERROR;
    }

    Param param_;
    OpIr irTable_;
    size_t maskIdx_ = NONE;
    size_t qLensIdx_ = NONE;
    size_t descaleIdx_ = NONE;
    size_t maskUseIdx_ = NONE;
    std::vector<int32_t> lens_;   // (int8 cache mode: the lengths of the last Setup)
    std::vector<int32_t> qLens_;
    std::vector<int32_t> causalUse_; // the maskUseStatus flags of the last Setup (empty: every sequence)
    bool useMask_ = false;           // the mask tensor is added to the scores
    bool maskFree_ = false;          // ... after its expansion from the MASK_FREE template
    bool causalRows_ = false;
    int64_t maskLen_ = 0;
    int32_t maskFreeRows_ = 0, maskFreeBatch_ = 0;
    uint64_t planBytes_ = 0, maskFreeTableOff_ = 0, maskFreeTableBytes_ = 0, maskFreeMaskOff_ = 0, maskFreeBytes_ = 0;
    uint32_t inputNum_ = 6;
    AtbmiPaPlan *plan_ = nullptr;
    AtbmiPaShape planShape_{};
};
} // namespace

template <> Status CreateOperation(const infer::MultiLatentAttentionParam &opParam, Operation **operation)
{
    if (operation == nullptr) {
        return ERROR_INVALID_PARAM;
    }
    if (!ParamRangeCheck(opParam)) {
        return ERROR_INVALID_PARAM;
    }
    if (opParam.calcType == Param::CALC_TYPE_PREFILL ? !ParamPrefillCheck(opParam) : !ParamCheck(opParam)) {
        return ERROR_INVALID_PARAM;
    }
    if (!ReservedIsZero(opParam)) {
        ATB_LOG(ERROR) << "MultiLatentAttentionParam rsv has a non-zero byte";
        return ERROR_INVALID_PARAM;
    }
    *operation = opParam.calcType == Param::CALC_TYPE_PREFILL
                     ? NewMultiLatentAttentionPrefillOperation(opParam)
                     : new (std::nothrow) MultiLatentAttentionOperation(opParam);
    if (*operation == nullptr) {
        return ERROR_OUT_OF_HOST_MEMORY;
    }
    return NO_ERROR;
}
} // namespace atb
