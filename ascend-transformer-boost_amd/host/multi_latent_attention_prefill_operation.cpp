// MultiLatentAttentionOperation with calcType CALC_TYPE_PREFILL on MI355X: attention of whole prompts over
// keys and values given as plain tensors (no block tables), 128 + 64 query / key channels and 128 value
// channels per head.
//
// Inputs [query, queryRope, key, keyRope, value, qSeqLen, kvSeqLen, (mask)]; one output shaped like query.
// Tensor counts, InferShape and the dim checks follow the reference operator (reference
// src/ops/ops_infer/multi_latent_attention/multi_latent_attention_operation.cpp: 245-266 counts, 268-283
// InferShape, 306-320 Setup checks, 622-672 InTensorDimCheckPrefill, 674-716 query, 718-771 key / value),
// the dtype tables its sections Prefill and MaskPrefill of ops_configs/atb_ops_info.ini (:6968-7020). Both
// length vectors are read from hostData during Setup and must agree unless the mask is CAUSAL_MASK, as in
// the reference runner (multi_latent_attention_ops_runner_prefill.cpp:98-110).
//
// What the masks mean here: MASK_FREE and CAUSAL_MASK hide key j from query i when j > i (MASK_FREE comes
// with the reference's fixed 512 x 512 strictly-upper-triangular mask tensor, reference
// tests/apitest/opstest/python/operations/multi_latent_attention/test_multi_latent_attention_prefill.py:373-391;
// its values say the same thing and are not read), SWA_NORM also hides j <= i - windowSize (:301-316).
// With CAUSAL_MASK the reference lets the two lengths of a sequence differ; its tests never do, and this
// implementation refuses such a pack during Setup.
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

constexpr size_t QUERY = 0, QUERY_ROPE = 1, KEY = 2, KEY_ROPE = 3, VALUE = 4, Q_SEQLEN = 5, KV_SEQLEN = 6, MASK = 7;
constexpr int64_t NOPE_DIM = 128; // channels of query / key / value per head
constexpr int64_t ROPE_DIM = 64;
constexpr int64_t MAX_BATCH = 8192;
constexpr int64_t COMPRESSED_MASK = 512;

bool HasMaskInput(const Param &p)
{
    return p.maskType != Param::UNDEFINED && p.maskType != Param::MASK_TYPE_CAUSAL_MASK;
}

OpIr MakeIr(const Param &p)
{
    OpIr ir;
    for (aclDataType q : {ACL_FLOAT16, ACL_BF16}) {
        IrCombo c;
        c.inDtypes = {q, q, q, q, q, ACL_INT32, ACL_INT32};
        if (HasMaskInput(p)) {
            c.inDtypes.push_back(q);
        }
        c.inFormats.assign(c.inDtypes.size(), ACL_FORMAT_ND);
        c.outDtypes = {q};
        c.outFormats = {ACL_FORMAT_ND};
        ir.push_back(c);
    }
    return ir;
}

class MultiLatentAttentionPrefillOperation : public OperationBase {
public:
    explicit MultiLatentAttentionPrefillOperation(const Param &param)
        : OperationBase("MultiLatentAttentionOperation"), param_(param), irTable_(MakeIr(param))
    {
        ir_ = &irTable_;
    }

    uint32_t GetInputNum() const override { return HasMaskInput(param_) ? 8 : 7; }
    uint32_t GetOutputNum() const override { return 1; }

protected:
    Status InferShapeImpl(const SVector<TensorDesc> &in, SVector<TensorDesc> &out) const override
    {
        out.at(0) = in.at(QUERY);
        out.at(0).dtype = in.at(QUERY_ROPE).dtype;
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
        // the output is shaped like the query (reference :312-319, tensor_check.cpp:77-88)
        const Dims &q = inTensors.at(QUERY).desc.shape;
        const Dims &o = outTensors.at(0).desc.shape;
        if (o.dimNum != q.dimNum) {
            ATB_LOG(ERROR) << "attenOut should have as many dims as query";
            return ERROR_INVALID_TENSOR_DIM_NUM;
        }
        for (uint64_t i = 0; i < o.dimNum; ++i) {
            if (o.dims[i] != q.dims[i]) {
                ATB_LOG(ERROR) << "attenOut should be shaped like query";
                return ERROR_INVALID_TENSOR_DIM;
            }
        }
        return NO_ERROR;
    }

    Status PlanImpl(const VariantPack &pack, uint64_t &workspaceSize) override
    {
        const Tensor &qLens = pack.inTensors.at(Q_SEQLEN);
        const Tensor &kvLens = pack.inTensors.at(KV_SEQLEN);
        if (!qLens.hostData || !kvLens.hostData) {
            ATB_LOG(ERROR) << "qSeqLen.hostData or kvSeqLen.hostData is null; the lengths are read on the host during Setup";
            return ERROR_INVALID_PARAM;
        }
        const int32_t batch = static_cast<int32_t>(qLens.desc.shape.dims[0]);
        const int32_t *ql = static_cast<const int32_t *>(qLens.hostData);
        const int32_t *kl = static_cast<const int32_t *>(kvLens.hostData);
        qLens_.assign(ql, ql + batch);
        kvLens_.assign(kl, kl + batch);
        int64_t qRows = 0, kRows = 0, longest = 0;
        for (int32_t b = 0; b < batch; ++b) {
            if (qLens_[b] < 0 || kvLens_[b] < 0) {
                ATB_LOG(ERROR) << "sequence " << b << " has negative length";
                return ERROR_INVALID_PARAM;
            }
            if (qLens_[b] != kvLens_[b]) {
                // (the reference refuses it unless the mask is CAUSAL_MASK; see the head of this file)
                ATB_LOG(ERROR) << "qSeqLen and kvSeqLen should be the same, sequence " << b << " has " << qLens_[b]
                               << " and " << kvLens_[b];
                return ERROR_INVALID_PARAM;
            }
            qRows += qLens_[b];
            kRows += kvLens_[b];
            longest = kvLens_[b] > longest ? kvLens_[b] : longest;
        }
        const Dims &q = pack.inTensors.at(QUERY).desc.shape;
        const Dims &k = pack.inTensors.at(KEY).desc.shape;
        if (qRows > q.dims[0]) {
            ATB_LOG(ERROR) << "qSeqLen adds up to " << qRows << " tokens, query holds " << q.dims[0];
            return ERROR_INVALID_PARAM;
        }
        // key / keyRope / value as [tokens, kvHeadNum, channels], or padded per sequence as
        // [batch, maxSeqLen, kvHeadNum * channels] (reference :722-737)
        const bool packed = k.dims[1] == param_.kvHeadNum && k.dims[2] == NOPE_DIM;
        kvPaddedRows_ = packed ? 0 : k.dims[1];
        if (packed ? kRows > k.dims[0] : longest > k.dims[1]) {
            ATB_LOG(ERROR) << "kvSeqLen does not fit the key tensor";
            return ERROR_INVALID_PARAM;
        }
        if (param_.maskType == Param::MASK_TYPE_SWA_NORM) {
            // one mask row and column per position of the longest sequence (reference kernel library
            // src/kernels/mixkernels/multi_latent_attention/mla_operation.cpp:184-204)
            const Dims &m = pack.inTensors.at(MASK).desc.shape;
            if (m.dimNum != 2 || m.dims[0] < longest || m.dims[1] < longest) {
                ATB_LOG(ERROR) << "the SWA_NORM mask should be [maxSeqLen, maxSeqLen]";
                return ERROR_INVALID_PARAM;
            }
        }
        AtbmiMlaPrefillCall call = MakeCall(pack);
        int rc = atbmi_mla_prefill_workspace_size(&call, &workspaceSize);
        if (rc != 0) {
            ATB_LOG(ERROR) << "MultiLatentAttention prefill plan: " << atbmi_last_error();
            return rc;
        }
        return NO_ERROR;
    }

    Status LaunchImpl(const VariantPack &pack, uint8_t *workspace, uint64_t workspaceSize,
                      aclrtStream stream) override
    {
        AtbmiMlaPrefillCall call = MakeCall(pack);
        int rc = atbmi_mla_prefill(&call, workspace, workspaceSize, stream);
        if (rc != 0) {
            ATB_LOG(ERROR) << "MultiLatentAttention prefill launch failed: " << atbmi_last_error();
        }
        return rc;
    }

private:
    AtbmiMlaPrefillCall MakeCall(const VariantPack &pack) const
    {
        AtbmiMlaPrefillCall c{};
        c.dtype = pack.inTensors.at(QUERY).desc.dtype == ACL_BF16 ? ATBMI_BF16 : ATBMI_F16;
        c.numHeads = param_.headNum;
        c.numKvHeads = param_.kvHeadNum;
        c.mask = param_.maskType == Param::UNDEFINED ? ATBMI_MLA_PREFILL_MASK_NONE
                 : param_.maskType == Param::MASK_TYPE_SWA_NORM ? ATBMI_MLA_PREFILL_MASK_WINDOW
                                                                : ATBMI_MLA_PREFILL_MASK_CAUSAL;
        c.windowSize = static_cast<int32_t>(param_.windowSize);
        c.qkScale = param_.qkScale;
        c.batch = static_cast<int32_t>(qLens_.size());
        c.kvPaddedRows = kvPaddedRows_;
        c.hostQLens = qLens_.data();
        c.hostKvLens = kvLens_.data();
        c.query = pack.inTensors.at(QUERY).deviceData;
        c.queryRope = pack.inTensors.at(QUERY_ROPE).deviceData;
        c.key = pack.inTensors.at(KEY).deviceData;
        c.keyRope = pack.inTensors.at(KEY_ROPE).deviceData;
        c.value = pack.inTensors.at(VALUE).deviceData;
        c.out = pack.outTensors.at(0).deviceData;
        return c;
    }

    // Reference :622-672 with :674-716 (query) and :718-771 (key, keyRope, value).
    Status DimCheck(const SVector<TensorDesc> &in) const
    {
        const Dims &q = in.at(QUERY).shape;
        const Dims &qr = in.at(QUERY_ROPE).shape;
        const Dims &k = in.at(KEY).shape;
        const Dims &kr = in.at(KEY_ROPE).shape;
        const Dims &v = in.at(VALUE).shape;
        const bool maskFree = param_.maskType == Param::MASK_TYPE_MASK_FREE;
        if ((q.dimNum != 2 && q.dimNum != 3) || qr.dimNum != q.dimNum || k.dimNum != 3 || kr.dimNum != 3 ||
            v.dimNum != 3 || in.at(Q_SEQLEN).shape.dimNum != 1 || in.at(KV_SEQLEN).shape.dimNum != 1 ||
            (maskFree && in.at(MASK).shape.dimNum != 2 && in.at(MASK).shape.dimNum != 3)) {
            ATB_LOG(ERROR) << "expected dims: query / queryRope 2 or 3, key / keyRope / value 3, qSeqLen / kvSeqLen 1, "
                              "mask 2 or 3";
            return ERROR_INVALID_TENSOR_DIM_NUM;
        }
        const int64_t batch = in.at(Q_SEQLEN).shape.dims[0];
        if (batch > MAX_BATCH) {
            ATB_LOG(ERROR) << "batch should be <= " << MAX_BATCH << ", got " << batch;
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (batch != in.at(KV_SEQLEN).shape.dims[0]) {
            ATB_LOG(ERROR) << "qSeqLen and kvSeqLen should have the same length";
            return ERROR_INVALID_TENSOR_DIM;
        }
        const int64_t heads = param_.headNum, kvHeads = param_.kvHeadNum;
        if (q.dimNum == 2 ? q.dims[1] != heads * NOPE_DIM : (q.dims[1] != heads || q.dims[2] != NOPE_DIM)) {
            ATB_LOG(ERROR) << "query should be [tokens, headNum * 128] or [tokens, headNum, 128]";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (qr.dims[0] != q.dims[0]) {
            ATB_LOG(ERROR) << "dim 0 of query and queryRope should be the same";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (qr.dimNum == 2 ? qr.dims[1] != heads * ROPE_DIM : (qr.dims[1] != heads || qr.dims[2] != ROPE_DIM)) {
            ATB_LOG(ERROR) << "queryRope should be [tokens, headNum * 64] or [tokens, headNum, 64]";
            return ERROR_INVALID_TENSOR_DIM;
        }
        const bool packed = k.dims[1] == kvHeads && k.dims[2] == NOPE_DIM;
        const bool padded = k.dims[0] == batch && k.dims[2] == kvHeads * NOPE_DIM;
        if (param_.maskType == Param::MASK_TYPE_CAUSAL_MASK ? !padded : (!packed && !padded)) {
            ATB_LOG(ERROR) << "key should be [tokens, kvHeadNum, 128] or [batch, maxSeqLen, kvHeadNum * 128]";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (kr.dims[0] != k.dims[0] || kr.dims[1] != k.dims[1] || kr.dims[2] != k.dims[2] / 2) {
            ATB_LOG(ERROR) << "keyRope should be shaped like key with half as many channels";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (v.dims[0] != k.dims[0] || v.dims[1] != k.dims[1] || v.dims[2] != k.dims[2]) {
            ATB_LOG(ERROR) << "value should be shaped like key";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (maskFree && in.at(MASK).shape.dimNum == 2 &&
            (in.at(MASK).shape.dims[0] != COMPRESSED_MASK || in.at(MASK).shape.dims[1] != COMPRESSED_MASK)) {
            ATB_LOG(ERROR) << "the MASK_FREE mask should be [512, 512]";
            return ERROR_INVALID_TENSOR_DIM;
        }
        return NO_ERROR;
    }

    Param param_;
    OpIr irTable_;
    std::vector<int32_t> qLens_;
    std::vector<int32_t> kvLens_;
    int64_t kvPaddedRows_ = 0;
};
} // namespace

// Called by CreateOperation<MultiLatentAttentionParam> once the param has passed the reference's checks.
Operation *NewMultiLatentAttentionPrefillOperation(const infer::MultiLatentAttentionParam &param)
{
    return new (std::nothrow) MultiLatentAttentionPrefillOperation(param);
}
} // namespace atb
