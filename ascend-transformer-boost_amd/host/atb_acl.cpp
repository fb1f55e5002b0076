// The tensor handle of the aclnn-style interfaces and the two-call C wrappers built on it
// (reference src/atb/utils/atb_acl_util.cpp:30-70 conversion of a handle into an atb::Tensor,
// src/ops/ops_infer/multi_latent_attention/atb_acl_mla.cpp:25-124,
// src/ops/ops_infer/paged_cache_load/atb_acl_paged_cache_load.cpp:20-86).
#include "atb/atb_acl.h"
#include <new>
#include <vector>
#include "atb/utils.h"
#include "log.h"

struct aclTensor {
    std::vector<int64_t> viewDims;
    std::vector<int64_t> strides;
    std::vector<int64_t> storageDims;
    int64_t offset = 0;
    aclDataType dataType = ACL_DT_UNDEFINED;
    aclFormat format = ACL_FORMAT_ND;
    void *data = nullptr;
};

namespace {
// device = false: the data pointer is host memory (contextLens, qSeqLen).
atb::Status ToAtbTensor(const aclTensor *src, atb::Tensor *dst, bool device)
{
    if (src == nullptr) {
        dst->hostData = nullptr;
        dst->deviceData = nullptr;
        return atb::NO_ERROR;
    }
    if (src->viewDims.size() > atb::MAX_DIM) {
        ATB_LOG(ERROR) << "tensor dimNum " << src->viewDims.size() << " is invalid, should be <= MAX_DIM(8)";
        return atb::ERROR_INVALID_TENSOR_DIM;
    }
    dst->desc.shape.dimNum = src->viewDims.size();
    for (size_t i = 0; i < src->viewDims.size(); ++i) {
        dst->desc.shape.dims[i] = src->viewDims[i];
    }
    dst->desc.format = src->format;
    dst->desc.dtype = src->dataType;
    dst->deviceData = device ? src->data : nullptr;
    dst->hostData = device ? nullptr : src->data;
    dst->dataSize = atb::Utils::GetTensorSize(dst->desc);
    return atb::NO_ERROR;
}

atb::Status RunExecute(const char *what, void *workspace, uint64_t workspaceSize, atb::Operation *op,
                       atb::Context *context)
{
    if (op == nullptr) {
        ATB_LOG(ERROR) << what << ": operation pointer is nullptr";
        return atb::ERROR_INVALID_OPERATION_ADDR;
    }
    atb::VariantPack pack; // empty: the tensors are the ones Setup bound
    return op->Execute(pack, static_cast<uint8_t *>(workspace), workspaceSize, context);
}
} // namespace

// A handle that does not convert (more than 8 dims) ends the call with the conversion's own
// status, as the reference's wrappers do (src/atb/atb_acl/atb_acl_mla.cpp:69-96).
#define ATB_ACL_CONVERT(expr)               \
    do {                                    \
        const atb::Status converted_ = (expr); \
        if (converted_ != atb::NO_ERROR) {  \
            return converted_;              \
        }                                   \
    } while (0)

extern "C" {

aclTensor *aclCreateTensor(const int64_t *viewDims, uint64_t viewDimsNum, aclDataType dataType, const int64_t *stride,
                           int64_t offset, aclFormat format, const int64_t *storageDims, uint64_t storageDimsNum,
                           void *tensorData)
{
    if ((viewDims == nullptr && viewDimsNum != 0) || viewDimsNum > 64) {
        return nullptr;
    }
    aclTensor *t = new (std::nothrow) aclTensor;
    if (t == nullptr) {
        return nullptr;
    }
    t->viewDims.assign(viewDims, viewDims + viewDimsNum);
    if (stride != nullptr) {
        t->strides.assign(stride, stride + viewDimsNum);
    }
    if (storageDims != nullptr) {
        t->storageDims.assign(storageDims, storageDims + storageDimsNum);
    }
    t->offset = offset;
    t->dataType = dataType;
    t->format = format;
    t->data = tensorData;
    return t;
}

aclnnStatus aclDestroyTensor(const aclTensor *tensor)
{
    delete tensor;
    return ACL_SUCCESS;
}

aclnnStatus aclGetViewShape(const aclTensor *tensor, int64_t **viewDims, uint64_t *viewDimsNum)
{
    if (tensor == nullptr || viewDims == nullptr || viewDimsNum == nullptr) {
        return ACL_ERROR_INVALID_PARAM;
    }
    *viewDimsNum = tensor->viewDims.size();
    *viewDims = new (std::nothrow) int64_t[tensor->viewDims.size() + 1];
    if (*viewDims == nullptr) {
        return ACL_ERROR_INVALID_PARAM;
    }
    for (size_t i = 0; i < tensor->viewDims.size(); ++i) {
        (*viewDims)[i] = tensor->viewDims[i];
    }
    return ACL_SUCCESS;
}

aclnnStatus aclGetDataType(const aclTensor *tensor, aclDataType *dataType)
{
    if (tensor == nullptr || dataType == nullptr) {
        return ACL_ERROR_INVALID_PARAM;
    }
    *dataType = tensor->dataType;
    return ACL_SUCCESS;
}

aclnnStatus aclGetFormat(const aclTensor *tensor, aclFormat *format)
{
    if (tensor == nullptr || format == nullptr) {
        return ACL_ERROR_INVALID_PARAM;
    }
    *format = tensor->format;
    return ACL_SUCCESS;
}

aclnnStatus aclGetRawTensorAddr(const aclTensor *tensor, void **addr)
{
    if (tensor == nullptr || addr == nullptr) {
        return ACL_ERROR_INVALID_PARAM;
    }
    *addr = tensor->data;
    return ACL_SUCCESS;
}

size_t aclDataTypeSize(aclDataType dataType)
{
    switch (dataType) {
        case ACL_INT8: case ACL_UINT8: case ACL_BOOL: return 1;
        case ACL_FLOAT16: case ACL_BF16: case ACL_INT16: case ACL_UINT16: return 2;
        case ACL_FLOAT: case ACL_INT32: case ACL_UINT32: return 4;
        case ACL_INT64: case ACL_UINT64: case ACL_DOUBLE: case ACL_COMPLEX64: return 8;
        case ACL_COMPLEX128: return 16;
        default: return 0;
    }
}

atb::Status AtbMLAGetWorkspaceSize(const aclTensor *qNope, const aclTensor *qRope, const aclTensor *ctKV,
                                   const aclTensor *kRope, const aclTensor *blockTables, const aclTensor *contextLens,
                                   const aclTensor *mask, const aclTensor *qSeqLen, const aclTensor *qkDescale,
                                   const aclTensor *pvDescale, int32_t headNum, float qkScale, int32_t kvHeadNum,
                                   int maskType, int calcType, uint8_t cacheMode, aclTensor *attenOut, aclTensor *lse,
                                   uint64_t *workspaceSize, atb::Operation **op, atb::Context *context)
{
    using Param = atb::infer::MultiLatentAttentionParam;
    Param param;
    param.headNum = headNum;
    param.qkScale = qkScale;
    param.kvHeadNum = kvHeadNum;
    param.maskType = Param::MaskType(maskType);
    param.calcType = Param::CalcType(calcType);
    param.cacheMode = Param::CacheMode(cacheMode);
    if (op == nullptr || workspaceSize == nullptr) {
        ATB_LOG(ERROR) << "AtbMLAGetWorkspaceSize: op and workspaceSize must not be null";
        return atb::ERROR_INVALID_OPERATION_ADDR;
    }
    if (*op == nullptr) {
        atb::Status st = atb::CreateOperation(param, op);
        if (st != atb::NO_ERROR) {
            ATB_LOG(ERROR) << "AtbMLAGetWorkspaceSize: creating the operation failed";
            return st;
        }
    }
    // The input list follows the operation's own: mask with a mask type, qSeqLen with the
    // several-query-tokens calcType, the two descales with the int8 cache mode.
    const bool int8Cache = param.cacheMode == Param::INT8_NZCACHE;
    const bool hasMask = param.maskType != Param::UNDEFINED;
    const bool hasQLens = param.calcType == Param::CALC_TYPE_SPEC;
    const bool hasLse = param.calcType == Param::CALC_TYPE_RING;
    atb::VariantPack pack;
    pack.inTensors.resize(6 + (hasMask ? 1 : 0) + (hasQLens ? 1 : 0) + (int8Cache ? 2 : 0));
    size_t i = 0;
    ATB_ACL_CONVERT(ToAtbTensor(qNope, &pack.inTensors[i++], true));
    ATB_ACL_CONVERT(ToAtbTensor(qRope, &pack.inTensors[i++], true));
    ATB_ACL_CONVERT(ToAtbTensor(ctKV, &pack.inTensors[i++], true));
    ATB_ACL_CONVERT(ToAtbTensor(kRope, &pack.inTensors[i++], true));
    ATB_ACL_CONVERT(ToAtbTensor(blockTables, &pack.inTensors[i++], true));
    ATB_ACL_CONVERT(ToAtbTensor(contextLens, &pack.inTensors[i++], false));
    if (hasMask) {
        ATB_ACL_CONVERT(ToAtbTensor(mask, &pack.inTensors[i++], true));
    }
    if (hasQLens) {
        ATB_ACL_CONVERT(ToAtbTensor(qSeqLen, &pack.inTensors[i++], false));
    }
    if (int8Cache) {
        ATB_ACL_CONVERT(ToAtbTensor(qkDescale, &pack.inTensors[i++], true));
        ATB_ACL_CONVERT(ToAtbTensor(pvDescale, &pack.inTensors[i++], true));
    }
    pack.outTensors.resize(hasLse ? 2 : 1);
    ATB_ACL_CONVERT(ToAtbTensor(attenOut, &pack.outTensors[0], true));
    if (hasLse) {
        ATB_ACL_CONVERT(ToAtbTensor(lse, &pack.outTensors[1], true));
    }
    return (*op)->Setup(pack, *workspaceSize, context);
}

atb::Status AtbMLA(void *workspace, uint64_t workspaceSize, atb::Operation *op, atb::Context *context)
{
    return RunExecute("AtbMLA", workspace, workspaceSize, op, context);
}

atb::Status AtbMLAPreFillGetWorkspaceSize(const aclTensor *q, const aclTensor *qRope, const aclTensor *k,
                                          const aclTensor *kRope, const aclTensor *v, const aclTensor *qSeqLen,
                                          const aclTensor *kvSeqLen, const aclTensor *mask, int32_t headNum,
                                          float qkScale, int32_t kvHeadNum, int maskType, uint8_t cacheMode,
                                          aclTensor *attenOut, uint64_t *workspaceSize, atb::Operation **op,
                                          atb::Context *context)
{
    using Param = atb::infer::MultiLatentAttentionParam;
    Param param;
    param.headNum = headNum;
    param.qkScale = qkScale;
    param.kvHeadNum = kvHeadNum;
    param.maskType = Param::MaskType(maskType);
    param.calcType = Param::CALC_TYPE_PREFILL;
    param.cacheMode = Param::CacheMode(cacheMode);
    if (op == nullptr || workspaceSize == nullptr) {
        ATB_LOG(ERROR) << "AtbMLAPreFillGetWorkspaceSize: op and workspaceSize must not be null";
        return atb::ERROR_INVALID_OPERATION_ADDR;
    }
    if (*op == nullptr) {
        atb::Status st = atb::CreateOperation(param, op);
        if (st != atb::NO_ERROR) {
            ATB_LOG(ERROR) << "AtbMLAPreFillGetWorkspaceSize: creating the operation failed";
            return st;
        }
    }
    // The mask travels with the mask types whose operation takes one (MASK_FREE; this wrapper has no
    // windowSize argument, so SWA_NORM never gets past creation); both length tensors are host tensors.
    const bool hasMask = param.maskType != Param::UNDEFINED && param.maskType != Param::MASK_TYPE_CAUSAL_MASK;
    atb::VariantPack pack;
    pack.inTensors.resize(hasMask ? 8 : 7);
    size_t i = 0;
    ATB_ACL_CONVERT(ToAtbTensor(q, &pack.inTensors[i++], true));
    ATB_ACL_CONVERT(ToAtbTensor(qRope, &pack.inTensors[i++], true));
    ATB_ACL_CONVERT(ToAtbTensor(k, &pack.inTensors[i++], true));
    ATB_ACL_CONVERT(ToAtbTensor(kRope, &pack.inTensors[i++], true));
    ATB_ACL_CONVERT(ToAtbTensor(v, &pack.inTensors[i++], true));
    ATB_ACL_CONVERT(ToAtbTensor(qSeqLen, &pack.inTensors[i++], false));
    ATB_ACL_CONVERT(ToAtbTensor(kvSeqLen, &pack.inTensors[i++], false));
    if (hasMask) {
        ATB_ACL_CONVERT(ToAtbTensor(mask, &pack.inTensors[i++], true));
    }
    pack.outTensors.resize(1);
    ATB_ACL_CONVERT(ToAtbTensor(attenOut, &pack.outTensors[0], true));
    return (*op)->Setup(pack, *workspaceSize, context);
}

atb::Status AtbMLAPreFill(void *workspace, uint64_t workspaceSize, atb::Operation *op, atb::Context *context)
{
    return RunExecute("AtbMLAPreFill", workspace, workspaceSize, op, context);
}

atb::Status AtbPagedCacheLoadGetWorkspaceSize(const aclTensor *keyCache, const aclTensor *valueCache,
                                              const aclTensor *blockTables, const aclTensor *contextLens,
                                              const aclTensor *key, const aclTensor *value, const aclTensor *seqStarts,
                                              int8_t kvCacheCfg, bool isSeqLensCumsumType, bool hasSeqStarts,
                                              uint64_t *workspaceSize, atb::Operation **op, atb::Context *context)
{
    atb::infer::PagedCacheLoadParam param;
    param.kvCacheCfg = atb::infer::PagedCacheLoadParam::KvCacheCfg(kvCacheCfg);
    param.isSeqLensCumsumMode = isSeqLensCumsumType;
    param.hasSeqStarts = hasSeqStarts;
    if (op == nullptr || workspaceSize == nullptr) {
        ATB_LOG(ERROR) << "AtbPagedCacheLoadGetWorkspaceSize: op and workspaceSize must not be null";
        return atb::ERROR_INVALID_OPERATION_ADDR;
    }
    if (*op == nullptr) {
        atb::Status st = atb::CreateOperation(param, op);
        if (st != atb::NO_ERROR) {
            ATB_LOG(ERROR) << "AtbPagedCacheLoadGetWorkspaceSize: creating the operation failed";
            return st;
        }
    }
    atb::VariantPack pack;
    pack.inTensors.resize(hasSeqStarts ? 7 : 6);
    size_t i = 0;
    ATB_ACL_CONVERT(ToAtbTensor(keyCache, &pack.inTensors[i++], true));
    ATB_ACL_CONVERT(ToAtbTensor(valueCache, &pack.inTensors[i++], true));
    ATB_ACL_CONVERT(ToAtbTensor(blockTables, &pack.inTensors[i++], true));
    ATB_ACL_CONVERT(ToAtbTensor(contextLens, &pack.inTensors[i++], true));
    ATB_ACL_CONVERT(ToAtbTensor(key, &pack.inTensors[i++], true));
    ATB_ACL_CONVERT(ToAtbTensor(value, &pack.inTensors[i++], true));
    if (hasSeqStarts) {
        ATB_ACL_CONVERT(ToAtbTensor(seqStarts, &pack.inTensors[i++], true));
    }
    pack.outTensors.resize(2);
    ATB_ACL_CONVERT(ToAtbTensor(key, &pack.outTensors[0], true));
    ATB_ACL_CONVERT(ToAtbTensor(value, &pack.outTensors[1], true));
    return (*op)->Setup(pack, *workspaceSize, context);
}

atb::Status AtbPagedCacheLoad(void *workspace, uint64_t workspaceSize, atb::Operation *op, atb::Context *context)
{
    return RunExecute("AtbPagedCacheLoad", workspace, workspaceSize, op, context);
}

} // extern "C"
