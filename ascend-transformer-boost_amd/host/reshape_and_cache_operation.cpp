// ReshapeAndCacheOperation on MI355X: parameter and shape validation as in
// the reference operator (reference
// src/ops/ops_infer/reshape_and_cache/reshape_and_cache_operation.cpp:43-99 create,
// :124-158 tensor counts / InferShape, :176-319 dim checks), launching the
// gfx950 copy kernel through the C ABI.
//
// Supported: K_CACHE_V_CACHE (key + value caches), also with head compression
// (COMPRESS_TYPE_KVHEAD: + wins, seqLens; COMPRESS_TYPE_KVHEAD_ROPE: + wins,
// seqLens, offsetIndex), K_CACHE_V_BYPASS (key cache only) and K_CACHE_V_CACHE_NZ
// (fractal-NZ caches, the layout MultiLatentAttention's NZCACHE / INT8_NZCACHE
// modes read; reference :321-377 KVCacheDimCheck910BNZ).
#include <new>
#include "atb/infer_op_params.h"
#include "atb/utils.h"
#include "atbmi_kernels.h"
#include "log.h"
#include "operation_base.h"

namespace atb {
namespace {
using Param = infer::ReshapeAndCacheParam;

// extra: the int32 inputs after slotMapping (reference ops_configs/atb_ops_info.ini:851-908)
OpIr MakeIr(bool siso, int extra = 0)
{
    OpIr ir;
    for (aclDataType t : {ACL_FLOAT16, ACL_INT8, ACL_BF16}) {
        IrCombo c;
        if (extra == 3 && t == ACL_INT8) {
            continue; // the window mean is built for 16-bit rows only
        }
        if (siso) {
            c.inDtypes = {t, t, ACL_INT32};
            c.outDtypes = {t};
        } else {
            c.inDtypes = {t, t, t, t, ACL_INT32};
            c.inDtypes.insert(c.inDtypes.end(), extra, ACL_INT32);
            c.outDtypes = {t, t};
        }
        c.inFormats.assign(c.inDtypes.size(), ACL_FORMAT_ND);
        c.outFormats.assign(c.outDtypes.size(), ACL_FORMAT_ND);
        ir.push_back(c);
    }
    return ir;
}

// Fractal-NZ caches (reference ops_configs/atb_ops_info.ini:829-850): int8 or 16-bit key rows with 16-bit value
// rows of either type.
OpIr MakeNzIr()
{
    OpIr ir;
    const aclDataType pairs[6][2] = {{ACL_INT8, ACL_FLOAT16}, {ACL_INT8, ACL_BF16},  {ACL_FLOAT16, ACL_FLOAT16},
                                     {ACL_BF16, ACL_BF16},    {ACL_FLOAT16, ACL_BF16}, {ACL_BF16, ACL_FLOAT16}};
    for (const auto &p : pairs) {
        IrCombo c;
        c.inDtypes = {p[0], p[1], p[0], p[1], ACL_INT32};
        c.outDtypes = {p[0], p[1]};
        c.inFormats = {ACL_FORMAT_ND, ACL_FORMAT_ND, ACL_FORMAT_FRACTAL_NZ, ACL_FORMAT_FRACTAL_NZ, ACL_FORMAT_ND};
        c.outFormats = {ACL_FORMAT_FRACTAL_NZ, ACL_FORMAT_FRACTAL_NZ};
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

class ReshapeAndCacheOperation : public OperationBase {
public:
    explicit ReshapeAndCacheOperation(const Param &param)
        : OperationBase("ReshapeAndCacheOperation"), param_(param), siso_(param.kvCacheCfg == Param::K_CACHE_V_BYPASS),
          nz_(param.kvCacheCfg == Param::K_CACHE_V_CACHE_NZ),
          extra_(param.compressType == Param::COMPRESS_TYPE_KVHEAD ? 2
                 : param.compressType == Param::COMPRESS_TYPE_KVHEAD_ROPE ? 3 : 0)
    {
        static const OpIr normal = MakeIr(false);
        static const OpIr single = MakeIr(true);
        static const OpIr keepLast = MakeIr(false, 2);
        static const OpIr meanWindow = MakeIr(false, 3);
        static const OpIr fractal = MakeNzIr();
        ir_ = nz_ ? &fractal : siso_ ? &single : extra_ == 2 ? &keepLast : extra_ == 3 ? &meanWindow : &normal;
    }

    // reference :124-136: + wins, seqLens (+ offsetIndex) under head compression
    uint32_t GetInputNum() const override { return siso_ ? 3 : 5 + extra_; }
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
        return siso_ ? DimCheckSiso(in) : nz_ ? DimCheckNz(in) : DimCheck(in);
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
        const size_t keyCacheIdx = siso_ ? 1 : 2;
        if (!SameDesc(in.at(keyCacheIdx), outTensors.at(0).desc) ||
            (!siso_ && !SameDesc(in.at(3), outTensors.at(1).desc))) {
            ATB_LOG(ERROR) << "ReshapeAndCache: output descs must equal the cache input descs";
            return ERROR_INVALID_TENSOR_DIM;
        }
        return NO_ERROR;
    }

    Status PlanImpl(const VariantPack &pack, uint64_t &workspaceSize) override
    {
        // The kernel-level checks of the reference
        // (src/kernels/mixkernels/reshape_and_cache/reshape_and_cache_operation.cpp:95-196):
        // slot count equals token count.
        const Tensor &slots = pack.inTensors.at(siso_ ? 2 : 4);
        if (extra_ > 0) {
            // reference kernel library reshape_and_cache_operation.cpp:198-229,246-275: one slot, window (and
            // offset) per (sequence, head) pair
            const Tensor &seqLens = pack.inTensors.at(6);
            if (pack.inTensors.at(5).desc.shape.dimNum != 1 || seqLens.desc.shape.dimNum != 1 ||
                (extra_ == 3 && pack.inTensors.at(7).desc.shape.dimNum != 1)) {
                ATB_LOG(ERROR) << "ReshapeAndCache: wins, seqLens and offsetIndex should have one dim";
                return ERROR_INVALID_PARAM;
            }
            const int64_t pairs = seqLens.desc.shape.dims[0] * pack.inTensors.at(0).desc.shape.dims[1];
            if (slots.desc.shape.dims[0] != pairs || pack.inTensors.at(5).desc.shape.dims[0] != pairs ||
                (extra_ == 3 && pack.inTensors.at(7).desc.shape.dims[0] != pairs)) {
                ATB_LOG(ERROR) << "ReshapeAndCache: slotMapping, wins and offsetIndex should have batch * numHeads = "
                               << pairs << " entries";
                return ERROR_INVALID_PARAM;
            }
            workspaceSize = 0;
            return NO_ERROR;
        }
        if (slots.desc.shape.dims[0] != pack.inTensors.at(0).desc.shape.dims[0]) {
            ATB_LOG(ERROR) << "ReshapeAndCache: slotMapping length must equal the token count";
            return ERROR_INVALID_PARAM;
        }
        workspaceSize = 0;
        return NO_ERROR;
    }

    Status LaunchImpl(const VariantPack &pack, uint8_t *, uint64_t, aclrtStream stream) override
    {
        const Tensor &key = pack.inTensors.at(0);
        const Tensor &keyCacheIn = pack.inTensors.at(siso_ ? 1 : 2);
        const Tensor &slots = pack.inTensors.at(siso_ ? 2 : 4);
        // Outputs are the caches themselves; callers alias them to the cache
        // inputs (the reference kernel never reads the cache inputs either,
        // op_kernel/reshape_and_cache_nd.cpp:21-28,91-98).
        const Tensor &keyCacheOut = pack.outTensors.at(0);
        const int64_t tokens = key.desc.shape.dims[0];
        const int64_t heads = key.desc.shape.dims[1];
        const int64_t dk = key.desc.shape.dims[2];
        const int64_t numSlots = keyCacheIn.desc.shape.dims[0] * keyCacheIn.desc.shape.dims[nz_ ? 2 : 1];
        const int32_t elemBytes = key.desc.dtype == ACL_INT8 ? 1 : 2;
        const void *value = nullptr;
        void *valueCache = nullptr;
        int64_t dv = 0;
        if (!siso_) {
            value = pack.inTensors.at(1).deviceData;
            valueCache = pack.outTensors.at(1).deviceData;
            dv = pack.inTensors.at(1).desc.shape.dims[2];
            if (!value || !valueCache) {
                ATB_LOG(ERROR) << "ReshapeAndCache: value / valueCache device pointer is null";
                return ERROR_INVALID_PARAM;
            }
        }
        if (!key.deviceData || !keyCacheOut.deviceData || !slots.deviceData) {
            ATB_LOG(ERROR) << "ReshapeAndCache: key / keyCache / slotMapping device pointer is null";
            return ERROR_INVALID_PARAM;
        }
        if (nz_) {
            const Tensor &valueIn = pack.inTensors.at(1);
            int rc = atbmi_reshape_and_cache_nz(key.deviceData, value, keyCacheOut.deviceData, valueCache,
                                                static_cast<const int32_t *>(slots.deviceData), tokens, heads * dk,
                                                valueIn.desc.shape.dims[1] * dv, keyCacheIn.desc.shape.dims[2],
                                                keyCacheIn.desc.shape.dims[0], elemBytes,
                                                valueIn.desc.dtype == ACL_INT8 ? 1 : 2, stream);
            if (rc != 0) {
                ATB_LOG(ERROR) << "ReshapeAndCache launch failed: " << atbmi_last_error();
            }
            return rc;
        }
        if (extra_ > 0) {
            const int32_t dtype = key.desc.dtype == ACL_INT8 ? ATBMI_INT8 : key.desc.dtype == ACL_BF16 ? ATBMI_BF16 : ATBMI_F16;
            int rc = atbmi_reshape_and_cache_compress(
                key.deviceData, value, keyCacheOut.deviceData, valueCache, static_cast<const int32_t *>(slots.deviceData),
                static_cast<const int32_t *>(pack.inTensors.at(5).deviceData),
                static_cast<const int32_t *>(pack.inTensors.at(6).deviceData),
                extra_ == 3 ? static_cast<const int32_t *>(pack.inTensors.at(7).deviceData) : nullptr,
                pack.inTensors.at(6).desc.shape.dims[0], heads, dk, tokens, numSlots, dtype, stream);
            if (rc != 0) {
                ATB_LOG(ERROR) << "ReshapeAndCache launch failed: " << atbmi_last_error();
            }
            return rc;
        }
        int rc = atbmi_reshape_and_cache(key.deviceData, value, keyCacheOut.deviceData, valueCache,
                                         static_cast<const int32_t *>(slots.deviceData), tokens, heads, dk, dv,
                                         numSlots, elemBytes, stream);
        if (rc != 0) {
            ATB_LOG(ERROR) << "ReshapeAndCache launch failed: " << atbmi_last_error();
        }
        return rc;
    }

private:
    // Reference reshape_and_cache_operation.cpp:217-252 (DimCheck) and :280-319 (KVCacheDimCheck910B).
    Status DimCheck(const SVector<TensorDesc> &in) const
    {
        if (in.at(0).shape.dimNum != 3 || in.at(1).shape.dimNum != 3 || in.at(2).shape.dimNum != 4 ||
            in.at(3).shape.dimNum != 4 || in.at(4).shape.dimNum != 1) {
            ATB_LOG(ERROR) << "ReshapeAndCache: expected dims 3/3/4/4/1";
            return ERROR_INVALID_TENSOR_DIM_NUM;
        }
        const Dims &k = in.at(0).shape;
        const Dims &v = in.at(1).shape;
        const Dims &kc = in.at(2).shape;
        const Dims &vc = in.at(3).shape;
        if (k.dims[0] != v.dims[0] || k.dims[1] != v.dims[1]) {
            ATB_LOG(ERROR) << "ReshapeAndCache: key and value must agree on tokens and heads";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (kc.dims[0] != vc.dims[0] || kc.dims[1] != vc.dims[1]) {
            ATB_LOG(ERROR) << "ReshapeAndCache: caches must agree on numBlocks and blockSize";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (extra_ > 0) {
            // reference :286-305: one head per cache slot, equal head sizes, a multiple of 32
            if (k.dims[2] != v.dims[2] || k.dims[2] != kc.dims[3] || k.dims[2] != vc.dims[3]) {
                ATB_LOG(ERROR) << "ReshapeAndCache: head compress key, value and cache headSizes should be same";
                return ERROR_INVALID_TENSOR_DIM;
            }
            if (kc.dims[2] != 1 || vc.dims[2] != 1) {
                ATB_LOG(ERROR) << "ReshapeAndCache: dim 2 of head compress keyCache and valueCache should be 1";
                return ERROR_INVALID_TENSOR_DIM;
            }
            if (k.dims[2] % 32 != 0) {
                ATB_LOG(ERROR) << "ReshapeAndCache: head compress headSizes must be a multiple of 32";
                return ERROR_INVALID_TENSOR_DIM;
            }
        } else if (k.dims[1] != kc.dims[2] || v.dims[1] != vc.dims[2]) {
            ATB_LOG(ERROR) << "ReshapeAndCache: head count of key/value must equal that of the caches";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (k.dims[2] != kc.dims[3] || v.dims[2] != vc.dims[3]) {
            ATB_LOG(ERROR) << "ReshapeAndCache: head size of key/value must equal that of the caches";
            return ERROR_INVALID_TENSOR_DIM;
        }
        return NO_ERROR;
    }

    // Reference reshape_and_cache_operation.cpp:254-278 (DimCheckSISO).
    Status DimCheckSiso(const SVector<TensorDesc> &in) const
    {
        if (in.at(0).shape.dimNum != 3 || in.at(1).shape.dimNum != 4 || in.at(2).shape.dimNum != 1) {
            ATB_LOG(ERROR) << "ReshapeAndCache: expected dims 3/4/1";
            return ERROR_INVALID_TENSOR_DIM_NUM;
        }
        const Dims &k = in.at(0).shape;
        const Dims &kc = in.at(1).shape;
        if (k.dims[0] != in.at(2).shape.dims[0] || k.dims[1] != kc.dims[2] || k.dims[2] != kc.dims[3]) {
            ATB_LOG(ERROR) << "ReshapeAndCache: key does not match keyCache / slotMapping";
            return ERROR_INVALID_TENSOR_DIM;
        }
        return NO_ERROR;
    }

    // Reference reshape_and_cache_operation.cpp:321-377 (KVCacheDimCheck910BNZ): caches
    // [numBlocks, heads * headSize / lastDim, blockSize, lastDim], lastDim 32 for an int8 key cache, else 16.
    Status DimCheckNz(const SVector<TensorDesc> &in) const
    {
        if (in.at(0).shape.dimNum != 3 || in.at(1).shape.dimNum != 3 || in.at(2).shape.dimNum != 4 ||
            in.at(3).shape.dimNum != 4 || in.at(4).shape.dimNum != 1) {
            ATB_LOG(ERROR) << "ReshapeAndCache: expected dims 3/3/4/4/1";
            return ERROR_INVALID_TENSOR_DIM_NUM;
        }
        const Dims &k = in.at(0).shape;
        const Dims &v = in.at(1).shape;
        const Dims &kc = in.at(2).shape;
        const Dims &vc = in.at(3).shape;
        if (k.dims[0] != v.dims[0] || k.dims[1] != v.dims[1]) {
            ATB_LOG(ERROR) << "ReshapeAndCache: key and value must agree on tokens and heads";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (kc.dims[2] != vc.dims[2]) {
            ATB_LOG(ERROR) << "ReshapeAndCache: blockSizes should be same";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (kc.dims[2] % 16 != 0) {
            ATB_LOG(ERROR) << "ReshapeAndCache: the blockSize of keyCache and valueCache should be 16-aligned";
            return ERROR_INVALID_TENSOR_DIM;
        }
        const int64_t keyLast = in.at(0).dtype == ACL_INT8 ? 32 : 16;
        if (k.dims[1] * k.dims[2] != kc.dims[1] * keyLast || kc.dims[3] != keyLast) {
            ATB_LOG(ERROR) << "ReshapeAndCache: NZ keyCache should be [blocks, heads * headSize / " << keyLast
                           << ", blockSize, " << keyLast << "]";
            return ERROR_INVALID_TENSOR_DIM;
        }
        if (v.dims[1] * v.dims[2] != vc.dims[1] * 16 || vc.dims[3] != 16) {
            ATB_LOG(ERROR) << "ReshapeAndCache: NZ valueCache should be [blocks, heads * headSize / 16, blockSize, 16]";
            return ERROR_INVALID_TENSOR_DIM;
        }
        // the kernel addresses both caches by one slot number (block = slot / blockSize)
        if (kc.dims[0] != vc.dims[0]) {
            ATB_LOG(ERROR) << "ReshapeAndCache: caches must agree on numBlocks";
            return ERROR_INVALID_TENSOR_DIM;
        }
        return NO_ERROR;
    }

    Param param_;
    bool siso_;
    bool nz_;
    uint32_t extra_; // int32 inputs after slotMapping: 2 (wins, seqLens) or 3 (+ offsetIndex) under head compression
};
} // namespace

template <> Status CreateOperation(const infer::ReshapeAndCacheParam &opParam, Operation **operation)
{
    if (operation == nullptr) {
        return ERROR_INVALID_PARAM;
    }
    if (!ReservedIsZero(opParam)) {
        ATB_LOG(ERROR) << "ReshapeAndCacheParam rsv has a non-zero byte";
        return ERROR_INVALID_PARAM;
    }
    if (opParam.compressType < Param::COMPRESS_TYPE_UNDEFINED || opParam.compressType > Param::COMPRESS_TYPE_KVHEAD_ROPE ||
        opParam.kvCacheCfg < Param::K_CACHE_V_CACHE || opParam.kvCacheCfg > Param::K_CACHE_V_CACHE_NZ) {
        ATB_LOG(ERROR) << "ReshapeAndCacheParam enum value out of range";
        return ERROR_INVALID_PARAM;
    }
    if (opParam.kvCacheCfg != Param::K_CACHE_V_CACHE && opParam.compressType != Param::COMPRESS_TYPE_UNDEFINED) {
        ATB_LOG(ERROR) << "ReshapeAndCacheParam: compressType needs K_CACHE_V_CACHE";
        return ERROR_INVALID_PARAM;
    }
    *operation = new (std::nothrow) ReshapeAndCacheOperation(opParam);
    if (*operation == nullptr) {
        return ERROR_OUT_OF_HOST_MEMORY;
    }
    return NO_ERROR;
}
} // namespace atb
