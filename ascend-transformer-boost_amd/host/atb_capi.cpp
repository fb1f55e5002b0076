// Flat C view of the atb::Operation API (see atb_capi.h).
#include "atb_capi.h"
#include <cstring>
#include <new>
#include <vector>
#include <exception>
#include <string>
#include "atb/atb_infer.h"

namespace {
atb::Tensor ToTensor(const AtbCTensor &c)
{
    atb::Tensor t;
    t.desc.dtype = static_cast<aclDataType>(c.dtype);
    t.desc.format = static_cast<aclFormat>(c.format);
    t.desc.shape.dimNum = c.dimNum;
    for (int i = 0; i < 8; ++i) {
        t.desc.shape.dims[i] = c.dims[i];
    }
    t.deviceData = c.deviceData;
    t.hostData = c.hostData;
    t.dataSize = c.dataSize;
    return t;
}

void FromDesc(const atb::TensorDesc &d, AtbCTensor &c)
{
    c.dtype = static_cast<int32_t>(d.dtype);
    c.format = static_cast<int32_t>(d.format);
    c.dimNum = d.shape.dimNum;
    for (int i = 0; i < 8; ++i) {
        c.dims[i] = d.shape.dims[i];
    }
}

bool FillPack(atb::VariantPack &pack, const AtbCTensor *in, uint32_t numIn, const AtbCTensor *out, uint32_t numOut)
{
    if ((numIn && !in) || (numOut && !out) || numIn > atb::MAX_SVECTOR_SIZE || numOut > atb::MAX_SVECTOR_SIZE) {
        return false;
    }
    for (uint32_t i = 0; i < numIn; ++i) {
        pack.inTensors.push_back(ToTensor(in[i]));
    }
    for (uint32_t i = 0; i < numOut; ++i) {
        pack.outTensors.push_back(ToTensor(out[i]));
    }
    return true;
}
} // namespace

extern "C" {

int32_t atb_c_create_context(void *stream, void **context)
{
    if (!context) {
        return atb::ERROR_INVALID_PARAM;
    }
    atb::Context *ctx = nullptr;
    atb::Status st = atb::CreateContext(&ctx);
    if (st != atb::NO_ERROR) {
        return st;
    }
    ctx->SetExecuteStream(stream);
    *context = ctx;
    return atb::NO_ERROR;
}

int32_t atb_c_context_set_stream(void *context, void *stream)
{
    return context ? static_cast<atb::Context *>(context)->SetExecuteStream(stream) : atb::ERROR_INVALID_PARAM;
}

int32_t atb_c_context_set_streams(void *context, void *const *streams, uint32_t count)
{
    if (!context || (!streams && count > 0)) {
        return atb::ERROR_INVALID_PARAM;
    }
    try {
        return static_cast<atb::Context *>(context)->SetExecuteStreams(std::vector<aclrtStream>(streams, streams + count));
    } catch (const std::bad_alloc &) {
        return atb::ERROR_OUT_OF_HOST_MEMORY;
    }
}

int32_t atb_c_context_set_execute_type(void *context, int32_t type)
{
    return context ? static_cast<atb::Context *>(context)->SetExecuteType(static_cast<atb::ExecuteType>(type))
                   : atb::ERROR_INVALID_PARAM;
}

int32_t atb_c_destroy_context(void *context)
{
    return atb::DestroyContext(static_cast<atb::Context *>(context));
}

int32_t atb_c_create_operation(const char *opName, const void *param, uint64_t paramSize, void **operation)
{
    if (!opName || !param) {
        return atb::ERROR_INVALID_PARAM;
    }
    atb::Operation **out = reinterpret_cast<atb::Operation **>(operation);
    if (!strcmp(opName, "PagedAttentionOperation") && paramSize == sizeof(atb::infer::PagedAttentionParam)) {
        atb::infer::PagedAttentionParam p;
        memcpy(static_cast<void *>(&p), param, sizeof(p));
        return atb::CreateOperation(p, out);
    }
    if (!strcmp(opName, "ReshapeAndCacheOperation") && paramSize == sizeof(atb::infer::ReshapeAndCacheParam)) {
        atb::infer::ReshapeAndCacheParam p;
        memcpy(static_cast<void *>(&p), param, sizeof(p));
        return atb::CreateOperation(p, out);
    }
    if (!strcmp(opName, "ReshapeAndCacheWithStrideOperation") &&
        paramSize == sizeof(atb::infer::ReshapeAndCacheWithStrideParam)) {
        atb::infer::ReshapeAndCacheWithStrideParam p;
        memcpy(static_cast<void *>(&p), param, sizeof(p));
        return atb::CreateOperation(p, out);
    }
    if (!strcmp(opName, "ReshapeAndCacheOmniOperation") && paramSize == sizeof(atb::infer::ReshapeAndCacheOmniParam)) {
        atb::infer::ReshapeAndCacheOmniParam p;
        memcpy(static_cast<void *>(&p), param, sizeof(p));
        return atb::CreateOperation(p, out);
    }
    if (!strcmp(opName, "NormRopeReshapeOperation") && paramSize == sizeof(atb::infer::NormRopeReshapeParam)) {
        atb::infer::NormRopeReshapeParam p;
        memcpy(static_cast<void *>(&p), param, sizeof(p));
        return atb::CreateOperation(p, out);
    }
    if (!strcmp(opName, "RopeOperation") && paramSize == sizeof(atb::infer::RopeParam)) {
        atb::infer::RopeParam p;
        memcpy(static_cast<void *>(&p), param, sizeof(p));
        return atb::CreateOperation(p, out);
    }
    if (!strcmp(opName, "ElewiseOperation") && paramSize == sizeof(atb::infer::ElewiseParam)) {
        atb::infer::ElewiseParam p;
        memcpy(static_cast<void *>(&p), param, sizeof(p));
        return atb::CreateOperation(p, out);
    }
    if (!strcmp(opName, "BlockCopyOperation") && paramSize == sizeof(atb::infer::BlockCopyParam)) {
        atb::infer::BlockCopyParam p;
        memcpy(static_cast<void *>(&p), param, sizeof(p));
        return atb::CreateOperation(p, out);
    }
    if (!strcmp(opName, "PagedCacheLoadOperation") && paramSize == sizeof(atb::infer::PagedCacheLoadParam)) {
        atb::infer::PagedCacheLoadParam p;
        memcpy(static_cast<void *>(&p), param, sizeof(p));
        return atb::CreateOperation(p, out);
    }
    if (!strcmp(opName, "MultiLatentAttentionOperation") &&
        paramSize == sizeof(atb::infer::MultiLatentAttentionParam)) {
        atb::infer::MultiLatentAttentionParam p;
        memcpy(static_cast<void *>(&p), param, sizeof(p));
        return atb::CreateOperation(p, out);
    }
    return atb::ERROR_INVALID_PARAM;
}

int32_t atb_c_op_set_stream_id(void *operation, uint32_t streamId)
{
    return atb::SetExecuteStreamId(static_cast<atb::Operation *>(operation), streamId);
}

uint32_t atb_c_op_get_stream_id(void *operation)
{
    return atb::GetExecuteStreamId(static_cast<atb::Operation *>(operation));
}

int32_t atb_c_destroy_operation(void *operation)
{
    return atb::DestroyOperation(static_cast<atb::Operation *>(operation));
}

uint32_t atb_c_op_input_num(void *operation)
{
    return operation ? static_cast<atb::Operation *>(operation)->GetInputNum() : 0;
}

uint32_t atb_c_op_output_num(void *operation)
{
    return operation ? static_cast<atb::Operation *>(operation)->GetOutputNum() : 0;
}

int32_t atb_c_op_name(void *operation, char *buf, uint64_t bufSize)
{
    if (!operation || !buf || bufSize == 0) {
        return atb::ERROR_INVALID_PARAM;
    }
    std::string name = static_cast<atb::Operation *>(operation)->GetName();
    strncpy(buf, name.c_str(), bufSize - 1);
    buf[bufSize - 1] = '\0';
    return atb::NO_ERROR;
}

int32_t atb_c_op_infer_shape(void *operation, const AtbCTensor *inDescs, uint32_t numIn, AtbCTensor *outDescs,
                             uint32_t outCapacity, uint32_t *numOut)
{
    if (!operation || (numIn && !inDescs) || numIn > atb::MAX_SVECTOR_SIZE) {
        return atb::ERROR_INVALID_PARAM;
    }
    try {
        atb::SVector<atb::TensorDesc> in;
        atb::SVector<atb::TensorDesc> out;
        for (uint32_t i = 0; i < numIn; ++i) {
            in.push_back(ToTensor(inDescs[i]).desc);
        }
        atb::Status st = static_cast<atb::Operation *>(operation)->InferShape(in, out);
        if (st != atb::NO_ERROR) {
            return st;
        }
        if (numOut) {
            *numOut = static_cast<uint32_t>(out.size());
        }
        for (uint32_t i = 0; i < out.size() && i < outCapacity && outDescs; ++i) {
            FromDesc(out.at(i), outDescs[i]);
        }
        return atb::NO_ERROR;
    } catch (const std::exception &) {
        return atb::ERROR_OUT_OF_HOST_MEMORY;
    }
}

int32_t atb_c_op_setup(void *operation, const AtbCTensor *inTensors, uint32_t numIn, const AtbCTensor *outTensors,
                       uint32_t numOut, uint64_t *workspaceSize, void *context)
{
    if (!operation || !workspaceSize) {
        return atb::ERROR_INVALID_PARAM;
    }
    try {
        atb::VariantPack pack;
        if (!FillPack(pack, inTensors, numIn, outTensors, numOut)) {
            return atb::ERROR_INVALID_PARAM;
        }
        uint64_t ws = 0;
        atb::Status st =
            static_cast<atb::Operation *>(operation)->Setup(pack, ws, static_cast<atb::Context *>(context));
        *workspaceSize = ws;
        return st;
    } catch (const std::exception &) {
        return atb::ERROR_OUT_OF_HOST_MEMORY;
    }
}

int32_t atb_c_op_execute(void *operation, const AtbCTensor *inTensors, uint32_t numIn,
                         const AtbCTensor *outTensors, uint32_t numOut, void *workspace, uint64_t workspaceSize,
                         void *context)
{
    if (!operation) {
        return atb::ERROR_INVALID_PARAM;
    }
    try {
        atb::VariantPack pack;
        if (!FillPack(pack, inTensors, numIn, outTensors, numOut)) {
            return atb::ERROR_INVALID_PARAM;
        }
        return static_cast<atb::Operation *>(operation)
            ->Execute(pack, static_cast<uint8_t *>(workspace), workspaceSize, static_cast<atb::Context *>(context));
    } catch (const std::exception &) {
        return atb::ERROR_RT_FAIL;
    }
}

uint64_t atb_c_tensor_size(const AtbCTensor *tensor)
{
    return tensor ? atb::Utils::GetTensorSize(ToTensor(*tensor).desc) : 0;
}

void atb_c_quant_param_convert(const float *src, uint64_t *dest, uint64_t itemCount)
{
    atb::Utils::QuantParamConvert(src, dest, itemCount);
}

uint64_t atb_c_sizeof_paged_attention_param(void)
{
    return sizeof(atb::infer::PagedAttentionParam);
}

uint64_t atb_c_sizeof_reshape_and_cache_param(void)
{
    return sizeof(atb::infer::ReshapeAndCacheParam);
}

uint64_t atb_c_sizeof_multi_latent_attention_param(void)
{
    return sizeof(atb::infer::MultiLatentAttentionParam);
}

} // extern "C"
