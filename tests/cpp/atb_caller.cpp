// A caller written against the reference's public C++ API only (atb/atb_infer.h): context, two
// operations, InferShape and Setup of a decode step, as an ATB user writes them. Built and run by
// tests/test_host_api.py on the CPU: Setup is host-only, so the device pointers are placeholders and
// Execute is not called. Prints "ok" and returns 0 when every call behaves as documented.
#include <cstdint>
#include <cstdio>
#include <vector>
#include "atb/atb_infer.h"

#define EXPECT(cond)                                                       \
    do {                                                                   \
        if (!(cond)) {                                                     \
            std::printf("%s:%d: %s failed\n", __FILE__, __LINE__, #cond); \
            return 1;                                                      \
        }                                                                  \
    } while (0)

static atb::Tensor MakeTensor(aclDataType dtype, std::vector<int64_t> dims, void *device, void *host = nullptr)
{
    atb::Tensor t;
    t.desc.dtype = dtype;
    t.desc.format = ACL_FORMAT_ND;
    t.desc.shape.dimNum = dims.size();
    for (size_t i = 0; i < dims.size(); ++i) {
        t.desc.shape.dims[i] = dims[i];
    }
    t.deviceData = device;
    t.hostData = host;
    t.dataSize = atb::Utils::GetTensorSize(t);
    return t;
}

int main()
{
    void *fake = reinterpret_cast<void *>(0x10000);
    atb::Context *context = nullptr;
    EXPECT(atb::CreateContext(&context) == atb::NO_ERROR && context != nullptr);
    EXPECT(context->SetExecuteStream(reinterpret_cast<aclrtStream>(0x1)) == atb::NO_ERROR);
    EXPECT(context->GetExecuteStream() == reinterpret_cast<aclrtStream>(0x1));

    // the cache write of a decode step: 4 tokens, 8 KV heads of 128 channels, 64 blocks of 128 slots
    atb::infer::ReshapeAndCacheParam cacheParam;
    atb::Operation *cacheWrite = nullptr;
    EXPECT(atb::CreateOperation(cacheParam, &cacheWrite) == atb::NO_ERROR);
    EXPECT(cacheWrite->GetName() == "ReshapeAndCacheOperation");
    EXPECT(cacheWrite->GetInputNum() == 5 && cacheWrite->GetOutputNum() == 2);
    atb::VariantPack cachePack;
    cachePack.inTensors = {MakeTensor(ACL_FLOAT16, {4, 8, 128}, fake), MakeTensor(ACL_FLOAT16, {4, 8, 128}, fake),
                           MakeTensor(ACL_FLOAT16, {64, 128, 8, 128}, fake),
                           MakeTensor(ACL_FLOAT16, {64, 128, 8, 128}, fake), MakeTensor(ACL_INT32, {4}, fake)};
    cachePack.outTensors = {cachePack.inTensors.at(2), cachePack.inTensors.at(3)};
    uint64_t workspaceSize = 1;
    EXPECT(cacheWrite->Setup(cachePack, workspaceSize, context) == atb::NO_ERROR && workspaceSize == 0);

    // the attention of the same step
    atb::infer::PagedAttentionParam param;
    param.headNum = 32;
    param.kvHeadNum = 8;
    param.qkScale = 0.08838834764831843f;
    atb::Operation *attention = nullptr;
    EXPECT(atb::CreateOperation(param, &attention) == atb::NO_ERROR);
    EXPECT(attention->GetInputNum() == 5 && attention->GetOutputNum() == 1);
    int32_t contextLens[4] = {100, 7, 512, 1};
    atb::SVector<atb::TensorDesc> inDescs;
    atb::VariantPack pack;
    pack.inTensors = {MakeTensor(ACL_FLOAT16, {4, 32, 128}, fake), MakeTensor(ACL_FLOAT16, {64, 128, 8, 128}, fake),
                      MakeTensor(ACL_FLOAT16, {64, 128, 8, 128}, fake), MakeTensor(ACL_INT32, {4, 4}, fake),
                      MakeTensor(ACL_INT32, {4}, fake, contextLens)};
    for (size_t i = 0; i < pack.inTensors.size(); ++i) {
        inDescs.push_back(pack.inTensors.at(i).desc);
    }
    atb::SVector<atb::TensorDesc> outDescs;
    EXPECT(attention->InferShape(inDescs, outDescs) == atb::NO_ERROR && outDescs.size() == 1);
    EXPECT(outDescs.at(0).shape.dimNum == 3 && outDescs.at(0).shape.dims[0] == 4 && outDescs.at(0).shape.dims[1] == 32 &&
           outDescs.at(0).shape.dims[2] == 128 && outDescs.at(0).dtype == ACL_FLOAT16);
    atb::Tensor out;
    out.desc = outDescs.at(0);
    out.deviceData = fake;
    out.dataSize = atb::Utils::GetTensorSize(out);
    pack.outTensors = {out};
    EXPECT(attention->Setup(pack, workspaceSize, context) == atb::NO_ERROR && workspaceSize > 0);
    // a context length beyond the block table is caught on the host, before anything is launched
    contextLens[2] = 4 * 128 + 1;
    EXPECT(attention->Setup(pack, workspaceSize, context) == atb::ERROR_INVALID_PARAM);
    // Execute without a successful Setup is refused
    EXPECT(attention->Execute(pack, nullptr, 0, context) != atb::NO_ERROR);
    // a wrong parameter is refused at creation and leaves no operation behind
    atb::infer::PagedAttentionParam bad = param;
    bad.headNum = 0;
    atb::Operation *none = nullptr;
    EXPECT(atb::CreateOperation(bad, &none) == atb::ERROR_INVALID_PARAM && none == nullptr);

    // the operation whose param can be read back and replaced (reference include/atb/operation.h:130,140)
    atb::infer::ReshapeAndCacheOmniParam omniParam;
    atb::Operation *omni = nullptr;
    EXPECT(atb::CreateOperation(omniParam, &omni) == atb::NO_ERROR && omni != nullptr);
    EXPECT(omni->GetName() == "ReshapeAndCacheOmniOperation" && omni->GetInputNum() == 8 && omni->GetOutputNum() == 2);
    atb::infer::ReshapeAndCacheOmniParam readBack;
    readBack.rsv[3] = 9;
    EXPECT(atb::CloneOperationParam(omni, readBack) == atb::NO_ERROR && readBack.rsv[3] == 0);
    EXPECT(atb::UpdateOperationParam(omni, omniParam) == atb::NO_ERROR);
    EXPECT(atb::CloneOperationParam(attention, readBack) == atb::ERROR_INVALID_PARAM);   // another operation's type
    EXPECT(atb::UpdateOperationParam(static_cast<atb::Operation *>(nullptr), omniParam) == atb::ERROR_INVALID_PARAM);
    EXPECT(atb::GetExecuteStreamId(omni) == 0 && atb::SetExecuteStreamId(omni, 2) == atb::NO_ERROR &&
           atb::GetExecuteStreamId(omni) == 2);
    EXPECT(atb::SetExecuteStreamId(nullptr, 1) == atb::ERROR_INVALID_PARAM);
    EXPECT(atb::DestroyOperation(omni) == atb::NO_ERROR);

    EXPECT(atb::DestroyOperation(attention) == atb::NO_ERROR);
    EXPECT(atb::DestroyOperation(cacheWrite) == atb::NO_ERROR);
    EXPECT(atb::DestroyContext(context) == atb::NO_ERROR);
    std::printf("ok\n");
    return 0;
}
