// A decode step executed on the GPU by a caller that uses only the reference's public C++ API
// (atb/atb_infer.h) plus the HIP runtime for memory and the stream: the counterpart of the reference's
// own demos (example/op_demo/reshape_and_cache/reshape_and_cache_inference_demo.cpp:111-114 and
// example/op_demo/paged_attention/paged_attention_inference_demo.cpp:83-127), which use the CANN runtime
// for the same purpose. CreateContext -> SetExecuteStream -> CreateOperation -> Setup -> Execute -> sync,
// first the cache write, then the attention, on inputs read from a file; the output and both caches go
// to a second file. tests/test_a_cpp_gpu_caller.py writes the first file, runs this program as a child
// process and compares the second file with the oracle.
//
//   atb_gpu_caller <input file> <output file>
//
// Input file: int32 header {magic 0x41544231, batch, heads, kvHeads, headSize, blockSize, numBlocks,
// maxBlocksPerSeq, dtype (1 fp16, 27 bf16)}, then contextLens[batch], blockTables[batch][maxBlocksPerSeq],
// slotMapping[batch] (int32), query[batch][heads][headSize], key / value[batch][kvHeads][headSize],
// keyCache / valueCache[numBlocks][blockSize][kvHeads][headSize] (16-bit). Output file: out, keyCache, valueCache.
#include <hip/hip_runtime_api.h>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <vector>
#include "atb/atb_infer.h"

#define CHECK_ATB(expr)                                                                    \
    do {                                                                                   \
        const atb::Status st_ = (expr);                                                    \
        if (st_ != atb::NO_ERROR) {                                                        \
            std::printf("%s:%d: %s returned %d\n", __FILE__, __LINE__, #expr, (int)st_);   \
            return 1;                                                                      \
        }                                                                                  \
    } while (0)
#define CHECK_HIP(expr)                                                                    \
    do {                                                                                   \
        const hipError_t e_ = (expr);                                                      \
        if (e_ != hipSuccess) {                                                            \
            std::printf("%s:%d: %s: %s\n", __FILE__, __LINE__, #expr, hipGetErrorString(e_)); \
            return 1;                                                                      \
        }                                                                                  \
    } while (0)

namespace {

struct Header {
    int32_t magic, batch, heads, kvHeads, headSize, blockSize, numBlocks, maxBlocks, dtype;
};

template <typename T> bool ReadArray(FILE *f, std::vector<T> &v, size_t n)
{
    v.resize(n);
    return std::fread(v.data(), sizeof(T), n, f) == n;
}

// A device tensor with the given shape, filled from `host`.
template <typename T>
int MakeDeviceTensor(aclDataType dtype, std::vector<int64_t> dims, const std::vector<T> &host, atb::Tensor &t)
{
    t.desc.dtype = dtype;
    t.desc.format = ACL_FORMAT_ND;
    t.desc.shape.dimNum = dims.size();
    for (size_t i = 0; i < dims.size(); ++i) {
        t.desc.shape.dims[i] = dims[i];
    }
    t.dataSize = atb::Utils::GetTensorSize(t);
    if (t.dataSize != host.size() * sizeof(T)) {
        std::printf("tensor of %llu bytes, %zu given\n", (unsigned long long)t.dataSize, host.size() * sizeof(T));
        return 1;
    }
    CHECK_HIP(hipMalloc(&t.deviceData, t.dataSize));
    CHECK_HIP(hipMemcpy(t.deviceData, host.data(), t.dataSize, hipMemcpyHostToDevice));
    return 0;
}

} // namespace

int main(int argc, char **argv)
{
    if (argc != 3) {
        std::printf("usage: %s <input file> <output file>\n", argv[0]);
        return 2;
    }
    FILE *in = std::fopen(argv[1], "rb");
    Header h{};
    if (!in || std::fread(&h, sizeof(h), 1, in) != 1 || h.magic != 0x41544231) {
        std::printf("cannot read %s\n", argv[1]);
        return 2;
    }
    std::vector<int32_t> contextLens, blockTables, slotMapping;
    std::vector<uint16_t> query, key, value, keyCache, valueCache;
    const size_t rowElems = static_cast<size_t>(h.kvHeads) * h.headSize;
    const size_t cacheElems = static_cast<size_t>(h.numBlocks) * h.blockSize * rowElems;
    if (!ReadArray(in, contextLens, h.batch) || !ReadArray(in, blockTables, static_cast<size_t>(h.batch) * h.maxBlocks) ||
        !ReadArray(in, slotMapping, h.batch) || !ReadArray(in, query, static_cast<size_t>(h.batch) * h.heads * h.headSize) ||
        !ReadArray(in, key, h.batch * rowElems) || !ReadArray(in, value, h.batch * rowElems) ||
        !ReadArray(in, keyCache, cacheElems) || !ReadArray(in, valueCache, cacheElems)) {
        std::printf("%s is truncated\n", argv[1]);
        return 2;
    }
    std::fclose(in);
    const aclDataType dtype = static_cast<aclDataType>(h.dtype);

    CHECK_HIP(hipSetDevice(0));
    atb::Context *context = nullptr;
    CHECK_ATB(atb::CreateContext(&context));
    hipStream_t stream = nullptr;
    CHECK_HIP(hipStreamCreate(&stream));
    CHECK_ATB(context->SetExecuteStream(stream));

    atb::Tensor tQuery, tKey, tValue, tKeyCache, tValueCache, tSlots, tTables, tLens, tOut;
    if (MakeDeviceTensor(dtype, {h.batch, h.heads, h.headSize}, query, tQuery) ||
        MakeDeviceTensor(dtype, {h.batch, h.kvHeads, h.headSize}, key, tKey) ||
        MakeDeviceTensor(dtype, {h.batch, h.kvHeads, h.headSize}, value, tValue) ||
        MakeDeviceTensor(dtype, {h.numBlocks, h.blockSize, h.kvHeads, h.headSize}, keyCache, tKeyCache) ||
        MakeDeviceTensor(dtype, {h.numBlocks, h.blockSize, h.kvHeads, h.headSize}, valueCache, tValueCache) ||
        MakeDeviceTensor(ACL_INT32, {h.batch}, slotMapping, tSlots) ||
        MakeDeviceTensor(ACL_INT32, {h.batch, h.maxBlocks}, blockTables, tTables) ||
        MakeDeviceTensor(ACL_INT32, {h.batch}, contextLens, tLens)) {
        return 1;
    }
    tLens.hostData = contextLens.data(); // the operation plans from the host copy of the lengths

    // ---- the cache write of the step
    atb::infer::ReshapeAndCacheParam cacheParam;
    atb::Operation *cacheWrite = nullptr;
    CHECK_ATB(atb::CreateOperation(cacheParam, &cacheWrite));
    atb::VariantPack cachePack;
    cachePack.inTensors = {tKey, tValue, tKeyCache, tValueCache, tSlots};
    cachePack.outTensors = {tKeyCache, tValueCache};
    uint64_t workspaceSize = 0;
    CHECK_ATB(cacheWrite->Setup(cachePack, workspaceSize, context));
    uint8_t *workspace = nullptr;
    if (workspaceSize > 0) {
        CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&workspace), workspaceSize));
    }
    CHECK_ATB(cacheWrite->Execute(cachePack, workspace, workspaceSize, context));

    // ---- the attention of the step, on the same stream
    atb::infer::PagedAttentionParam param;
    param.headNum = h.heads;
    param.kvHeadNum = h.kvHeads;
    param.qkScale = 1.0f / std::sqrt(static_cast<float>(h.headSize));
    atb::Operation *attention = nullptr;
    CHECK_ATB(atb::CreateOperation(param, &attention));
    atb::VariantPack pack;
    pack.inTensors = {tQuery, tKeyCache, tValueCache, tTables, tLens};
    atb::SVector<atb::TensorDesc> inDescs, outDescs;
    for (size_t i = 0; i < pack.inTensors.size(); ++i) {
        inDescs.push_back(pack.inTensors.at(i).desc);
    }
    CHECK_ATB(attention->InferShape(inDescs, outDescs));
    tOut.desc = outDescs.at(0);
    tOut.dataSize = atb::Utils::GetTensorSize(tOut);
    CHECK_HIP(hipMalloc(&tOut.deviceData, tOut.dataSize));
    CHECK_HIP(hipMemset(tOut.deviceData, 0, tOut.dataSize));
    pack.outTensors = {tOut};
    uint64_t attentionWorkspace = 0;
    CHECK_ATB(attention->Setup(pack, attentionWorkspace, context));
    uint8_t *attentionWs = nullptr;
    if (attentionWorkspace > 0) {
        CHECK_HIP(hipMalloc(reinterpret_cast<void **>(&attentionWs), attentionWorkspace));
    }
    CHECK_ATB(attention->Execute(pack, attentionWs, attentionWorkspace, context));
    CHECK_HIP(hipStreamSynchronize(stream));

    // ---- results
    std::vector<uint16_t> out(tOut.dataSize / 2);
    CHECK_HIP(hipMemcpy(out.data(), tOut.deviceData, tOut.dataSize, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(keyCache.data(), tKeyCache.deviceData, tKeyCache.dataSize, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(valueCache.data(), tValueCache.deviceData, tValueCache.dataSize, hipMemcpyDeviceToHost));
    FILE *dump = std::fopen(argv[2], "wb");
    if (!dump || std::fwrite(out.data(), 2, out.size(), dump) != out.size() ||
        std::fwrite(keyCache.data(), 2, keyCache.size(), dump) != keyCache.size() ||
        std::fwrite(valueCache.data(), 2, valueCache.size(), dump) != valueCache.size()) {
        std::printf("cannot write %s\n", argv[2]);
        return 2;
    }
    std::fclose(dump);

    for (atb::Tensor *t : {&tQuery, &tKey, &tValue, &tKeyCache, &tValueCache, &tSlots, &tTables, &tLens, &tOut}) {
        CHECK_HIP(hipFree(t->deviceData));
    }
    if (workspace) {
        CHECK_HIP(hipFree(workspace));
    }
    if (attentionWs) {
        CHECK_HIP(hipFree(attentionWs));
    }
    CHECK_ATB(atb::DestroyOperation(attention)); // operations first, the context after them
    CHECK_ATB(atb::DestroyOperation(cacheWrite));
    CHECK_HIP(hipStreamDestroy(stream));
    CHECK_ATB(atb::DestroyContext(context));
    std::printf("ok workspace %llu\n", (unsigned long long)attentionWorkspace);
    return 0;
}
