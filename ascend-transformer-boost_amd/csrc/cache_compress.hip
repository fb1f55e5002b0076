// KV-cache write under head compression for gfx950: every (sequence, KV head)
// pair keeps its own stretch of consecutive cache slots in caches shaped
// [numBlocks, blockSize, 1, headSize] (one head per slot).
//
//   keep-last (COMPRESS_TYPE_KVHEAD): pair i = b * heads + h copies the last
//     wins[i] tokens of sequence b, head h, to slots slotMapping[i] ... in
//     order (reference golden tests/apitest/kernelstest/mix/test_reshape_and_cache_wins.py:61-88,
//     device kernel src/kernels/mixkernels/reshape_and_cache/op_kernel/reshape_and_cache_compress.cpp).
//   mean-window (COMPRESS_TYPE_KVHEAD_ROPE): with o = offsetIndex[i] >= 0 the
//     tokens before o are copied, the wins[i] tokens from o on are replaced by
//     their mean in one slot, the tokens after them follow; o == -1 copies the
//     whole sequence (golden test_reshape_and_cache_wins_rope.py:78-131, device
//     kernel op_kernel/reshape_and_cache_compress_rope.cpp:30-108: fp32 sum in
//     token order, one fp32 division by the window length, round to nearest even).
//
// Pure data movement apart from the mean: 16-byte pieces, consecutive lanes on
// consecutive pieces of a token row. Sequence starts are the prefix sums of
// seqLens, taken by every workgroup for its own sequence (the batch is small).
#include <hip/hip_runtime.h>
#include "atbmi_common.h"
#include "atbmi_kernels.h"

namespace atbmi {
namespace {

constexpr int CC_THREADS = 256;

bool Aligned(const void *p, uintptr_t a)
{
    return reinterpret_cast<uintptr_t>(p) % a == 0;
}

struct CompressArgs {
    const uint8_t *src[2]; // key, value: [tokens][heads][headSize]
    uint8_t *dst[2];       // keyCache, valueCache: [slots][headSize]
    const int32_t *slots;  // [batch * heads] first slot of the pair, < 0: skip
    const int32_t *wins;   // [batch * heads]
    const int32_t *seqLens; // [batch]
    const int32_t *offsets; // [batch * heads], mean-window only
    int32_t heads;
    int32_t rowBytes;  // headSize * element size, a multiple of 16
    int64_t numTokens; // rows of key / value
    int64_t numSlots;
};

// Tokens of the sequences before b, as every lane's return value.
__device__ __forceinline__ int64_t SequenceStart(const int32_t *seqLens, int b, int64_t *scratch)
{
    int64_t part = 0;
    for (int k = threadIdx.x; k < b; k += CC_THREADS) {
        part += seqLens[k];
    }
    for (int off = WAVE / 2; off > 0; off >>= 1) {
        part += __shfl_xor(part, off, WAVE);
    }
    if (threadIdx.x % WAVE == 0) {
        scratch[threadIdx.x / WAVE] = part;
    }
    __syncthreads();
    int64_t total = 0;
    for (int w = 0; w < CC_THREADS / WAVE; ++w) {
        total += scratch[w];
    }
    return total;
}

// Copies `count` token rows of head h, from token `srcTok` on, to slots `dstSlot` on; the workgroups
// of one pair (gridDim.y of them) share the rows. Rows outside the tensors are left out.
__device__ __forceinline__ void CopyRows(const CompressArgs &a, int which, int h, int64_t srcTok, int64_t dstSlot,
                                         int64_t count)
{
    const int pieces = a.rowBytes / 16;
    const int64_t total = count * pieces;
    for (int64_t at = static_cast<int64_t>(blockIdx.y) * CC_THREADS + threadIdx.x; at < total;
         at += static_cast<int64_t>(gridDim.y) * CC_THREADS) {
        const int64_t j = at / pieces;
        const int p = static_cast<int>(at % pieces);
        const int64_t tok = srcTok + j;
        const int64_t slot = dstSlot + j;
        if (tok < 0 || tok >= a.numTokens || slot < 0 || slot >= a.numSlots) {
            continue;
        }
        const uint4 v = *reinterpret_cast<const uint4 *>(a.src[which] + (tok * a.heads + h) * a.rowBytes + p * 16);
        *reinterpret_cast<uint4 *>(a.dst[which] + slot * a.rowBytes + p * 16) = v;
    }
}

// grid (pairs, workers per pair, key | value)
__global__ __launch_bounds__(CC_THREADS) void CompressKeepLastKernel(const CompressArgs a)
{
    __shared__ int64_t scratch[CC_THREADS / WAVE];
    const int pair = blockIdx.x;
    const int32_t slot = a.slots[pair];
    if (slot < 0) {
        return;
    }
    const int b = pair / a.heads;
    const int h = pair % a.heads;
    const int64_t end = SequenceStart(a.seqLens, b, scratch) + a.seqLens[b];
    const int64_t win = a.wins[pair];
    CopyRows(a, blockIdx.z, h, end - win, slot, win);
}

template <bool BF16>
__global__ __launch_bounds__(CC_THREADS) void CompressMeanWindowKernel(const CompressArgs a)
{
    __shared__ int64_t scratch[CC_THREADS / WAVE];
    const int pair = blockIdx.x;
    const int32_t slot = a.slots[pair];
    if (slot < 0) {
        return;
    }
    const int b = pair / a.heads;
    const int h = pair % a.heads;
    const int which = blockIdx.z;
    const int64_t start = SequenceStart(a.seqLens, b, scratch);
    const int64_t len = a.seqLens[b];
    const int64_t off = a.offsets[pair];
    const int64_t win = a.wins[pair];
    if (off < 0) {
        CopyRows(a, which, h, start, slot, len);
        return;
    }
    CopyRows(a, which, h, start, slot, min(off, len));
    if (win <= 0) {
        CopyRows(a, which, h, start + off, slot + off, len - off);
        return;
    }
    CopyRows(a, which, h, start + off + win, slot + off + 1, len - off - win);
    if (blockIdx.y != 0 || off >= len || slot + off >= a.numSlots) {
        return;
    }
    // The mean of the window: a thread owns a channel and adds its values in token order.
    const int channels = a.rowBytes / 2;
    const uint16_t *src = reinterpret_cast<const uint16_t *>(a.src[which]);
    uint16_t *dst = reinterpret_cast<uint16_t *>(a.dst[which]);
    for (int c = threadIdx.x; c < channels; c += CC_THREADS) {
        float sum = 0.0f;
        const int64_t first = start + off;
#pragma unroll 8
        for (int64_t k = 0; k < win; ++k) {
            const int64_t tok = first + k;
            if (tok < a.numTokens) {
                const uint16_t raw = src[(tok * a.heads + h) * channels + c];
                sum += BF16 ? Bf16ToFloat(raw) : HalfBitsToFloat(raw);
            }
        }
        const float mean = sum / static_cast<float>(static_cast<int32_t>(win));
        dst[(slot + off) * channels + c] = BF16 ? FloatToBf16(mean) : FloatToHalfBits(mean);
    }
}

} // namespace
} // namespace atbmi

using namespace atbmi;

extern "C" int atbmi_reshape_and_cache_compress(const void *key, const void *value, void *keyCache, void *valueCache,
                                                const int32_t *slotMapping, const int32_t *wins,
                                                const int32_t *seqLens, const int32_t *offsetIndex, int64_t batch,
                                                int64_t numHeads, int64_t headSize, int64_t numTokens,
                                                int64_t numSlots, int32_t dtype, void *stream)
{
    if (!key || !value || !keyCache || !valueCache || !slotMapping || !wins || !seqLens) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache_compress: key, value, the caches, slotMapping, wins and seqLens "
                                       "must be non-null");
    }
    if (dtype != ATBMI_F16 && dtype != ATBMI_BF16 && dtype != ATBMI_INT8) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache_compress: dtype %d", dtype);
    }
    if (offsetIndex && dtype == ATBMI_INT8) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache_compress: the mean of a window needs fp16 or bf16 rows");
    }
    if (batch < 0 || numHeads <= 0 || headSize <= 0 || numTokens < 0 || numSlots <= 0) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache_compress: bad extents");
    }
    if (headSize % 32 != 0) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache_compress: headSize %lld is not a multiple of 32",
                    (long long)headSize);
    }
    const int64_t pairs = batch * numHeads;
    if (pairs > 0x7fffffffLL || numHeads > 0x7fffffffLL || headSize > (1 << 20)) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache_compress: extents out of range");
    }
    for (const void *p : {key, value, static_cast<const void *>(keyCache), static_cast<const void *>(valueCache)}) {
        if (!Aligned(p, 16)) {
            return Fail(ERR_INVALID_PARAM, "reshape_and_cache_compress: tensors must start on 16-byte boundaries");
        }
    }
    if (pairs == 0 || numTokens == 0) {
        return OK;
    }
    CompressArgs a{};
    a.src[0] = static_cast<const uint8_t *>(key);
    a.src[1] = static_cast<const uint8_t *>(value);
    a.dst[0] = static_cast<uint8_t *>(keyCache);
    a.dst[1] = static_cast<uint8_t *>(valueCache);
    a.slots = slotMapping;
    a.wins = wins;
    a.seqLens = seqLens;
    a.offsets = offsetIndex;
    a.heads = static_cast<int32_t>(numHeads);
    a.rowBytes = static_cast<int32_t>(headSize * (dtype == ATBMI_INT8 ? 1 : 2));
    a.numTokens = numTokens;
    a.numSlots = numSlots;
    // workers per pair: enough for an average sequence at 64 rows each, the lengths themselves are on the device
    const int64_t rowsPerPair = (numTokens + batch - 1) / batch;
    int64_t workers = (rowsPerPair + 63) / 64;
    workers = workers < 1 ? 1 : (workers > 64 ? 64 : workers);
    dim3 grid(static_cast<unsigned>(pairs), static_cast<unsigned>(workers), 2);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (!offsetIndex) {
        CompressKeepLastKernel<<<grid, CC_THREADS, 0, s>>>(a);
    } else if (dtype == ATBMI_BF16) {
        CompressMeanWindowKernel<true><<<grid, CC_THREADS, 0, s>>>(a);
    } else {
        CompressMeanWindowKernel<false><<<grid, CC_THREADS, 0, s>>>(a);
    }
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}
