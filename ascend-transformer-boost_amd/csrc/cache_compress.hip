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
//   drop-window (ReshapeAndCacheOmniOperation): as mean-window, but the window leaves nothing behind: the tokens
//     before o, then at once the tokens from o + wins[i] on (golden
//     tests/framework/python/CsvOpsTestTool/data_generation.py:9797-9846 and
//     tests/apitest/kernelstest/mix/test_reshape_and_cache_omni_compress.py:80-116, device kernel
//     op_kernel/reshape_and_cache_omni_compress.cpp:87-110 with reshape_and_cache_base.h:276-289).
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
constexpr int MEAN_STAGE_BYTES = 32768; // token rows of a window staged in LDS at a time
constexpr int MEAN_MAX_CHANNELS = 1024; // head size the window mean is built for

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
    const int32_t *offsets; // [batch * heads], first token of the window (mean-window, drop-window)
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

// Copies `count` token rows of head h, from token `srcTok` on, to slots `dstSlot` on; `workers`
// workgroups of the pair share the rows, this one is number `worker`. Rows outside the tensors are left out.
__device__ __forceinline__ void CopyRows(const CompressArgs &a, int which, int h, int64_t srcTok, int64_t dstSlot,
                                         int64_t count, int worker, int workers)
{
    const int pieces = a.rowBytes / 16;
    const int64_t total = count * pieces;
    for (int64_t at = static_cast<int64_t>(worker) * CC_THREADS + threadIdx.x; at < total;
         at += static_cast<int64_t>(workers) * CC_THREADS) {
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
    CopyRows(a, blockIdx.z, h, end - win, slot, win, blockIdx.y, gridDim.y);
}

// The window [off, off + win) of the sequence is left out, the tokens after it close up.
__global__ __launch_bounds__(CC_THREADS) void CompressDropWindowKernel(const CompressArgs a)
{
    __shared__ int64_t scratch[CC_THREADS / WAVE];
    const int pair = blockIdx.x;
    const int32_t slot = a.slots[pair];
    if (slot < 0) {
        return;
    }
    const int b = pair / a.heads;
    const int h = pair % a.heads;
    const int64_t start = SequenceStart(a.seqLens, b, scratch);
    const int64_t len = a.seqLens[b];
    const int64_t off = a.offsets[pair];
    const int64_t win = a.wins[pair];
    if (off < 0 || win <= 0 || off >= len) { // no window: the whole sequence as it is
        CopyRows(a, blockIdx.z, h, start, slot, len, blockIdx.y, gridDim.y);
        return;
    }
    // one run of rows for the workers to share: row j comes from token j, or from j + win once past the window
    const int64_t after = len - off - win > 0 ? len - off - win : 0;
    const int pieces = a.rowBytes / 16;
    const int64_t total = (off + after) * pieces;
    const int which = blockIdx.z;
    for (int64_t at = static_cast<int64_t>(blockIdx.y) * CC_THREADS + threadIdx.x; at < total;
         at += static_cast<int64_t>(gridDim.y) * CC_THREADS) {
        const int64_t j = at / pieces;
        const int p = static_cast<int>(at % pieces);
        const int64_t tok = start + (j < off ? j : j + win);
        const int64_t dst = slot + j;
        if (tok < 0 || tok >= a.numTokens || dst >= a.numSlots) {
            continue;
        }
        const uint4 v = *reinterpret_cast<const uint4 *>(a.src[which] + (tok * a.heads + h) * a.rowBytes + p * 16);
        *reinterpret_cast<uint4 *>(a.dst[which] + dst * a.rowBytes + p * 16) = v;
    }
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
    if (off < 0 || win <= 0 || off >= len) { // no window: the whole sequence as it is
        CopyRows(a, which, h, start, slot, len, blockIdx.y, gridDim.y);
        return;
    }
    // The first workgroup of the pair takes the mean (the long pole: it starts at once), the others copy.
    const bool solo = gridDim.y == 1;
    if (blockIdx.y != 0 || solo) {
        const int worker = solo ? 0 : blockIdx.y - 1;
        const int workers = solo ? 1 : gridDim.y - 1;
        CopyRows(a, which, h, start, slot, off, worker, workers);
        CopyRows(a, which, h, start + off + win, slot + off + 1, len - off - win, worker, workers);
    }
    if (blockIdx.y != 0 || slot + off >= a.numSlots) {
        return;
    }
    // The mean of the window. The order of the fp32 additions is fixed (token order), so the work of a
    // channel cannot be split: the workgroup stages a run of token rows in LDS with all its lanes (16-byte
    // pieces, many loads in flight), then every thread adds up its channels from there.
    __shared__ __align__(16) uint8_t stage[MEAN_STAGE_BYTES];
    const int channels = a.rowBytes / 2;
    const int pieces = a.rowBytes / 16;
    const int chunkTokens = MEAN_STAGE_BYTES / a.rowBytes;
    const int64_t first = start + off;
    const int64_t inRange = a.numTokens - first < win ? a.numTokens - first : win;
    const uint8_t *src = a.src[which];
    const uint16_t *staged = reinterpret_cast<const uint16_t *>(stage);
    float sum[MEAN_MAX_CHANNELS / CC_THREADS];
#pragma unroll
    for (int i = 0; i < MEAN_MAX_CHANNELS / CC_THREADS; ++i) {
        sum[i] = 0.0f;
    }
    // The rows of the next run travel while this one is added up: a run's loads are asked for one run ahead and
    // wait in registers (one workgroup has nothing else to hide their latency behind).
    constexpr int HELD = MEAN_STAGE_BYTES / 16 / CC_THREADS; // 16-byte pieces per thread and run
    auto countOf = [&](int64_t k0) {
        return static_cast<int>(inRange - k0 < chunkTokens ? inRange - k0 : chunkTokens);
    };
#define ATBMI_REQUEST_RUN(k0_, count_)                                                                        \
    _Pragma("unroll") for (int u = 0; u < HELD; ++u)                                                          \
    { /* lanes past the run's end repeat its last piece */                                                    \
        const int last = (count_) * pieces - 1;                                                               \
        const int at = threadIdx.x + u * CC_THREADS < last ? threadIdx.x + u * CC_THREADS : last;             \
        held[u] = *reinterpret_cast<const Piece *>(src + ((first + (k0_) + at / pieces) * a.heads + h) * a.rowBytes + \
                                                   (at % pieces) * 16);                                       \
    }
    // (a plain vector type: arrays of the runtime's uint4 structure that live across loop iterations stay in memory)
    typedef unsigned int Piece __attribute__((ext_vector_type(4)));
    Piece held[HELD];
    if (inRange > 0) {
        ATBMI_REQUEST_RUN(0, countOf(0))
    }
    for (int64_t k0 = 0; k0 < inRange; k0 += chunkTokens) {
        const int count = countOf(k0);
        __syncthreads(); // the previous run has been added up
#pragma unroll
        for (int u = 0; u < HELD; ++u) {
            const int at = threadIdx.x + u * CC_THREADS;
            if (at < count * pieces) {
                *reinterpret_cast<Piece *>(stage + static_cast<size_t>(at) * 16) = held[u];
            }
        }
        if (k0 + chunkTokens < inRange) {
            ATBMI_REQUEST_RUN(k0 + chunkTokens, countOf(k0 + chunkTokens))
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < MEAN_MAX_CHANNELS / CC_THREADS; ++i) {
            const int c = threadIdx.x + i * CC_THREADS;
            if (c < channels) {
                float acc = sum[i];
                int j = 0;
                for (; j + 16 <= count; j += 16) { // sixteen LDS reads in flight, then the additions in order
                    uint16_t raw[16];
#pragma unroll
                    for (int u = 0; u < 16; ++u) {
                        raw[u] = staged[(j + u) * channels + c];
                    }
#pragma unroll
                    for (int u = 0; u < 16; ++u) {
                        acc += BF16 ? Bf16ToFloat(raw[u]) : HalfBitsToFloat(raw[u]);
                    }
                }
                for (; j < count; ++j) {
                    const uint16_t raw = staged[j * channels + c];
                    acc += BF16 ? Bf16ToFloat(raw) : HalfBitsToFloat(raw);
                }
                sum[i] = acc;
            }
        }
    }
#undef ATBMI_REQUEST_RUN
    uint16_t *dst = reinterpret_cast<uint16_t *>(a.dst[which]);
#pragma unroll
    for (int i = 0; i < MEAN_MAX_CHANNELS / CC_THREADS; ++i) {
        const int c = threadIdx.x + i * CC_THREADS;
        if (c < channels) {
            const float mean = sum[i] / static_cast<float>(static_cast<int32_t>(win));
            dst[(slot + off) * channels + c] = BF16 ? FloatToBf16(mean) : FloatToHalfBits(mean);
        }
    }
}

} // namespace
} // namespace atbmi

using namespace atbmi;

namespace {
enum CompressMode { KEEP_LAST, MEAN_WINDOW, DROP_WINDOW };

int CompressImpl(const char *name, CompressMode mode, const void *key, const void *value, void *keyCache,
                 void *valueCache, const int32_t *slotMapping, const int32_t *wins, const int32_t *seqLens,
                 const int32_t *offsetIndex, int64_t batch, int64_t numHeads, int64_t headSize, int64_t numTokens,
                 int64_t numSlots, int32_t dtype, void *stream)
{
    if (!key || !value || !keyCache || !valueCache || !slotMapping || !wins || !seqLens) {
        return Fail(ERR_INVALID_PARAM, "%s: key, value, the caches, slotMapping, wins and seqLens must be non-null", name);
    }
    if (mode == DROP_WINDOW && !offsetIndex) {
        return Fail(ERR_INVALID_PARAM, "%s: offsetIndex must be non-null", name);
    }
    if (dtype != ATBMI_F16 && dtype != ATBMI_BF16 && dtype != ATBMI_INT8) {
        return Fail(ERR_INVALID_PARAM, "%s: dtype %d", name, dtype);
    }
    if (mode == MEAN_WINDOW && dtype == ATBMI_INT8) {
        return Fail(ERR_INVALID_PARAM, "%s: the mean of a window needs fp16 or bf16 rows", name);
    }
    if (batch < 0 || numHeads <= 0 || headSize <= 0 || numTokens < 0 || numSlots <= 0) {
        return Fail(ERR_INVALID_PARAM, "%s: bad extents", name);
    }
    if (mode == MEAN_WINDOW && headSize > MEAN_MAX_CHANNELS) {
        return Fail(ERR_INVALID_PARAM, "%s: the window mean is built for head sizes up to %d, got %lld", name,
                    MEAN_MAX_CHANNELS, (long long)headSize);
    }
    if (headSize % 32 != 0) {
        return Fail(ERR_INVALID_PARAM, "%s: headSize %lld is not a multiple of 32", name, (long long)headSize);
    }
    const int64_t pairs = batch * numHeads;
    if (pairs > 0x7fffffffLL || numHeads > 0x7fffffffLL || headSize > (1 << 20)) {
        return Fail(ERR_INVALID_PARAM, "%s: extents out of range", name);
    }
    for (const void *p : {key, value, static_cast<const void *>(keyCache), static_cast<const void *>(valueCache)}) {
        if (!Aligned(p, 16)) {
            return Fail(ERR_INVALID_PARAM, "%s: tensors must start on 16-byte boundaries", name);
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
    workers += mode == MEAN_WINDOW ? 1 : 0; // the one that takes the window's mean
    dim3 grid(static_cast<unsigned>(pairs), static_cast<unsigned>(workers), 2);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (mode == KEEP_LAST) {
        CompressKeepLastKernel<<<grid, CC_THREADS, 0, s>>>(a);
    } else if (mode == DROP_WINDOW) {
        CompressDropWindowKernel<<<grid, CC_THREADS, 0, s>>>(a);
    } else if (dtype == ATBMI_BF16) {
        CompressMeanWindowKernel<true><<<grid, CC_THREADS, 0, s>>>(a);
    } else {
        CompressMeanWindowKernel<false><<<grid, CC_THREADS, 0, s>>>(a);
    }
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}
} // namespace

extern "C" int atbmi_reshape_and_cache_compress(const void *key, const void *value, void *keyCache, void *valueCache,
                                                const int32_t *slotMapping, const int32_t *wins,
                                                const int32_t *seqLens, const int32_t *offsetIndex, int64_t batch,
                                                int64_t numHeads, int64_t headSize, int64_t numTokens,
                                                int64_t numSlots, int32_t dtype, void *stream)
{
    return CompressImpl("reshape_and_cache_compress", offsetIndex ? MEAN_WINDOW : KEEP_LAST, key, value, keyCache,
                        valueCache, slotMapping, wins, seqLens, offsetIndex, batch, numHeads, headSize, numTokens,
                        numSlots, dtype, stream);
}

extern "C" int atbmi_reshape_and_cache_omni(const void *key, const void *value, void *keyCache, void *valueCache,
                                            const int32_t *slotMapping, const int32_t *wins, const int32_t *seqLens,
                                            const int32_t *offsetIndex, int64_t batch, int64_t numHeads,
                                            int64_t headSize, int64_t numTokens, int64_t numSlots, int32_t dtype,
                                            void *stream)
{
    return CompressImpl("reshape_and_cache_omni", DROP_WINDOW, key, value, keyCache, valueCache, slotMapping, wins,
                        seqLens, offsetIndex, batch, numHeads, headSize, numTokens, numSlots, dtype, stream);
}
