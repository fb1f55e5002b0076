// KV-cache block movement kernels for gfx950: BlockCopy (whole cache blocks
// copied to other blocks of the same caches) and PagedCacheLoad (the rows of
// every sequence gathered from the paged caches into contiguous tensors, the
// reverse of ReshapeAndCache).
//
// Both are plain HBM-bound byte movers: every access is a full-width vector
// access (16 bytes per lane when sizes and addresses allow it), consecutive
// lanes touch consecutive addresses, and a launch has many more workgroups
// than the chip has CUs.
#include <algorithm>
#include "atbmi_common.h"

namespace atbmi {
namespace {

constexpr int MOVE_THREADS = 256;
constexpr int PIECES_PER_THREAD = 4; // a workgroup moves 256 * 4 vectors: 16 KB with 16-byte vectors

typedef uint32_t Vec16 __attribute__((ext_vector_type(4)));
typedef uint32_t Vec8 __attribute__((ext_vector_type(2)));

// Every byte is written once: the non-temporal hint keeps the stream from displacing what the
// attention kernels want to find in the caches. (BlockCopy's loads stay ordinary: a source block with
// several destinations is then fetched from HBM once; with the hint on the loads it ran at less than
// half the rate.)
template <typename VecT> __device__ __forceinline__ void StoreOnce(VecT *p, VecT v)
{
    __builtin_nontemporal_store(v, p);
}

inline bool Aligned(const void *p, uintptr_t a)
{
    return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}

// grid.x = piece of the block, grid.y = destination index, grid.z = 0 (key cache) / 1 (value cache).
// Destination j takes the block of source i, the first i with cumSum[i] > j.
template <typename VecT>
__global__ __launch_bounds__(MOVE_THREADS) void BlockCopyKernel(uint8_t *__restrict__ keyCache,
                                                                uint8_t *__restrict__ valueCache,
                                                                const int32_t *__restrict__ srcBlocks,
                                                                const int32_t *__restrict__ dstBlocks,
                                                                const int32_t *__restrict__ cumSum, int32_t srcCount,
                                                                int64_t numBlocks, int64_t kBlockBytes,
                                                                int64_t vBlockBytes)
{
    const int j = blockIdx.y;
    int lo = 0, hi = srcCount; // first i in [0, srcCount) with cumSum[i] > j
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (cumSum[mid] > j) {
            hi = mid;
        } else {
            lo = mid + 1;
        }
    }
    if (lo >= srcCount) {
        return; // past the last source's share: nothing names this destination
    }
    const int64_t src = srcBlocks[lo];
    const int64_t dst = dstBlocks[j];
    if (src < 0 || src >= numBlocks || dst < 0 || dst >= numBlocks || src == dst) {
        return;
    }
    const bool isValue = blockIdx.z == 1;
    const int64_t blockBytes = isValue ? vBlockBytes : kBlockBytes;
    uint8_t *cache = isValue ? valueCache : keyCache;
    const VecT *from = reinterpret_cast<const VecT *>(cache + src * blockBytes);
    VecT *to = reinterpret_cast<VecT *>(cache + dst * blockBytes);
    const int64_t n = blockBytes / static_cast<int64_t>(sizeof(VecT));
    const int64_t base = static_cast<int64_t>(blockIdx.x) * (MOVE_THREADS * PIECES_PER_THREAD) + threadIdx.x;
    VecT v[PIECES_PER_THREAD];
#pragma unroll
    for (int p = 0; p < PIECES_PER_THREAD; ++p) { // all loads first
        const int64_t i = base + p * MOVE_THREADS;
        if (i < n) {
            v[p] = from[i]; // (a source with several destinations is read again: let it stay cached)
        }
    }
#pragma unroll
    for (int p = 0; p < PIECES_PER_THREAD; ++p) {
        const int64_t i = base + p * MOVE_THREADS;
        if (i < n) {
            StoreOnce(to + i, v[p]);
        }
    }
}

// grid.x = 8-token group of a sequence, grid.y = sequence, grid.z = 0 (key) / 1 (value). Small groups on
// purpose: a workgroup requests everything it moves at once and ends (16 KB with 2 KB rows, as BlockCopy);
// with 32 or 128 tokens a workgroup, several rounds of loads then stores each, the same copy ran at 64 % and
// 59 % of the HBM peak instead of 72 %.
// Token t of sequence b sits in block tables[b][seqStarts[b] / blockSize + t / blockSize] at offset
// t % blockSize and goes to output row (tokens of the sequences before b) + t. A negative block id
// leaves the output row as it is.
constexpr int LOAD_TOKENS = 8;

// Where vector `col` of cache row `r` (= block * blockSize + offset) sits, in vectors from the cache's base.
// Token-major caches: rows follow each other. Fractal-NZ caches [blocks, pieces, blockSize, piece]: the row is cut
// into pieces of perPiece vectors, and a block holds piece 0 of all its rows, then piece 1, ...
template <bool NZ>
__device__ __forceinline__ int64_t CacheVector(int64_t r, int col, int perRow, int perPiece, int blockSize)
{
    if (!NZ) {
        return r * perRow + col;
    }
    const int64_t blk = r / blockSize;
    const int64_t off = r - blk * blockSize;
    const int piece = col / perPiece;
    return ((blk * (perRow / perPiece) + piece) * blockSize + off) * perPiece + (col - piece * perPiece);
}

template <typename VecT, bool NZ>
__global__ __launch_bounds__(MOVE_THREADS) void PagedCacheLoadKernel(
    const uint8_t *__restrict__ keyCache, const uint8_t *__restrict__ valueCache,
    const int32_t *__restrict__ tables, const int32_t *__restrict__ lens, const int32_t *__restrict__ seqStarts,
    uint8_t *__restrict__ key, uint8_t *__restrict__ value, int32_t maxBlocksPerSeq, int32_t blockSize,
    int64_t numBlocks, int64_t kRowBytes, int64_t vRowBytes, int64_t outRows, int32_t cumsumMode,
    int32_t kPieceBytes, int32_t vPieceBytes)
{
    const int b = blockIdx.y;
    const int t0 = blockIdx.x * LOAD_TOKENS;
    // Everything the workgroup has to look up is requested at once: the lengths before this sequence
    // (their sum is its first output row), its own length and the block ids of this group's tokens; one
    // memory round trip instead of three in a row, which is most of what a group of this size costs.
    __shared__ int64_t total;
    __shared__ int64_t srcRow[LOAD_TOKENS]; // cache row of each of the group's tokens (-1: leave the output row alone)
    const int firstBlock = seqStarts ? seqStarts[b] / blockSize : 0;
    int64_t before = 0; // this lane's share of the lengths before sequence b
    int32_t len;
    if (cumsumMode) {
        before = lens[b];
        len = lens[b + 1] - static_cast<int32_t>(before);
    } else {
        if (threadIdx.x < WAVE) {
            for (int i = threadIdx.x; i < b; i += WAVE) {
                before += lens[i];
            }
        }
        len = lens[b];
    }
    int64_t blk = -1;
    if (threadIdx.x < LOAD_TOKENS) {
        const int tableIdx = firstBlock + (t0 + static_cast<int>(threadIdx.x)) / blockSize;
        if (tableIdx < maxBlocksPerSeq) {
            blk = tables[static_cast<int64_t>(b) * maxBlocksPerSeq + tableIdx];
        }
    }
    if (t0 >= len) {
        return;
    }
    if (!cumsumMode && threadIdx.x < WAVE) {
        for (int off = 32; off > 0; off >>= 1) {
            before += __shfl_xor(before, off, WAVE);
        }
    }
    const int64_t begin = cumsumMode ? before : __shfl(before, 0, WAVE); // (valid in the first wave; the others read `total`)
    if (threadIdx.x == 0) {
        total = begin;
    }
    const int tokens = min(LOAD_TOKENS, len - t0);
    if (threadIdx.x < LOAD_TOKENS) {
        const int t = t0 + threadIdx.x;
        int64_t r = -1;
        if (static_cast<int>(threadIdx.x) < tokens && blk >= 0 && blk < numBlocks && begin + t < outRows) {
            r = blk * blockSize + t % blockSize;
        }
        srcRow[threadIdx.x] = r;
    }
    __syncthreads();
    const int64_t firstRow = total;
    const bool isValue = blockIdx.z == 1;
    const int64_t rowBytes = isValue ? vRowBytes : kRowBytes;
    const uint8_t *cache = isValue ? valueCache : keyCache;
    uint8_t *out = isValue ? value : key;
    const int perRow = static_cast<int>(rowBytes / static_cast<int64_t>(sizeof(VecT)));
    const int perPiece = NZ ? (isValue ? vPieceBytes : kPieceBytes) / static_cast<int>(sizeof(VecT)) : perRow;
    const VecT *from = reinterpret_cast<const VecT *>(cache);
    VecT *to = reinterpret_cast<VecT *>(out + (firstRow + t0) * rowBytes);
    // A thread keeps its column and walks down the rows: the division that finds (row, column) is done once,
    // not per vector moved. Short rows: several rows per pass of the workgroup; long rows: several passes a row.
    constexpr int BATCH = 4;
    if (perRow <= MOVE_THREADS) {
        const int rowsPerPass = MOVE_THREADS / perRow;
        const int col = threadIdx.x % perRow;
        const int row0 = threadIdx.x / perRow;
        if (row0 >= rowsPerPass) {
            return; // (threads past the last whole row of a pass)
        }
        for (int tok0 = row0; tok0 < tokens; tok0 += rowsPerPass * BATCH) {
            VecT v[BATCH];
            bool live[BATCH];
#pragma unroll
            for (int k = 0; k < BATCH; ++k) { // all loads first
                const int tok = tok0 + k * rowsPerPass;
                live[k] = false;
                if (tok < tokens) {
                    const int64_t r = srcRow[tok];
                    if (r >= 0) {
                        live[k] = true;
                        // (token-major rows are read once, in whole cache lines: the non-temporal hint is worth 3 %;
                        // on the 32-byte pieces of the fractal layout it costs 40 %)
                        const VecT *at = from + CacheVector<NZ>(r, col, perRow, perPiece, blockSize);
                        v[k] = NZ ? *at : __builtin_nontemporal_load(at);
                    }
                }
            }
#pragma unroll
            for (int k = 0; k < BATCH; ++k) {
                if (live[k]) {
                    StoreOnce(to + static_cast<int64_t>(tok0 + k * rowsPerPass) * perRow + col, v[k]);
                }
            }
        }
        return;
    }
    for (int tok = 0; tok < tokens; ++tok) {
        const int64_t r = srcRow[tok];
        if (r < 0) {
            continue;
        }
        VecT *dst = to + static_cast<int64_t>(tok) * perRow;
        for (int c0 = threadIdx.x; c0 < perRow; c0 += MOVE_THREADS * BATCH) {
            VecT v[BATCH];
#pragma unroll
            for (int k = 0; k < BATCH; ++k) {
                const int c = c0 + k * MOVE_THREADS;
                if (c < perRow) {
                    v[k] = from[CacheVector<NZ>(r, c, perRow, perPiece, blockSize)];
                }
            }
#pragma unroll
            for (int k = 0; k < BATCH; ++k) {
                const int c = c0 + k * MOVE_THREADS;
                if (c < perRow) {
                    StoreOnce(dst + c, v[k]);
                }
            }
        }
    }
}

// Widest power-of-two vector (<= 16 bytes) that divides both sizes and that every pointer is aligned to.
template <typename... Ptrs> uintptr_t CommonAlign(int64_t a, int64_t b, Ptrs... ptrs)
{
    uintptr_t align = 16;
    const void *all[] = {ptrs...};
    for (;;) {
        bool ok = a % static_cast<int64_t>(align) == 0 && b % static_cast<int64_t>(align) == 0;
        for (const void *p : all) {
            ok = ok && (p == nullptr || Aligned(p, align));
        }
        if (ok || align == 1) {
            return align;
        }
        align >>= 1;
    }
}

} // namespace

extern "C" int atbmi_block_copy(void *keyCache, void *valueCache, const int32_t *srcBlocks, const int32_t *dstBlocks,
                                const int32_t *cumSum, int64_t srcCount, int64_t dstCount, int64_t numBlocks,
                                int64_t keyBlockBytes, int64_t valueBlockBytes, void *stream)
{
    if (!keyCache || !srcBlocks || !dstBlocks || !cumSum) {
        return Fail(ERR_INVALID_PARAM, "block_copy: keyCache, srcBlocks, dstBlocks and cumSum must be non-null");
    }
    if (srcCount < 0 || dstCount < 0 || numBlocks <= 0 || keyBlockBytes <= 0 || (valueCache && valueBlockBytes <= 0)) {
        return Fail(ERR_INVALID_PARAM, "block_copy: bad extents");
    }
    if (srcCount == 0 || dstCount == 0) {
        return OK;
    }
    if (srcCount > 0x7fffffffLL || dstCount > 65535) {
        return Fail(ERR_INVALID_PARAM, "block_copy: %lld sources / %lld destinations are more than one launch takes",
                    (long long)srcCount, (long long)dstCount);
    }
    const int64_t vBytes = valueCache ? valueBlockBytes : keyBlockBytes;
    const uintptr_t align = CommonAlign(keyBlockBytes, vBytes, keyCache, valueCache);
    const int64_t maxBytes = std::max(keyBlockBytes, vBytes);
    const int64_t perWg = static_cast<int64_t>(MOVE_THREADS) * PIECES_PER_THREAD * static_cast<int64_t>(align);
    const int64_t pieces = (maxBytes + perWg - 1) / perWg;
    if (pieces > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "block_copy: blocks of %lld bytes are too large", (long long)maxBytes);
    }
    dim3 grid(static_cast<unsigned>(pieces), static_cast<unsigned>(dstCount), valueCache ? 2 : 1);
    hipStream_t s = static_cast<hipStream_t>(stream);
    uint8_t *k8 = static_cast<uint8_t *>(keyCache);
    uint8_t *v8 = static_cast<uint8_t *>(valueCache);
    const int32_t n = static_cast<int32_t>(srcCount);
#define ATBMI_LAUNCH_BLOCK_COPY(T) \
    BlockCopyKernel<T><<<grid, MOVE_THREADS, 0, s>>>(k8, v8, srcBlocks, dstBlocks, cumSum, n, numBlocks, keyBlockBytes, vBytes)
    switch (align) {
        case 16: ATBMI_LAUNCH_BLOCK_COPY(Vec16); break;
        case 8: ATBMI_LAUNCH_BLOCK_COPY(Vec8); break;
        case 4: ATBMI_LAUNCH_BLOCK_COPY(uint32_t); break;
        case 2: ATBMI_LAUNCH_BLOCK_COPY(uint16_t); break;
        default: ATBMI_LAUNCH_BLOCK_COPY(uint8_t); break;
    }
#undef ATBMI_LAUNCH_BLOCK_COPY
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}

// Shared by the token-major and the fractal-NZ entry points: piece sizes of 0 mean token-major caches.
static int LaunchPagedCacheLoad(const char *who, const void *keyCache, const void *valueCache,
                                const int32_t *blockTables, const int32_t *seqLens, const int32_t *seqStarts,
                                void *key, void *value, int64_t batch, int64_t maxBlocksPerSeq, int64_t blockSize,
                                int64_t numBlocks, int64_t keyRowBytes, int64_t valueRowBytes, int64_t keyPieceBytes,
                                int64_t valuePieceBytes, int64_t outRows, int64_t maxSeqLen, int32_t cumsumMode,
                                void *stream)
{
    if (!keyCache || !valueCache || !blockTables || !seqLens || !key || !value) {
        return Fail(ERR_INVALID_PARAM, "%s: caches, blockTables, seqLens, key and value must be non-null", who);
    }
    if (batch < 0 || maxBlocksPerSeq <= 0 || blockSize <= 0 || numBlocks <= 0 || keyRowBytes <= 0 ||
        valueRowBytes <= 0 || outRows < 0 || maxSeqLen < 0) {
        return Fail(ERR_INVALID_PARAM, "%s: bad extents", who);
    }
    const bool nz = keyPieceBytes > 0;
    if (nz && (valuePieceBytes <= 0 || keyRowBytes % keyPieceBytes != 0 || valueRowBytes % valuePieceBytes != 0)) {
        return Fail(ERR_INVALID_PARAM, "%s: rows of %lld / %lld bytes are not whole pieces of %lld / %lld bytes", who,
                    (long long)keyRowBytes, (long long)valueRowBytes, (long long)keyPieceBytes,
                    (long long)valuePieceBytes);
    }
    if (batch == 0 || outRows == 0 || maxSeqLen == 0) {
        return OK;
    }
    const int64_t groups = (maxSeqLen + LOAD_TOKENS - 1) / LOAD_TOKENS;
    if (batch > 65535 || groups > 0x7fffffffLL || maxBlocksPerSeq > 0x7fffffffLL || blockSize > 0x7fffffffLL ||
        keyRowBytes > (1 << 24) || valueRowBytes > (1 << 24)) {
        return Fail(ERR_INVALID_PARAM, "%s: %lld sequences of up to %lld tokens are more than one launch takes", who,
                    (long long)batch, (long long)maxSeqLen);
    }
    // a vector never straddles two pieces
    const uintptr_t align = nz ? CommonAlign(keyPieceBytes, valuePieceBytes, keyCache, valueCache, key, value)
                               : CommonAlign(keyRowBytes, valueRowBytes, keyCache, valueCache, key, value);
    dim3 grid(static_cast<unsigned>(groups), static_cast<unsigned>(batch), 2);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint8_t *kc8 = static_cast<const uint8_t *>(keyCache);
    const uint8_t *vc8 = static_cast<const uint8_t *>(valueCache);
    uint8_t *k8 = static_cast<uint8_t *>(key);
    uint8_t *v8 = static_cast<uint8_t *>(value);
#define ATBMI_LAUNCH_CACHE_LOAD_AS(T, NZ)                                                                         \
    PagedCacheLoadKernel<T, NZ><<<grid, MOVE_THREADS, 0, s>>>(                                                    \
        kc8, vc8, blockTables, seqLens, seqStarts, k8, v8, static_cast<int32_t>(maxBlocksPerSeq),                 \
        static_cast<int32_t>(blockSize), numBlocks, keyRowBytes, valueRowBytes, outRows, cumsumMode,              \
        static_cast<int32_t>(keyPieceBytes), static_cast<int32_t>(valuePieceBytes))
#define ATBMI_LAUNCH_CACHE_LOAD(T)              \
    if (nz) {                                   \
        ATBMI_LAUNCH_CACHE_LOAD_AS(T, true);    \
    } else {                                    \
        ATBMI_LAUNCH_CACHE_LOAD_AS(T, false);   \
    }
    switch (align) {
        case 16: ATBMI_LAUNCH_CACHE_LOAD(Vec16); break;
        case 8: ATBMI_LAUNCH_CACHE_LOAD(Vec8); break;
        case 4: ATBMI_LAUNCH_CACHE_LOAD(uint32_t); break;
        case 2: ATBMI_LAUNCH_CACHE_LOAD(uint16_t); break;
        default: ATBMI_LAUNCH_CACHE_LOAD(uint8_t); break;
    }
#undef ATBMI_LAUNCH_CACHE_LOAD
#undef ATBMI_LAUNCH_CACHE_LOAD_AS
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}

extern "C" int atbmi_paged_cache_load(const void *keyCache, const void *valueCache, const int32_t *blockTables,
                                      const int32_t *seqLens, const int32_t *seqStarts, void *key, void *value,
                                      int64_t batch, int64_t maxBlocksPerSeq, int64_t blockSize, int64_t numBlocks,
                                      int64_t keyRowBytes, int64_t valueRowBytes, int64_t outRows,
                                      int64_t maxSeqLen, int32_t cumsumMode, void *stream)
{
    return LaunchPagedCacheLoad("paged_cache_load", keyCache, valueCache, blockTables, seqLens, seqStarts, key, value,
                                batch, maxBlocksPerSeq, blockSize, numBlocks, keyRowBytes, valueRowBytes, 0, 0, outRows,
                                maxSeqLen, cumsumMode, stream);
}

extern "C" int atbmi_paged_cache_load_nz(const void *keyCache, const void *valueCache, const int32_t *blockTables,
                                         const int32_t *seqLens, void *key, void *value, int64_t batch,
                                         int64_t maxBlocksPerSeq, int64_t blockSize, int64_t numBlocks,
                                         int64_t keyRowBytes, int64_t valueRowBytes, int64_t keyPieceBytes,
                                         int64_t valuePieceBytes, int64_t outRows, int64_t maxSeqLen, void *stream)
{
    if (keyPieceBytes <= 0 || valuePieceBytes <= 0) {
        return Fail(ERR_INVALID_PARAM, "paged_cache_load_nz: piece sizes must be positive");
    }
    return LaunchPagedCacheLoad("paged_cache_load_nz", keyCache, valueCache, blockTables, seqLens, nullptr, key, value,
                                batch, maxBlocksPerSeq, blockSize, numBlocks, keyRowBytes, valueRowBytes, keyPieceBytes,
                                valuePieceBytes, outRows, maxSeqLen, 0, stream);
}

} // namespace atbmi
