// Shared host/device helpers of the MI355X kernel layer.
#ifndef ATBMI_COMMON_H
#define ATBMI_COMMON_H
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include "atbmi_kernels.h"

namespace atbmi {

// Return codes are atb::ErrorType values.
constexpr int OK = 0;
constexpr int ERR_INVALID_PARAM = 1;
constexpr int ERR_RT_FAIL = 4;
constexpr int ERR_OUT_OF_DEVICE_MEMORY = 26;
constexpr int ERR_OUT_OF_HOST_MEMORY = 27;

constexpr int WAVE = 64;

// Records the message atbmi_last_error() hands back and returns `code`.
int Fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

// Compute units of the current device (256 when no device can be asked: plans are also made on hosts without a GPU).
int DeviceComputeUnits();

#define ATBMI_HIP_CHECK(expr)                                                                       \
    do {                                                                                            \
        hipError_t e_ = (expr);                                                                     \
        if (e_ != hipSuccess) {                                                                     \
            return ::atbmi::Fail(::atbmi::ERR_RT_FAIL, "%s failed: %s", #expr, hipGetErrorString(e_)); \
        }                                                                                           \
    } while (0)

// One physical work item of the split-K plan: the token range
// [tokBegin, tokEnd) of one sequence, handled by one workgroup per KV head.
struct PaWorkItem {
    int32_t qRow;        // row of q / out
    int32_t seq;         // row of blockTables (and of logN)
    int32_t tokBegin;
    int32_t tokEnd;
    int32_t partialBase; // first partial slot this item writes
    int32_t direct;      // 1: the only chunk of its sequence, write `out` directly
    int32_t maskRow;     // row of the mask (in units of maskBatchStride) this query row uses
    int32_t pad1;
};

// Per non-empty sequence: where its partials live, for the merge kernel.
struct PaSeqInfo {
    int32_t qRow;
    int32_t firstPartial;
    int32_t numPartials;
    int32_t ctxLen;
};

// Kernel arguments shared by the attention kernels and the merge kernel.
struct PaArgs {
    const void *q;
    const void *kc;
    const void *vc;
    const int32_t *tables;
    const float *kScale;
    const int32_t *kOff;
    const float *vScale;
    const int32_t *vOff;
    void *out;
    const PaWorkItem *items;
    const PaSeqInfo *seqs;
    float *partO;   // [numPartials][H][Dv] normalised partial outputs: fp32 for the scalar kernel's chunks; the stream
                    // plans of the MFMA kernels keep 16-bit values of the query's type there (half the bytes a wave
                    // writes at a row boundary, for rows that end in a 16-bit output anyway)
    float *partLse; // [numPartials][H] log2-domain log-sum-exp
    int32_t H, G, D, Dv;
    int32_t blockSize, maxBlocksPerSeq;
    int32_t qIsBf16;
    int32_t groupSize; // H / G
    float qkScale;
    float qScale; // 0 when unused
    // Element (slot r, head g, channel c) of a cache sits at r * rowStride + g * headStride + c, where the
    // slot of token `off` of block `blk` is blk * blockRows + off. Token-major blocks [blockSize][G][D]:
    // rowStride G*D, headStride D, blockRows blockSize. Head-major blocks [G][blockSize][D]: rowStride D,
    // headStride blockSize*D, blockRows G*blockSize.
    int64_t kRowStride; // key cache
    int64_t vRowStride; // value cache (the key cache's when V aliases K)
    int32_t vHeadStride; // value cache (D - ropeDim when V aliases K)
    int32_t finishV;     // 1: partial outputs are still in int8 units; the final write applies vScale (int8 caches
                         // without offsets and without head compression; otherwise the attention kernel descales them)
    // Additive score bias (null: none), in the query's type: the score of the sequence in batch row b,
    // head h, token t gets mask[b * maskBatchStride + h * maskHeadStride + t] added after scaling.
    const void *mask;
    int64_t maskBatchStride;
    int64_t maskHeadStride;
    int32_t maskLen;     // tokens per mask row
    int32_t maskVec;     // 1: every mask row starts on an 8-byte boundary (4-token vector loads are legal)
    const float *logN;   // per batch row factor on qkScale (null: none)
    int32_t scaleStride; // floats between consecutive kScale / vScale entries: 1, or 2 for uint64-packed ones
    int32_t maskRowStep; // mask rows between consecutive query tokens of one sequence (0: they share a row)
    // Split latent layout (null / 0: none): the last ropeDim of the D channels of every query row live in
    // qRope [rows][H][ropeDim] and those of every key row in kRope [slots][G][ropeDim]; q and kc then
    // hold rows of D - ropeDim channels.
    const void *qRope;
    const void *kRope;
    int64_t ropeRowStride; // elements between consecutive tokens in kRope (G * ropeDim)
    int32_t ropeDim;
    int32_t blockRows;   // cache slots per block (see kRowStride)
    int32_t kHeadStride; // elements between the KV heads of one key-cache slot (see kRowStride)
    int32_t descaleHeads; // > 0: sequence b takes slice b % descaleHeads of the descale vectors instead of its KV head's
    const float *razor;   // [slots] added to q.k before the score scale (null: none)
    void *lse;           // [rows][H] in the query's type: natural-log log-sum-exp of the scaled scores (null: none)
    int32_t nzShift;     // > 0: fractal-NZ caches of the split latent layout, log2 of the block size; channel c of
                         // the token at offset t of block b sits at ((b * (dn / 16) + c / 16) << nzShift) * 16 + t * 16 +
                         // c % 16 (dn channels per row of that cache)
};

// ---- Plan of the MFMA kernel ------------------------------------------------
// The KV rows of all non-empty sequences, cut into 32-token steps, form one
// linear step space [0, totalSteps). It is divided evenly into numWaveRanges
// contiguous ranges; one wave walks one range for one KV head (or one tile of
// 16 query heads of it), crossing sequence boundaries where they fall. The
// device only needs where each sequence starts in that space. A sequence with
// several query tokens appears once per token, each with the whole context.
constexpr int PA_INLINE_SEQS = 160;   // plans up to this many query rows travel in the kernel arguments
constexpr int PA_INLINE_RANGES = 512; // workgroup ranges whose first sequence is tabulated inline

// One pass over a sequence's context: for its single decode token, or for up to
// PaStreamPlan::foldTokens of its consecutive query tokens (speculative /
// multi-token decoding), which share the pass as extra columns of the head tile.
// A sequence with more query tokens than that appears once per such group.
struct PaSeq {
    int32_t tableRow;  // row of blockTables and of logN (index of the sequence in the batch)
    int32_t ctxLen;    // tokens
    int32_t stepBegin; // first step of this pass in the linear step space
    int32_t maskRow;   // row of the mask (in units of maskBatchStride) of its first query token
    int32_t qRow;      // row of q / out of its first query token
    int32_t nTok;      // query tokens in this pass
};

struct PaStreamPlan {
    const PaSeq *seqs;        // numSeqs + 1 entries (the last one only carries stepBegin = totalSteps);
                              // null: use inlineSeqs
    const uint16_t *firstSeq; // per workgroup range: sequence holding its first step; null: use inlineFirst
    int32_t numSeqs;          // passes (PaSeq entries)
    int32_t totalSteps;
    int32_t numWaveRanges;    // at most numWgRanges * tokenSlices and at most totalSteps: no range is empty
    int32_t numWgRanges;
    int32_t tokenSlices;      // consecutive wave ranges one workgroup covers (waves / headsPerWg)
    int32_t headsPerWg;       // virtual heads (KV head x query-head tile) one workgroup covers
    int32_t headGroups;       // virtual heads / headsPerWg
    int32_t headTiles;        // query-head tiles per KV head
    int32_t foldTokens;       // query tokens of one sequence that may share a head tile (1: none do);
                              // a partial slot then holds foldTokens x H rows
    int32_t maxRangesPerRow;  // most wave ranges any one pass spans (the merge kernel sizes itself by it)
    int32_t rowStartSteps;    // steps at the head of every pass that stand for no tokens: what starting a row costs a
                              // wave (its query, the block table, a cold first tile, the partial row it leaves), so
                              // that equal ranges are equal work. Step s of a pass holds the tokens of its step
                              // s - rowStartSteps; a range that only has such steps of a pass leaves an empty partial row.
    PaSeq inlineSeqs[PA_INLINE_SEQS + 1];
    uint16_t inlineFirst[PA_INLINE_RANGES];
};

// First step of wave range `wr`: ranges differ by at most one step. (The products fit 32 bits for all but
// enormous plans, and a 32-bit division is a fraction of the instructions of a 64-bit one on the GPU; both
// forms give the same quotient.)
__host__ __device__ __forceinline__ int32_t PaRangeBegin(int32_t wr, int32_t totalSteps, int32_t numWaveRanges)
{
    const int64_t product = static_cast<int64_t>(wr) * totalSteps;
    if (product < 0x7fffffffLL) {
        return static_cast<int32_t>(static_cast<uint32_t>(product) / static_cast<uint32_t>(numWaveRanges));
    }
    return static_cast<int32_t>(product / numWaveRanges);
}

// The wave range that holds step `s`.
__host__ __device__ __forceinline__ int32_t PaRangeOf(int32_t s, int32_t totalSteps, int32_t numWaveRanges)
{
    const int64_t product = (static_cast<int64_t>(s) + 1) * numWaveRanges - 1;
    if (product < 0x7fffffffLL) {
        return static_cast<int32_t>(static_cast<uint32_t>(product) / static_cast<uint32_t>(totalSteps));
    }
    return static_cast<int32_t>(product / totalSteps);
}

__device__ __forceinline__ float Bf16ToFloat(uint16_t v)
{
    return __uint_as_float(static_cast<uint32_t>(v) << 16);
}

// Round-to-nearest-even fp32 -> bf16, NaN kept quiet.
__device__ __forceinline__ uint16_t FloatToBf16(float f)
{
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        return static_cast<uint16_t>((u >> 16) | 0x40u);
    }
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

__device__ __forceinline__ float HalfBitsToFloat(uint16_t v)
{
    return static_cast<float>(__builtin_bit_cast(_Float16, v));
}

__device__ __forceinline__ uint16_t FloatToHalfBits(float f)
{
    return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
}

__device__ __forceinline__ float Load16(const void *p, int64_t idx, bool bf16)
{
    uint16_t raw = reinterpret_cast<const uint16_t *>(p)[idx];
    return bf16 ? Bf16ToFloat(raw) : HalfBitsToFloat(raw);
}

__device__ __forceinline__ void Store16(void *p, int64_t idx, float v, bool bf16)
{
    reinterpret_cast<uint16_t *>(p)[idx] = bf16 ? FloatToBf16(v) : FloatToHalfBits(v);
}

} // namespace atbmi
#endif
