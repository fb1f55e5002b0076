// Split-KV merge kernel: combines the partial attention results of one
// sequence into its output row.
//
// Every partial p holds a normalised output O_p (fp32) and a log-sum-exp in
// base 2, lse_p = m_p + log2(l_p). With M = max_p lse_p and
// w_p = 2^(lse_p - M) the merged row is sum_p w_p O_p / sum_p w_p, the same
// combination the reference applies to its per-core partials (reference
// src/kernels/mixkernels/pagedattention/op_kernel/paged_attention_decoder_nd_common.cce:6568-6760,
// :7959-7975). An empty partial carries lse = -inf and weighs 0.
//
// One workgroup per (sequence, query head); threads own output channels.
#include "pa_internal.h"

namespace atbmi {
namespace {

constexpr int REDUCE_THREADS = 128;
constexpr float LN2 = 0.6931471805599453f; // the partial log-sum-exps are kept in base 2

__global__ __launch_bounds__(REDUCE_THREADS) void PaReduceKernel(const PaArgs a)
{
    const PaSeqInfo s = a.seqs[blockIdx.x / a.H];
    const int h = blockIdx.x % a.H;
    const int np = s.numPartials;
    const float *lse = a.partLse + static_cast<int64_t>(s.firstPartial) * a.H + h;

    float mx = -INFINITY;
    for (int p = 0; p < np; ++p) {
        mx = fmaxf(mx, lse[static_cast<int64_t>(p) * a.H]);
    }
    float total = 0.0f;
    // (a chunk a -inf mask emptied has lse == -inf and weighs nothing, even when every chunk is like that)
    auto weightOf = [mx](float v) { return v == -INFINITY ? 0.0f : exp2f(v - mx); };
    for (int p = 0; p < np; ++p) {
        total += weightOf(lse[static_cast<int64_t>(p) * a.H]);
    }
    const float inv = total > 0.0f ? 1.0f / total : 0.0f;
    const int g = h / a.groupSize;
    const bool bf16 = a.qIsBf16 != 0;
    if (a.lse && threadIdx.x == 0) {
        Store16(a.lse, static_cast<int64_t>(s.qRow) * a.H + h, (mx + log2f(total)) * LN2, bf16);
    }

    for (int d = threadIdx.x; d < a.Dv; d += REDUCE_THREADS) {
        float acc = 0.0f;
        for (int p = 0; p < np; ++p) {
            const float w = weightOf(lse[static_cast<int64_t>(p) * a.H]);
            const int64_t ph = (static_cast<int64_t>(s.firstPartial) + p) * a.H + h;
            acc += w * a.partO[ph * a.Dv + d];
        }
        acc *= inv;
        if (a.finishV) {
            const int c = g * a.Dv + d;
            acc = (acc + (a.vOff ? static_cast<float>(a.vOff[c]) : 0.0f)) * a.vScale[c * a.scaleStride];
        }
        Store16(a.out, (static_cast<int64_t>(s.qRow) * a.H + h) * a.Dv + d, acc, bf16);
    }
}

// Stream plan: the partials of a pass live in the slots of the wave ranges that
// intersect its steps; a pass inside one range was written directly by that
// wave. Slot 2wr holds the row a range starts in, slot 2wr+1 the row it ends
// in, so only the first range of a pass can use an odd slot; a slot holds
// foldTokens x H partial rows.
// A thread owns four consecutive channels of one output row (pass, query token,
// head): it takes the maximum of the row's log-sum-exps, then adds up the
// weighted partial rows with 16-byte loads. A workgroup of 128 threads covers as
// many whole rows as fit (four for 128 channels, one for 512).
// The partial rows are 16-bit values of the query's type; a thread owns eight channels.

// A thread's piece of one partial row, kept as loaded (16 bytes) until it is accumulated.
struct PartialPiece {
    static constexpr int CH = 8;
    uint32_t raw[4];
    __device__ __forceinline__ void Clear() { raw[0] = raw[1] = raw[2] = raw[3] = 0u; }
    __device__ __forceinline__ void Load(const float *partO, int64_t elem)
    {
        const uint4 x = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(partO) + elem);
        raw[0] = x.x; raw[1] = x.y; raw[2] = x.z; raw[3] = x.w;
    }
    __device__ __forceinline__ float Get(int e, bool bf16) const
    {
        const uint32_t w = raw[e >> 1];
        if (bf16) {
            return __uint_as_float((e & 1) ? (w & 0xffff0000u) : (w << 16));
        }
        return HalfBitsToFloat(static_cast<uint16_t>((e & 1) ? (w >> 16) : (w & 0xffffu)));
    }
};

template <bool BF16>
__global__ __launch_bounds__(REDUCE_THREADS) void PaStreamReduceKernel(const PaArgs a, const PaStreamPlan p)
{
    constexpr int CH = PartialPiece::CH;                              // channels per thread
    const int vecs = a.Dv / CH;                                       // threads per row
    const int rowsPerWg = vecs >= REDUCE_THREADS ? 1 : REDUCE_THREADS / vecs;
    const int rowsPerSlot = a.H * p.foldTokens;
    const int tid = threadIdx.x;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * rowsPerWg + (vecs >= REDUCE_THREADS ? 0 : tid / vecs);
    if (row >= static_cast<int64_t>(p.numSeqs) * rowsPerSlot || (vecs < REDUCE_THREADS && tid >= rowsPerWg * vecs)) {
        return;
    }
    const int b = static_cast<int>(row / rowsPerSlot);
    const int tok = static_cast<int>(row % rowsPerSlot) / a.H;
    const int h = static_cast<int>(row % a.H);
    const PaSeq sq = p.seqs ? p.seqs[b] : p.inlineSeqs[b];
    if (tok >= sq.nTok) {
        return;
    }
    const int begin = sq.stepBegin;
    const int end = (p.seqs ? p.seqs[b + 1] : p.inlineSeqs[b + 1]).stepBegin;
    const int wrFirst = PaRangeOf(begin, p.totalSteps, p.numWaveRanges);
    const int wrLast = PaRangeOf(end - 1, p.totalSteps, p.numWaveRanges);
    if (wrFirst == wrLast) {
        return;
    }
    const int firstOdd = PaRangeBegin(wrFirst, p.totalSteps, p.numWaveRanges) >= begin ? 0 : 1;
    const int64_t stride = 2 * static_cast<int64_t>(rowsPerSlot);
    // partial row of the k-th range, k >= 1
    const int64_t phEven = 2 * static_cast<int64_t>(wrFirst) * rowsPerSlot + static_cast<int64_t>(tok) * a.H + h;
    const int64_t ph0 = phEven + static_cast<int64_t>(firstOdd) * rowsPerSlot;
    const int count = wrLast - wrFirst + 1;
    auto rowOf = [&](int k) { return k == 0 ? ph0 : phEven + k * stride; };

    const int g = h / a.groupSize;
    constexpr bool bf16 = BF16;
    const int64_t outRow = static_cast<int64_t>(sq.qRow + tok) * a.H + h;
    // 2^x on the hardware unit: -inf gives 0, which is what an empty range must weigh
    auto pow2 = [](float x) { return __builtin_amdgcn_exp2f(x); };
    // The ranges of a row are taken MAX_HELD at a time: their log-sum-exps and the thread's pieces of their
    // partial rows are requested together and held as loaded, one memory round trip for nearly every row;
    // a longer row carries its running maximum and sums from one group of ranges to the next.
    constexpr int MAX_HELD = 8;
#pragma unroll 1
    for (int c = vecs >= REDUCE_THREADS ? tid : tid % vecs; c < vecs; c += REDUCE_THREADS) {
        float acc[CH];
#pragma unroll
        for (int e = 0; e < CH; ++e) {
            acc[e] = 0.0f;
        }
        float sum = 0.0f;
        float mx = -INFINITY;
#pragma unroll 1
        for (int k0 = 0; k0 < count; k0 += MAX_HELD) {
            float lseHeld[MAX_HELD];
            PartialPiece piece[MAX_HELD];
#pragma unroll
            for (int k = 0; k < MAX_HELD; ++k) {
                lseHeld[k] = -INFINITY;
                piece[k].Clear();
                if (k0 + k < count) {
                    const int64_t ph = rowOf(k0 + k);
                    lseHeld[k] = a.partLse[ph];
                    piece[k].Load(a.partO, ph * a.Dv + c * CH);
                }
            }
            float mNew = mx;
#pragma unroll
            for (int k = 0; k < MAX_HELD; ++k) {
                mNew = fmaxf(mNew, lseHeld[k]);
            }
            if (k0 > 0 && mNew > mx) { // (mx is finite here or everything so far weighed nothing)
                const float keep = pow2(mx - mNew);
                sum *= keep;
#pragma unroll
                for (int e = 0; e < CH; ++e) {
                    acc[e] *= keep;
                }
            }
            mx = mNew;
#pragma unroll
            for (int k = 0; k < MAX_HELD; ++k) {
                // a range that a -inf mask emptied (and a slot past the row's ranges) weighs nothing
                const float w = mx == -INFINITY ? 0.0f : pow2(lseHeld[k] - mx);
                sum += w;
#pragma unroll
                for (int e = 0; e < CH; ++e) {
                    acc[e] += w * piece[k].Get(e, bf16);
                }
            }
        }
        const float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
        uint16_t bits[CH];
#pragma unroll
        for (int e = 0; e < CH; ++e) {
            float o = acc[e] * inv;
            if (a.finishV) {
                const int ch = g * a.Dv + c * CH + e;
                o = (o + (a.vOff ? static_cast<float>(a.vOff[ch]) : 0.0f)) * a.vScale[ch * a.scaleStride];
            }
            bits[e] = bf16 ? FloatToBf16(o) : FloatToHalfBits(o);
        }
        uint32_t packed[CH / 2];
#pragma unroll
        for (int e = 0; e < CH / 2; ++e) {
            packed[e] = static_cast<uint32_t>(bits[2 * e]) | (static_cast<uint32_t>(bits[2 * e + 1]) << 16);
        }
        uint16_t *dst = reinterpret_cast<uint16_t *>(a.out) + outRow * a.Dv + c * CH;
        *reinterpret_cast<uint4 *>(dst) = uint4{packed[0], packed[1], packed[2], packed[3]};
        if (a.lse && c == 0) {
            Store16(a.lse, outRow, (mx + log2f(sum)) * LN2, bf16);
        }
    }
}

// The same merge for plans whose rows span many ranges (a few long sequences in a batch): SLICES threads share each
// piece of an output row, thread s taking the ranges s, s + SLICES, ... eight at a time; each ends with a maximum, a
// sum of weights and a weighted sum of its own, and the first of them joins these through LDS. A row of 40 ranges is
// then two memory round trips, not five. Partial rows of up to 256 channels.
constexpr int SLICES = 4;
template <bool BF16>
__global__ __launch_bounds__(REDUCE_THREADS) void PaStreamReduceSlicedKernel(const PaArgs a, const PaStreamPlan p)
{
    constexpr int CH = PartialPiece::CH;
    constexpr int MAX_HELD = 8;
    __shared__ float joined[REDUCE_THREADS * (CH + 2)];
    const int vecs = a.Dv / CH;                  // pieces per row
    const int rowThreads = vecs * SLICES;
    const int rowsPerWg = REDUCE_THREADS / rowThreads; // (>= 1: the launcher sends wider rows to the other kernel)
    const int rowsPerSlot = a.H * p.foldTokens;
    const int tid = threadIdx.x;
    const int slice = (tid / vecs) % SLICES;
    const int c = tid % vecs;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * rowsPerWg + tid / rowThreads;
    // (every thread stays to the barrier; a thread without a row to merge works on nothing)
    bool active = tid < rowsPerWg * rowThreads && row < static_cast<int64_t>(p.numSeqs) * rowsPerSlot;
    const int b = active ? static_cast<int>(row / rowsPerSlot) : 0;
    const int tok = active ? static_cast<int>(row % rowsPerSlot) / a.H : 0;
    const int h = active ? static_cast<int>(row % a.H) : 0;
    const PaSeq sq = p.seqs ? p.seqs[b] : p.inlineSeqs[b];
    const int begin = sq.stepBegin;
    const int end = (p.seqs ? p.seqs[b + 1] : p.inlineSeqs[b + 1]).stepBegin;
    const int wrFirst = PaRangeOf(begin, p.totalSteps, p.numWaveRanges);
    const int wrLast = PaRangeOf(end - 1, p.totalSteps, p.numWaveRanges);
    active = active && tok < sq.nTok && wrFirst != wrLast;
    const int firstOdd = PaRangeBegin(wrFirst, p.totalSteps, p.numWaveRanges) >= begin ? 0 : 1;
    const int64_t stride = 2 * static_cast<int64_t>(rowsPerSlot);
    const int64_t phEven = 2 * static_cast<int64_t>(wrFirst) * rowsPerSlot + static_cast<int64_t>(tok) * a.H + h;
    const int64_t ph0 = phEven + static_cast<int64_t>(firstOdd) * rowsPerSlot;
    const int count = active ? wrLast - wrFirst + 1 : 0;
    auto rowOf = [&](int k) { return k == 0 ? ph0 : phEven + k * stride; };
    auto pow2 = [](float x) { return __builtin_amdgcn_exp2f(x); };

    float acc[CH];
#pragma unroll
    for (int e = 0; e < CH; ++e) {
        acc[e] = 0.0f;
    }
    float sum = 0.0f;
    float mx = -INFINITY;
#pragma unroll 1
    for (int k0 = slice; k0 < count; k0 += MAX_HELD * SLICES) {
        float lseHeld[MAX_HELD];
        PartialPiece piece[MAX_HELD];
#pragma unroll
        for (int k = 0; k < MAX_HELD; ++k) {
            lseHeld[k] = -INFINITY;
            piece[k].Clear();
            if (k0 + k * SLICES < count) {
                const int64_t ph = rowOf(k0 + k * SLICES);
                lseHeld[k] = a.partLse[ph];
                piece[k].Load(a.partO, ph * a.Dv + c * CH);
            }
        }
        float mNew = mx;
#pragma unroll
        for (int k = 0; k < MAX_HELD; ++k) {
            mNew = fmaxf(mNew, lseHeld[k]);
        }
        if (k0 > slice && mNew > mx) {
            const float keep = pow2(mx - mNew);
            sum *= keep;
#pragma unroll
            for (int e = 0; e < CH; ++e) {
                acc[e] *= keep;
            }
        }
        mx = mNew;
#pragma unroll
        for (int k = 0; k < MAX_HELD; ++k) {
            const float w = mx == -INFINITY ? 0.0f : pow2(lseHeld[k] - mx);
            sum += w;
#pragma unroll
            for (int e = 0; e < CH; ++e) {
                acc[e] += w * piece[k].Get(e, BF16);
            }
        }
    }
    float *mine = joined + tid * (CH + 2);
    mine[0] = mx;
    mine[1] = sum;
#pragma unroll
    for (int e = 0; e < CH; ++e) {
        mine[2 + e] = acc[e];
    }
    __syncthreads();
    if (!active || slice != 0) {
        return;
    }
    // join the slices: the usual rescaling to the common maximum
    float top = mx;
#pragma unroll
    for (int s = 1; s < SLICES; ++s) {
        top = fmaxf(top, joined[(tid + s * vecs) * (CH + 2)]);
    }
    const float own = top == -INFINITY ? 0.0f : pow2(mx - top);
    sum *= own;
#pragma unroll
    for (int e = 0; e < CH; ++e) {
        acc[e] *= own;
    }
#pragma unroll
    for (int s = 1; s < SLICES; ++s) {
        const float *other = joined + (tid + s * vecs) * (CH + 2);
        const float w = top == -INFINITY ? 0.0f : pow2(other[0] - top);
        sum += w * other[1];
#pragma unroll
        for (int e = 0; e < CH; ++e) {
            acc[e] += w * other[2 + e];
        }
    }
    const int g = h / a.groupSize;
    const int64_t outRow = static_cast<int64_t>(sq.qRow + tok) * a.H + h;
    const float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
    uint16_t bits[CH];
#pragma unroll
    for (int e = 0; e < CH; ++e) {
        float o = acc[e] * inv;
        if (a.finishV) {
            const int ch = g * a.Dv + c * CH + e;
            o = (o + (a.vOff ? static_cast<float>(a.vOff[ch]) : 0.0f)) * a.vScale[ch * a.scaleStride];
        }
        bits[e] = BF16 ? FloatToBf16(o) : FloatToHalfBits(o);
    }
    uint32_t packed[CH / 2];
#pragma unroll
    for (int e = 0; e < CH / 2; ++e) {
        packed[e] = static_cast<uint32_t>(bits[2 * e]) | (static_cast<uint32_t>(bits[2 * e + 1]) << 16);
    }
    uint16_t *dst = reinterpret_cast<uint16_t *>(a.out) + outRow * a.Dv + c * CH;
    *reinterpret_cast<uint4 *>(dst) = uint4{packed[0], packed[1], packed[2], packed[3]};
    if (a.lse && c == 0) {
        Store16(a.lse, outRow, (top + log2f(sum)) * LN2, BF16);
    }
}

} // namespace

int LaunchPaStreamReduce(const AtbmiPaShape &shape, const PaArgs &args, const PaStreamPlan &plan,
                         hipStream_t stream)
{
    (void)shape;
    constexpr int CH = PartialPiece::CH;
    if (args.Dv % CH != 0) {
        return Fail(ERR_INVALID_PARAM, "pa_reduce: %d channels a row, not a multiple of %d", args.Dv, CH);
    }
    const int vecs = args.Dv / CH;
    const int rowsPerWg = vecs >= REDUCE_THREADS ? 1 : REDUCE_THREADS / vecs;
    const int64_t rows = static_cast<int64_t>(plan.numSeqs) * plan.foldTokens * args.H;
    const int64_t grid = (rows + rowsPerWg - 1) / rowsPerWg;
    if (grid <= 0) {
        return OK;
    }
    if (grid > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "pa_reduce: grid of %lld workgroups is out of range", (long long)grid);
    }
    if (plan.maxRangesPerRow > 8 && vecs * SLICES <= REDUCE_THREADS) {
        const int slicedRowsPerWg = REDUCE_THREADS / (vecs * SLICES);
        const int64_t slicedGrid = (rows + slicedRowsPerWg - 1) / slicedRowsPerWg;
        if (slicedGrid <= 0x7fffffffLL) {
            const unsigned slicedBlocks = static_cast<unsigned>(slicedGrid);
            if (args.qIsBf16) {
                PaStreamReduceSlicedKernel<true><<<slicedBlocks, REDUCE_THREADS, 0, stream>>>(args, plan);
            } else {
                PaStreamReduceSlicedKernel<false><<<slicedBlocks, REDUCE_THREADS, 0, stream>>>(args, plan);
            }
            ATBMI_HIP_CHECK(hipGetLastError());
            return OK;
        }
    }
    const unsigned blocks = static_cast<unsigned>(grid);
    if (args.qIsBf16) {
        PaStreamReduceKernel<true><<<blocks, REDUCE_THREADS, 0, stream>>>(args, plan);
    } else {
        PaStreamReduceKernel<false><<<blocks, REDUCE_THREADS, 0, stream>>>(args, plan);
    }
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}

int LaunchPaReduce(const AtbmiPaShape &shape, const PaArgs &args, int numSeqs, hipStream_t stream)
{
    (void)shape;
    if (numSeqs <= 0) {
        return OK;
    }
    const int64_t grid = static_cast<int64_t>(numSeqs) * args.H;
    if (grid > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "pa_reduce: grid of %lld workgroups is out of range", (long long)grid);
    }
    PaReduceKernel<<<static_cast<unsigned>(grid), REDUCE_THREADS, 0, stream>>>(args);
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}

} // namespace atbmi
