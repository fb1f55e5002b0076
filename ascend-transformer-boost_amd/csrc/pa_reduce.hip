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
typedef float ReduceF4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(REDUCE_THREADS) void PaStreamReduceKernel(const PaArgs a, const PaStreamPlan p)
{
    const int vecs = a.Dv / 4;                                        // threads per row
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
    const bool bf16 = a.qIsBf16 != 0;
    const int64_t outRow = static_cast<int64_t>(sq.qRow + tok) * a.H + h;
    // Rows of up to MAX_HELD ranges (nearly all): the log-sum-exps and the thread's pieces of the partial
    // rows are requested together and held in registers, one memory round trip; longer rows take the
    // log-sum-exps first and the pieces in a second pass.
    constexpr int MAX_HELD = 8;
    const bool held = count <= MAX_HELD;
    float lseHeld[MAX_HELD];
    float mx = -INFINITY;
    if (!held) {
        for (int k = 0; k < count; ++k) {
            mx = fmaxf(mx, a.partLse[rowOf(k)]);
        }
    }
    for (int c4 = vecs >= REDUCE_THREADS ? tid : tid % vecs; c4 < vecs; c4 += REDUCE_THREADS) {
        ReduceF4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
        float sum = 0.0f;
        if (held) {
            ReduceF4 piece[MAX_HELD];
#pragma unroll
            for (int k = 0; k < MAX_HELD; ++k) {
                lseHeld[k] = -INFINITY;
                piece[k] = ReduceF4{0.0f, 0.0f, 0.0f, 0.0f};
                if (k < count) {
                    const int64_t ph = rowOf(k);
                    lseHeld[k] = a.partLse[ph];
                    piece[k] = *reinterpret_cast<const ReduceF4 *>(a.partO + ph * a.Dv + c4 * 4);
                }
            }
            mx = -INFINITY;
#pragma unroll
            for (int k = 0; k < MAX_HELD; ++k) {
                mx = fmaxf(mx, lseHeld[k]);
            }
#pragma unroll
            for (int k = 0; k < MAX_HELD; ++k) {
                // a range that a -inf mask emptied (and a slot past the row's ranges) weighs nothing
                const float w = lseHeld[k] == -INFINITY ? 0.0f : exp2f(lseHeld[k] - mx);
                sum += w;
                acc += w * piece[k];
            }
        } else {
#pragma unroll 4
            for (int k = 0; k < count; ++k) {
                const int64_t ph = rowOf(k);
                const float lse = a.partLse[ph];
                const float w = lse == -INFINITY ? 0.0f : exp2f(lse - mx); // a range a -inf mask emptied weighs nothing
                sum += w;
                acc += w * *reinterpret_cast<const ReduceF4 *>(a.partO + ph * a.Dv + c4 * 4);
            }
        }
        const float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
        float o[4] = {acc[0] * inv, acc[1] * inv, acc[2] * inv, acc[3] * inv};
        if (a.finishV) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int ch = g * a.Dv + c4 * 4 + e;
                o[e] = (o[e] + (a.vOff ? static_cast<float>(a.vOff[ch]) : 0.0f)) * a.vScale[ch * a.scaleStride];
            }
        }
        uint16_t bits[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            bits[e] = bf16 ? FloatToBf16(o[e]) : FloatToHalfBits(o[e]);
        }
        uint2 packed;
        packed.x = static_cast<uint32_t>(bits[0]) | (static_cast<uint32_t>(bits[1]) << 16);
        packed.y = static_cast<uint32_t>(bits[2]) | (static_cast<uint32_t>(bits[3]) << 16);
        *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(a.out) + outRow * a.Dv + c4 * 4) = packed;
        if (a.lse && c4 == 0) {
            Store16(a.lse, outRow, (mx + log2f(sum)) * LN2, bf16);
        }
    }
}

} // namespace

int LaunchPaStreamReduce(const AtbmiPaShape &shape, const PaArgs &args, const PaStreamPlan &plan,
                         hipStream_t stream)
{
    (void)shape;
    const int vecs = args.Dv / 4;
    const int rowsPerWg = vecs >= REDUCE_THREADS ? 1 : REDUCE_THREADS / vecs;
    const int64_t rows = static_cast<int64_t>(plan.numSeqs) * plan.foldTokens * args.H;
    const int64_t grid = (rows + rowsPerWg - 1) / rowsPerWg;
    if (grid <= 0) {
        return OK;
    }
    if (grid > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "pa_reduce: grid of %lld workgroups is out of range", (long long)grid);
    }
    PaStreamReduceKernel<<<static_cast<unsigned>(grid), REDUCE_THREADS, 0, stream>>>(args, plan);
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
