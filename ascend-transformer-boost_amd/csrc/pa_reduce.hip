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
    for (int p = 0; p < np; ++p) {
        total += exp2f(lse[static_cast<int64_t>(p) * a.H] - mx);
    }
    const float inv = total > 0.0f ? 1.0f / total : 0.0f;
    const int g = h / a.groupSize;
    const bool bf16 = a.qIsBf16 != 0;

    for (int d = threadIdx.x; d < a.Dv; d += REDUCE_THREADS) {
        float acc = 0.0f;
        for (int p = 0; p < np; ++p) {
            const float w = exp2f(lse[static_cast<int64_t>(p) * a.H] - mx);
            const int64_t ph = (static_cast<int64_t>(s.firstPartial) + p) * a.H + h;
            acc += w * a.partO[ph * a.Dv + d];
        }
        acc *= inv;
        if (a.finishV) {
            const int c = g * a.Dv + d;
            acc = (acc + (a.vOff ? static_cast<float>(a.vOff[c]) : 0.0f)) * a.vScale[c];
        }
        Store16(a.out, (static_cast<int64_t>(s.qRow) * a.H + h) * a.Dv + d, acc, bf16);
    }
}

// Stream plan: the partials of sequence b live in the slots of the wave
// ranges that intersect its steps; a sequence inside one range was written
// directly by that wave.
__global__ __launch_bounds__(REDUCE_THREADS) void PaStreamReduceKernel(const PaArgs a, const PaStreamPlan p)
{
    const int b = blockIdx.x / a.H;
    const int h = blockIdx.x % a.H;
    const int begin = (p.seqs ? p.seqs[b] : p.inlineSeqs[b]).stepBegin;
    const int end = (p.seqs ? p.seqs[b + 1] : p.inlineSeqs[b + 1]).stepBegin;
    const int wrFirst = PaRangeOf(begin, p.totalSteps, p.numWaveRanges);
    const int wrLast = PaRangeOf(end - 1, p.totalSteps, p.numWaveRanges);
    if (wrFirst == wrLast) {
        return;
    }
    // slot 2wr holds the row a range starts in, slot 2wr+1 the row it ends in
    auto slotOf = [&](int wr) {
        return 2 * wr + (PaRangeBegin(wr, p.totalSteps, p.numWaveRanges) >= begin ? 0 : 1);
    };
    float mx = -INFINITY;
    for (int wr = wrFirst; wr <= wrLast; ++wr) {
        mx = fmaxf(mx, a.partLse[static_cast<int64_t>(slotOf(wr)) * a.H + h]);
    }
    float total = 0.0f;
    for (int wr = wrFirst; wr <= wrLast; ++wr) {
        total += exp2f(a.partLse[static_cast<int64_t>(slotOf(wr)) * a.H + h] - mx);
    }
    const float inv = 1.0f / total;
    const int g = h / a.groupSize;
    const bool bf16 = a.qIsBf16 != 0;
    for (int d = threadIdx.x; d < a.Dv; d += REDUCE_THREADS) {
        float acc = 0.0f;
        for (int wr = wrFirst; wr <= wrLast; ++wr) {
            const int64_t ph = static_cast<int64_t>(slotOf(wr)) * a.H + h;
            acc += exp2f(a.partLse[ph] - mx) * a.partO[ph * a.Dv + d];
        }
        acc *= inv;
        if (a.finishV) {
            const int c = g * a.Dv + d;
            acc = (acc + (a.vOff ? static_cast<float>(a.vOff[c]) : 0.0f)) * a.vScale[c];
        }
        Store16(a.out, (static_cast<int64_t>(b) * a.H + h) * a.Dv + d, acc, bf16);
    }
}

} // namespace

int LaunchPaStreamReduce(const AtbmiPaShape &shape, const PaArgs &args, const PaStreamPlan &plan,
                         hipStream_t stream)
{
    (void)shape;
    const int64_t grid = static_cast<int64_t>(plan.numSeqs) * args.H;
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
