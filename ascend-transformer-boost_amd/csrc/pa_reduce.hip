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

// Stream plan: the partials of sequence b live in the slots of the wave
// ranges that intersect its steps; a sequence inside one range was written
// directly by that wave. One workgroup merges one (sequence, query head).
// Slot 2wr holds the row a range starts in, slot 2wr+1 the row it ends in, so
// only the first range of a sequence can use an odd slot.
// The weights 2^(lse_k - max) are computed once, 128 ranges at a time by the
// 128 threads, and kept in LDS; threads then own output channels.
__global__ __launch_bounds__(REDUCE_THREADS) void PaStreamReduceKernel(const PaArgs a, const PaStreamPlan p)
{
    __shared__ float weight[REDUCE_THREADS];
    __shared__ float red[REDUCE_THREADS / WAVE];
    // one workgroup per (pass, query token of it, head); a slot holds foldTokens x H partial rows
    const int rowsPerSlot = a.H * p.foldTokens;
    const int b = blockIdx.x / rowsPerSlot;
    const int tok = blockIdx.x % rowsPerSlot / a.H;
    const int h = blockIdx.x % a.H;
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
    const int tid = threadIdx.x;
    auto rowOf = [&](int k) { return k == 0 ? ph0 : phEven + k * stride; };
    auto blockMax = [&](float v) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            v = fmaxf(v, __shfl_xor(v, off, WAVE));
        }
        __syncthreads();
        if (tid % WAVE == 0) {
            red[tid / WAVE] = v;
        }
        __syncthreads();
        return fmaxf(red[0], red[1]);
    };
    auto blockSum = [&](float v) {
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            v += __shfl_xor(v, off, WAVE);
        }
        __syncthreads();
        if (tid % WAVE == 0) {
            red[tid / WAVE] = v;
        }
        __syncthreads();
        return red[0] + red[1];
    };

    float mx = -INFINITY;
    for (int k = tid; k < count; k += REDUCE_THREADS) {
        mx = fmaxf(mx, a.partLse[rowOf(k)]);
    }
    mx = blockMax(mx);

    const int g = h / a.groupSize;
    const bool bf16 = a.qIsBf16 != 0;
    // channels handled by this thread: tid, tid + 128, ... (at most 5 for Dv <= 576)
    float acc[5] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    float total = 0.0f;
    for (int k0 = 0; k0 < count; k0 += REDUCE_THREADS) {
        const int kn = min(REDUCE_THREADS, count - k0);
        __syncthreads();
        float w = 0.0f;
        if (tid < kn) {
            const float lse = a.partLse[rowOf(k0 + tid)];
            w = lse == -INFINITY ? 0.0f : exp2f(lse - mx); // a range a -inf mask emptied weighs nothing
            weight[tid] = w;
        }
        total += w;
        __syncthreads();
#pragma unroll
        for (int c = 0; c < 5; ++c) {
            const int d = tid + c * REDUCE_THREADS;
            if (d < a.Dv) {
                float s = 0.0f;
#pragma unroll 4
                for (int k = 0; k < kn; ++k) {
                    s += weight[k] * a.partO[rowOf(k0 + k) * a.Dv + d];
                }
                acc[c] += s;
            }
        }
    }
    const float sum = blockSum(total);
    const float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
    if (a.lse && tid == 0) {
        Store16(a.lse, static_cast<int64_t>(sq.qRow + tok) * a.H + h, (mx + log2f(sum)) * LN2, a.qIsBf16 != 0);
    }
#pragma unroll
    for (int c = 0; c < 5; ++c) {
        const int d = tid + c * REDUCE_THREADS;
        if (d < a.Dv) {
            float o = acc[c] * inv;
            if (a.finishV) {
                const int ch = g * a.Dv + d;
                o = (o + (a.vOff ? static_cast<float>(a.vOff[ch]) : 0.0f)) * a.vScale[ch * a.scaleStride];
            }
            Store16(a.out, (static_cast<int64_t>(sq.qRow + tok) * a.H + h) * a.Dv + d, o, bf16);
        }
    }
}

} // namespace

int LaunchPaStreamReduce(const AtbmiPaShape &shape, const PaArgs &args, const PaStreamPlan &plan,
                         hipStream_t stream)
{
    (void)shape;
    const int64_t grid = static_cast<int64_t>(plan.numSeqs) * plan.foldTokens * args.H;
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
