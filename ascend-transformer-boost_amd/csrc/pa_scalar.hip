// Scalar (VALU) paged decode-attention kernel for gfx950.
//
// The fallback for shapes the MFMA kernel is not built for: any head size up
// to 576, any block size, any GQA group. fp32 arithmetic throughout, in the
// same order of operations as the reference golden (int8 rows are dequantised
// as (q + offset) * scale in fp32; reference
// tests/apitest/kernelstest/mix/test_paged_attention_common.py:85-108,229-276).
//
// One workgroup = one (work item, KV head, tile of up to 8 query heads).
// Its four waves take tokens round-robin; a wave spreads the channels of one
// K/V row over its 64 lanes (lane L owns channels L, L+64, ...), so a row is
// read as consecutive 2- or 1-byte elements by consecutive lanes. Each wave
// keeps its own online-softmax state and writes its own partial; the merge
// kernel combines them.
#include "pa_internal.h"

namespace atbmi {
namespace {

constexpr int HT = PA_SCALAR_HEAD_TILE;

__device__ __forceinline__ float WaveSum(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        v += __shfl_xor(v, off, WAVE);
    }
    return v;
}

// KV8 = true: int8 cache rows; false: 16-bit rows of the query's type.
template <bool KV8, int EPL>
__global__ __launch_bounds__(PA_SCALAR_WAVES * WAVE) void PaScalarKernel(const PaArgs a)
{
    const int g = blockIdx.x % a.G;
    const int headTiles = (a.groupSize + HT - 1) / HT;
    const int rest = blockIdx.x / a.G;
    const int ht = rest % headTiles;
    const PaWorkItem it = a.items[rest / headTiles];
    const int wave = threadIdx.x / WAVE;
    const int lane = threadIdx.x % WAVE;
    const bool bf16 = a.qIsBf16 != 0;
    const int h0 = g * a.groupSize + ht * HT;
    const int nh = min(HT, a.groupSize - ht * HT);
    constexpr float LOG2E = 1.4426950408889634f;
    const float scale2 = a.qkScale * LOG2E * (a.logN ? a.logN[it.seq] : 1.0f);
    // additive score bias of this sequence and head tile (base-2 units once multiplied by LOG2E)
    const int64_t maskRow = a.mask ? static_cast<int64_t>(it.maskRow) * a.maskBatchStride : 0;

    const int gs = a.descaleHeads > 0 ? it.seq % a.descaleHeads : g; // descale slice (see PaArgs::descaleHeads)
    const int dn = a.D - a.ropeDim; // channels held by q / kc themselves (all of them unless the layout is split)
    float q[HT][EPL];
#pragma unroll
    for (int hh = 0; hh < HT; ++hh) {
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            const int d = lane + WAVE * e;
            float v = 0.0f;
            if (hh < nh && d < a.D) {
                const int64_t qh = static_cast<int64_t>(it.qRow) * a.H + h0 + hh;
                v = d < dn ? Load16(a.q, qh * dn + d, bf16) : Load16(a.qRope, qh * a.ropeDim + d - dn, bf16);
                if (a.qScale != 0.0f) {
                    // the reference pre-multiplies Q in its own dtype
                    v *= a.qScale;
                    v = bf16 ? Bf16ToFloat(FloatToBf16(v)) : HalfBitsToFloat(FloatToHalfBits(v));
                }
            }
            q[hh][e] = v;
        }
    }

    float kS[EPL], kO[EPL], vS[EPL], vO[EPL];
#pragma unroll
    for (int e = 0; e < EPL; ++e) {
        const int d = lane + WAVE * e;
        kS[e] = 1.0f; kO[e] = 0.0f; vS[e] = 1.0f; vO[e] = 0.0f;
        if (KV8) {
            if (d < a.D) {
                kS[e] = a.kScale[(gs * a.D + d) * a.scaleStride];
                kO[e] = a.kOff ? static_cast<float>(a.kOff[gs * a.D + d]) : 0.0f;
            }
            if (d < a.Dv) {
                vS[e] = a.vScale[(gs * a.Dv + d) * a.scaleStride];
                vO[e] = a.vOff ? static_cast<float>(a.vOff[gs * a.Dv + d]) : 0.0f;
            }
        }
    }

    float m[HT], l[HT], acc[HT][EPL];
#pragma unroll
    for (int hh = 0; hh < HT; ++hh) {
        m[hh] = -INFINITY;
        l[hh] = 0.0f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            acc[hh][e] = 0.0f;
        }
    }

    const int32_t *table = a.tables + static_cast<int64_t>(it.seq) * a.maxBlocksPerSeq;
    for (int t = it.tokBegin + wave; t < it.tokEnd; t += PA_SCALAR_WAVES) {
        const int64_t blk = table[t / a.blockSize];
        const int off = t % a.blockSize;
        const int64_t row = blk * a.blockRows + off;
        int64_t kBase = row * a.kRowStride + static_cast<int64_t>(g) * a.kHeadStride;
        int64_t rBase = row * a.ropeRowStride + static_cast<int64_t>(g) * a.ropeDim - dn;
        int64_t vBase = row * a.vRowStride + static_cast<int64_t>(g) * a.vHeadStride;
        // Fractal-NZ caches: a block is (channels / 16) slabs of blockSize x 16; element d then sits
        // ((d / 16) << nzShift) * 16 + d % 16 past the token's place in the first slab.
        const bool nz = a.nzShift > 0;
        if (nz) {
            kBase = blk * a.blockSize * dn + off * 16;
            vBase = kBase;
            rBase = blk * a.blockSize * a.ropeDim + off * 16;
        }
        auto nzOff = [&](int d) { return (static_cast<int64_t>(d >> 4) << a.nzShift) * 16 + (d & 15); };
        const float razor = a.razor ? a.razor[row] : 0.0f;
        float k[EPL], v[EPL];
#pragma unroll
        for (int e = 0; e < EPL; ++e) {
            const int d = lane + WAVE * e;
            k[e] = 0.0f;
            v[e] = 0.0f;
            if (KV8) {
                if (d < a.D) {
                    k[e] = (static_cast<float>(reinterpret_cast<const int8_t *>(a.kc)[kBase + d]) + kO[e]) * kS[e];
                }
                if (d < a.Dv) {
                    v[e] = (static_cast<float>(reinterpret_cast<const int8_t *>(a.vc)[vBase + d]) + vO[e]) * vS[e];
                }
            } else {
                if (d < a.D) {
                    if (nz) {
                        k[e] = d < dn ? Load16(a.kc, kBase + nzOff(d), bf16) : Load16(a.kRope, rBase + nzOff(d - dn), bf16);
                    } else {
                        k[e] = d < dn ? Load16(a.kc, kBase + d, bf16) : Load16(a.kRope, rBase + d, bf16);
                    }
                }
                if (d < a.Dv) {
                    v[e] = Load16(a.vc, nz ? vBase + nzOff(d) : vBase + d, bf16);
                }
            }
        }
#pragma unroll
        for (int hh = 0; hh < HT; ++hh) {
            if (hh < nh) {
                float s = 0.0f;
#pragma unroll
                for (int e = 0; e < EPL; ++e) {
                    s += q[hh][e] * k[e];
                }
                s = (WaveSum(s) + razor) * scale2;
                if (a.mask) {
                    s += Load16(a.mask, maskRow + static_cast<int64_t>(h0 + hh) * a.maskHeadStride + t, bf16) * LOG2E;
                }
                const float mNew = fmaxf(m[hh], s);
                // (a bias of -inf takes the token out; nothing to rescale while the row is still empty)
                const float corr = m[hh] == -INFINITY ? 0.0f : exp2f(m[hh] - mNew);
                const float p = s == -INFINITY ? 0.0f : exp2f(s - mNew);
                m[hh] = mNew;
                l[hh] = l[hh] * corr + p;
#pragma unroll
                for (int e = 0; e < EPL; ++e) {
                    acc[hh][e] = acc[hh][e] * corr + p * v[e];
                }
            }
        }
    }

    const int64_t part = static_cast<int64_t>(it.partialBase) + wave;
#pragma unroll
    for (int hh = 0; hh < HT; ++hh) {
        if (hh < nh) {
            const int64_t ph = part * a.H + h0 + hh;
            const float inv = l[hh] > 0.0f ? 1.0f / l[hh] : 0.0f;
#pragma unroll
            for (int e = 0; e < EPL; ++e) {
                const int d = lane + WAVE * e;
                if (d < a.Dv) {
                    a.partO[ph * a.Dv + d] = acc[hh][e] * inv;
                }
            }
            if (lane == 0) {
                a.partLse[ph] = l[hh] > 0.0f ? m[hh] + log2f(l[hh]) : -INFINITY;
            }
        }
    }
}

template <bool KV8>
int LaunchScalarByWidth(const AtbmiPaShape &shape, const PaArgs &args, unsigned grid, hipStream_t stream)
{
    const int width = shape.headDimK > shape.headDimV ? shape.headDimK : shape.headDimV;
    constexpr int threads = PA_SCALAR_WAVES * WAVE;
    if (width <= 64) {
        PaScalarKernel<KV8, 1><<<grid, threads, 0, stream>>>(args);
    } else if (width <= 128) {
        PaScalarKernel<KV8, 2><<<grid, threads, 0, stream>>>(args);
    } else if (width <= 256) {
        PaScalarKernel<KV8, 4><<<grid, threads, 0, stream>>>(args);
    } else if (width <= 576) {
        PaScalarKernel<KV8, 9><<<grid, threads, 0, stream>>>(args);
    } else {
        return Fail(ERR_INVALID_PARAM, "pa_decode: head size %d exceeds 576", width);
    }
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}

} // namespace

int LaunchPaScalar(const AtbmiPaShape &shape, const PaArgs &args, int numItems, hipStream_t stream)
{
    const int headTiles = (args.groupSize + HT - 1) / HT;
    const int64_t grid = static_cast<int64_t>(numItems) * headTiles * args.G;
    if (grid <= 0 || grid > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: grid of %lld workgroups is out of range", (long long)grid);
    }
    if (shape.kvDtype == ATBMI_INT8) {
        return LaunchScalarByWidth<true>(shape, args, static_cast<unsigned>(grid), stream);
    }
    return LaunchScalarByWidth<false>(shape, args, static_cast<unsigned>(grid), stream);
}

} // namespace atbmi
