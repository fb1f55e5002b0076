// Rotary position embedding of the query and key rows of a step, gfx950.
//
// Every row of q [tokens, hiddenQ] and k [tokens, hiddenK] is cut into units of headDim channels
// (headDim = the row size of the cos / sin tables); a unit is cut into rotaryCoeff / 2 chunks of
// 2 * stride channels, stride = headDim / rotaryCoeff, and inside a chunk channel i of the first
// half pairs with channel i of the second half:
//     out[lo] = x[lo] * cos[lo'] - x[hi] * sin[lo']
//     out[hi] = x[hi] * cos[hi'] + x[lo] * sin[hi']        (lo', hi' = the channels' offsets in the unit)
// rotaryCoeff 2 is "rotate half", rotaryCoeff = headDim the interleaved form (stride 1), 4 rotates the
// two halves of a head separately. Row r of the tables belongs to token r (cosFormat 0) or to
// position r of every sequence (cosFormat 1: the sequence lengths give each token its position).
//
// An HBM-bound elementwise kernel: a thread owns one pair of 16-byte pieces (8 channels of the
// first half of a chunk and their 8 partners), so every byte of q and k is read once and written
// once, by the same thread (the outputs may be the inputs). Strides below 8 channels take one
// pair of elements per thread. Arithmetic is fp32, rounded once.
#include <algorithm>
#include "atbmi_common.h"

namespace atbmi {
namespace {

constexpr int ROPE_THREADS = 256;

struct RopeArgs {
    const uint16_t *q, *k;
    const void *cosTab, *sinTab;
    const int32_t *seqLens;
    uint16_t *qOut, *kOut;
    int64_t numTokens, cosRows;
    int32_t hiddenQ, hiddenK, headDim, stride, batch, cosFormat;
};

__device__ __forceinline__ float Tab(const void *tab, int64_t idx, bool tabFloat, bool bf16)
{
    return tabFloat ? reinterpret_cast<const float *>(tab)[idx] : Load16(tab, idx, bf16);
}

// Eight consecutive table entries from a 16-byte aligned position.
template <bool BF16, bool TAB_FLOAT> __device__ __forceinline__ void Tab8(const void *tab, int64_t idx, float (&out)[8])
{
    if constexpr (TAB_FLOAT) {
        const float4 lo = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(tab) + idx);
        const float4 hi = *reinterpret_cast<const float4 *>(reinterpret_cast<const float *>(tab) + idx + 4);
        out[0] = lo.x; out[1] = lo.y; out[2] = lo.z; out[3] = lo.w;
        out[4] = hi.x; out[5] = hi.y; out[6] = hi.z; out[7] = hi.w;
    } else {
        const uint4 v = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(tab) + idx);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const uint16_t h = static_cast<uint16_t>(w[e >> 1] >> (16 * (e & 1)));
            out[e] = BF16 ? Bf16ToFloat(h) : HalfBitsToFloat(h);
        }
    }
}

// Table row of a token: its own index, or its position inside its sequence (-1: the token lies
// past the last sequence, or its position past the table).
__device__ __forceinline__ int64_t TableRow(const RopeArgs &a, int64_t token)
{
    if (a.cosFormat == 0) {
        return token < a.cosRows ? token : -1;
    }
    int64_t begin = 0;
    for (int b = 0; b < a.batch; ++b) {
        const int64_t len = a.seqLens[b];
        if (token < begin + len) {
            const int64_t pos = token - begin;
            return pos < a.cosRows ? pos : -1;
        }
        begin += len;
    }
    return -1;
}

// PIECE = 8: 16-byte pieces (stride a multiple of 8 channels); PIECE = 1: single elements.
template <int PIECE, bool BF16, bool TAB_FLOAT>
__global__ __launch_bounds__(ROPE_THREADS) void RopeKernel(const RopeArgs a)
{
    const int pairsPerToken = (a.hiddenQ + a.hiddenK) / 2 / PIECE;
    const int64_t total = a.numTokens * pairsPerToken;
    const int64_t step = static_cast<int64_t>(gridDim.x) * ROPE_THREADS;
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * ROPE_THREADS + threadIdx.x; idx < total; idx += step) {
        const int64_t token = idx / pairsPerToken;
        int pair = static_cast<int>(idx - token * pairsPerToken) * PIECE; // index among the first-half channels of the token
        const int64_t row = TableRow(a, token);
        if (row < 0) {
            continue;
        }
        const bool isK = pair >= a.hiddenQ / 2;
        if (isK) {
            pair -= a.hiddenQ / 2;
        }
        const int hidden = isK ? a.hiddenK : a.hiddenQ;
        // pair -> (chunk, offset inside the chunk's first half) -> channel
        const int chunk = pair / a.stride;
        const int lo = chunk * 2 * a.stride + (pair - chunk * a.stride);
        const int hi = lo + a.stride;
        const int loInUnit = lo % a.headDim;
        const int hiInUnit = loInUnit + a.stride;
        const uint16_t *src = (isK ? a.k : a.q) + token * hidden;
        uint16_t *dst = (isK ? a.kOut : a.qOut) + token * hidden;
        const int64_t tab = row * a.headDim;
        if constexpr (PIECE == 8) {
            const uint4 xl = *reinterpret_cast<const uint4 *>(src + lo);
            const uint4 xh = *reinterpret_cast<const uint4 *>(src + hi);
            const uint32_t wl[4] = {xl.x, xl.y, xl.z, xl.w}, wh[4] = {xh.x, xh.y, xh.z, xh.w};
            float cl[8], sl[8], ch[8], sh[8];
            Tab8<BF16, TAB_FLOAT>(a.cosTab, tab + loInUnit, cl);
            Tab8<BF16, TAB_FLOAT>(a.sinTab, tab + loInUnit, sl);
            Tab8<BF16, TAB_FLOAT>(a.cosTab, tab + hiInUnit, ch);
            Tab8<BF16, TAB_FLOAT>(a.sinTab, tab + hiInUnit, sh);
            uint32_t ol[4], oh[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float rl[2], rh[2];
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const uint16_t bl = static_cast<uint16_t>(wl[e] >> (16 * h)), bh = static_cast<uint16_t>(wh[e] >> (16 * h));
                    const float vl = BF16 ? Bf16ToFloat(bl) : HalfBitsToFloat(bl);
                    const float vh = BF16 ? Bf16ToFloat(bh) : HalfBitsToFloat(bh);
                    const int c = 2 * e + h;
                    // two products and a sum, each rounded: no fused multiply-add, as in the golden
                    rl[h] = __fadd_rn(__fmul_rn(vl, cl[c]), __fmul_rn(-vh, sl[c]));
                    rh[h] = __fadd_rn(__fmul_rn(vh, ch[c]), __fmul_rn(vl, sh[c]));
                }
                ol[e] = (BF16 ? FloatToBf16(rl[0]) : FloatToHalfBits(rl[0])) |
                        (static_cast<uint32_t>(BF16 ? FloatToBf16(rl[1]) : FloatToHalfBits(rl[1])) << 16);
                oh[e] = (BF16 ? FloatToBf16(rh[0]) : FloatToHalfBits(rh[0])) |
                        (static_cast<uint32_t>(BF16 ? FloatToBf16(rh[1]) : FloatToHalfBits(rh[1])) << 16);
            }
            *reinterpret_cast<uint4 *>(dst + lo) = uint4{ol[0], ol[1], ol[2], ol[3]};
            *reinterpret_cast<uint4 *>(dst + hi) = uint4{oh[0], oh[1], oh[2], oh[3]};
        } else {
            const float vl = Load16(src, lo, BF16), vh = Load16(src, hi, BF16);
            const float rl = __fadd_rn(__fmul_rn(vl, Tab(a.cosTab, tab + loInUnit, TAB_FLOAT, BF16)),
                                       __fmul_rn(-vh, Tab(a.sinTab, tab + loInUnit, TAB_FLOAT, BF16)));
            const float rh = __fadd_rn(__fmul_rn(vh, Tab(a.cosTab, tab + hiInUnit, TAB_FLOAT, BF16)),
                                       __fmul_rn(vl, Tab(a.sinTab, tab + hiInUnit, TAB_FLOAT, BF16)));
            Store16(dst, lo, rl, BF16);
            Store16(dst, hi, rh, BF16);
        }
    }
}

template <int PIECE> void LaunchRope(const RopeArgs &a, bool bf16, bool tabFloat, unsigned grid, hipStream_t s)
{
    if (tabFloat) {
        RopeKernel<PIECE, false, true><<<grid, ROPE_THREADS, 0, s>>>(a); // fp32 tables go with fp16 rows only
    } else if (bf16) {
        RopeKernel<PIECE, true, false><<<grid, ROPE_THREADS, 0, s>>>(a);
    } else {
        RopeKernel<PIECE, false, false><<<grid, ROPE_THREADS, 0, s>>>(a);
    }
}

bool Aligned16(const void *p)
{
    return (reinterpret_cast<uintptr_t>(p) & 15) == 0;
}

} // namespace
} // namespace atbmi

using namespace atbmi;

extern "C" int atbmi_rope(const void *q, const void *k, const void *cosTable, const void *sinTable,
                          const int32_t *seqLens, void *qOut, void *kOut, int64_t numTokens, int64_t hiddenQ,
                          int64_t hiddenK, int64_t headDim, int64_t tableRows, int64_t batch, int32_t rotaryCoeff,
                          int32_t cosFormat, int32_t dtype, int32_t tableIsFloat, void *stream)
{
    if (!q || !k || !cosTable || !sinTable || !qOut || !kOut) {
        return Fail(ERR_INVALID_PARAM, "rope: q, k, cos, sin and the outputs must be non-null");
    }
    if (dtype != ATBMI_F16 && dtype != ATBMI_BF16) {
        return Fail(ERR_INVALID_PARAM, "rope: q and k must be fp16 or bf16");
    }
    if (tableIsFloat && dtype != ATBMI_F16) {
        return Fail(ERR_INVALID_PARAM, "rope: fp32 cos / sin tables go with fp16 rows only");
    }
    if (numTokens < 0 || hiddenQ <= 0 || hiddenK <= 0 || headDim <= 0 || tableRows < 0 || batch < 0 ||
        hiddenQ > (1 << 24) || hiddenK > (1 << 24) || batch > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "rope: bad extents");
    }
    if (rotaryCoeff < 2 || rotaryCoeff % 2 != 0 || headDim % rotaryCoeff != 0) {
        return Fail(ERR_INVALID_PARAM, "rope: rotaryCoeff %d must be even and divide the table row size %lld",
                    rotaryCoeff, (long long)headDim);
    }
    if (hiddenQ % headDim != 0 || hiddenK % headDim != 0) {
        return Fail(ERR_INVALID_PARAM, "rope: row sizes %lld / %lld must be multiples of the table row size %lld",
                    (long long)hiddenQ, (long long)hiddenK, (long long)headDim);
    }
    if (cosFormat != 0 && cosFormat != 1) {
        return Fail(ERR_INVALID_PARAM, "rope: cosFormat must be 0 or 1, got %d", cosFormat);
    }
    if (cosFormat == 1 && (!seqLens || batch == 0)) {
        return Fail(ERR_INVALID_PARAM, "rope: cosFormat 1 needs the sequence lengths");
    }
    if (numTokens == 0) {
        return OK;
    }
    RopeArgs a;
    a.q = static_cast<const uint16_t *>(q);
    a.k = static_cast<const uint16_t *>(k);
    a.cosTab = cosTable;
    a.sinTab = sinTable;
    a.seqLens = seqLens;
    a.qOut = static_cast<uint16_t *>(qOut);
    a.kOut = static_cast<uint16_t *>(kOut);
    a.numTokens = numTokens;
    a.cosRows = tableRows;
    a.hiddenQ = static_cast<int32_t>(hiddenQ);
    a.hiddenK = static_cast<int32_t>(hiddenK);
    a.headDim = static_cast<int32_t>(headDim);
    a.stride = static_cast<int32_t>(headDim / rotaryCoeff);
    a.batch = static_cast<int32_t>(batch);
    a.cosFormat = cosFormat;
    const bool wide = a.stride % 8 == 0 && Aligned16(q) && Aligned16(k) && Aligned16(qOut) && Aligned16(kOut) &&
                      Aligned16(cosTable) && Aligned16(sinTable);
    const int piece = wide ? 8 : 1;
    const int64_t total = numTokens * ((hiddenQ + hiddenK) / 2 / piece);
    const unsigned grid = static_cast<unsigned>(std::min<int64_t>((total + ROPE_THREADS - 1) / ROPE_THREADS, 1 << 20));
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (wide) {
        LaunchRope<8>(a, dtype == ATBMI_BF16, tableIsFloat != 0, grid, s);
    } else {
        LaunchRope<1>(a, dtype == ATBMI_BF16, tableIsFloat != 0, grid, s);
    }
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}
