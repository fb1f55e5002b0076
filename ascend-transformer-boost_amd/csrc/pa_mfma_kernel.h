// MFMA paged decode-attention kernel for gfx950 (MI355X).
//
// Work decomposition
//   One workgroup (4 waves) = one KV chunk of one sequence, one KV head, one
//   tile of up to 16 query heads. The waves take 32-token steps of the chunk
//   round-robin and never synchronise inside the loop: each wave keeps its own
//   online-softmax state and its own K/V tile in LDS; the four states are
//   merged once at the end.
//
// Data path per wave and step (32 tokens)
//   HBM -> VGPR : the 32 K rows and 32 V rows of this KV head, 16 bytes per
//                 lane and consecutive lanes on consecutive addresses, so every
//                 row is read as whole 128-byte lines exactly once. The loads
//                 of step i+1 are issued before step i is computed.
//   VGPR -> LDS : rows are written row-major with a padded pitch (int8 rows
//                 are widened to fp16 on the way: x ^ 0x80 is spliced under
//                 the exponent 0x6400 and 1152 is subtracted, which is exact).
//   QK^T        : S^T[token, head] = K . Q^T on v_mfma_f32_16x16x32. K is the A
//                 operand (ds_read_b128 per lane), Q^T stays in registers as B.
//                 The accumulator then holds 4 consecutive tokens of one head
//                 per lane, which is exactly the B-operand layout of the next
//                 MFMA, so P never moves between lanes.
//   softmax     : base-2 online softmax; the row maximum needs two cross-lane
//                 exchanges (lanes l, l^16, l^32, l^48 hold one head).
//   PV          : O^T[d, head] += V^T . P^T, V^T read from the row-major LDS
//                 tile with the transposing ds_read_b64_tr_b16.
//
// int8 caches: the per-channel K descale is folded into Q once (q' = q * s_k),
// K offsets shift every score of a head by the same constant and cancel in the
// softmax, V is accumulated in integer units and (acc + off_v) * s_v is applied
// when the final row is written.
#ifndef ATBMI_PA_MFMA_KERNEL_H
#define ATBMI_PA_MFMA_KERNEL_H
#include "pa_internal.h"

namespace atbmi {
namespace mfma {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int STEP = PA_MFMA_STEP;   // tokens per wave step
constexpr int NW = PA_MFMA_WAVES;    // waves per workgroup
constexpr int HT = PA_MFMA_HEAD_TILE;
constexpr int K_PAD = 8;             // halves of padding per K tile row (16 B)
constexpr int V_PAD = 16;            // halves of padding per V tile row (32 B)

template <bool BF16> __device__ __forceinline__ f32x4 Mma(u32x4 a, u32x4 b, f32x4 c)
{
    if constexpr (BF16) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b),
                                                       c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c,
                                                      0, 0, 0);
    }
}

template <bool BF16> __device__ __forceinline__ uint32_t Pack2(float lo, float hi)
{
    if constexpr (BF16) {
        bf16x2 v = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
        return __builtin_bit_cast(uint32_t, v);
    } else {
        f16x2 v = {static_cast<_Float16>(lo), static_cast<_Float16>(hi)};
        return __builtin_bit_cast(uint32_t, v);
    }
}

__device__ __forceinline__ float Unpack(uint32_t word, int half, bool bf16)
{
    const uint16_t bits = static_cast<uint16_t>(half ? (word >> 16) : (word & 0xffffu));
    return bf16 ? Bf16ToFloat(bits) : HalfBitsToFloat(bits);
}

// 4 int8 in one dword -> 4 fp16 in two dwords, exact.
__device__ __forceinline__ u32x2 Int8x4ToHalf(uint32_t w)
{
    const uint32_t x = w ^ 0x80808080u;                       // bytes now hold value + 128
    const uint32_t e = 0x64646464u;                           // fp16 high byte 0x64: 0x64xx = 1024 + xx
    const uint32_t a = __builtin_amdgcn_perm(e, x, 0x04010400u); // {x.b0, 0x64, x.b1, 0x64}
    const uint32_t b = __builtin_amdgcn_perm(e, x, 0x04030402u); // {x.b2, 0x64, x.b3, 0x64}
    const f16x2 bias = {static_cast<_Float16>(1152.0f), static_cast<_Float16>(1152.0f)};
    u32x2 r;
    r[0] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, a) - bias);
    r[1] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, b) - bias);
    return r;
}

// 16 int8 (one 16-byte piece) -> 16 fp16 (two 16-byte pieces).
__device__ __forceinline__ void WidenPiece(u32x4 piece, u32x4 &lo, u32x4 &hi)
{
    const u32x2 a = Int8x4ToHalf(piece[0]);
    const u32x2 b = Int8x4ToHalf(piece[1]);
    const u32x2 c = Int8x4ToHalf(piece[2]);
    const u32x2 d = Int8x4ToHalf(piece[3]);
    lo = u32x4{a[0], a[1], b[0], b[1]};
    hi = u32x4{c[0], c[1], d[0], d[1]};
}

__device__ __forceinline__ u32x4 LoadGlobal16(const void *p)
{
    return *reinterpret_cast<const u32x4 *>(p);
}

// LDS bytes one workgroup needs.
template <bool KV8, int D, int DV, bool MLA> constexpr int LdsBytes()
{
    constexpr int kTile = STEP * (D + K_PAD) * 2;
    constexpr int vTile = MLA ? 0 : STEP * (DV + V_PAD) * 2;
    constexpr int tiles = NW * (kTile + vTile);
    constexpr int merge = NW * HT * (DV + 4) * 4 + 2 * NW * HT * 4;
    return tiles > merge ? tiles : merge;
}

// BF16: MFMA operand type (bf16 when the cache is bf16, fp16 otherwise).
// KV8 : int8 cache rows. MLA: V is the first DV channels of the K row.
// PF  : keep the next step's rows in registers while computing this one.
template <bool BF16, bool KV8, int D, int DV, bool MLA, bool PF>
__global__ __launch_bounds__(NW *WAVE) void PaMfmaKernel(const PaArgs a, const int numStreams)
{
    static_assert(D % 32 == 0 && DV % 16 == 0, "head sizes must fit the MFMA tiles");
    static_assert(!KV8 || DV % 32 == 0, "int8 rows are staged 16 channels at a time");
    static_assert(!(MLA && KV8), "combined cache is 16-bit only");
    constexpr int KP = D + K_PAD;                 // K tile pitch in halves
    constexpr int VP = MLA ? KP : DV + V_PAD;     // V tile pitch in halves
    constexpr int K_TILE_BYTES = STEP * KP * 2;
    constexpr int V_TILE_BYTES = MLA ? 0 : STEP * VP * 2;
    constexpr int NQ = D / 32;                    // QK MFMAs per 16-token sub-tile
    constexpr int NO = DV / 16;                   // PV MFMAs (output tiles of 16 channels)
    constexpr int ESZ = KV8 ? 1 : 2;              // bytes per cache element
    constexpr int KPR = D * ESZ / 16;             // 16-byte pieces per K row
    constexpr int VPR = DV * ESZ / 16;
    constexpr int NKP = STEP * KPR / WAVE;        // K pieces per lane and step
    constexpr int NVP = MLA ? 0 : STEP * VPR / WAVE;
    static_assert((STEP * KPR) % WAVE == 0 && (MLA || (STEP * VPR) % WAVE == 0), "pieces must split evenly");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    // blockIdx -> (stream = work item x KV head, head tile). The head tiles of
    // one stream read the same K/V rows: they are placed 8 workgroups apart so
    // that they run on the same XCD (workgroups go to XCDs round-robin) and
    // share its L2.
    const int headTiles = (a.groupSize + HT - 1) / HT;
    const int bx = blockIdx.x;
    const int octet = bx / (8 * headTiles);
    const int within = bx % (8 * headTiles);
    const int ht = within / 8;
    const int stream = octet * 8 + (within % 8);
    if (stream >= numStreams) {
        return;
    }
    const int g = stream % a.G;
    const PaWorkItem it = a.items[stream / a.G];

    const int lane = threadIdx.x % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int n = lane & 15;  // head (B operand / accumulator column), token or channel (A operand row)
    const int kg = lane >> 4; // k-group: which 8 contraction values / 4 accumulator rows this lane holds
    const bool qBf16 = a.qIsBf16 != 0;
    const int h0 = g * a.groupSize + ht * HT;
    const int nh = min(HT, a.groupSize - ht * HT);

    unsigned char *kTile = smem + wave * (K_TILE_BYTES + V_TILE_BYTES);
    unsigned char *vTile = MLA ? kTile : kTile + K_TILE_BYTES;

    // ---- Q^T as B operand: lane (n, kg) holds q[h0+n][32j + 8kg .. +8) for j < NQ
    u32x4 qreg[NQ];
    {
        const bool plain = !KV8 && a.qScale == 0.0f; // raw bits are already the operand
        const uint16_t *qrow =
            reinterpret_cast<const uint16_t *>(a.q) + (static_cast<int64_t>(it.qRow) * a.H + h0 + n) * D;
#pragma unroll
        for (int j = 0; j < NQ; ++j) {
            const int d0 = j * 32 + kg * 8;
            u32x4 raw = {0u, 0u, 0u, 0u};
            if (n < nh) {
                raw = LoadGlobal16(qrow + d0);
            }
            if (!plain) {
                float f[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    f[e] = Unpack(raw[e >> 1], e & 1, qBf16);
                    if (a.qScale != 0.0f) {
                        f[e] *= a.qScale;
                        f[e] = qBf16 ? Bf16ToFloat(FloatToBf16(f[e])) : HalfBitsToFloat(FloatToHalfBits(f[e]));
                    }
                    if (KV8) {
                        f[e] *= a.kScale[g * D + d0 + e];
                    }
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    raw[e] = Pack2<BF16>(f[2 * e], f[2 * e + 1]);
                }
            }
            qreg[j] = raw;
        }
    }

    constexpr float LOG2E = 1.4426950408889634f;
    const float scale2 = a.qkScale * LOG2E;
    float m = -INFINITY; // running maximum (base-2 exponent units) of head n
    float l = 0.0f;      // this lane's share of the running denominator
    f32x4 acc[NO];
#pragma unroll
    for (int i = 0; i < NO; ++i) {
        acc[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }

    const int32_t *table = a.tables + static_cast<int64_t>(it.seq) * a.maxBlocksPerSeq;
    const unsigned char *kcBase = reinterpret_cast<const unsigned char *>(a.kc);
    const unsigned char *vcBase = reinterpret_cast<const unsigned char *>(a.vc);

    // Issues the loads of the 32 rows starting at token t; rows at or past
    // tokEnd come back as zeros and their block-table entries are not read.
    auto loadStep = [&](int t, u32x4 *kp, u32x4 *vp) {
        int64_t rowBase[2];
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            const int ts = t + 16 * s;
            rowBase[s] = 0;
            if (ts < it.tokEnd) {
                rowBase[s] = static_cast<int64_t>(table[ts / a.blockSize]) * a.blockSize + (ts % a.blockSize);
            }
        }
#pragma unroll
        for (int i = 0; i < NKP; ++i) {
            const int p = i * WAVE + lane;
            const int row = p / KPR;
            const int col = p % KPR;
            u32x4 v = {0u, 0u, 0u, 0u};
            if (t + row < it.tokEnd) {
                const int64_t r = rowBase[row >> 4] + (row & 15);
                v = LoadGlobal16(kcBase + (r * a.kRowStride + static_cast<int64_t>(g) * D) * ESZ + col * 16);
            }
            kp[i] = v;
        }
#pragma unroll
        for (int i = 0; i < NVP; ++i) {
            const int p = i * WAVE + lane;
            const int row = p / VPR;
            const int col = p % VPR;
            u32x4 v = {0u, 0u, 0u, 0u};
            if (t + row < it.tokEnd) {
                const int64_t r = rowBase[row >> 4] + (row & 15);
                v = LoadGlobal16(vcBase + (r * a.vRowStride + static_cast<int64_t>(g) * a.vHeadStride) * ESZ + col * 16);
            }
            vp[i] = v;
        }
    };

    // Writes staged rows into this wave's LDS tiles (int8 widened to fp16).
    auto storeStep = [&](const u32x4 *kp, const u32x4 *vp) {
#pragma unroll
        for (int i = 0; i < NKP; ++i) {
            const int p = i * WAVE + lane;
            const int row = p / KPR;
            const int col = p % KPR;
            if constexpr (KV8) {
                u32x4 lo, hi;
                WidenPiece(kp[i], lo, hi);
                u32x4 *dst = reinterpret_cast<u32x4 *>(kTile + row * (KP * 2) + col * 32);
                dst[0] = lo;
                dst[1] = hi;
            } else {
                *reinterpret_cast<u32x4 *>(kTile + row * (KP * 2) + col * 16) = kp[i];
            }
        }
#pragma unroll
        for (int i = 0; i < NVP; ++i) {
            const int p = i * WAVE + lane;
            const int row = p / VPR;
            const int col = p % VPR;
            if constexpr (KV8) {
                u32x4 lo, hi;
                WidenPiece(vp[i], lo, hi);
                u32x4 *dst = reinterpret_cast<u32x4 *>(vTile + row * (VP * 2) + col * 32);
                dst[0] = lo;
                dst[1] = hi;
            } else {
                *reinterpret_cast<u32x4 *>(vTile + row * (VP * 2) + col * 16) = vp[i];
            }
        }
    };

    constexpr int NKR = PF ? NKP : 1;
    constexpr int NVR = PF ? (NVP > 0 ? NVP : 1) : 1;
    u32x4 kStage[NKR];
    u32x4 vStage[NVR];

    const int tFirst = it.tokBegin + wave * STEP;
    if constexpr (PF) {
        if (tFirst < it.tokEnd) {
            loadStep(tFirst, kStage, vStage);
        }
    }

    for (int t = tFirst; t < it.tokEnd; t += NW * STEP) {
        if constexpr (PF) {
            storeStep(kStage, vStage);
            if (t + NW * STEP < it.tokEnd) {
                loadStep(t + NW * STEP, kStage, vStage);
            }
        } else {
            // Large rows: stage a few pieces at a time to bound register use.
            int64_t rowBase[2];
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const int ts = t + 16 * s;
                rowBase[s] = 0;
                if (ts < it.tokEnd) {
                    rowBase[s] = static_cast<int64_t>(table[ts / a.blockSize]) * a.blockSize + (ts % a.blockSize);
                }
            }
            constexpr int BATCH = 6;
            static_assert(!KV8, "the unstaged path handles 16-bit rows only");
#pragma unroll
            for (int i0 = 0; i0 < NKP; i0 += BATCH) {
                u32x4 tmp[BATCH];
#pragma unroll
                for (int b = 0; b < BATCH; ++b) {
                    const int i = i0 + b;
                    tmp[b] = u32x4{0u, 0u, 0u, 0u};
                    if (i < NKP) {
                        const int p = i * WAVE + lane;
                        const int row = p / KPR;
                        const int col = p % KPR;
                        if (t + row < it.tokEnd) {
                            const int64_t r = rowBase[row >> 4] + (row & 15);
                            tmp[b] = LoadGlobal16(kcBase + (r * a.kRowStride + static_cast<int64_t>(g) * D) * 2 + col * 16);
                        }
                    }
                }
#pragma unroll
                for (int b = 0; b < BATCH; ++b) {
                    const int i = i0 + b;
                    if (i < NKP) {
                        const int p = i * WAVE + lane;
                        *reinterpret_cast<u32x4 *>(kTile + (p / KPR) * (KP * 2) + (p % KPR) * 16) = tmp[b];
                    }
                }
            }
#pragma unroll
            for (int i0 = 0; i0 < NVP; i0 += BATCH) {
                u32x4 tmp[BATCH];
#pragma unroll
                for (int b = 0; b < BATCH; ++b) {
                    const int i = i0 + b;
                    tmp[b] = u32x4{0u, 0u, 0u, 0u};
                    if (i < NVP) {
                        const int p = i * WAVE + lane;
                        const int row = p / VPR;
                        const int col = p % VPR;
                        if (t + row < it.tokEnd) {
                            const int64_t r = rowBase[row >> 4] + (row & 15);
                            tmp[b] = LoadGlobal16(vcBase + (r * a.vRowStride + static_cast<int64_t>(g) * a.vHeadStride) * 2 + col * 16);
                        }
                    }
                }
#pragma unroll
                for (int b = 0; b < BATCH; ++b) {
                    const int i = i0 + b;
                    if (i < NVP) {
                        const int p = i * WAVE + lane;
                        *reinterpret_cast<u32x4 *>(vTile + (p / VPR) * (VP * 2) + (p % VPR) * 16) = tmp[b];
                    }
                }
            }
        }
        // The tile is private to this wave: LDS executes a wave's accesses in
        // order, only the compiler has to be kept from moving reads above writes.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        // ---- S^T = K . Q^T for the two 16-token sub-tiles
        f32x4 s[2];
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            s[sub] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            const unsigned char *krow = kTile + (sub * 16 + n) * (KP * 2) + kg * 16;
#pragma unroll
            for (int j = 0; j < NQ; ++j) {
                const u32x4 kop = *reinterpret_cast<const u32x4 *>(krow + j * 64);
                s[sub] = Mma<BF16>(kop, qreg[j], s[sub]);
            }
        }

        // ---- online softmax in base 2; lane holds tokens t + 16 sub + 4 kg + r of head n
        float x[8];
        float mloc = -INFINITY;
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int tok = t + sub * 16 + kg * 4 + r;
                const float v = tok < it.tokEnd ? s[sub][r] * scale2 : -INFINITY;
                x[sub * 4 + r] = v;
                mloc = fmaxf(mloc, v);
            }
        }
        mloc = fmaxf(mloc, __shfl_xor(mloc, 16, WAVE));
        mloc = fmaxf(mloc, __shfl_xor(mloc, 32, WAVE));
        const float mNew = fmaxf(m, mloc); // finite: every step holds at least one valid token
        const float corr = exp2f(m - mNew);
        m = mNew;
        float psum = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            x[e] = exp2f(x[e] - mNew);
            psum += x[e];
        }
        l = l * corr + psum;
#pragma unroll
        for (int i = 0; i < NO; ++i) {
            acc[i] *= corr;
        }
        u32x4 pop; // P^T as B operand: k = {sub 0: r 0..3, sub 1: r 0..3}
        pop[0] = Pack2<BF16>(x[0], x[1]);
        pop[1] = Pack2<BF16>(x[2], x[3]);
        pop[2] = Pack2<BF16>(x[4], x[5]);
        pop[3] = Pack2<BF16>(x[6], x[7]);

        // ---- O^T += V^T . P^T. The transposing read hands lane (n, kg) the four
        // tokens 4kg..4kg+3 of channel 16 i + n when lane (n, kg) points at
        // token 4kg + n/4, channels 16 i + 4 (n%4) .. +4.
        const unsigned char *vrow = vTile + (kg * 4 + (n >> 2)) * (VP * 2) + (n & 3) * 8;
#pragma unroll
        for (int i = 0; i < NO; ++i) {
            const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) i16x4 *)(vrow + i * 32));
            const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) i16x4 *)(vrow + 16 * (VP * 2) + i * 32));
            u32x4 vop;
            const u32x2 lo2 = __builtin_bit_cast(u32x2, lo);
            const u32x2 hi2 = __builtin_bit_cast(u32x2, hi);
            vop[0] = lo2[0];
            vop[1] = lo2[1];
            vop[2] = hi2[0];
            vop[3] = hi2[1];
            acc[i] = Mma<BF16>(vop, pop, acc[i]);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }

    // ---- merge the four waves
    l += __shfl_xor(l, 16, WAVE);
    l += __shfl_xor(l, 32, WAVE);
    __syncthreads(); // every wave is done with its tiles; the space is reused
    constexpr int OP = DV + 4; // floats per (wave, head) row of the merge area
    float *mergeO = reinterpret_cast<float *>(smem);
    float *mergeM = mergeO + NW * HT * OP;
    float *mergeL = mergeM + NW * HT;
#pragma unroll
    for (int i = 0; i < NO; ++i) {
        *reinterpret_cast<f32x4 *>(mergeO + (wave * HT + n) * OP + i * 16 + kg * 4) = acc[i];
    }
    if (kg == 0) {
        mergeM[wave * HT + n] = m;
        mergeL[wave * HT + n] = l;
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < HT * DV; idx += NW * WAVE) {
        const int hh = idx / DV;
        const int d = idx % DV;
        if (hh >= nh) {
            continue;
        }
        float mx = -INFINITY;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            mx = fmaxf(mx, mergeM[w * HT + hh]);
        }
        float den = 0.0f;
        float num = 0.0f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            const float wgt = exp2f(mergeM[w * HT + hh] - mx); // 0 for a wave that saw no token
            den += wgt * mergeL[w * HT + hh];
            num += wgt * mergeO[(w * HT + hh) * OP + d];
        }
        float o = num / den;
        const int h = h0 + hh;
        if (it.direct) {
            if (KV8) {
                const int c = g * DV + d;
                o = (o + (a.vOff ? static_cast<float>(a.vOff[c]) : 0.0f)) * a.vScale[c];
            }
            Store16(a.out, (static_cast<int64_t>(it.qRow) * a.H + h) * DV + d, o, qBf16);
        } else {
            const int64_t ph = static_cast<int64_t>(it.partialBase) * a.H + h;
            a.partO[ph * DV + d] = o;
            if (d == 0) {
                a.partLse[ph] = mx + log2f(den);
            }
        }
    }
}

template <bool BF16, bool KV8, int D, int DV, bool MLA, bool PF>
int Launch(const PaArgs &args, int numItems, hipStream_t stream)
{
    auto kernel = PaMfmaKernel<BF16, KV8, D, DV, MLA, PF>;
    constexpr int lds = LdsBytes<KV8, D, DV, MLA>();
    static bool configured = false; // one attribute call per instantiation and process
    if (!configured) {
        ATBMI_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        configured = true;
    }
    const int headTiles = (args.groupSize + HT - 1) / HT;
    const int64_t streams = static_cast<int64_t>(numItems) * args.G;
    const int64_t grid = (streams + 7) / 8 * 8 * headTiles;
    if (grid <= 0 || grid > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: grid of %lld workgroups is out of range", (long long)grid);
    }
    kernel<<<static_cast<unsigned>(grid), NW * WAVE, lds, stream>>>(args, static_cast<int>(streams));
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}

} // namespace mfma
} // namespace atbmi
#endif
