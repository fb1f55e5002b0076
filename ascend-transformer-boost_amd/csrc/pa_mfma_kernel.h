// MFMA paged decode-attention kernel for gfx950 (MI355X).
//
// Work decomposition ("stream" split-KV)
//   The KV rows of all sequences, in 32-token steps, form one linear step
//   space. It is cut into equal contiguous ranges, one per wave and KV head:
//   every wave gets the same number of steps (+-1) whatever the length
//   distribution of the batch, so there is no tail of half-empty rounds and no
//   per-chunk workgroup launch. A range that crosses a sequence boundary makes
//   the wave finish one (partial or complete) attention row and start the next.
//   The waves of a workgroup cover the KV heads of the SAME token range, so a
//   CU pulls whole contiguous [token][head][channel] cache rows out of HBM.
//   Waves never synchronise: each owns its K/V tile in LDS and its softmax
//   state; rows that span several ranges are merged by the reduce kernel.
//
// Data path per wave and step (32 tokens)
//   HBM -> VGPR : the 32 K rows and 32 V rows of this KV head, 16 bytes per
//                 lane and consecutive lanes on consecutive addresses, so every
//                 row is read as whole 128-byte lines exactly once. The loads
//                 of step i+1 are issued before step i is computed.
//   VGPR -> LDS : rows are written row-major with a padded pitch (int8 rows
//                 are widened to fp16 on the way: x ^ 0x80 spliced under the
//                 exponent byte 0x64, i.e. value + 1152, exactly).
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
constexpr int HT = PA_MFMA_HEAD_TILE;
constexpr int K_PAD = 8;             // halves of padding per K tile row (16 B)
constexpr int V_PAD = 16;            // halves of padding per V tile row (32 B)

// Four consecutive per-channel descales from channel c on. stride 1: a plain float array; stride 2:
// the low halves of 8-byte packed entries. Read as whole 16-byte vectors either way: one address per
// four channels keeps the many descale loads of a row from crowding the register file.
__device__ __forceinline__ f32x4 LoadScale4(const float *scales, int c, int stride)
{
    typedef float Vec4 __attribute__((ext_vector_type(4), aligned(4)));
    if (stride == 1) {
        const Vec4 v = *reinterpret_cast<const Vec4 *>(scales + c);
        return f32x4{v[0], v[1], v[2], v[3]};
    }
    const Vec4 lo = *reinterpret_cast<const Vec4 *>(scales + 2 * c);
    const Vec4 hi = *reinterpret_cast<const Vec4 *>(scales + 2 * c + 4);
    return f32x4{lo[0], lo[2], hi[0], hi[2]};
}

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

// int8 rows enter the matrix cores as fp16 numbers equal to value + INT8_BIAS:
// x ^ 0x80 (value + 128 as an unsigned byte) spliced under the fp16 high byte
// 0x64 reads as 1024 + (value + 128). The bias is never subtracted per element:
// in Q.K^T it adds the same constant to every score of a head, which the
// softmax cancels, and in P.V it adds INT8_BIAS times the sum of P, which is
// removed once per output element after the normalisation.
constexpr float INT8_BIAS = 1152.0f;

// 4 int8 in one dword -> 4 biased fp16 in two dwords.
__device__ __forceinline__ u32x2 Int8x4ToHalf(uint32_t w)
{
    const uint32_t x = w ^ 0x80808080u;
    const uint32_t e = 0x64646464u;
    u32x2 r;
    r[0] = __builtin_amdgcn_perm(e, x, 0x04010400u); // {x.b0, 0x64, x.b1, 0x64}
    r[1] = __builtin_amdgcn_perm(e, x, 0x04030402u); // {x.b2, 0x64, x.b3, 0x64}
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

// 2^x on the hardware unit directly: arguments here are <= 0 (or -inf) and a
// result below the normal range may flush to zero.
__device__ __forceinline__ float Exp2(float x)
{
    return __builtin_amdgcn_exp2f(x);
}

__device__ __forceinline__ u32x4 LoadGlobal16(const void *p)
{
    return *reinterpret_cast<const u32x4 *>(p);
}

// Cache rows are read once per call: the non-temporal hint keeps them from
// displacing anything in L2 / the memory-side cache, which is worth ~15% of
// HBM read bandwidth on this access pattern.
__device__ __forceinline__ u32x4 LoadStream16(const void *p)
{
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
}

// LDS bytes one wave needs for its K and V tiles.
template <int D, int DV, bool MLA> constexpr int WaveLdsBytes()
{
    constexpr int kTile = STEP * (D + K_PAD) * 2;
    constexpr int vTile = MLA ? 0 : STEP * (DV + V_PAD) * 2;
    return kTile + vTile;
}

__device__ __forceinline__ PaSeq PlanSeq(const PaStreamPlan &p, int i)
{
    return p.seqs ? p.seqs[i] : p.inlineSeqs[i];
}

// BF16: MFMA operand type (bf16 when the cache is bf16, fp16 otherwise).
// KV8 : int8 cache rows. MLA: V is the first DV channels of the K row.
// PF  : keep the next step's rows in registers while computing this one.
// NW  : waves per workgroup.
// SHARED: the waves of a workgroup are the query-head tiles of ONE KV head and token range (MLA with
//       many heads): the K tile is staged once per workgroup, double-buffered, and read by all waves.
// EXT : with the additive mask, the per-sequence log-N scale and several query tokens folded into one
//       tile. Calls that use none of them run the EXT = false build, which keeps those values out of
//       its registers (the int8 builds sit at the register limit of their occupancy).
template <bool BF16, bool KV8, int D, int DV, bool MLA, bool PF, int NW, bool SHARED, bool EXT>
__global__ __launch_bounds__(NW *WAVE) void PaMfmaKernel(const PaArgs a, const PaStreamPlan p)
{
    static_assert(D % 32 == 0 && DV % 16 == 0, "head sizes must fit the MFMA tiles");
    static_assert(!KV8 || DV % 32 == 0, "int8 rows are staged 16 channels at a time");
    static_assert(!(MLA && KV8), "combined cache is 16-bit only");
    static_assert(!SHARED || MLA, "the shared-tile mode is built for the combined (MLA) cache");
    constexpr int KP = D + K_PAD;                 // K tile pitch in halves
    constexpr int VP = MLA ? KP : DV + V_PAD;     // V tile pitch in halves
    constexpr int K_TILE_BYTES = STEP * KP * 2;
    constexpr int NQ = D / 32;                    // QK MFMAs per 16-token sub-tile
    constexpr int NO = DV / 16;                   // PV MFMAs (output tiles of 16 channels)
    constexpr bool BIG = NQ > 8 || NO > 16;       // wide rows: operand fetch is pipelined by hand
    constexpr int KD = 2;                         // ... this many MFMA pairs ahead for K
    constexpr int VD = 3;                         // ... and this many MFMAs ahead for V
    constexpr int ESZ = KV8 ? 1 : 2;              // bytes per cache element
    constexpr int KPR = D * ESZ / 16;             // 16-byte pieces per K row
    constexpr int VPR = DV * ESZ / 16;
    constexpr int NKP = STEP * KPR / WAVE;        // K pieces per lane and step
    constexpr int NVP = MLA ? 0 : STEP * VPR / WAVE;
    static_assert((STEP * KPR) % WAVE == 0 && (MLA || (STEP * VPR) % WAVE == 0), "pieces must split evenly");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    // eight private-tile waves: the steps each wave has left, behind the tiles (see the step loop)
    constexpr bool BALANCED = NW == 8 && !SHARED;
    volatile int *stepsLeft = reinterpret_cast<volatile int *>(smem + NW * WaveLdsBytes<D, DV, MLA>());

    const int lane = threadIdx.x % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int n = lane & 15;  // head (B operand / accumulator column), token or channel (A operand row)
    const int kg = lane >> 4; // k-group: which 8 contraction values / 4 accumulator rows this lane holds
    const bool qBf16 = a.qIsBf16 != 0;

    // Workgroup -> (token range, group of virtual heads); wave -> (virtual head, slice of the range).
    // Workgroups go to the 8 XCDs round-robin; the head groups of one token range read the
    // same cache rows, so they sit 8 workgroup ids apart: same XCD, same L2, launched together.
    const int octet = blockIdx.x / (8 * p.headGroups);
    const int within = blockIdx.x % (8 * p.headGroups);
    const int hgIdx = within / 8;
    const int wgRange = octet * 8 + within % 8;
    if (wgRange >= p.numWgRanges) {
        return;
    }
    const int vh = hgIdx * p.headsPerWg + wave % p.headsPerWg;
    const int g = vh / p.headTiles;
    const int ht = vh % p.headTiles;
    const int wr = wgRange * p.tokenSlices + wave / p.headsPerWg;
    if (wr >= p.numWaveRanges) {
        return;
    }
    const int s0 = PaRangeBegin(wr, p.totalSteps, p.numWaveRanges);
    const int s1 = PaRangeBegin(wr + 1, p.totalSteps, p.numWaveRanges);
    if (s0 >= s1) {
        return;
    }
    const int h0 = g * a.groupSize + ht * HT;
    const int nhTile = min(HT, a.groupSize - ht * HT);

    unsigned char *kTile = SHARED ? smem : smem + wave * WaveLdsBytes<D, DV, MLA>();
    unsigned char *vTile = MLA ? kTile : kTile + K_TILE_BYTES;
    const unsigned char *kcBase = reinterpret_cast<const unsigned char *>(a.kc);
    const unsigned char *vcBase = reinterpret_cast<const unsigned char *>(a.vc);
    // Split latent layout (combined cache only): the last ropeDim channels of a key row come from a
    // cache of their own, those of a query row from a tensor of their own.
    const unsigned char *krBase = reinterpret_cast<const unsigned char *>(a.kRope);
    const int dn = MLA ? D - a.ropeDim : D;  // channels per row of q and of the key cache itself
    const int nopePieces = dn / 8;           // 16-byte pieces of a key row that the key cache holds
    // Address of piece `col` of the key row at cache slot r.
    auto keyPiece = [&](int64_t r, int col) -> const unsigned char * {
        if (MLA && a.nzShift > 0) {
            // fractal-NZ: slabs of blockSize x 16 channels; a 16-byte piece is half a slab row
            const int64_t blk = r >> a.nzShift;
            const int64_t off = r & ((1 << a.nzShift) - 1);
            if (col >= nopePieces) {
                const int c = col - nopePieces;
                return krBase + ((((blk * (a.ropeDim >> 4) + (c >> 1)) << a.nzShift) + off) * 16 + (c & 1) * 8) * 2;
            }
            return kcBase + ((((blk * (dn >> 4) + (col >> 1)) << a.nzShift) + off) * 16 + (col & 1) * 8) * 2;
        }
        if (MLA && col >= nopePieces) {
            return krBase + (r * a.ropeRowStride + static_cast<int64_t>(g) * a.ropeDim) * 2 + (col - nopePieces) * 16;
        }
        return kcBase + (r * a.kRowStride + static_cast<int64_t>(g) * a.kHeadStride) * ESZ + col * 16;
    };
    constexpr float LOG2E = 1.4426950408889634f;
    const float scale2 = a.qkScale * LOG2E;
    const uint32_t onePair = BF16 ? 0x3f803f80u : 0x3c003c00u; // {1.0, 1.0} in the operand type
    const u32x4 ones = {onePair, onePair, onePair, onePair};

    int seqIdx = p.firstSeq ? p.firstSeq[wgRange] : p.inlineFirst[wgRange];
    while (PlanSeq(p, seqIdx + 1).stepBegin <= s0) {
        ++seqIdx;
    }

    for (; seqIdx < p.numSeqs; ++seqIdx) {
        const PaSeq sq = PlanSeq(p, seqIdx);
        if (sq.stepBegin >= s1) {
            break;
        }
        const int seqEnd = PlanSeq(p, seqIdx + 1).stepBegin;
        const int segBegin = max(s0, sq.stepBegin);
        const int segEnd = min(s1, seqEnd);
        const int tokBegin = max(0, segBegin - sq.stepBegin - p.rowStartSteps) * STEP;
        const int tokEnd = min(sq.ctxLen, max(0, segEnd - sq.stepBegin - p.rowStartSteps) * STEP);
        const bool complete = segBegin == sq.stepBegin && segEnd == seqEnd;
        if (tokBegin >= tokEnd) {
            // the range ends inside the steps that stand for the start of the row (PaStreamPlan::rowStartSteps): the
            // merge kernel reads this range's slot like any other, so it must say "no tokens"
            const bool folded = EXT && p.foldTokens > 1;
            const int columns = folded ? sq.nTok * a.groupSize : nhTile;
            if (n < columns) {
                const int tok = folded ? n / a.groupSize : 0;
                const int head = h0 + (folded ? n - tok * a.groupSize : n);
                const int slot = 2 * wr + (segBegin == s0 ? 0 : 1);
                const int64_t ph = (static_cast<int64_t>(slot) * (EXT ? p.foldTokens : 1) + tok) * a.H + head;
#pragma unroll
                for (int i = 0; i < DV / 16; ++i) {
                    *reinterpret_cast<u32x2 *>(reinterpret_cast<uint16_t *>(a.partO) + ph * DV + i * 16 + kg * 4) =
                        u32x2{0u, 0u};
                }
                if (kg == 0) {
                    a.partLse[ph] = -INFINITY;
                }
            }
            continue;
        }
        // Column n of the tile is head h0 + n of the pass's query token, or, when the plan folds
        // several query tokens of a sequence into one tile (small GQA groups), head h0 + n % group
        // of its query token n / group.
        const bool fold = EXT && p.foldTokens > 1;
        int nh = nhTile;
        if (fold) {
            nh = sq.nTok * a.groupSize;
        }
        const int nc = EXT ? min(n, nh - 1) : n; // columns past the tile's end borrow its last one where they must read
        int colTok = 0, colHead = nc;
        if (fold) {
            colTok = nc / a.groupSize;
            colHead = nc - colTok * a.groupSize;
        }
        const int qRow = sq.qRow + colTok;
        // SCALE_TYPE_LOGN: a per-sequence factor on the score scale, indexed like the block tables
        const float scaleSeq = EXT && a.logN ? scale2 * a.logN[sq.tableRow] : scale2;
        // additive score bias of this column's query token and head
        const uint16_t *maskRow = nullptr;
        if (EXT && a.mask) {
            maskRow = reinterpret_cast<const uint16_t *>(a.mask) +
                      static_cast<int64_t>(sq.maskRow + colTok * a.maskRowStep) * a.maskBatchStride +
                      static_cast<int64_t>(h0 + colHead) * a.maskHeadStride;
        }

        // descale slice of this sequence: its KV head's, or, under head compression, the model KV head it stands for
        const int gs = EXT && a.descaleHeads > 0 ? sq.tableRow % a.descaleHeads : g;

        // ---- Q^T as B operand: lane (n, kg) holds q[column n][32j + 8kg .. +8) for j < NQ
        u32x4 qreg[NQ];
        {
            const int64_t qh = static_cast<int64_t>(qRow) * a.H + h0 + colHead;
            const uint16_t *qrow = reinterpret_cast<const uint16_t *>(a.q) + qh * dn;
            const uint16_t *qrope = reinterpret_cast<const uint16_t *>(a.qRope) + qh * a.ropeDim - dn;
#pragma unroll
            for (int j = 0; j < NQ; ++j) { // all loads first, so their latencies overlap
                qreg[j] = u32x4{0u, 0u, 0u, 0u};
                if (n < nh) {
                    qreg[j] = LoadGlobal16((MLA && j * 32 >= dn ? qrope : qrow) + j * 32 + kg * 8);
                }
            }
        }
        // The operand form of Q (the q pre-scale rounded in the query's type, the K descales of an int8 cache folded in).
        // Called behind the loads of the segment's first step, so that the waits in here overlap with those.
        auto prepareQ = [&]() {
            const bool plain = !KV8 && a.qScale == 0.0f; // raw bits are already the operand
            if (!plain) {
#pragma unroll
                for (int j = 0; j < NQ; ++j) {
                    const int d0 = j * 32 + kg * 8;
                    float f[8];
                    f32x4 ks[2] = {f32x4{1.0f, 1.0f, 1.0f, 1.0f}, f32x4{1.0f, 1.0f, 1.0f, 1.0f}};
                    if (KV8) {
                        ks[0] = LoadScale4(a.kScale, gs * D + d0, a.scaleStride);
                        ks[1] = LoadScale4(a.kScale, gs * D + d0 + 4, a.scaleStride);
                    }
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        f[e] = Unpack(qreg[j][e >> 1], e & 1, qBf16);
                        if (a.qScale != 0.0f) {
                            f[e] *= a.qScale;
                            f[e] = qBf16 ? Bf16ToFloat(FloatToBf16(f[e])) : HalfBitsToFloat(FloatToHalfBits(f[e]));
                        }
                        if (KV8) {
                            f[e] *= ks[e >> 2][e & 3];
                        }
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        qreg[j][e] = Pack2<BF16>(f[2 * e], f[2 * e + 1]);
                    }
                }
            }
        };

        float m = -INFINITY; // running maximum (base-2 exponent units) of head n
        f32x4 accL = {0.0f, 0.0f, 0.0f, 0.0f}; // running denominator of head n (the same in all four entries)
        f32x4 acc[NO];
#pragma unroll
        for (int i = 0; i < NO; ++i) {
            acc[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }

        const int32_t *table = a.tables + static_cast<int64_t>(sq.tableRow) * a.maxBlocksPerSeq;

        // Block ids of this segment, 64 at a time, one per lane: a step then gets
        // its block id with a cross-lane read instead of a dependent memory load.
        const int blocksNeeded = (tokEnd + a.blockSize - 1) / a.blockSize; // entries past this are never read
        int cacheBase = tokBegin / a.blockSize;
        int blkCache = (cacheBase + lane < blocksNeeded) ? table[cacheBase + lane] : 0;
        // The load cursor: block index and offset inside the block of the next
        // 16-token sub-tile to fetch (a sub-tile never straddles cache blocks).
        int curBlk = cacheBase;
        int curOff = tokBegin % a.blockSize;

        // Cache slot of the first token of the next two sub-tiles; advances the cursor.
        auto nextRows = [&](int64_t *rowBase) {
#pragma unroll
            for (int sub = 0; sub < 2; ++sub) {
                if (curBlk >= cacheBase + WAVE) {
                    cacheBase = curBlk;
                    blkCache = (cacheBase + lane < blocksNeeded) ? table[cacheBase + lane] : 0;
                }
                const int blk = __builtin_amdgcn_readlane(blkCache, curBlk - cacheBase);
                rowBase[sub] = static_cast<int64_t>(blk) * a.blockRows + curOff;
                curOff += 16;
                if (curOff >= a.blockSize) {
                    curOff = 0;
                    ++curBlk;
                }
            }
        };
        // Loads of a step. When the 16-byte pieces of a row divide the wave evenly,
        // load i of a full step covers whole consecutive rows of one sub-tile: its
        // address is a wave-uniform base plus a per-lane offset that never changes.
        // Otherwise (or in the last, partial step, where rows at or past tokEnd are
        // not touched and read as zeros) every lane computes its own row.
        constexpr bool K_UNIFORM = WAVE % KPR == 0;
        constexpr bool V_UNIFORM = !MLA && WAVE % VPR == 0;
        constexpr int K_RPL = K_UNIFORM ? WAVE / KPR : 1; // rows per load
        constexpr int V_RPL = V_UNIFORM ? WAVE / VPR : 1;
        const uint32_t laneOffK = static_cast<uint32_t>(
            (static_cast<int64_t>(lane / KPR) * a.kRowStride + static_cast<int64_t>(g) * a.kHeadStride) * ESZ +
            (lane % KPR) * 16);
        const uint32_t laneOffV = static_cast<uint32_t>(
            (static_cast<int64_t>(lane / VPR) * a.vRowStride + static_cast<int64_t>(g) * a.vHeadStride) * ESZ +
            (lane % VPR) * 16);
        auto loadK = [&](int t, const int64_t *rowBase, int i, bool full) -> u32x4 {
            if constexpr (K_UNIFORM) {
                if (full) {
                    const int row0 = i * K_RPL;
                    const unsigned char *base = kcBase + (rowBase[row0 >> 4] + (row0 & 15)) * a.kRowStride * ESZ;
                    return LoadStream16(base + laneOffK);
                }
            }
            const int pc = i * WAVE + lane;
            const int row = pc / KPR;
            const int col = pc % KPR;
            u32x4 v = {0u, 0u, 0u, 0u};
            if (full || t + row < tokEnd) {
                const int64_t r = rowBase[row >> 4] + (row & 15);
                v = LoadStream16(keyPiece(r, col));
            }
            return v;
        };
        auto loadV = [&](int t, const int64_t *rowBase, int i, bool full) -> u32x4 {
            if constexpr (V_UNIFORM) {
                if (full) {
                    const int row0 = i * V_RPL;
                    const unsigned char *base = vcBase + (rowBase[row0 >> 4] + (row0 & 15)) * a.vRowStride * ESZ;
                    return LoadStream16(base + laneOffV);
                }
            }
            const int pc = i * WAVE + lane;
            const int row = pc / VPR;
            const int col = pc % VPR;
            u32x4 v = {0u, 0u, 0u, 0u};
            if (full || t + row < tokEnd) {
                const int64_t r = rowBase[row >> 4] + (row & 15);
                v = LoadStream16(vcBase + (r * a.vRowStride + static_cast<int64_t>(g) * a.vHeadStride) * ESZ +
                                 col * 16);
            }
            return v;
        };
        // Writes one staged 16-byte piece into an LDS tile (int8 widened to fp16).
        auto storePiece = [&](unsigned char *tile, int pitchHalves, int piecesPerRow, int i, u32x4 piece) {
            const int pc = i * WAVE + lane;
            const int row = pc / piecesPerRow;
            const int col = pc % piecesPerRow;
            if constexpr (KV8) {
                u32x4 lo, hi;
                WidenPiece(piece, lo, hi);
                u32x4 *dst = reinterpret_cast<u32x4 *>(tile + row * (pitchHalves * 2) + col * 32);
                dst[0] = lo;
                dst[1] = hi;
            } else {
                *reinterpret_cast<u32x4 *>(tile + row * (pitchHalves * 2) + col * 16) = piece;
            }
        };

        constexpr int NKR = PF ? NKP : 1;
        constexpr int NVR = (PF && NVP > 0) ? NVP : 1;
        u32x4 kStage[NKR];
        u32x4 vStage[NVR];
        // Issues the loads of the step at token t into the stage registers.
        auto loadStage = [&](int t) {
            if constexpr (PF) {
                int64_t rowBase[2];
                nextRows(rowBase);
                if (t + STEP <= tokEnd) {
    #pragma unroll
                    for (int i = 0; i < NKP; ++i) {
                        kStage[i] = loadK(t, rowBase, i, true);
                    }
    #pragma unroll
                    for (int i = 0; i < NVP; ++i) {
                        vStage[i] = loadV(t, rowBase, i, true);
                    }
                } else {
    #pragma unroll
                    for (int i = 0; i < NKP; ++i) {
                        kStage[i] = loadK(t, rowBase, i, false);
                    }
    #pragma unroll
                    for (int i = 0; i < NVP; ++i) {
                        vStage[i] = loadV(t, rowBase, i, false);
                    }
                }
            }
        };
        if constexpr (PF && !SHARED) {
            loadStage(tokBegin);
        }
        prepareQ();

        // One 32-token step of attention for this wave's heads, on the tile at kT / vT.
        auto computeStep = [&](int t, const unsigned char *kT, const unsigned char *vT) {
                // The bias of this lane's 8 tokens is requested before the MFMAs and used after them.
                u32x2 bias[2] = {u32x2{0u, 0u}, u32x2{0u, 0u}};
                if (maskRow) {
#pragma unroll
                    for (int sub = 0; sub < 2; ++sub) {
                        const int tok0 = t + sub * 16 + kg * 4;
                        if (a.maskVec && tok0 + 4 <= a.maskLen) {
                            bias[sub] = *reinterpret_cast<const u32x2 *>(maskRow + tok0);
                        } else {
                            uint32_t h[4];
#pragma unroll
                            for (int r = 0; r < 4; ++r) {
                                h[r] = tok0 + r < a.maskLen ? maskRow[tok0 + r] : 0u;
                            }
                            bias[sub] = u32x2{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
                        }
                    }
                }
                // ---- S^T = K . Q^T for the two 16-token sub-tiles
                f32x4 s[2] = {f32x4{0.0f, 0.0f, 0.0f, 0.0f}, f32x4{0.0f, 0.0f, 0.0f, 0.0f}};
                const unsigned char *krow = kT + n * (KP * 2) + kg * 16;
                if constexpr (BIG) {
                    // Wide rows: operands are fetched two MFMAs ahead and the order is pinned,
                    // otherwise the scheduler hoists every LDS read and spills.
                    u32x4 ka[KD + 1], kb[KD + 1];
#pragma unroll
                    for (int j = 0; j < KD && j < NQ; ++j) {
                        ka[j] = *reinterpret_cast<const u32x4 *>(krow + j * 64);
                        kb[j] = *reinterpret_cast<const u32x4 *>(krow + 16 * (KP * 2) + j * 64);
                    }
#pragma unroll
                    for (int j = 0; j < NQ; ++j) {
                        if (j + KD < NQ) {
                            ka[(j + KD) % (KD + 1)] = *reinterpret_cast<const u32x4 *>(krow + (j + KD) * 64);
                            kb[(j + KD) % (KD + 1)] =
                                *reinterpret_cast<const u32x4 *>(krow + 16 * (KP * 2) + (j + KD) * 64);
                        }
                        s[0] = Mma<BF16>(ka[j % (KD + 1)], qreg[j], s[0]);
                        s[1] = Mma<BF16>(kb[j % (KD + 1)], qreg[j], s[1]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                } else {
#pragma unroll
                    for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
                        for (int j = 0; j < NQ; ++j) {
                            const u32x4 kop = *reinterpret_cast<const u32x4 *>(krow + sub * 16 * (KP * 2) + j * 64);
                            s[sub] = Mma<BF16>(kop, qreg[j], s[sub]);
                        }
                    }
                }

                // ---- online softmax in base 2; lane holds tokens t + 16 sub + 4 kg + r of head n
                float x[8];
    #pragma unroll
                for (int e = 0; e < 8; ++e) {
                    x[e] = s[e >> 2][e & 3];
                }
                if (EXT && a.razor) {
                    // per-slot score offsets of this lane's 8 tokens, added before the scale (a 16-token
                    // sub-tile lies in one block)
#pragma unroll
                    for (int sub = 0; sub < 2; ++sub) {
                        const int tok0 = t + sub * 16;
                        if (tok0 < tokEnd) {
                            const int64_t slot = static_cast<int64_t>(table[tok0 / a.blockSize]) * a.blockSize +
                                                 tok0 % a.blockSize + kg * 4;
#pragma unroll
                            for (int r = 0; r < 4; ++r) {
                                x[sub * 4 + r] += a.razor[slot + r];
                            }
                        }
                    }
                }
    #pragma unroll
                for (int e = 0; e < 8; ++e) {
                    x[e] *= scaleSeq;
                }
                if (maskRow) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        x[e] += Unpack(bias[e >> 2][(e >> 1) & 1], e & 1, qBf16) * LOG2E;
                    }
                }
                if (t + STEP > tokEnd) { // last step of the segment: mask the tokens past its end
    #pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const int tok = t + (e >> 2) * 16 + kg * 4 + (e & 3);
                        x[e] = tok < tokEnd ? x[e] : -INFINITY;
                    }
                }
                float mloc = fmaxf(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])), fmaxf(fmaxf(x[4], x[5]), fmaxf(x[6], x[7])));
                mloc = fmaxf(mloc, __shfl_xor(mloc, 16, WAVE));
                mloc = fmaxf(mloc, __shfl_xor(mloc, 32, WAVE));
                // without a mask mloc is finite from the first step on (every step holds a valid token);
                // a bias of -inf may leave a head without any token yet: m then stays -inf
                if (__builtin_amdgcn_ballot_w64(mloc > m) != 0) { // some head's maximum grew: rescale
                    const float mNew = fmaxf(m, mloc);
                    const float corr = EXT && mNew == -INFINITY ? 1.0f : Exp2(m - mNew);
                    m = mNew;
                    accL *= corr;
    #pragma unroll
                    for (int i = 0; i < NO; ++i) {
                        acc[i] *= corr;
                    }
                }
                const float mRef = EXT && m == -INFINITY ? 0.0f : m; // (-inf) - (-inf) would be NaN
    #pragma unroll
                for (int e = 0; e < 8; ++e) {
                    x[e] = Exp2(x[e] - mRef);
                }
                u32x4 pop; // P^T as B operand: k = {sub 0: r 0..3, sub 1: r 0..3}
                pop[0] = Pack2<BF16>(x[0], x[1]);
                pop[1] = Pack2<BF16>(x[2], x[3]);
                pop[2] = Pack2<BF16>(x[4], x[5]);
                pop[3] = Pack2<BF16>(x[6], x[7]);
                // The denominator is the sum of the rounded P that multiplies V, taken by
                // the matrix core itself from a row of ones: numerator and denominator
                // then see exactly the same weights.
                accL = Mma<BF16>(ones, pop, accL);

                // ---- O^T += V^T . P^T. The transposing read hands lane (n, kg) the four
                // tokens 4kg..4kg+3 of channel 16 i + n when lane (n, kg) points at
                // token 4kg + n/4, channels 16 i + 4 (n%4) .. +4.
                const unsigned char *vrow = vT + (kg * 4 + (n >> 2)) * (VP * 2) + (n & 3) * 8;
                auto readV = [&](int i) -> u32x4 {
                    const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (__attribute__((address_space(3))) i16x4 *)(vrow + i * 32));
                    const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (__attribute__((address_space(3))) i16x4 *)(vrow + 16 * (VP * 2) + i * 32));
                    const u32x2 lo2 = __builtin_bit_cast(u32x2, lo);
                    const u32x2 hi2 = __builtin_bit_cast(u32x2, hi);
                    return u32x4{lo2[0], lo2[1], hi2[0], hi2[1]};
                };
                if constexpr (BIG) {
                    u32x4 vop[VD + 1];
#pragma unroll
                    for (int i = 0; i < VD && i < NO; ++i) {
                        vop[i] = readV(i);
                    }
#pragma unroll
                    for (int i = 0; i < NO; ++i) {
                        if (i + VD < NO) {
                            vop[(i + VD) % (VD + 1)] = readV(i + VD);
                        }
                        acc[i] = Mma<BF16>(vop[i % (VD + 1)], pop, acc[i]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < NO; ++i) {
                        acc[i] = Mma<BF16>(readV(i), pop, acc[i]);
                    }
                }
        };

        if constexpr (SHARED) {
            // Cooperative staging: the NW*64 threads fetch the 32 latent rows of a step
            // together (whole rows, consecutive threads on consecutive 16-byte pieces),
            // one step ahead in registers, into the buffer the waves are not reading.
            constexpr int NT = NW * WAVE;
            constexpr int PIECES = STEP * KPR;
            constexpr int NSP = (PIECES + NT - 1) / NT;
            u32x4 stage[NSP];
            const int tid = threadIdx.x;
            auto coopLoad = [&](int t) {
                int64_t rowBase[2];
                nextRows(rowBase);
#pragma unroll
                for (int i = 0; i < NSP; ++i) {
                    const int pc = i * NT + tid;
                    const int row = pc / KPR;
                    const int col = pc % KPR;
                    stage[i] = u32x4{0u, 0u, 0u, 0u};
                    if (pc < PIECES && t + row < tokEnd) {
                        const int64_t r = rowBase[row >> 4] + (row & 15);
                        // plain load: the other head groups of this range fetch the same rows from L2
                        stage[i] = LoadGlobal16(keyPiece(r, col));
                    }
                }
            };
            auto coopStore = [&](unsigned char *tile) {
#pragma unroll
                for (int i = 0; i < NSP; ++i) {
                    const int pc = i * NT + tid;
                    if (pc < PIECES) {
                        *reinterpret_cast<u32x4 *>(tile + (pc / KPR) * (KP * 2) + (pc % KPR) * 16) = stage[i];
                    }
                }
            };
            int buf = 0;
            coopLoad(tokBegin);
            coopStore(smem);
            __syncthreads();
            for (int t = tokBegin; t < tokEnd; t += STEP) {
                const bool more = t + STEP < tokEnd;
                if (more) {
                    coopLoad(t + STEP);
                }
                const unsigned char *cur = smem + buf * K_TILE_BYTES;
                computeStep(t, cur, cur);
                if (more) {
                    coopStore(smem + (buf ^ 1) * K_TILE_BYTES);
                }
                __syncthreads(); // everyone is done with `cur`, the other buffer is complete
                buf ^= 1;
            }
        } else {
            for (int t = tokBegin; t < tokEnd; t += STEP) {
                if constexpr (BALANCED) {
                    // Two waves share a SIMD (wave w and w ^ 4), and its arbiter lets the older one issue first
                    // whenever both are ready. With the memory system saturated that is worth 15 % more rows per
                    // microsecond to waves 0-3, which then leave 13 us before their siblings and the launch ends with
                    // half its requests in flight. Each wave publishes the steps it still has to do and takes the
                    // higher issue priority while it has more left than its sibling (ties go to the younger wave).
                    const int left = __builtin_amdgcn_readfirstlane(s1 - segBegin - (t - tokBegin) / STEP);
                    if (lane == 0) {
                        stepsLeft[wave] = left;
                    }
                    const int sibling = __builtin_amdgcn_readfirstlane(stepsLeft[wave ^ 4]);
                    if (left > sibling || (left == sibling && wave >= 4)) {
                        __builtin_amdgcn_s_setprio(1);
                    } else {
                        __builtin_amdgcn_s_setprio(0);
                    }
                }
                if constexpr (PF) {
#pragma unroll
                    for (int i = 0; i < NKP; ++i) {
                        storePiece(kTile, KP, KPR, i, kStage[i]);
                    }
#pragma unroll
                    for (int i = 0; i < NVP; ++i) {
                        storePiece(vTile, VP, VPR, i, vStage[i]);
                    }
                    if (t + STEP < tokEnd) {
                        loadStage(t + STEP);
                    }
                } else {
                    // Large rows: stage a few pieces at a time to bound register use.
                    constexpr int BATCH = 6;
                    int64_t rowBase[2];
                    nextRows(rowBase);
                    const bool full = t + STEP <= tokEnd;
#pragma unroll
                    for (int i0 = 0; i0 < NKP; i0 += BATCH) {
                        u32x4 tmp[BATCH];
#pragma unroll
                        for (int b = 0; b < BATCH; ++b) {
                            if (i0 + b < NKP) {
                                tmp[b] = loadK(t, rowBase, i0 + b, full);
                            }
                        }
#pragma unroll
                        for (int b = 0; b < BATCH; ++b) {
                            if (i0 + b < NKP) {
                                storePiece(kTile, KP, KPR, i0 + b, tmp[b]);
                            }
                        }
                    }
#pragma unroll
                    for (int i0 = 0; i0 < NVP; i0 += BATCH) {
                        u32x4 tmp[BATCH];
#pragma unroll
                        for (int b = 0; b < BATCH; ++b) {
                            if (i0 + b < NVP) {
                                tmp[b] = loadV(t, rowBase, i0 + b, full);
                            }
                        }
#pragma unroll
                        for (int b = 0; b < BATCH; ++b) {
                            if (i0 + b < NVP) {
                                storePiece(vTile, VP, VPR, i0 + b, tmp[b]);
                            }
                        }
                    }
                }
                // The tile is private to this wave: LDS executes a wave's accesses in
                // order, only the compiler has to be kept from moving reads above writes.
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

                computeStep(t, kTile, vTile);
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
            }
        }

        // ---- finish the row (or this wave's share of it)
        const float l = accL[0];
        const float inv = EXT && l == 0.0f ? 0.0f : 1.0f / l; // l == 0: a -inf mask took every token out
        const float bias = KV8 ? INT8_BIAS : 0.0f; // see Int8x4ToHalf
        if (n < nh) {
            const int h = h0 + colHead;
            if (complete) {
                uint16_t *orow = reinterpret_cast<uint16_t *>(a.out) + (static_cast<int64_t>(qRow) * a.H + h) * DV;
#pragma unroll
                for (int i = 0; i < NO; ++i) {
                    const int d = i * 16 + kg * 4;
                    float o[4];
                    f32x4 vs = {1.0f, 1.0f, 1.0f, 1.0f};
                    if (KV8) {
                        vs = LoadScale4(a.vScale, gs * DV + d, a.scaleStride);
                    }
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        o[r] = acc[i][r] * inv - bias;
                        if (KV8) {
                            const int c = gs * DV + d + r;
                            o[r] = (o[r] + (a.vOff ? static_cast<float>(a.vOff[c]) : 0.0f)) * vs[r];
                        }
                    }
                    u32x2 packed;
                    if (qBf16) {
                        packed[0] = Pack2<true>(o[0], o[1]);
                        packed[1] = Pack2<true>(o[2], o[3]);
                    } else {
                        packed[0] = Pack2<false>(o[0], o[1]);
                        packed[1] = Pack2<false>(o[2], o[3]);
                    }
                    *reinterpret_cast<u32x2 *>(orow + d) = packed;
                }
                if (a.lse && kg == 0) {
                    Store16(a.lse, static_cast<int64_t>(qRow) * a.H + h, (m + log2f(l)) * 0.6931471805599453f, qBf16);
                }
            } else {
                const int slot = 2 * wr + (segBegin == s0 ? 0 : 1);
                const int64_t ph = (static_cast<int64_t>(slot) * (EXT ? p.foldTokens : 1) + colTok) * a.H + h;
#pragma unroll
                for (int i = 0; i < NO; ++i) {
                    f32x4 o = acc[i] * inv - bias;
                    if (KV8 && !a.finishV) {
                        // descale here (an affine map of rows whose merge weights sum to one commutes with the
                        // merge): under head compression the merge kernel cannot tell the slice, and with offsets
                        // the sum must be taken before the row is rounded to 16 bits
                        const int c = gs * DV + i * 16 + kg * 4;
                        const f32x4 vs = LoadScale4(a.vScale, c, a.scaleStride);
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            o[r] = (o[r] + (a.vOff ? static_cast<float>(a.vOff[c + r]) : 0.0f)) * vs[r];
                        }
                    }
                    // partial rows travel in the query's 16-bit type
                    u32x2 packed;
                    if (qBf16) {
                        packed[0] = Pack2<true>(o[0], o[1]);
                        packed[1] = Pack2<true>(o[2], o[3]);
                    } else {
                        packed[0] = Pack2<false>(o[0], o[1]);
                        packed[1] = Pack2<false>(o[2], o[3]);
                    }
                    *reinterpret_cast<u32x2 *>(reinterpret_cast<uint16_t *>(a.partO) + ph * DV + i * 16 + kg * 4) = packed;
                }
                if (kg == 0) {
                    a.partLse[ph] = m + log2f(l);
                }
            }
        }
    }
    if (BALANCED && lane == 0) {
        stepsLeft[wave] = 0; // the sibling keeps the higher priority from here on
    }
}

template <bool BF16, bool KV8, int D, int DV, bool MLA, bool PF, int NW, bool SHARED, bool EXT>
int LaunchBuild(const PaArgs &args, const PaStreamPlan &plan, hipStream_t stream)
{
    auto kernel = PaMfmaKernel<BF16, KV8, D, DV, MLA, PF, NW, SHARED, EXT>;
    constexpr int lds = SHARED ? 2 * WaveLdsBytes<D, DV, MLA>() : NW * WaveLdsBytes<D, DV, MLA>() + 64; // + stepsLeft
    static_assert(lds <= 160 * 1024, "tiles exceed the 160 KB of LDS per CU");
    const int configured = ConfigureKernelLds(reinterpret_cast<const void *>(kernel), lds);
    if (configured != OK) {
        return configured;
    }
    if (plan.headsPerWg * plan.tokenSlices != NW || (SHARED && plan.tokenSlices != 1)) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: plan made for %d waves, kernel has %d",
                    plan.headsPerWg * plan.tokenSlices, NW);
    }
    const int64_t grid = (static_cast<int64_t>(plan.numWgRanges) + 7) / 8 * 8 * plan.headGroups;
    if (grid <= 0 || grid > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: grid of %lld workgroups is out of range", (long long)grid);
    }
    kernel<<<static_cast<unsigned>(grid), NW * WAVE, lds, stream>>>(args, plan);
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}

// The combined-cache builds always carry the extensions (their callers use masks and several query
// tokens routinely and they are not register-bound); the others come in both forms.
template <bool BF16, bool KV8, int D, int DV, bool MLA, bool PF, int NW, bool SHARED = false>
int Launch(const PaArgs &args, const PaStreamPlan &plan, hipStream_t stream)
{
    if (MLA || args.mask != nullptr || args.logN != nullptr || plan.foldTokens > 1 || args.razor != nullptr ||
        args.descaleHeads > 0) {
        return LaunchBuild<BF16, KV8, D, DV, MLA, PF, NW, SHARED, true>(args, plan, stream);
    }
    return LaunchBuild<BF16, KV8, D, DV, MLA, PF, NW, SHARED, MLA>(args, plan, stream);
}

} // namespace mfma
} // namespace atbmi
#endif
