// PagedAttention decode with int8 queries over int8 caches (PagedAttentionParam::quantType TYPE_QUANT_QKV_ONLINE /
// TYPE_QUANT_QKV_OFFLINE) for gfx950 (reference operator src/ops/ops_infer/paged_attention/
// paged_attention_operation.cpp:250-275,429-436, kernel library checks src/kernels/mixkernels/pagedattention/
// paged_attention_operation.cpp:357-403; golden tests/apitest/kernelstest/mix/test_paged_attention_common.py:
// 104-110, 147-168, 171-229, 256-276).
//
// Arithmetic, per sequence and query head h of KV head g = h / (heads / kvHeads), as the golden has it:
//   score   = (int32 dot of the int8 query and the int8 key row) x kDescale[h], times qkScale, plus the mask;
//   weights = exp(score - running max), quantised per tile of tokens to int8: online against the largest weight
//             of the tile, rint(fp16(w / (wmax / 127))), offline with the given factor, rint(fp16(w x pScale[h]));
//   values  = int32 dot of the int8 weights and the int8 value rows, times vDescale[h] x wmax / 127 (online) or
//             vDescale[h] (offline); tiles are joined by the usual online rescaling, the denominator adds up the
//             unquantised weights.
// The tile is 64 tokens here. (The golden's tile follows the Ascend kernel's own block size and split; its
// tests compare against the whole context as one tile by the double-golden criterion, so the tile is not a
// property of the operator.) Every integer product is exact (v_mfma_i32_16x16x64_i8; sums stay below 2^24).
//
// A wave owns one KV head and up to 16 of its query heads (a "pair": KV head, tile of 16 query heads) and works on
// its own: its own two LDS tiles, softmax state and accumulators, no workgroup barrier. A workgroup is up to eight
// waves, the pairs of the SAME tokens: together they read whole token slots, [kvHeads x D] contiguous bytes a
// token, at about the same time, which is what the memory system delivers fastest (a workgroup that reads one KV
// head alone picks 128 of every 1024 bytes). The launch has as many workgroups as the chip holds at once; each
// walks its share of the context tokens of all sequences, piece after piece (a piece: consecutive tiles of one
// sequence), with the rows of the next piece's first tile requested during the last tile of the piece before.
//   scores   four MFMA row blocks st = 0 .. 3; row m of block st is token 16 (m / 4) + 4 st + m % 4, so that lane
//            (head n, kg) ends up with the scores of tokens 16 kg .. 16 kg + 15 (its 4 x 4 results in the order
//            j = 4 st + e). The key rows are stored to LDS in that order (row 16 st + m), the reads stay
//            conflict-free;
//   softmax  in the lane's registers; a head's four lanes (kg = 0 .. 3) exchange maxima and sums through the
//            cross-lane network; the 16 int8 weights of a lane ARE its B operand of the value product
//            (contraction index 16 kg + j = token);
//   values   O^T[channel, head] += V^T . P^T, V^T read from the token-major rows by the transposing
//            ds_read_b64_tr_b8, two reads a tile of 16 channels.
// Operand layout of v_mfma_i32_16x16x64_i8: lane (n = lane % 16, kg = lane / 16) supplies the 16 contraction values
// 16 kg .. 16 kg + 15 of row n (A) / column n (B) and receives D[4 kg + e][n], e = 0 .. 3.
// A sequence that lies in one piece is written directly; the pieces of the others leave normalised fp32 rows and
// natural-log log-sum-exps for a merge kernel (the golden cuts and merges the same way, :171-229).
#include <algorithm>
#include <type_traits>
#include <vector>
#include "pa_internal.h"
#include "upload_ring.h"

namespace atbmi {
namespace int8q {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int TILE = 128; // tokens in the unit that AtbmiPaInt8QCall::pieceTiles counts
constexpr int TW = 64;    // tokens of a wave's tile: their weights are quantised together
constexpr int HT = 16;    // query heads of a wave (the N extent of the MFMA)
template <int D> constexpr int WaveLdsBytes() { return 2 * TW * (D + 16); } // key and value tile, rows padded by 16 bytes
template <int D> constexpr int MaxWaves() { return D <= 128 ? 8 : 4; }      // (LDS: 18 KB a wave for D = 128, 35 KB for 256)

// One piece of a sequence with a non-empty context: its block-table row, the tokens [tokBegin, tokEnd) of its
// context (tokBegin a multiple of the tile; an empty range pads the table), row of query / out, mask row, and the
// first of its partial rows (-1: the piece is the whole sequence and writes the output itself).
struct Row {
    int32_t tableRow;
    int32_t tokBegin;
    int32_t tokEnd;
    int32_t qRow;
    int32_t maskRow;
    int32_t partial;
    int32_t streamFirst; // entry w of the table holds the index of the first piece of stream w (the pieces of a stream
                         // follow one another; the table has one entry more than there are streams)
    int32_t pad;
};

// A sequence that was cut: row of out, its first partial row and how many pieces it has.
struct MergeRow {
    int32_t qRow;
    int32_t firstPartial;
    int32_t numPartials;
    int32_t pad;
};

struct Args {
    const int8_t *q8;
    const int8_t *k8;
    const int8_t *v8;
    const int32_t *tables;
    const float *kDescale;
    const float *vDescale;
    const float *pScale; // offline quantisation only
    const void *mask;
    void *out;
    const Row *rows;
    const MergeRow *mergeRows;
    uint16_t *partO; // [partial rows][kvHeads x headTiles][16 heads][D], normalised, in the output's type
    float *partLse; // [partial rows][kvHeads x headTiles][16 heads]
    int64_t maskSeqStride;  // elements between the mask rows of two sequences (0: shared)
    int64_t maskHeadStride; // elements between the mask rows of two heads (0: shared)
    int32_t H;
    int32_t G;
    int32_t maxBlocksPerSeq;
    int32_t blockSize;
    int32_t bf16; // outputs (and mask values) are bf16 instead of fp16
    float qkScale;
};

// Cache rows are read once per call: the non-temporal hint keeps them from displacing anything in L2 / the
// memory-side cache.
__device__ __forceinline__ u32x4 LoadStream16(const void *p)
{
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
}

__device__ __forceinline__ float QuadMax(float x) // over the lanes n, n + 16, n + 32, n + 48
{
    x = fmaxf(x, __shfl_xor(x, 16));
    return fmaxf(x, __shfl_xor(x, 32));
}
__device__ __forceinline__ float QuadSum(float x)
{
    x += __shfl_xor(x, 16);
    return x + __shfl_xor(x, 32);
}

template <int D, bool OFFLINE, bool MASK, bool WHOLE>
__global__ __launch_bounds__(MaxWaves<D>() * WAVE) void PaInt8QKernel(const Args a)
{
    constexpr int PITCH = D + 16;
    constexpr int PPR = D / 16;     // 16-byte pieces per row = loads per tile, lane and cache
    constexpr int RPL = WAVE / PPR; // rows per load instruction
    constexpr int CT = D / 16;      // channel tiles of 16
    constexpr int MW = 9;           // aligned 32-bit words that hold a lane's 16 mask values
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int n = lane & 15;
    const int kg = lane >> 4;
    const int group = a.H / a.G;
    const int headTiles = (group + HT - 1) / HT;
    const int vheads = a.G * headTiles; // (KV head, head tile) pairs: one wave each
    const int wavesPerWg = blockDim.x / WAVE;
    const int vgroups = (vheads + wavesPerWg - 1) / wavesPerWg;
    // A workgroup walks the pieces of one stream, one after the other (rows[stream].streamFirst .. of the next one)
    const int stream = blockIdx.x / vgroups;
    const int vh = (blockIdx.x % vgroups) * wavesPerWg + wave;
    int piece = a.rows[stream].streamFirst;
    const int pieceEnd = a.rows[stream + 1].streamFirst;
    if (piece >= pieceEnd || vh >= vheads) {
        return; // (no barriers anywhere: leaving is safe)
    }
    const int g = vh / headTiles;
    const int ht = vh % headTiles;
    const int nh = min(HT, group - ht * HT);
    const int h0 = g * group + ht * HT;
    const bool liveHead = n < nh;
    const int hn = h0 + min(n, nh - 1);
    const int64_t slotBytes = static_cast<int64_t>(a.G) * D;
    unsigned char *kTile = smem + wave * WaveLdsBytes<D>();
    unsigned char *vTile = kTile + TW * PITCH;
    const int ldTok = lane / PPR;
    const int ldPiece = lane % PPR;
    const int64_t laneAt = static_cast<int64_t>(g) * D + ldPiece * 16;
    const float kDescale = a.kDescale[hn];
    const float vDescale = a.vDescale[hn];
    const float pScale = OFFLINE ? a.pScale[hn] : 0.0f;

    // Rows of the piece table and block ids come through scalar loads: they are the same for the whole wave, and a
    // scalar load is not counted with the vector loads, so looking a block up never waits for cache rows that are
    // on their way.
    auto rowAt = [&](int index) {
        i32x8 v;
        const Row *at = a.rows + index;
        asm volatile("s_load_dwordx8 %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(at) : "memory");
        return Row{v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7]};
    };
    auto blockIdOf = [&](const Row &r, int blk) {
        int id;
        const int32_t *at = a.tables + static_cast<int64_t>(r.tableRow) * a.maxBlocksPerSeq + blk;
        asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(id) : "s"(at) : "memory");
        return id;
    };
    auto queryOf = [&](const Row &r, i32x4(&q8)[D / 64]) {
#pragma unroll
        for (int j = 0; j < D / 64; ++j) {
            // (lanes past the last head of the tile repeat it; what they compute is never stored)
            q8[j] = *reinterpret_cast<const i32x4 *>(a.q8 + (static_cast<int64_t>(r.qRow) * a.H + hn) * D + j * 64 + kg * 16);
        }
    };

    // ---- requests: key rows are asked for two tiles ahead of the arithmetic and value rows one tile ahead, each on a
    // position of its own in the stream. Past the end of the stream a request asks for one row of the last tile
    // again: no request is ever skipped, so the number of loads on their way at any point of the loop is known when
    // the kernel is compiled and a wait names exactly the loads it needs.
    struct Cursor {
        int piece;
        Row row;
        int tok;
        bool live;
    };
    auto request = [&](const int8_t *cache, Cursor &c, u32x4(&r)[PPR]) {
        const int t0 = c.tok;
        if constexpr (WHOLE) {
            // (the tile's first slot is the same for the whole wave: a base in scalar registers and a small offset a lane)
            const int blk = t0 / a.blockSize;
            const int64_t first = static_cast<int64_t>(blockIdOf(c.row, blk)) * a.blockSize + (t0 - blk * a.blockSize);
            const int8_t *base = cache + first * slotBytes;
            const int last = c.live ? c.row.tokEnd - 1 - t0 : 0;
#pragma unroll
            for (int q = 0; q < PPR; ++q) {
                const uint32_t at = static_cast<uint32_t>(min(q * RPL + ldTok, last)) * static_cast<uint32_t>(slotBytes) +
                                    static_cast<uint32_t>(laneAt);
                r[q] = LoadStream16(base + at);
            }
        } else {
            const int32_t *table = a.tables + static_cast<int64_t>(c.row.tableRow) * a.maxBlocksPerSeq;
#pragma unroll
            for (int q = 0; q < PPR; ++q) {
                const int tok = c.live ? min(t0 + q * RPL + ldTok, c.row.tokEnd - 1) : t0;
                const int blk = tok / a.blockSize;
                r[q] = LoadStream16(cache + (static_cast<int64_t>(table[blk]) * a.blockSize + (tok - blk * a.blockSize)) * slotBytes +
                                    laneAt);
            }
        }
        if (c.live) {
            if (c.tok + TW < c.row.tokEnd) {
                c.tok += TW;
            } else if (c.piece + 1 < pieceEnd) {
                c.row = rowAt(++c.piece);
                c.tok = c.row.tokBegin;
            } else {
                c.live = false;
            }
        }
    };
    auto storeRows = [&](const u32x4(&kr)[PPR], const u32x4(&vr)[PPR]) {
#pragma unroll
        for (int q = 0; q < PPR; ++q) {
            const int tok = q * RPL + ldTok;
            const int krow = 16 * ((tok >> 2) & 3) + 4 * (tok >> 4) + (tok & 3);
            *reinterpret_cast<u32x4 *>(kTile + krow * PITCH + ldPiece * 16) = kr[q];
            *reinterpret_cast<u32x4 *>(vTile + tok * PITCH + ldPiece * 16) = vr[q];
        }
    };
    // mask values of tokens t0 + 16 kg .. + 15 of head n: the nine aligned words around them, asked for a tile ahead
    auto maskRowOf = [&](const Row &r) {
        return reinterpret_cast<const uint16_t *>(a.mask) + static_cast<int64_t>(r.maskRow) * a.maskSeqStride +
               static_cast<int64_t>(hn) * a.maskHeadStride;
    };
    uint32_t maskNext[MW] = {}, maskBits[MW] = {};
    auto requestMask = [&](const Row &r, int t0) {
        if constexpr (MASK) {
            const uint16_t *maskRow = maskRowOf(r);
            const uintptr_t last = reinterpret_cast<uintptr_t>(maskRow + r.tokEnd - 1) & ~static_cast<uintptr_t>(3);
            const uintptr_t first = reinterpret_cast<uintptr_t>(maskRow + t0 + 16 * kg) & ~static_cast<uintptr_t>(3);
#pragma unroll
            for (int k = 0; k < MW; ++k) {
                const uintptr_t at = first + 4 * k;
                maskNext[k] = *reinterpret_cast<const uint32_t *>(at < last ? at : last);
            }
        }
    };

    // ---- the arithmetic: piece `piece` with row cur, at token tok; nxt is the row of the piece after it (or cur again)
    Row cur = rowAt(piece);
    Row nxt = rowAt(min(piece + 1, pieceEnd - 1));
    i32x4 q8[D / 64], q8n[D / 64];
    queryOf(cur, q8);
    queryOf(nxt, q8n);
    int tok = cur.tokBegin;
    float runMax = -INFINITY;
    float runSum = 0.0f;
    f32x4 acc[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        acc[ct] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    Cursor keyAt{piece, cur, cur.tokBegin, true};
    Cursor valueAt = keyAt;
    u32x4 kA[PPR], kB[PPR], vr[PPR];
    requestMask(cur, tok);
    request(a.k8, keyAt, kA);
    request(a.v8, valueAt, vr);
    request(a.k8, keyAt, kB);
    storeRows(kA, vr);
#pragma unroll
    for (int k = 0; k < MW; ++k) {
        maskBits[k] = maskNext[k];
    }
    // One tile: LDS holds its rows, kNow are the key rows of the tile after it (on their way since the step before),
    // kLater takes those of the tile after that, vr the value rows of the tile after this one. Returns false after
    // the last tile of the stream.
    auto step = [&](u32x4(&kNow)[PPR], u32x4(&kLater)[PPR]) -> bool {
        const int t0 = tok;
        const bool lastOfPiece = t0 + TW >= cur.tokEnd;
        requestMask(lastOfPiece ? nxt : cur, lastOfPiece ? nxt.tokBegin : t0 + TW);
        request(a.v8, valueAt, vr);
        request(a.k8, keyAt, kLater);
        // ---- scores of tokens t0 + 16 kg + j, j = 4 st + e
        float w[16];
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            i32x4 dot = {0, 0, 0, 0};
#pragma unroll
            for (int j = 0; j < D / 64; ++j) {
                const i32x4 kk = *reinterpret_cast<const i32x4 *>(kTile + (16 * st + n) * PITCH + j * 64 + kg * 16);
                dot = __builtin_amdgcn_mfma_i32_16x16x64_i8(kk, q8[j], dot, 0, 0, 0);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int j = 4 * st + e;
                float bias = 0.0f;
                if constexpr (MASK) {
                    // value j sits 2 j bytes (+ 2 when the first one starts in the upper half of its word) into the words
                    const uint32_t shift = (reinterpret_cast<uintptr_t>(maskRowOf(cur) + t0 + 16 * kg) & 2) * 8;
                    const uint32_t pair = __builtin_amdgcn_alignbit(maskBits[j / 2 + 1], maskBits[j / 2], shift);
                    const uint16_t half = static_cast<uint16_t>(j % 2 ? pair >> 16 : pair);
                    bias = a.bf16 ? Bf16ToFloat(half) : HalfBitsToFloat(half);
                }
                w[j] = static_cast<float>(dot[e]) * kDescale * a.qkScale + bias;
            }
        }
        if (t0 + TW > cur.tokEnd) {
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                w[j] = t0 + 16 * kg + j < cur.tokEnd ? w[j] : -INFINITY;
            }
        }
        // ---- weights
        float tileMax = -INFINITY;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            tileMax = fmaxf(tileMax, w[j]);
        }
        tileMax = QuadMax(tileMax);
        const float newMax = fmaxf(runMax, tileMax);
        const bool any = newMax > -INFINITY; // (a mask of -inf can hide everything seen so far)
        float sum = 0.0f, wmax = 0.0f;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            w[j] = any ? __expf(w[j] - newMax) : 0.0f;
            sum += w[j];
            wmax = fmaxf(wmax, w[j]);
        }
        sum = QuadSum(sum);
        wmax = QuadMax(wmax);
        const float keep = (any && runMax > -INFINITY) ? __expf(runMax - newMax) : 0.0f;
        runSum = runSum * keep + sum;
        runMax = newMax;
        uint32_t packed[4] = {};
        float vscale;
        if constexpr (OFFLINE) {
            // rint(fp16(w x pScale)), with the given factor
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const float p = rintf(static_cast<float>(static_cast<_Float16>(w[j] * pScale)));
                packed[j / 4] = __builtin_amdgcn_cvt_pk_u8_f32(p, j % 4, packed[j / 4]);
            }
            vscale = vDescale;
        } else {
            // rint(fp16(w / step)), 0 .. 127. The quotient by a multiplication with 1 / step and one fused correction
            // (the division's own sequence without its rescaling); a step too small for that takes the division.
            const float step = wmax / 127.0f;
            if (step >= 1.0e-30f) {
                const float y = __builtin_amdgcn_rcpf(step);
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const float q0 = w[j] * y;
                    const float q = __builtin_fmaf(__builtin_fmaf(-q0, step, w[j]), y, q0);
                    const float p = rintf(static_cast<float>(static_cast<_Float16>(q)));
                    packed[j / 4] = __builtin_amdgcn_cvt_pk_u8_f32(p, j % 4, packed[j / 4]);
                }
            } else if (wmax > 0.0f) {
#pragma unroll
                for (int j = 0; j < 16; ++j) {
                    const float p = rintf(static_cast<float>(static_cast<_Float16>(__fdiv_rn(w[j], step))));
                    packed[j / 4] = __builtin_amdgcn_cvt_pk_u8_f32(p, j % 4, packed[j / 4]);
                }
            }
            vscale = vDescale * wmax / 127.0f;
        }
        // ---- values: O^T[channel, head] += V^T . P^T; the transposing read hands lane (channel n, kg) the bytes of
        // tokens r .. r + 7 when lane n of the group points at token r + n / 2, channels (n % 2) * 8 .. + 8
        const i32x4 pw = {static_cast<int>(packed[0]), static_cast<int>(packed[1]), static_cast<int>(packed[2]),
                          static_cast<int>(packed[3])};
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            const unsigned char *vp = vTile + (kg * 16 + (n >> 1)) * PITCH + ct * 16 + (n & 1) * 8;
            const i32x2 lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) i32x2 *)(vp));
            const i32x2 hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) i32x2 *)(vp + 8 * PITCH));
            const i32x4 vt = i32x4{lo[0], lo[1], hi[0], hi[1]};
            const i32x4 iacc = __builtin_amdgcn_mfma_i32_16x16x64_i8(vt, pw, i32x4{0, 0, 0, 0}, 0, 0, 0);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                acc[ct][e] = acc[ct][e] * keep + static_cast<float>(iacc[e]) * vscale;
            }
        }
        bool go = true;
        if (lastOfPiece) {
            // ---- acc / sum, to the output or, for a piece of a sequence, to its partial row with log(sum) + max
            if (liveHead) {
                const float inv = runSum > 0.0f ? 1.0f / runSum : 0.0f;
                if (cur.partial >= 0) {
                    const int64_t slot = (static_cast<int64_t>(cur.partial) * a.G + g) * headTiles + ht;
                    // (in the output's 16-bit type: a normalised row that ends in that type anyway; half the bytes a wave
                    // writes between two pieces of its stream)
                    uint16_t *prow = a.partO + (slot * HT + n) * D + kg * 4;
#pragma unroll
                    for (int ct = 0; ct < CT; ++ct) {
                        uint16_t bits[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float o = acc[ct][e] * inv;
                            bits[e] = a.bf16 ? FloatToBf16(o) : FloatToHalfBits(o);
                        }
                        uint2 row2;
                        row2.x = static_cast<uint32_t>(bits[0]) | (static_cast<uint32_t>(bits[1]) << 16);
                        row2.y = static_cast<uint32_t>(bits[2]) | (static_cast<uint32_t>(bits[3]) << 16);
                        *reinterpret_cast<uint2 *>(prow + ct * 16) = row2;
                    }
                    if (kg == 0) {
                        a.partLse[slot * HT + n] = runSum > 0.0f ? __logf(runSum) + runMax : -INFINITY;
                    }
                } else {
                    uint16_t *orow = reinterpret_cast<uint16_t *>(a.out) + (static_cast<int64_t>(cur.qRow) * a.H + h0 + n) * D + kg * 4;
#pragma unroll
                    for (int ct = 0; ct < CT; ++ct) {
                        uint16_t bits[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const float o = acc[ct][e] * inv;
                            bits[e] = a.bf16 ? FloatToBf16(o) : FloatToHalfBits(o);
                        }
                        uint2 out2;
                        out2.x = static_cast<uint32_t>(bits[0]) | (static_cast<uint32_t>(bits[1]) << 16);
                        out2.y = static_cast<uint32_t>(bits[2]) | (static_cast<uint32_t>(bits[3]) << 16);
                        *reinterpret_cast<uint2 *>(orow + ct * 16) = out2;
                    }
                }
            }
            // ---- on to the next piece of the stream
            go = piece + 1 < pieceEnd;
            ++piece;
            cur = nxt;
            nxt = rowAt(min(piece + 1, pieceEnd - 1));
            tok = cur.tokBegin;
#pragma unroll
            for (int j = 0; j < D / 64; ++j) {
                q8[j] = q8n[j];
            }
            queryOf(nxt, q8n);
            runMax = -INFINITY;
            runSum = 0.0f;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                acc[ct] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            }
        } else {
            tok = t0 + TW;
        }
        // ---- the next tile: its rows arrived while this one was worked on
        storeRows(kNow, vr);
        if constexpr (MASK) {
#pragma unroll
            for (int k = 0; k < MW; ++k) {
                maskBits[k] = maskNext[k];
            }
        }
        return go;
    };
    while (step(kB, kA) && step(kA, kB)) {
    }
}

// Joins the pieces of a cut sequence: out = sum_p exp(lse_p - L) O_p, L = log sum_p exp(lse_p) (reference golden
// test_paged_attention_common.py:217-228). A thread takes four channels of one head's row (16-byte loads of the
// partial rows, one 8-byte store); a workgroup of 256 threads takes as many heads of one cut sequence as fit (eight
// for 128 channels); grid.x = cut sequences x ceil(heads / heads a workgroup).
constexpr int MERGE_THREADS = 256;
__global__ __launch_bounds__(MERGE_THREADS) void PaInt8QMergeKernel(const Args a, int D)
{
    const int perHead = D / 4;                      // threads a head
    const int headsPerWg = MERGE_THREADS / perHead; // 16, 8 or 4
    const int wgsPerRow = (a.H + headsPerWg - 1) / headsPerWg;
    const MergeRow m = a.mergeRows[blockIdx.x / wgsPerRow];
    const int h = (blockIdx.x % wgsPerRow) * headsPerWg + static_cast<int>(threadIdx.x) / perHead;
    if (h >= a.H) {
        return;
    }
    const int d = (static_cast<int>(threadIdx.x) % perHead) * 4;
    const int group = a.H / a.G;
    const int headTiles = (group + HT - 1) / HT;
    const int g = h / group;
    const int ht = (h % group) / HT;
    const int n = (h % group) % HT;
    const int64_t perPartial = static_cast<int64_t>(a.G) * headTiles * HT; // head rows of one partial row
    const int64_t first = (static_cast<int64_t>(m.firstPartial) * a.G + g) * headTiles * HT + ht * HT + n;
    float mx = -INFINITY;
    for (int p = 0; p < m.numPartials; ++p) {
        mx = fmaxf(mx, a.partLse[first + p * perPartial]);
    }
    // (a piece a -inf mask emptied has lse == -inf and weighs nothing, even when every piece is like that)
    auto weightOf = [mx](float v) { return v == -INFINITY ? 0.0f : __expf(v - mx); };
    float total = 0.0f;
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int p = 0; p < m.numPartials; ++p) {
        const float w = weightOf(a.partLse[first + p * perPartial]);
        total += w;
        const uint2 raw = *reinterpret_cast<const uint2 *>(a.partO + (first + p * perPartial) * D + d);
        const uint32_t words[2] = {raw.x, raw.y};
        f32x4 row;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint16_t bits = static_cast<uint16_t>(words[e >> 1] >> ((e & 1) * 16));
            row[e] = a.bf16 ? Bf16ToFloat(bits) : HalfBitsToFloat(bits);
        }
        acc += row * w;
    }
    const float inv = total > 0.0f ? 1.0f / total : 0.0f;
    uint16_t bits[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float o = acc[e] * inv;
        bits[e] = a.bf16 ? FloatToBf16(o) : FloatToHalfBits(o);
    }
    uint2 out2;
    out2.x = static_cast<uint32_t>(bits[0]) | (static_cast<uint32_t>(bits[1]) << 16);
    out2.y = static_cast<uint32_t>(bits[2]) | (static_cast<uint32_t>(bits[3]) << 16);
    *reinterpret_cast<uint2 *>(reinterpret_cast<uint16_t *>(a.out) + (static_cast<int64_t>(m.qRow) * a.H + h) * D + d) = out2;
}

// Checks the call and lists its sequences (those of length 0, or switched off, take no query row).
int BuildRows(const AtbmiPaInt8QCall *c, std::vector<Row> *rows)
{
    if (!c || !c->hostContextLens) {
        return Fail(ERR_INVALID_PARAM, "pa_int8q: null call or context lengths");
    }
    if (c->outDtype != ATBMI_F16 && c->outDtype != ATBMI_BF16) {
        return Fail(ERR_INVALID_PARAM, "pa_int8q: the output is fp16 or bf16, got %d", c->outDtype);
    }
    if (c->numHeads <= 0 || c->numKvHeads <= 0 || c->numHeads % c->numKvHeads != 0) {
        return Fail(ERR_INVALID_PARAM, "pa_int8q: %d heads over %d KV heads", c->numHeads, c->numKvHeads);
    }
    if (c->headDim != 64 && c->headDim != 128 && c->headDim != 256) {
        return Fail(ERR_INVALID_PARAM, "pa_int8q: head size %d (64, 128 and 256 are built)", c->headDim);
    }
    if (c->batch < 0 || c->numBlocks <= 0 || c->maxBlocksPerSeq <= 0 || c->blockSize <= 0 || !(c->qkScale > 0.0f) ||
        (c->hasMask && c->maskLen <= 0) || c->maskSeqStride < 0 || c->maskHeadStride < 0 || c->pieceTiles < 0) {
        return Fail(ERR_INVALID_PARAM,
                    "pa_int8q: batch %d, %d blocks of %d tokens, %d blocks a sequence, qkScale %g, mask length %d",
                    c->batch, c->numBlocks, c->blockSize, c->maxBlocksPerSeq, c->qkScale, c->maskLen);
    }
    if (c->hasMask && (reinterpret_cast<uintptr_t>(c->mask) % 4 != 0 || c->maskSeqStride % 2 != 0 || c->maskHeadStride % 2 != 0 ||
                       c->maskLen % 2 != 0)) {
        // the kernel fetches mask values as aligned 32-bit words: a row that starts on an odd element would make it
        // read two bytes in front of the row, and one that ends on an even element two bytes behind it
        return Fail(ERR_INVALID_PARAM, "pa_int8q: the mask must start on a 4-byte boundary and have even strides (%lld, %lld) "
                                       "and an even row length (%d)", (long long)c->maskSeqStride, (long long)c->maskHeadStride,
                    c->maskLen);
    }
    int64_t qRow = 0;
    for (int32_t b = 0; b < c->batch; ++b) {
        const int32_t ctx = c->hostContextLens[b];
        if (ctx < 0) {
            return Fail(ERR_INVALID_PARAM, "pa_int8q: sequence %d has context %d", b, ctx);
        }
        if (ctx > static_cast<int64_t>(c->maxBlocksPerSeq) * c->blockSize) {
            return Fail(ERR_INVALID_PARAM, "pa_int8q: context %d of sequence %d exceeds its %d blocks", ctx, b,
                        c->maxBlocksPerSeq);
        }
        if (c->hasMask && ctx > c->maskLen) {
            return Fail(ERR_INVALID_PARAM, "pa_int8q: context %d of sequence %d exceeds the mask's %d positions", ctx, b,
                        c->maskLen);
        }
        if (ctx == 0) {
            continue;
        }
        if (qRow > 0x7fffffffLL) {
            return Fail(ERR_INVALID_PARAM, "pa_int8q: more than 2^31 query rows");
        }
        if (rows) {
            rows->push_back(Row{b, 0, ctx, static_cast<int32_t>(qRow), c->maskRowByQuery ? static_cast<int32_t>(qRow) : b,
                                -1, 0, 0});
        }
        ++qRow;
    }
    if (qRow > c->numQueryRows) {
        return Fail(ERR_INVALID_PARAM, "pa_int8q: the lengths ask for %lld query rows, the tensors hold %d",
                    (long long)qRow, c->numQueryRows);
    }
    return OK;
}

// What a call lays out in its workspace: the piece table as the kernel walks it, the table of cut sequences, and the
// partial rows.
struct Layout {
    std::vector<Row> pieces;     // stream after stream, and at least streams + 1 entries
    int64_t streams = 0;         // workgroups (times Shape::groups) that walk the pieces
    std::vector<MergeRow> merges;
    int64_t numPartials = 0;     // partial rows (each holds Shape::pairs x 16 head rows)
    uint64_t mergeOffset = 0, partOOffset = 0, partLseOffset = 0, bytes = 0;
};

// How the (KV head, tile of 16 query heads) pairs of a call are spread over workgroups.
struct Shape {
    int headTiles = 1;
    int pairs = 1;
    int groups = 1;  // workgroups a stream: the pairs in groups of `waves`
    int waves = 1;   // waves a workgroup
    bool whole = false; // a block holds whole tiles
};

Shape ShapeOf(const AtbmiPaInt8QCall *c)
{
    Shape sh;
    sh.headTiles = (c->numHeads / c->numKvHeads + HT - 1) / HT;
    sh.pairs = c->numKvHeads * sh.headTiles;
    const int most = c->headDim <= 128 ? 8 : 4;
    sh.groups = (sh.pairs + most - 1) / most;
    sh.waves = (sh.pairs + sh.groups - 1) / sh.groups;
    sh.whole = c->blockSize % TW == 0;
    return sh;
}

// Cuts sequence r into pieces at the token positions in `cuts` (ascending, inside the sequence) and appends them.
void CutSequence(const Row &r, const std::vector<int64_t> &cuts, Layout *lay, std::vector<Row> *out)
{
    const bool cut = !cuts.empty();
    if (cut) {
        lay->merges.push_back(MergeRow{r.qRow, static_cast<int32_t>(lay->numPartials), static_cast<int32_t>(cuts.size() + 1), 0});
    }
    int64_t begin = 0;
    for (size_t i = 0; i <= cuts.size(); ++i) {
        Row piece = r;
        piece.tokBegin = static_cast<int32_t>(begin);
        piece.tokEnd = static_cast<int32_t>(i < cuts.size() ? cuts[i] : r.tokEnd);
        piece.partial = cut ? static_cast<int32_t>(lay->numPartials++) : -1;
        out->push_back(piece);
        begin = piece.tokEnd;
    }
}

// Cuts the sequences into pieces of whole tiles and lays the piece table out stream after stream. There are as many
// streams as the chip holds workgroups at once (eight waves a CU, fewer where LDS says so), but no more than one for
// every four tiles.
// pieceTiles = 0: the tiles of all sequences, one sequence after the other, are one list that is cut into equal
//   shares, one for each stream; a sequence is cut where a share ends inside it.
// pieceTiles = c > 0: a sequence of n units of 128 tokens becomes ceil(n / c) pieces of ceil(n / pieces) units; the
//   pieces go to the streams in turn from the longest to the shortest.
Layout PlanPieces(const AtbmiPaInt8QCall *c, const std::vector<Row> &seqs)
{
    Layout lay;
    const Shape sh = ShapeOf(c);
    int64_t tiles = 0;
    for (const Row &r : seqs) {
        tiles += (r.tokEnd + TW - 1) / TW;
    }
    const int64_t waveLds = 2 * TW * (c->headDim + 16);
    const int64_t perCu = std::max<int64_t>(1, std::min<int64_t>(8 / sh.waves, 160 * 1024 / (sh.waves * waveLds)));
    lay.streams = std::max<int64_t>(1, std::min<int64_t>(tiles / 4, DeviceComputeUnits() * perCu / sh.groups));
    auto shareBegin = [&](int64_t w) { return tiles * w / lay.streams; };
    std::vector<std::vector<Row>> perStream(lay.streams);
    std::vector<Row> pieces;
    std::vector<int64_t> cuts;
    if (c->pieceTiles > 0) {
        for (const Row &r : seqs) {
            const int64_t n = (r.tokEnd + TILE - 1) / TILE;
            const int64_t parts = (n + c->pieceTiles - 1) / c->pieceTiles;
            const int64_t each = (n + parts - 1) / parts;
            cuts.clear();
            for (int64_t i = 1; i * each < n; ++i) {
                cuts.push_back(i * each * TILE);
            }
            CutSequence(r, cuts, &lay, &pieces);
        }
        std::stable_sort(pieces.begin(), pieces.end(), [](const Row &x, const Row &y) {
            return x.tokEnd - x.tokBegin > y.tokEnd - y.tokBegin;
        });
        for (size_t i = 0; i < pieces.size(); ++i) {
            perStream[i % lay.streams].push_back(pieces[i]);
        }
    } else {
        int64_t at = 0; // tiles before this sequence
        for (const Row &r : seqs) {
            const int64_t n = (r.tokEnd + TW - 1) / TW;
            // the streams whose shares begin inside the sequence: (first, last]
            int64_t first = (at * lay.streams + tiles - 1) / tiles; // smallest w with shareBegin(w) >= at ..
            while (first > 0 && shareBegin(first - 1) >= at) {
                --first;
            }
            while (first < lay.streams && shareBegin(first) < at) {
                ++first;
            }
            cuts.clear();
            for (int64_t w = first; w < lay.streams && shareBegin(w) < at + n; ++w) {
                if (shareBegin(w) > at) {
                    cuts.push_back((shareBegin(w) - at) * TW);
                }
            }
            pieces.clear();
            CutSequence(r, cuts, &lay, &pieces);
            int64_t stream = first > 0 ? first - 1 : 0; // the stream the sequence's first tile belongs to
            while (stream + 1 < lay.streams && shareBegin(stream + 1) <= at) {
                ++stream;
            }
            int64_t tile = at;
            for (const Row &p : pieces) {
                while (stream + 1 < lay.streams && shareBegin(stream + 1) <= tile) {
                    ++stream;
                }
                perStream[stream].push_back(p);
                tile += (p.tokEnd - p.tokBegin + TW - 1) / TW;
            }
            at += n;
        }
    }
    std::vector<int32_t> first;
    for (const std::vector<Row> &list : perStream) {
        first.push_back(static_cast<int32_t>(lay.pieces.size()));
        lay.pieces.insert(lay.pieces.end(), list.begin(), list.end());
    }
    first.push_back(static_cast<int32_t>(lay.pieces.size()));
    lay.pieces.resize(std::max(lay.pieces.size(), first.size()), Row{0, 0, 0, 0, 0, -1, 0, 0});
    for (size_t w = 0; w < first.size(); ++w) {
        lay.pieces[w].streamFirst = first[w];
    }
    auto align = [](uint64_t v) { return (v + 255) / 256 * 256; };
    lay.mergeOffset = align(lay.pieces.size() * sizeof(Row));
    lay.partOOffset = align(lay.mergeOffset + lay.merges.size() * sizeof(MergeRow));
    const uint64_t headRows = static_cast<uint64_t>(lay.numPartials) * sh.pairs * HT;
    lay.partLseOffset = align(lay.partOOffset + headRows * c->headDim * sizeof(uint16_t));
    lay.bytes = lay.partLseOffset + headRows * sizeof(float);
    return lay;
}

template <int D> int Launch(const AtbmiPaInt8QCall *call, const Args &a, const Layout &lay, hipStream_t s)
{
    const Shape sh = ShapeOf(call);
    // the kernel variant, one compile-time switch after the other
    void (*kernel)(Args) = nullptr;
    auto with = [](bool flag, auto &&next) {
        if (flag) {
            next(std::true_type{});
        } else {
            next(std::false_type{});
        }
    };
    with(call->offline != 0, [&](auto off) {
        with(a.mask != nullptr, [&](auto msk) {
            with(sh.whole, [&](auto who) {
                kernel = PaInt8QKernel<D, decltype(off)::value, decltype(msk)::value, decltype(who)::value>;
            });
        });
    });
    const int64_t numMerges = static_cast<int64_t>(lay.merges.size());
    const int64_t grid = lay.streams * sh.groups;
    if (grid > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "pa_int8q: %lld workgroups", (long long)grid);
    }
    const int threads = sh.waves * WAVE;
    const int ldsBytes = sh.waves * WaveLdsBytes<D>();
    int rc = ConfigureKernelLds(reinterpret_cast<const void *>(kernel), ldsBytes);
    if (rc != OK) {
        return rc;
    }
    TimedLaunch timed;
    rc = TimedLaunchBegin(s, &timed);
    if (rc != OK) {
        return rc;
    }
    kernel<<<static_cast<unsigned>(grid), threads, ldsBytes, s>>>(a);
    ATBMI_HIP_CHECK(hipGetLastError());
    rc = TimedLaunchKernelDone(s, timed);
    if (rc != OK) {
        return rc;
    }
    if (numMerges > 0) {
        const int headsPerWg = MERGE_THREADS / (D / 4);
        const unsigned mergeGrid = static_cast<unsigned>(numMerges * ((a.H + headsPerWg - 1) / headsPerWg));
        PaInt8QMergeKernel<<<mergeGrid, MERGE_THREADS, 0, s>>>(a, D);
        ATBMI_HIP_CHECK(hipGetLastError());
    }
    return TimedLaunchEnd(s, timed, numMerges > 0);
}

} // namespace int8q
} // namespace atbmi

using namespace atbmi;

extern "C" int atbmi_pa_int8q_workspace_size(const AtbmiPaInt8QCall *call, uint64_t *bytes)
{
    if (!bytes) {
        return Fail(ERR_INVALID_PARAM, "pa_int8q_workspace_size: null result pointer");
    }
    std::vector<int8q::Row> rows;
    const int rc = int8q::BuildRows(call, &rows);
    if (rc != OK) {
        return rc;
    }
    *bytes = int8q::PlanPieces(call, rows).bytes;
    return OK;
}

extern "C" int atbmi_pa_int8q_decode(const AtbmiPaInt8QCall *call, void *workspaceDevice, uint64_t workspaceBytes,
                                     void *stream)
{
    std::vector<int8q::Row> rows;
    int rc = int8q::BuildRows(call, &rows);
    if (rc != OK) {
        return rc;
    }
    if (rows.empty()) {
        return OK;
    }
    if (!call->query || !call->keyCache || !call->valueCache || !call->blockTables || !call->kDescale ||
        !call->vDescale || !call->out || (call->hasMask && !call->mask) || (call->offline && !call->pScale)) {
        return Fail(ERR_INVALID_PARAM, "pa_int8q: null tensor pointer");
    }
    const int8q::Layout lay = int8q::PlanPieces(call, rows);
    if (!workspaceDevice || workspaceBytes < lay.bytes) {
        return Fail(ERR_INVALID_PARAM, "pa_int8q: workspace of %llu bytes, %llu needed", (unsigned long long)workspaceBytes,
                    (unsigned long long)lay.bytes);
    }
    if (static_cast<int64_t>(lay.merges.size()) * call->numHeads > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "pa_int8q: %lld rows to merge", (long long)lay.merges.size() * call->numHeads);
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    unsigned char *ws = static_cast<unsigned char *>(workspaceDevice);
    rc = UploadTable(lay.pieces.data(), lay.pieces.size() * sizeof(int8q::Row), ws, s);
    if (rc == OK && !lay.merges.empty()) {
        rc = UploadTable(lay.merges.data(), lay.merges.size() * sizeof(int8q::MergeRow), ws + lay.mergeOffset, s);
    }
    if (rc != OK) {
        return rc;
    }
    int8q::Args a{};
    a.q8 = static_cast<const int8_t *>(call->query);
    a.k8 = static_cast<const int8_t *>(call->keyCache);
    a.v8 = static_cast<const int8_t *>(call->valueCache);
    a.tables = call->blockTables;
    a.kDescale = call->kDescale;
    a.vDescale = call->vDescale;
    a.pScale = call->offline ? call->pScale : nullptr;
    a.mask = call->hasMask ? call->mask : nullptr;
    a.out = call->out;
    a.rows = reinterpret_cast<const int8q::Row *>(ws);
    a.mergeRows = reinterpret_cast<const int8q::MergeRow *>(ws + lay.mergeOffset);
    a.partO = reinterpret_cast<uint16_t *>(ws + lay.partOOffset);
    a.partLse = reinterpret_cast<float *>(ws + lay.partLseOffset);
    a.maskSeqStride = call->maskSeqStride;
    a.maskHeadStride = call->maskHeadStride;
    a.H = call->numHeads;
    a.G = call->numKvHeads;
    a.maxBlocksPerSeq = call->maxBlocksPerSeq;
    a.blockSize = call->blockSize;
    a.bf16 = call->outDtype == ATBMI_BF16 ? 1 : 0;
    a.qkScale = call->qkScale;
    switch (call->headDim) {
        case 64: return int8q::Launch<64>(call, a, lay, s);
        case 128: return int8q::Launch<128>(call, a, lay, s);
        default: return int8q::Launch<256>(call, a, lay, s);
    }
}
