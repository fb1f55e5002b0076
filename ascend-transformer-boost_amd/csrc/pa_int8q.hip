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
// The tile is 128 tokens here. (The golden's tile follows the Ascend kernel's own block size and split; its
// tests compare against the whole context as one tile by the double-golden criterion, so the tile is not a
// property of the operator.) Every integer product is exact (v_mfma_i32_16x16x64_i8; sums stay below 2^24).
//
// A workgroup of four waves owns one piece of a sequence, one KV head and up to 16 of its query heads and walks the
// piece tile by tile. Key rows are requested into registers two tiles ahead of their scores, value rows one tile ahead, and
// both are stored to LDS (token-major, padded pitch) right after the scores of a tile: the key rows of the next tile
// and the value rows of this one. A tile then needs two workgroup barriers, after the scores and after the weights.
//   scores  wave w for tokens 32 w .. 32 w + 31: S^T[token, head] = K . Q^T (K rows from LDS as A, the query
//           resident in registers as B);
//   softmax 16 lanes a head, 8 tokens a lane (32 lanes with 4 tokens when a KV head has at most 8 query heads);
//           int8 weights P[head][token] go to LDS;
//   values  wave w for channels (D / 4) w .. : O^T[channel, head] += V^T . P^T, V^T read from the token-major rows by
//           the transposing ds_read_b64_tr_b8, P^T as 16 consecutive bytes of a head's weights.
// Operand layout of v_mfma_i32_16x16x64_i8: lane (n = lane % 16, kg = lane / 16) supplies the 16 contraction values
// 16 kg .. 16 kg + 15 of row n (A) / column n (B) and receives D[4 kg + e][n], e = 0 .. 3.
// Long contexts are cut into pieces of whole tiles (64 at most), sized so that the launch has a few workgroups per
// place on the chip; a sequence in one piece is written directly, the others leave normalised fp32 rows and natural-log
// log-sum-exps for a merge kernel (the golden cuts and merges the same way, :171-229).
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
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int TILE = 128;    // tokens per tile
constexpr int HT = 16;       // query heads per workgroup (the N extent of the MFMA)
constexpr int THREADS = 256; // four waves
constexpr int NWAVES = THREADS / WAVE;
constexpr int MAX_PIECE_TILES = 64; // a piece's block ids fit one register of a wave (see the kernel)
constexpr int S_PITCH = (TILE + 4) * 4; // 16 heads' 16-byte writes touch every bank once
constexpr int P_PITCH = TILE + 16;      // likewise for 16 heads' 16-byte reads
static_assert(TILE == NWAVES * 32, "four waves share a tile this way");

template <int D> struct Lds {
    static constexpr int PITCH = D + 16; // row pitch of the key and value tiles: 16 rows' 16-byte reads touch every bank once
    static constexpr int K = 0;                  // the key rows of a tile
    static constexpr int V = K + TILE * PITCH;   // the value rows of a tile
    static constexpr int S = V + TILE * PITCH;   // [16] fp32 scores
    static constexpr int P = S + HT * S_PITCH;   // [16] int8 weights
    static constexpr int STAT = P + HT * P_PITCH; // [16] {keep, value scale, 1 / sum, -}
    static constexpr int BYTES = STAT + HT * 16;
    static_assert(BYTES <= 160 * 1024 && S % 16 == 0 && P % 16 == 0 && STAT % 16 == 0, "LDS layout");
};

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
    int32_t pad[2];
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
    float *partO;   // [partial rows][kvHeads x headTiles][16 heads][D], normalised
    float *partLse; // [partial rows][kvHeads x headTiles][16 heads]
    int64_t maskSeqStride;  // elements between the mask rows of two sequences (0: shared)
    int64_t maskHeadStride; // elements between the mask rows of two heads (0: shared)
    int32_t H;
    int32_t G;
    int32_t numRows;
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

// All-reduce over the 16 lanes of a row (lanes 16 r .. 16 r + 15) by rotations inside the row.
template <int ROR> __device__ __forceinline__ float RowRotate(float x)
{
    const int v = __builtin_bit_cast(int, x);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(v, v, 0x120 + ROR, 0xf, 0xf, true));
}
__device__ __forceinline__ float RowMax(float x)
{
    x = fmaxf(x, RowRotate<8>(x));
    x = fmaxf(x, RowRotate<4>(x));
    x = fmaxf(x, RowRotate<2>(x));
    return fmaxf(x, RowRotate<1>(x));
}
__device__ __forceinline__ float RowSum(float x)
{
    x += RowRotate<8>(x);
    x += RowRotate<4>(x);
    x += RowRotate<2>(x);
    return x + RowRotate<1>(x);
}
// Both rows of a pair (rows 0 and 1, 2 and 3) of a value: the lane's own and, through the cross-lane network, that of
// the lane 16 further on or back.
__device__ __forceinline__ void PairOfRows(float x, float &a, float &b)
{
    a = x;
    b = __shfl_xor(x, 16);
}
// All-reduce over the LANES (16 or 32) lanes of a head.
template <int LANES> __device__ __forceinline__ float HeadMax(float x)
{
    x = RowMax(x);
    if constexpr (LANES == 32) {
        float a, b;
        PairOfRows(x, a, b);
        x = fmaxf(a, b);
    }
    return x;
}
template <int LANES> __device__ __forceinline__ float HeadSum(float x)
{
    x = RowSum(x);
    if constexpr (LANES == 32) {
        float a, b;
        PairOfRows(x, a, b);
        x = a + b;
    }
    return x;
}

// NARROW: no KV head has more than 8 query heads; the softmax then gives a head 32 lanes with 4 tokens each instead of
// 16 lanes with 8, and the rows of heads 8 .. 15 stay zero.
template <int D, bool OFFLINE, bool MASK, bool NARROW, bool WHOLE>
__global__ __launch_bounds__(THREADS) void PaInt8QKernel(const Args a)
{
    using L = Lds<D>;
    constexpr int CH = NARROW ? 32 : 16; // softmax: lanes a head
    constexpr int TPL = TILE / CH;       // softmax: tokens a lane
    constexpr int PPR = D / 16;              // 16-byte pieces per row
    constexpr int ROWS_PER_PASS = THREADS / PPR;
    constexpr int PASSES = TILE / ROWS_PER_PASS;
    constexpr int CT = D / 16 / NWAVES;      // channel tiles of 16 a wave
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int n = lane & 15;  // MFMA row (A) / column (B, D) of this lane
    const int kg = lane >> 4; // which 16 contraction values / 4 result rows this lane holds
    const int group = a.H / a.G;
    const int headTiles = (group + HT - 1) / HT;
    // workgroups go round the eight XCDs: XCD x takes the x-th eighth of the row table, so the workgroups of a
    // sequence, whose KV heads lie side by side in the cache rows, share one L2 (the host deals the sequences out to
    // the eighths longest first, see OrderRows)
    const int work = (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8;
    const Row row = a.rows[work / (a.G * headTiles)];
    if (row.tokEnd <= row.tokBegin) {
        return; // padding of an eighth
    }
    const int g = (work / headTiles) % a.G;
    const int ht = work % headTiles;
    const int nh = min(HT, group - ht * HT); // heads past the last one compute on zeros and store nothing
    const int h0 = g * group + ht * HT;
    const int32_t *table = a.tables + static_cast<int64_t>(row.tableRow) * a.maxBlocksPerSeq;
    const int numTiles = (row.tokEnd - row.tokBegin + TILE - 1) / TILE;
    const int64_t slotBytes = static_cast<int64_t>(a.G) * D; // one token's rows of all KV heads

    // ---- requests for a tile: this thread's pieces of the key and value rows (tokens past the context repeat the last one)
    const int ldTok = tid / PPR;
    const int ldPiece = tid % PPR;
    // WHOLE: a block holds whole tiles (block sizes 128, 256, ..), so a tile lies in one block and its first slot is
    // the same for the whole workgroup; otherwise every token looks its block up. With WHOLE the block ids of the
    // piece are read once, before the loop: lane l keeps table entry firstBlock + l (the host cuts pieces of at most
    // 64 tiles), and a request takes its id out of that register. No load and no branch then stands between the row
    // requests of one pass and of the next. Requests are never skipped either: past the last tile of the piece every
    // lane asks for its piece of one row of the last tile again (a few cache lines that are in L2), so that the
    // number of loads in flight at any point of the loop is known when the kernel is compiled and the waits in front
    // of the LDS stores name exactly the loads they need, instead of draining everything that is on its way.
    const int64_t laneAt = static_cast<int64_t>(g) * D + ldPiece * 16;
    const int firstBlock = WHOLE ? row.tokBegin / a.blockSize : 0;
    const int cachedIds = table[min(firstBlock + lane, a.maxBlocksPerSeq - 1)];
    const int lastTile = row.tokBegin + (numTiles - 1) * TILE;
    auto requestRows = [&](const int8_t *cache, int tile0, u32x4(&r)[PASSES]) {
        const bool live = tile0 <= lastTile;
        const int t0 = min(tile0, lastTile);
        if constexpr (WHOLE) {
            const int blk = __builtin_amdgcn_readfirstlane(t0 / a.blockSize);
            const int id = __builtin_amdgcn_readlane(cachedIds, blk - firstBlock);
            const int64_t first = static_cast<int64_t>(id) * a.blockSize + (t0 - blk * a.blockSize);
            const int last = live ? row.tokEnd - 1 - t0 : 0; // (tokens past the piece repeat its last one)
#pragma unroll
            for (int p = 0; p < PASSES; ++p) {
                r[p] = LoadStream16(cache + (first + min(p * ROWS_PER_PASS + ldTok, last)) * slotBytes + laneAt);
            }
        } else {
#pragma unroll
            for (int p = 0; p < PASSES; ++p) {
                const int tok = live ? min(t0 + p * ROWS_PER_PASS + ldTok, row.tokEnd - 1) : t0;
                const int blk = tok / a.blockSize;
                const int64_t slot = static_cast<int64_t>(table[blk]) * a.blockSize + (tok - blk * a.blockSize);
                r[p] = LoadStream16(cache + slot * slotBytes + laneAt);
            }
        }
    };
    auto storeRows = [&](int buffer, const u32x4(&r)[PASSES]) {
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            *reinterpret_cast<u32x4 *>(smem + buffer + (p * ROWS_PER_PASS + ldTok) * L::PITCH + ldPiece * 16) = r[p];
        }
    };
    // Rows are asked for a tile and a half ahead: while tile i is worked on, set A holds the key rows of tile i + 1
    // and the value rows of tile i (both stored to LDS once the scores of tile i are done), set B takes the key rows
    // of tile i + 2 and the value rows of tile i + 1; the sets swap roles every tile.
    u32x4 kA[PASSES], vA[PASSES], kB[PASSES], vB[PASSES];
    requestRows(a.k8, row.tokBegin, kA);

    // ---- Q^T as B operands: lane (n, kg) holds q8[head n][64 j + 16 kg .. + 16)
    i32x4 q8[D / 64];
    const bool liveHead = n < nh;
    const int hn = h0 + min(n, nh - 1);
#pragma unroll
    for (int j = 0; j < D / 64; ++j) {
        q8[j] = *reinterpret_cast<const i32x4 *>(a.q8 + (static_cast<int64_t>(row.qRow) * a.H + hn) * D + j * 64 + kg * 16);
        if (!liveHead) {
            q8[j] = i32x4{0, 0, 0, 0};
        }
    }
    const float descale = a.kDescale[hn];
    const uint16_t *maskRow = nullptr;
    if constexpr (MASK) {
        maskRow = reinterpret_cast<const uint16_t *>(a.mask) + static_cast<int64_t>(row.maskRow) * a.maskSeqStride +
                  static_cast<int64_t>(hn) * a.maskHeadStride;
    }
    // softmax: lane (head tid / CH, tokens 4 (tid % CH) .. + 4, and with 16 lanes a head 64 more on); a head's lanes
    // all hold its running maximum and sum
    const int smHead = tid / CH;
    const int smTok = (tid % CH) * 4;
    const int smH = h0 + min(smHead, nh - 1);
    const float smVDescale = a.vDescale[smH];
    const float smPScale = OFFLINE ? a.pScale[smH] : 0.0f;
    float runMax = -INFINITY;
    float runSum = 0.0f;
    // values: channels 16 (CT wave + ct) + 4 kg + e of head n
    f32x4 acc[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        acc[ct] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    // this lane's mask values of a tile: tokens 32 wave + 16 rt + 4 kg + e of head n. What is loaded is the aligned
    // 32-bit word that holds the value; the half is taken out where the value is used, so that nothing has to wait
    // for the load before then.
    uint32_t maskNext[2][4] = {};
    auto maskAddress = [&](int t0, int rt, int e) {
        return reinterpret_cast<uintptr_t>(maskRow + min(t0 + wave * 32 + rt * 16 + kg * 4 + e, row.tokEnd - 1));
    };
    auto requestMask = [&](int t0) {
        if constexpr (MASK) {
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    maskNext[rt][e] = *reinterpret_cast<const uint32_t *>(maskAddress(t0, rt, e) & ~static_cast<uintptr_t>(3));
                }
            }
        }
    };
    requestMask(row.tokBegin);
    storeRows(L::K, kA);
    requestRows(a.v8, row.tokBegin, vA);
    requestRows(a.k8, row.tokBegin + TILE, kA);
    if constexpr (NARROW) { // the weights and factors of heads 8 .. 15, which the softmax never writes
        for (int i = tid; i < (HT / 2) * (P_PITCH / 4); i += THREADS) {
            reinterpret_cast<uint32_t *>(smem + L::P + (HT / 2) * P_PITCH)[i] = 0u;
        }
        if (tid < (HT / 2) * 4) {
            reinterpret_cast<float *>(smem + L::STAT)[(HT / 2) * 4 + tid] = 0.0f;
        }
    }
    __syncthreads();

    // the mask values of the tile being worked on (see the end of a pass)
    uint32_t maskBits[2][4];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            maskBits[rt][e] = maskNext[rt][e];
        }
    }
    // One tile: LDS holds its key rows; kNow are the key rows of the next tile and vNow its own value rows, on their
    // way since the pass before; kLater / vLater take what the pass after this one will store. Two barriers a tile:
    // whatever a phase overwrites was last read two phases earlier.
    auto pass = [&](const int i, u32x4(&kNow)[PASSES], u32x4(&vNow)[PASSES], u32x4(&kLater)[PASSES], u32x4(&vLater)[PASSES]) {
        const int t0 = row.tokBegin + i * TILE;
        requestMask(t0 + TILE);
        requestRows(a.v8, t0 + TILE, vLater);
        requestRows(a.k8, t0 + 2 * TILE, kLater);
        // ---- scores of tokens 32 wave .. + 31
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
            const int tokBase = wave * 32 + rt * 16;
            const int tok = t0 + tokBase + kg * 4; // this lane's four tokens
            i32x4 dot = {0, 0, 0, 0};
#pragma unroll
            for (int j = 0; j < D / 64; ++j) {
                const i32x4 kk = *reinterpret_cast<const i32x4 *>(smem + L::K + (tokBase + n) * L::PITCH + j * 64 + kg * 16);
                dot = __builtin_amdgcn_mfma_i32_16x16x64_i8(kk, q8[j], dot, 0, 0, 0);
            }
            f32x4 sc;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float bias = 0.0f;
                if constexpr (MASK) {
                    const uint16_t half = static_cast<uint16_t>(maskBits[rt][e] >> ((maskAddress(t0, rt, e) & 2) * 8));
                    bias = a.bf16 ? Bf16ToFloat(half) : HalfBitsToFloat(half);
                }
                sc[e] = static_cast<float>(dot[e]) * descale * a.qkScale + bias;
            }
            if (t0 + TILE > row.tokEnd) { // the last tile of the piece: tokens past its end weigh nothing
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    sc[e] = tok + e < row.tokEnd ? sc[e] : -INFINITY;
                }
            }
            *reinterpret_cast<f32x4 *>(smem + L::S + n * S_PITCH + (tokBase + kg * 4) * 4) = sc;
        }
        __syncthreads(); // the key rows are scored, and everybody is done with the values of the tile before
        storeRows(L::K, kNow); // (after the last tile: rows nobody reads)
        storeRows(L::V, vNow);
        // ---- weights of the tile
        {
            float w[TPL];
            const float *srow = reinterpret_cast<const float *>(smem + L::S + smHead * S_PITCH) + smTok;
            float tileMax = -INFINITY;
#pragma unroll
            for (int k = 0; k < TPL; k += 4) {
                const f32x4 v = *reinterpret_cast<const f32x4 *>(srow + k * CH);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    w[k + e] = v[e];
                    tileMax = fmaxf(tileMax, v[e]);
                }
            }
            tileMax = HeadMax<CH>(tileMax);
            const float newMax = fmaxf(runMax, tileMax);
            const bool any = newMax > -INFINITY; // (a mask of -inf can hide everything seen so far)
            float sum = 0.0f, wmax = 0.0f;
#pragma unroll
            for (int k = 0; k < TPL; ++k) {
                w[k] = any ? __expf(w[k] - newMax) : 0.0f;
                sum += w[k];
                wmax = fmaxf(wmax, w[k]);
            }
            sum = HeadSum<CH>(sum);
            wmax = HeadMax<CH>(wmax);
            const float keep = (any && runMax > -INFINITY) ? __expf(runMax - newMax) : 0.0f;
            runSum = runSum * keep + sum;
            runMax = newMax;
            uint32_t packed[TPL / 4] = {};
            float vscale;
            if constexpr (OFFLINE) {
                // rint(fp16(w x pScale)), with the given factor
#pragma unroll
                for (int k = 0; k < TPL; ++k) {
                    const float p = rintf(static_cast<float>(static_cast<_Float16>(w[k] * smPScale)));
                    packed[k / 4] = __builtin_amdgcn_cvt_pk_u8_f32(p, k % 4, packed[k / 4]);
                }
                vscale = smVDescale;
            } else {
                // rint(fp16(w / step)), 0 .. 127. The quotient by a multiplication with 1 / step and one fused
                // correction (the division's own sequence without its rescaling); a step too small for that takes
                // the division.
                const float step = wmax / 127.0f;
                if (step >= 1.0e-30f) {
                    const float y = __builtin_amdgcn_rcpf(step);
#pragma unroll
                    for (int k = 0; k < TPL; ++k) {
                        const float q0 = w[k] * y;
                        const float q = __builtin_fmaf(__builtin_fmaf(-q0, step, w[k]), y, q0);
                        const float p = rintf(static_cast<float>(static_cast<_Float16>(q)));
                        packed[k / 4] = __builtin_amdgcn_cvt_pk_u8_f32(p, k % 4, packed[k / 4]);
                    }
                } else if (wmax > 0.0f) {
#pragma unroll
                    for (int k = 0; k < TPL; ++k) {
                        const float p = rintf(static_cast<float>(static_cast<_Float16>(__fdiv_rn(w[k], step))));
                        packed[k / 4] = __builtin_amdgcn_cvt_pk_u8_f32(p, k % 4, packed[k / 4]);
                    }
                }
                vscale = smVDescale * wmax / 127.0f;
            }
            unsigned char *prow = smem + L::P + smHead * P_PITCH + smTok;
#pragma unroll
            for (int k = 0; k < TPL / 4; ++k) {
                *reinterpret_cast<uint32_t *>(prow + k * CH * 4) = packed[k];
            }
            if (tid % CH == 0) {
                float *stat = reinterpret_cast<float *>(smem + L::STAT) + smHead * 4;
                stat[0] = keep;
                stat[1] = vscale;
            }
        }
        __syncthreads();
        // ---- values: O^T[channel, head] += V^T . P^T
        {
            const float *stat = reinterpret_cast<const float *>(smem + L::STAT) + n * 4;
            const float keep = stat[0];
            const float vscale = stat[1];
            i32x4 pw[TILE / 64];
#pragma unroll
            for (int hh = 0; hh < TILE / 64; ++hh) {
                pw[hh] = *reinterpret_cast<const i32x4 *>(smem + L::P + n * P_PITCH + hh * 64 + kg * 16);
            }
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const int cb = (wave * CT + ct) * 16;
                i32x4 iacc = {0, 0, 0, 0};
#pragma unroll
                for (int hh = 0; hh < TILE / 64; ++hh) {
                    // the transposing read hands lane (channel n, kg) the bytes of tokens r .. r + 7 when lane n of
                    // the group points at token r + n / 2, channels (n % 2) * 8 .. + 8
                    const unsigned char *vp =
                        smem + L::V + (hh * 64 + kg * 16 + (n >> 1)) * L::PITCH + cb + (n & 1) * 8;
                    const i32x2 lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) i32x2 *)(vp));
                    const i32x2 hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                        (__attribute__((address_space(3))) i32x2 *)(vp + 8 * L::PITCH));
                    const i32x4 vt = i32x4{lo[0], lo[1], hi[0], hi[1]};
                    iacc = __builtin_amdgcn_mfma_i32_16x16x64_i8(vt, pw[hh], iacc, 0, 0, 0);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    acc[ct][e] = acc[ct][e] * keep + static_cast<float>(iacc[e]) * vscale;
                }
            }
        }
        // The mask values of the next tile were asked for at the top of this pass, before its rows; they are taken
        // over here, a whole pass later, so that waiting for them does not hold anything up (loads come back in
        // order: earlier in the pass this wait would have been a wait for the rows asked for after them).
        if constexpr (MASK) {
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    maskBits[rt][e] = maskNext[rt][e];
                    asm volatile("" : "+v"(maskBits[rt][e]));
                }
            }
        }
    };
    // (pairs of tiles without a way round the second one: a path that skips it would reach the loop's head with the
    // first one's requests still on their way, and the compiler would wait for them there on every round)
    int tile = 0;
    for (; tile + 1 < numTiles; tile += 2) {
        pass(tile, kA, vA, kB, vB);
        pass(tile + 1, kB, vB, kA, vA);
    }
    if (tile < numTiles) {
        pass(tile, kA, vA, kB, vB);
    }
    // ---- the rows: acc / sum, to the output or, for a piece of a sequence, to its partial row with log(sum) + max
    if (tid % CH == 0) {
        float *stat = reinterpret_cast<float *>(smem + L::STAT) + smHead * 4;
        stat[2] = runSum > 0.0f ? 1.0f / runSum : 0.0f;
        stat[3] = runSum > 0.0f ? __logf(runSum) + runMax : -INFINITY;
    }
    __syncthreads();
    const float inv = reinterpret_cast<const float *>(smem + L::STAT)[n * 4 + 2];
    if (row.partial >= 0) {
        const int64_t slot = (static_cast<int64_t>(row.partial) * a.G + g) * headTiles + ht;
        float *prow = a.partO + (slot * HT + n) * D + kg * 4;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            *reinterpret_cast<f32x4 *>(prow + (wave * CT + ct) * 16) = acc[ct] * inv;
        }
        if (tid < HT) {
            a.partLse[slot * HT + tid] = reinterpret_cast<const float *>(smem + L::STAT)[tid * 4 + 3];
        }
    } else if (liveHead) {
        uint16_t *orow = reinterpret_cast<uint16_t *>(a.out) + (static_cast<int64_t>(row.qRow) * a.H + h0 + n) * D + kg * 4;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            uint16_t bits[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float o = acc[ct][e] * inv;
                bits[e] = a.bf16 ? FloatToBf16(o) : FloatToHalfBits(o);
            }
            uint2 w;
            w.x = static_cast<uint32_t>(bits[0]) | (static_cast<uint32_t>(bits[1]) << 16);
            w.y = static_cast<uint32_t>(bits[2]) | (static_cast<uint32_t>(bits[3]) << 16);
            *reinterpret_cast<uint2 *>(orow + (wave * CT + ct) * 16) = w;
        }
    }
}

// Joins the pieces of a cut sequence: out = sum_p exp(lse_p - L) O_p, L = log sum_p exp(lse_p) (reference golden
// test_paged_attention_common.py:217-228). grid.x = (cut sequence, head); a thread takes channels of the row.
constexpr int MERGE_THREADS = 128;
__global__ __launch_bounds__(MERGE_THREADS) void PaInt8QMergeKernel(const Args a, int D)
{
    const MergeRow m = a.mergeRows[blockIdx.x / a.H];
    const int h = blockIdx.x % a.H;
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
    for (int p = 0; p < m.numPartials; ++p) {
        total += weightOf(a.partLse[first + p * perPartial]);
    }
    const float inv = total > 0.0f ? 1.0f / total : 0.0f;
    uint16_t *orow = reinterpret_cast<uint16_t *>(a.out) + (static_cast<int64_t>(m.qRow) * a.H + h) * D;
    for (int d = threadIdx.x; d < D; d += MERGE_THREADS) {
        float acc = 0.0f;
        for (int p = 0; p < m.numPartials; ++p) {
            acc += weightOf(a.partLse[first + p * perPartial]) * a.partO[(first + p * perPartial) * D + d];
        }
        const float o = acc * inv;
        orow[d] = a.bf16 ? FloatToBf16(o) : FloatToHalfBits(o);
    }
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
            rows->push_back(Row{b, 0, ctx, static_cast<int32_t>(qRow), b, -1, {0, 0}});
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
    std::vector<Row> pieces;     // eight equal parts, one per XCD, padded with empty pieces
    std::vector<MergeRow> merges;
    int64_t numPartials = 0;     // partial rows (each holds kvHeads x headTiles x 16 head rows)
    uint64_t mergeOffset = 0, partOOffset = 0, partLseOffset = 0, bytes = 0;
};

// Cuts the sequences into pieces of whole tiles and deals them out to the eight parts of the table in turn from the
// longest to the shortest (every part starts with its longest piece, and the parts carry about the same number of
// tokens). The piece length aims at four workgroups for each of the 1024 places the chip has for them (256 CUs, four
// workgroups of this kernel each), at no less than four tiles and at no more than MAX_PIECE_TILES.
Layout PlanPieces(const AtbmiPaInt8QCall *c, const std::vector<Row> &seqs)
{
    Layout lay;
    const int64_t headTiles = (c->numHeads / c->numKvHeads + HT - 1) / HT;
    const int64_t perPiece = static_cast<int64_t>(c->numKvHeads) * headTiles; // workgroups of one piece
    int64_t tiles = 0;
    for (const Row &r : seqs) {
        tiles += (r.tokEnd + TILE - 1) / TILE;
    }
    const int64_t target = 4 * 1024;
    const int64_t chunk = std::min<int64_t>(
        MAX_PIECE_TILES, c->pieceTiles > 0 ? c->pieceTiles : std::max<int64_t>(4, (tiles * perPiece + target - 1) / target));
    for (const Row &r : seqs) {
        const int64_t n = (r.tokEnd + TILE - 1) / TILE;
        const int64_t parts = (n + chunk - 1) / chunk;
        const int64_t each = (n + parts - 1) / parts;
        if (parts > 1) {
            lay.merges.push_back(MergeRow{r.qRow, static_cast<int32_t>(lay.numPartials), 0, 0});
        }
        for (int64_t i = 0; i * each < n; ++i) {
            Row piece = r;
            piece.tokBegin = static_cast<int32_t>(i * each * TILE);
            piece.tokEnd = static_cast<int32_t>(std::min<int64_t>(r.tokEnd, (i + 1) * each * TILE));
            piece.partial = parts > 1 ? static_cast<int32_t>(lay.numPartials++) : -1;
            if (parts > 1) {
                ++lay.merges.back().numPartials;
            }
            lay.pieces.push_back(piece);
        }
    }
    std::stable_sort(lay.pieces.begin(), lay.pieces.end(), [](const Row &x, const Row &y) {
        return x.tokEnd - x.tokBegin > y.tokEnd - y.tokBegin;
    });
    const size_t each = (lay.pieces.size() + 7) / 8;
    std::vector<Row> table(each * 8, Row{0, 0, 0, 0, 0, -1, {0, 0}});
    for (size_t i = 0; i < lay.pieces.size(); ++i) {
        table[(i % 8) * each + i / 8] = lay.pieces[i];
    }
    lay.pieces.swap(table);
    auto align = [](uint64_t v) { return (v + 255) / 256 * 256; };
    lay.mergeOffset = align(lay.pieces.size() * sizeof(Row));
    lay.partOOffset = align(lay.mergeOffset + lay.merges.size() * sizeof(MergeRow));
    const uint64_t headRows = static_cast<uint64_t>(lay.numPartials) * perPiece * HT;
    lay.partLseOffset = align(lay.partOOffset + headRows * c->headDim * sizeof(float));
    lay.bytes = lay.partLseOffset + headRows * sizeof(float);
    return lay;
}

template <int D> int Launch(const AtbmiPaInt8QCall *call, const Args &a, int64_t grid, int64_t numMerges, hipStream_t s)
{
    const bool narrow = call->numHeads / call->numKvHeads <= HT / 2;
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
            with(narrow, [&](auto nar) {
                with(call->blockSize % TILE == 0, [&](auto who) {
                    kernel = PaInt8QKernel<D, decltype(off)::value, decltype(msk)::value, decltype(nar)::value, decltype(who)::value>;
                });
            });
        });
    });
    int rc = ConfigureKernelLds(reinterpret_cast<const void *>(kernel), Lds<D>::BYTES);
    if (rc != OK) {
        return rc;
    }
    TimedLaunch timed;
    rc = TimedLaunchBegin(s, &timed);
    if (rc != OK) {
        return rc;
    }
    kernel<<<static_cast<unsigned>(grid), THREADS, Lds<D>::BYTES, s>>>(a);
    ATBMI_HIP_CHECK(hipGetLastError());
    rc = TimedLaunchKernelDone(s, timed);
    if (rc != OK) {
        return rc;
    }
    if (numMerges > 0) {
        const unsigned mergeGrid = static_cast<unsigned>(numMerges * a.H);
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
    const int group = call->numHeads / call->numKvHeads;
    const int headTiles = (group + int8q::HT - 1) / int8q::HT;
    const int64_t grid = static_cast<int64_t>(lay.pieces.size()) * call->numKvHeads * headTiles; // (a multiple of 8)
    if (grid > 0x7fffffffLL || static_cast<int64_t>(lay.merges.size()) * call->numHeads > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "pa_int8q: %lld workgroups", (long long)grid);
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
    a.partO = reinterpret_cast<float *>(ws + lay.partOOffset);
    a.partLse = reinterpret_cast<float *>(ws + lay.partLseOffset);
    a.maskSeqStride = call->maskSeqStride;
    a.maskHeadStride = call->maskHeadStride;
    a.H = call->numHeads;
    a.G = call->numKvHeads;
    a.numRows = static_cast<int32_t>(lay.pieces.size());
    a.maxBlocksPerSeq = call->maxBlocksPerSeq;
    a.blockSize = call->blockSize;
    a.bf16 = call->outDtype == ATBMI_BF16 ? 1 : 0;
    a.qkScale = call->qkScale;
    switch (call->headDim) {
        case 64: return int8q::Launch<64>(call, a, grid, static_cast<int64_t>(lay.merges.size()), s);
        case 128: return int8q::Launch<128>(call, a, grid, static_cast<int64_t>(lay.merges.size()), s);
        default: return int8q::Launch<256>(call, a, grid, static_cast<int64_t>(lay.merges.size()), s);
    }
}
