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
// A workgroup of four waves owns one sequence, one KV head and up to 16 of its query heads and walks the context
// tile by tile. Key and value rows of tile i + 1 are requested into registers before the arithmetic of tile i and
// stored to LDS after it, token-major with a padded pitch.
//   scores  wave w for tokens 32 w .. 32 w + 31: S^T[token, head] = K . Q^T (K rows from LDS as A, the query
//           resident in registers as B);
//   softmax 16 lanes a head, 8 tokens a lane; int8 weights P[head][token] go to LDS;
//   values  wave w for channels (D / 4) w .. : O^T[channel, head] += V^T . P^T, V^T read from the token-major rows by
//           the transposing ds_read_b64_tr_b8, P^T as 16 consecutive bytes of a head's weights.
// Operand layout of v_mfma_i32_16x16x64_i8: lane (n = lane % 16, kg = lane / 16) supplies the 16 contraction values
// 16 kg .. 16 kg + 15 of row n (A) / column n (B) and receives D[4 kg + e][n], e = 0 .. 3.
// One pass per sequence (no split over the context): the launch has batch x kvHeads x ceil(group / 16) workgroups.
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
constexpr int CH = THREADS / HT;  // softmax: lanes a head
constexpr int TPL = TILE / CH;    // softmax: tokens a lane
constexpr int S_PITCH = (TILE + 4) * 4; // 16 heads' 16-byte writes touch every bank once
constexpr int P_PITCH = TILE + 16;      // likewise for 16 heads' 16-byte reads
static_assert(CH == 16 && TPL == 8 && TILE == NWAVES * 32, "four waves share a tile this way");

template <int D> struct Lds {
    static constexpr int PITCH = D + 16; // row pitch of the key and value tiles: 16 rows' 16-byte reads touch every bank once
    static constexpr int K = 0;
    static constexpr int V = K + TILE * PITCH;
    static constexpr int S = V + TILE * PITCH;   // [16] fp32 scores
    static constexpr int P = S + HT * S_PITCH;   // [16] int8 weights
    static constexpr int STAT = P + HT * P_PITCH; // [16] {keep, value scale, 1 / sum, -}
    static constexpr int BYTES = STAT + HT * 16;
    static_assert(BYTES <= 160 * 1024 && S % 16 == 0 && P % 16 == 0 && STAT % 16 == 0, "LDS layout");
};

// One sequence with a non-empty context: its block-table row, context length, row of query / out, mask row.
struct Row {
    int32_t tableRow;
    int32_t ctxLen;
    int32_t qRow;
    int32_t maskRow;
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
    int64_t maskSeqStride;  // elements between the mask rows of two sequences (0: shared)
    int64_t maskHeadStride; // elements between the mask rows of two heads (0: shared)
    int32_t H;
    int32_t G;
    int32_t numRows;
    int32_t maxBlocksPerSeq;
    int32_t blockSize;
    float qkScale;
};

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

template <int D, bool BF16, bool OFFLINE>
__global__ __launch_bounds__(THREADS) void PaInt8QKernel(const Args a)
{
    using L = Lds<D>;
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
    // workgroups go round the eight XCDs: the workgroups of a sequence, whose KV heads lie side by side in the
    // cache rows, take neighbouring places on one XCD and share its L2
    const int work = (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8;
    if (work >= a.numRows * a.G * headTiles) {
        return;
    }
    const Row row = a.rows[work / (a.G * headTiles)];
    const int g = (work / headTiles) % a.G;
    const int ht = work % headTiles;
    const int nh = min(HT, group - ht * HT); // heads past the last one compute on zeros and store nothing
    const int h0 = g * group + ht * HT;
    const int32_t *table = a.tables + static_cast<int64_t>(row.tableRow) * a.maxBlocksPerSeq;
    const int numTiles = (row.ctxLen + TILE - 1) / TILE;
    const int64_t slotBytes = static_cast<int64_t>(a.G) * D; // one token's rows of all KV heads

    // ---- requests for a tile: this thread's pieces of the key and value rows (tokens past the context repeat the last one)
    const int ldTok = tid / PPR;
    const int ldPiece = tid % PPR;
    auto requestTile = [&](int t0, u32x4(&kr)[PASSES], u32x4(&vr)[PASSES]) {
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            const int tok = min(t0 + p * ROWS_PER_PASS + ldTok, row.ctxLen - 1);
            const int64_t slot = static_cast<int64_t>(table[tok / a.blockSize]) * a.blockSize + tok % a.blockSize;
            const int64_t at = slot * slotBytes + g * D + ldPiece * 16;
            kr[p] = *reinterpret_cast<const u32x4 *>(a.k8 + at);
            vr[p] = *reinterpret_cast<const u32x4 *>(a.v8 + at);
        }
    };
    auto storeTile = [&](const u32x4(&kr)[PASSES], const u32x4(&vr)[PASSES]) {
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            const int at = (p * ROWS_PER_PASS + ldTok) * L::PITCH + ldPiece * 16;
            *reinterpret_cast<u32x4 *>(smem + L::K + at) = kr[p];
            *reinterpret_cast<u32x4 *>(smem + L::V + at) = vr[p];
        }
    };
    u32x4 kNext[PASSES], vNext[PASSES];
    requestTile(0, kNext, vNext);

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
    if (a.mask) {
        maskRow = reinterpret_cast<const uint16_t *>(a.mask) + static_cast<int64_t>(row.maskRow) * a.maskSeqStride +
                  static_cast<int64_t>(hn) * a.maskHeadStride;
    }
    // softmax: lane (head tid / 16, tokens 4 (tid % 16) .. + 4 and 64 more on); a head's lanes all hold its running
    // maximum and sum
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
    storeTile(kNext, vNext);
    __syncthreads();

    for (int i = 0; i < numTiles; ++i) {
        const int t0 = i * TILE;
        const bool more = i + 1 < numTiles;
        if (more) {
            requestTile(t0 + TILE, kNext, vNext);
        }
        // ---- scores of tokens 32 wave .. + 31
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
            const int tokBase = wave * 32 + rt * 16;
            const int tok = t0 + tokBase + kg * 4; // this lane's four tokens
            uint32_t maskBits[4] = {0u, 0u, 0u, 0u};
            if (maskRow) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    maskBits[e] = maskRow[min(tok + e, row.ctxLen - 1)];
                }
            }
            i32x4 dot = {0, 0, 0, 0};
#pragma unroll
            for (int j = 0; j < D / 64; ++j) {
                const i32x4 kk = *reinterpret_cast<const i32x4 *>(smem + L::K + (tokBase + n) * L::PITCH + j * 64 + kg * 16);
                dot = __builtin_amdgcn_mfma_i32_16x16x64_i8(kk, q8[j], dot, 0, 0, 0);
            }
            f32x4 sc;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const bool live = tok + e < row.ctxLen;
                float bias = 0.0f;
                if (maskRow) {
                    bias = BF16 ? Bf16ToFloat(static_cast<uint16_t>(maskBits[e]))
                                : HalfBitsToFloat(static_cast<uint16_t>(maskBits[e]));
                }
                const float x = static_cast<float>(dot[e]) * descale * a.qkScale + bias;
                sc[e] = live ? x : -INFINITY;
            }
            *reinterpret_cast<f32x4 *>(smem + L::S + n * S_PITCH + (tokBase + kg * 4) * 4) = sc;
        }
        __syncthreads();
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
            tileMax = RowMax(tileMax);
            const float newMax = fmaxf(runMax, tileMax);
            const bool any = newMax > -INFINITY; // (a mask of -inf can hide everything seen so far)
            float sum = 0.0f, wmax = 0.0f;
#pragma unroll
            for (int k = 0; k < TPL; ++k) {
                w[k] = any ? __expf(w[k] - newMax) : 0.0f;
                sum += w[k];
                wmax = fmaxf(wmax, w[k]);
            }
            sum = RowSum(sum);
            wmax = RowMax(wmax);
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
        __syncthreads(); // everybody has left the tile
        if (more) {
            storeTile(kNext, vNext);
            __syncthreads();
        }
    }
    // ---- the rows: acc / sum
    if (tid % CH == 0) {
        float *stat = reinterpret_cast<float *>(smem + L::STAT) + smHead * 4;
        stat[2] = runSum > 0.0f ? 1.0f / runSum : 0.0f;
    }
    __syncthreads();
    if (liveHead) {
        const float inv = reinterpret_cast<const float *>(smem + L::STAT)[n * 4 + 2];
        uint16_t *orow = reinterpret_cast<uint16_t *>(a.out) + (static_cast<int64_t>(row.qRow) * a.H + h0 + n) * D + kg * 4;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            uint16_t bits[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float o = acc[ct][e] * inv;
                bits[e] = BF16 ? FloatToBf16(o) : FloatToHalfBits(o);
            }
            uint2 w;
            w.x = static_cast<uint32_t>(bits[0]) | (static_cast<uint32_t>(bits[1]) << 16);
            w.y = static_cast<uint32_t>(bits[2]) | (static_cast<uint32_t>(bits[3]) << 16);
            *reinterpret_cast<uint2 *>(orow + (wave * CT + ct) * 16) = w;
        }
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
        (c->hasMask && c->maskLen <= 0) || c->maskSeqStride < 0 || c->maskHeadStride < 0) {
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
            rows->push_back(Row{b, ctx, static_cast<int32_t>(qRow), b});
        }
        ++qRow;
    }
    if (qRow > c->numQueryRows) {
        return Fail(ERR_INVALID_PARAM, "pa_int8q: the lengths ask for %lld query rows, the tensors hold %d",
                    (long long)qRow, c->numQueryRows);
    }
    return OK;
}

template <int D> int Launch(const AtbmiPaInt8QCall *call, const Args &a, int64_t grid, hipStream_t s)
{
    const bool bf16 = call->outDtype == ATBMI_BF16;
    const bool offline = call->offline != 0;
    auto kernel = bf16 ? (offline ? PaInt8QKernel<D, true, true> : PaInt8QKernel<D, true, false>)
                       : (offline ? PaInt8QKernel<D, false, true> : PaInt8QKernel<D, false, false>);
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
    return rc != OK ? rc : TimedLaunchEnd(s, timed, false);
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
    *bytes = rows.size() * sizeof(int8q::Row);
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
    const size_t bytes = rows.size() * sizeof(int8q::Row);
    if (!workspaceDevice || workspaceBytes < bytes) {
        return Fail(ERR_INVALID_PARAM, "pa_int8q: workspace of %llu bytes, %llu needed", (unsigned long long)workspaceBytes,
                    (unsigned long long)bytes);
    }
    const int group = call->numHeads / call->numKvHeads;
    const int headTiles = (group + int8q::HT - 1) / int8q::HT;
    const int64_t grid = (static_cast<int64_t>(rows.size()) * call->numKvHeads * headTiles + 7) / 8 * 8;
    if (grid > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "pa_int8q: %lld workgroups", (long long)grid);
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    rc = UploadTable(rows.data(), bytes, workspaceDevice, s);
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
    a.rows = static_cast<const int8q::Row *>(workspaceDevice);
    a.maskSeqStride = call->maskSeqStride;
    a.maskHeadStride = call->maskHeadStride;
    a.H = call->numHeads;
    a.G = call->numKvHeads;
    a.numRows = static_cast<int32_t>(rows.size());
    a.maxBlocksPerSeq = call->maxBlocksPerSeq;
    a.blockSize = call->blockSize;
    a.qkScale = call->qkScale;
    switch (call->headDim) {
        case 64: return int8q::Launch<64>(call, a, grid, s);
        case 128: return int8q::Launch<128>(call, a, grid, s);
        default: return int8q::Launch<256>(call, a, grid, s);
    }
}
