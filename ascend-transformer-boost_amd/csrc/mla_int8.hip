// Decode attention of MultiLatentAttention over the int8 fractal-NZ cache (cacheMode INT8_NZCACHE) for gfx950
// (reference operator src/ops/ops_infer/multi_latent_attention, device kernel
// src/kernels/mixkernels/multi_latent_attention/op_kernel/mla_int8.cce; golden
// tests/apitest/opstest/python/operations/multi_latent_attention/test_multi_latent_attention_int8nz.py:115-121,
// 179-262, 276-286).
//
// Arithmetic, per query row and head, as the golden has it:
//   score   = (int32 dot of the int8 query and the int8 cache row) x qkDescale[head]  +  fp32 dot of the 64
//             rotary channels, the sum times qkScale, plus the mask;
//   weights = exp(score - running max), quantised per tile of 128 tokens (one cache block) to int8 against the
//             largest weight of the tile: rint(fp16(w / (wmax / 127)));
//   values  = int32 dot of the int8 weights and the int8 cache rows (the first 512 channels are the values),
//             times pvDescale[head] x wmax / 127; tiles are joined by the usual online rescaling, the
//             denominator adds up the unquantised weights.
// Every integer product is exact (v_dot4_i32_i8 into int32; a tile's sums stay below 2^24).
//
// A workgroup of eight waves owns one query row and 16 heads (8 when there are no more) and walks the row's context block by block:
//   load    the block's int8 rows and rotary rows from the NZ layout into row-major LDS tiles;
//   scores  thread (token, quarter of the heads): its row against its query heads, each cache dword reused for
//           all of them;
//   softmax one wave per head (or per two), two tokens a lane;
//   values  thread (4 channels, quarter of the heads): four cache rows at a time, their bytes transposed in
//           registers so that one dot4 covers four tokens.
// Four barriers a block and no overlap of the load with the arithmetic: built for exact agreement with the
// golden first.
#include <vector>
#include "pa_internal.h"
#include "upload_ring.h"

namespace atbmi {
namespace mlaint8 {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int TILE = 128;            // tokens per tile = the block size of the cache
constexpr int DN = 512;              // int8 channels (keys and values)
constexpr int DR = 64;               // rotary channels (16-bit)
constexpr int THREADS = 512;         // eight waves, two a SIMD: one's LDS round trips hide behind the other's arithmetic
constexpr int K_PITCH = DN + 16;     // bytes; 16-byte reads of 16 consecutive rows touch every bank once
constexpr int R_PITCH = DR * 2 + 16;
// LDS of a workgroup with HT heads: the two tiles, the query (int8 rows, fp32 rotary rows), the tile's scores,
// its int8 weights and four numbers per head {keep, value scale, 1 / sum, lse}.
template <int HT> struct Lds {
    static constexpr int K = 0;
    static constexpr int R = K + TILE * K_PITCH;
    static constexpr int Q8 = R + TILE * R_PITCH;
    static constexpr int QR = Q8 + HT * DN;
    static constexpr int S = QR + HT * DR * 4;
    static constexpr int P = S + HT * TILE * 4;
    static constexpr int STAT = P + HT * TILE;
    static constexpr int BYTES = STAT + HT * 16;
    static_assert(BYTES <= 160 * 1024 && R % 16 == 0 && Q8 % 16 == 0 && S % 16 == 0, "LDS layout");
};

// One query row: its sequence's block-table row and context length, the row of query / out, the mask row.
struct Row {
    int32_t tableRow;
    int32_t ctxLen;
    int32_t qRow;
    int32_t pad;
};

struct Args {
    const int8_t *q8;
    const void *qRope;
    const int8_t *kv8;
    const void *kRope;
    const int32_t *tables;
    const float *qkDescale;
    const float *pvDescale;
    const void *mask;
    void *out;
    float *lse;
    const Row *rows;
    int32_t H;
    int32_t maxBlocksPerSeq;
    int32_t maskLen;
    int32_t bf16;
    float qkScale;
};

__device__ __forceinline__ float Load16AsFloat(uint32_t bits, bool bf16)
{
    return bf16 ? Bf16ToFloat(static_cast<uint16_t>(bits)) : HalfBitsToFloat(static_cast<uint16_t>(bits));
}

// HT heads per workgroup (8 or 16): a thread takes HT / 4 heads in the score and value phases, a wave HT / 8
// in the softmax.
template <int HT> __global__ __launch_bounds__(THREADS) void MlaInt8Kernel(const Args a)
{
    using L = Lds<HT>;
    constexpr int LDS_K = L::K, LDS_R = L::R, LDS_Q8 = L::Q8, LDS_QR = L::QR, LDS_S = L::S, LDS_P = L::P,
                  LDS_STAT = L::STAT;
    constexpr int HPT = HT / 4; // heads per thread
    constexpr int HPW = HT / 8; // heads per wave
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = tid / WAVE;
    const int headTiles = a.H / HT;
    const Row row = a.rows[blockIdx.x / headTiles];
    const int h0 = (blockIdx.x % headTiles) * HT;
    const bool bf16 = a.bf16 != 0;
    const int32_t *table = a.tables + static_cast<int64_t>(row.tableRow) * a.maxBlocksPerSeq;

    // ---- the query of the eight heads: int8 rows as they are, rotary rows as fp32
    {
        const int8_t *q8 = a.q8 + (static_cast<int64_t>(row.qRow) * a.H + h0) * DN;
        if (tid < HT * DN / 16) {
            *reinterpret_cast<u32x4 *>(smem + LDS_Q8 + tid * 16) = *reinterpret_cast<const u32x4 *>(q8 + tid * 16);
        }
        const uint16_t *qr = reinterpret_cast<const uint16_t *>(a.qRope) + (static_cast<int64_t>(row.qRow) * a.H + h0) * DR;
        float *dst = reinterpret_cast<float *>(smem + LDS_QR);
        for (int i = tid; i < HT * DR; i += THREADS) {
            dst[i] = Load16AsFloat(qr[i], bf16);
        }
    }

    // scores: thread (token, group of four heads)
    const int tok = tid & (TILE - 1);
    const int hs = (tid / TILE) * HPT;
    // softmax: this wave's two heads; the running maximum, sum and per-tile factors live in its lanes
    float runMax[HPW], runSum[HPW];
#pragma unroll
    for (int i = 0; i < HPW; ++i) {
        runMax[i] = -INFINITY;
        runSum[i] = 0.0f;
    }
    // values: thread (4 channels, group of four heads)
    const int col = tid & (TILE - 1); // dword column of a cache row
    float acc[HPT][4];
#pragma unroll
    for (int h = 0; h < HPT; ++h) {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            acc[h][b] = 0.0f;
        }
    }
    float descale[HPT];
#pragma unroll
    for (int h = 0; h < HPT; ++h) {
        descale[h] = a.qkDescale[h0 + hs + h];
    }
    const uint16_t *maskRow = a.mask ? reinterpret_cast<const uint16_t *>(a.mask) + static_cast<int64_t>(row.qRow) * a.maskLen
                                     : nullptr;

    for (int t0 = 0; t0 < row.ctxLen; t0 += TILE) {
        const int64_t blk = table[t0 / TILE];
        __syncthreads(); // the tiles (and, the first time, the query) are free / written
        // ---- the block, NZ [channels / 32][128][32] int8 and [4][128][16] 16-bit, into row-major tiles
        {
            const u32x4 *src = reinterpret_cast<const u32x4 *>(a.kv8 + blk * (TILE * DN));
#pragma unroll 4
            for (int v = tid; v < TILE * DN / 16; v += THREADS) {
                const int slab = v / (TILE * 2);
                const int r = (v % (TILE * 2)) / 2;
                *reinterpret_cast<u32x4 *>(smem + LDS_K + r * K_PITCH + slab * 32 + (v & 1) * 16) =
                    src[v];
            }
            const u32x4 *srcR = reinterpret_cast<const u32x4 *>(reinterpret_cast<const unsigned char *>(a.kRope) +
                                                                blk * (TILE * DR * 2));
            for (int v = tid; v < TILE * DR * 2 / 16; v += THREADS) {
                const int slab = v / (TILE * 2);
                const int r = (v % (TILE * 2)) / 2;
                *reinterpret_cast<u32x4 *>(smem + LDS_R + r * R_PITCH + slab * 32 + (v & 1) * 16) =
                    srcR[v];
            }
        }
        __syncthreads();
        // ---- scores of token `tok` for heads hs .. hs + 3
        {
            int dot[HPT] = {};
            const unsigned char *krow = smem + LDS_K + tok * K_PITCH;
#pragma unroll 4
            for (int j = 0; j < DN / 16; ++j) {
                const u32x4 kk = *reinterpret_cast<const u32x4 *>(krow + j * 16);
#pragma unroll
                for (int h = 0; h < HPT; ++h) {
                    const u32x4 qq = *reinterpret_cast<const u32x4 *>(smem + LDS_Q8 + (hs + h) * DN + j * 16);
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        dot[h] = __builtin_amdgcn_sdot4(static_cast<int>(kk[d]), static_cast<int>(qq[d]), dot[h], false);
                    }
                }
            }
            float rope[HPT] = {};
            const unsigned char *rrow = smem + LDS_R + tok * R_PITCH;
#pragma unroll 2
            for (int j = 0; j < DR / 8; ++j) {
                const u32x4 rr = *reinterpret_cast<const u32x4 *>(rrow + j * 16);
                float kf[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    kf[e] = Load16AsFloat((e & 1) ? (rr[e >> 1] >> 16) : (rr[e >> 1] & 0xffffu), bf16);
                }
#pragma unroll
                for (int h = 0; h < HPT; ++h) {
                    const float *qf = reinterpret_cast<const float *>(smem + LDS_QR) + (hs + h) * DR + j * 8;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        rope[h] = __builtin_fmaf(qf[e], kf[e], rope[h]);
                    }
                }
            }
            const bool live = t0 + tok < row.ctxLen;
            const float bias = (maskRow && live) ? Load16AsFloat(maskRow[t0 + tok], bf16) : 0.0f;
#pragma unroll
            for (int h = 0; h < HPT; ++h) {
                float s = (static_cast<float>(dot[h]) * descale[h] + rope[h]) * a.qkScale + bias;
                reinterpret_cast<float *>(smem + LDS_S)[(hs + h) * TILE + tok] = live ? s : -INFINITY;
            }
        }
        __syncthreads();
        // ---- weights of the tile for heads 2 wave, 2 wave + 1
#pragma unroll
        for (int i = 0; i < HPW; ++i) {
            const int h = HPW * wave + i;
            const float *srow = reinterpret_cast<const float *>(smem + LDS_S) + h * TILE;
            const float s0 = srow[lane], s1 = srow[lane + WAVE];
            float tileMax = fmaxf(s0, s1);
            for (int off = 32; off > 0; off >>= 1) {
                tileMax = fmaxf(tileMax, __shfl_xor(tileMax, off));
            }
            const float newMax = fmaxf(runMax[i], tileMax);
            const bool any = newMax > -INFINITY; // (a mask of -inf can hide everything seen so far)
            const float w0 = any ? __expf(s0 - newMax) : 0.0f;
            const float w1 = any ? __expf(s1 - newMax) : 0.0f;
            float sum = w0 + w1;
            float wmax = fmaxf(w0, w1);
            for (int off = 32; off > 0; off >>= 1) {
                sum += __shfl_xor(sum, off);
                wmax = fmaxf(wmax, __shfl_xor(wmax, off));
            }
            const float keep = (any && runMax[i] > -INFINITY) ? __expf(runMax[i] - newMax) : 0.0f;
            runSum[i] = runSum[i] * keep + sum;
            runMax[i] = newMax;
            const float step = wmax / 127.0f;
            int p0 = 0, p1 = 0;
            if (wmax > 0.0f) {
                p0 = static_cast<int>(rintf(static_cast<float>(static_cast<_Float16>(__fdiv_rn(w0, step)))));
                p1 = static_cast<int>(rintf(static_cast<float>(static_cast<_Float16>(__fdiv_rn(w1, step)))));
            }
            reinterpret_cast<int8_t *>(smem + LDS_P)[h * TILE + lane] = static_cast<int8_t>(p0);
            reinterpret_cast<int8_t *>(smem + LDS_P)[h * TILE + lane + WAVE] = static_cast<int8_t>(p1);
            if (lane == 0) {
                float *stat = reinterpret_cast<float *>(smem + LDS_STAT) + h * 4;
                stat[0] = keep;
                stat[1] = a.pvDescale[h0 + h] * wmax / 127.0f;
            }
        }
        __syncthreads();
        // ---- values: channels 4 col .. 4 col + 3 for heads hs .. hs + 3
        {
            int iacc[HPT][4];
#pragma unroll
            for (int h = 0; h < HPT; ++h) {
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    iacc[h][b] = 0;
                }
            }
            const unsigned char *kcol = smem + LDS_K + col * 4;
#pragma unroll 2
            for (int t4 = 0; t4 < TILE / 4; ++t4) {
                uint32_t r[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    r[i] = *reinterpret_cast<const uint32_t *>(kcol + (t4 * 4 + i) * K_PITCH);
                }
                // bytes of four rows transposed: kt[b] = {r0.b, r1.b, r2.b, r3.b}
                const uint32_t x01lo = __builtin_amdgcn_perm(r[1], r[0], 0x05010400u);
                const uint32_t x01hi = __builtin_amdgcn_perm(r[1], r[0], 0x07030602u);
                const uint32_t x23lo = __builtin_amdgcn_perm(r[3], r[2], 0x05010400u);
                const uint32_t x23hi = __builtin_amdgcn_perm(r[3], r[2], 0x07030602u);
                uint32_t kt[4];
                kt[0] = __builtin_amdgcn_perm(x23lo, x01lo, 0x05040100u);
                kt[1] = __builtin_amdgcn_perm(x23lo, x01lo, 0x07060302u);
                kt[2] = __builtin_amdgcn_perm(x23hi, x01hi, 0x05040100u);
                kt[3] = __builtin_amdgcn_perm(x23hi, x01hi, 0x07060302u);
#pragma unroll
                for (int h = 0; h < HPT; ++h) {
                    const uint32_t pw = *reinterpret_cast<const uint32_t *>(smem + LDS_P + (hs + h) * TILE + t4 * 4);
#pragma unroll
                    for (int b = 0; b < 4; ++b) {
                        iacc[h][b] = __builtin_amdgcn_sdot4(static_cast<int>(kt[b]), static_cast<int>(pw), iacc[h][b], false);
                    }
                }
            }
#pragma unroll
            for (int h = 0; h < HPT; ++h) {
                const float *stat = reinterpret_cast<const float *>(smem + LDS_STAT) + (hs + h) * 4;
                const float keep = stat[0], vscale = stat[1];
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    acc[h][b] = acc[h][b] * keep + static_cast<float>(iacc[h][b]) * vscale;
                }
            }
        }
    }
    // ---- the rows: acc / sum, and log(sum) + max
    __syncthreads();
    if (lane == 0) {
#pragma unroll
        for (int i = 0; i < HPW; ++i) {
            float *stat = reinterpret_cast<float *>(smem + LDS_STAT) + (HPW * wave + i) * 4;
            stat[2] = runSum[i] > 0.0f ? 1.0f / runSum[i] : 0.0f;
            stat[3] = runSum[i] > 0.0f ? logf(runSum[i]) + runMax[i] : -INFINITY;
        }
    }
    __syncthreads();
#pragma unroll
    for (int h = 0; h < HPT; ++h) {
        const float inv = reinterpret_cast<const float *>(smem + LDS_STAT)[(hs + h) * 4 + 2];
        uint16_t bits[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const float o = acc[h][b] * inv;
            bits[b] = bf16 ? FloatToBf16(o) : FloatToHalfBits(o);
        }
        uint2 w;
        w.x = static_cast<uint32_t>(bits[0]) | (static_cast<uint32_t>(bits[1]) << 16);
        w.y = static_cast<uint32_t>(bits[2]) | (static_cast<uint32_t>(bits[3]) << 16);
        uint16_t *dst = reinterpret_cast<uint16_t *>(a.out) + (static_cast<int64_t>(row.qRow) * a.H + h0 + hs + h) * DN + col * 4;
        *reinterpret_cast<uint2 *>(dst) = w;
    }
    if (a.lse && tid < HT) {
        a.lse[static_cast<int64_t>(row.qRow) * a.H + h0 + tid] = reinterpret_cast<const float *>(smem + LDS_STAT)[tid * 4 + 3];
    }
}

// Checks the call and lists its query rows (sequences of length 0 take none).
int BuildRows(const AtbmiMlaInt8Call *c, std::vector<Row> *rows)
{
    if (!c || !c->hostContextLens) {
        return Fail(ERR_INVALID_PARAM, "mla_int8: null call or context lengths");
    }
    if (c->outDtype != ATBMI_F16 && c->outDtype != ATBMI_BF16) {
        return Fail(ERR_INVALID_PARAM, "mla_int8: the 16-bit tensors are fp16 or bf16, got %d", c->outDtype);
    }
    if (c->numHeads <= 0 || c->numHeads % 8 != 0) {
        return Fail(ERR_INVALID_PARAM, "mla_int8: %d heads (a multiple of 8)", c->numHeads);
    }
    if (c->blockSize != TILE) {
        return Fail(ERR_INVALID_PARAM, "mla_int8: block size %d (the int8 cache has blocks of %d tokens)", c->blockSize, TILE);
    }
    if (c->batch < 0 || c->numBlocks <= 0 || c->maxBlocksPerSeq <= 0 || !(c->qkScale > 0.0f) ||
        (c->hasMask && c->maskLen <= 0)) {
        return Fail(ERR_INVALID_PARAM, "mla_int8: batch %d, %d blocks, %d blocks a sequence, qkScale %g, mask length %d",
                    c->batch, c->numBlocks, c->maxBlocksPerSeq, c->qkScale, c->maskLen);
    }
    int64_t qRow = 0;
    for (int32_t b = 0; b < c->batch; ++b) {
        const int32_t ctx = c->hostContextLens[b];
        const int32_t nq = c->hostQueryLens ? c->hostQueryLens[b] : 1;
        if (ctx < 0 || nq < 0) {
            return Fail(ERR_INVALID_PARAM, "mla_int8: sequence %d has context %d and %d query tokens", b, ctx, nq);
        }
        if (ctx > static_cast<int64_t>(c->maxBlocksPerSeq) * c->blockSize) {
            return Fail(ERR_INVALID_PARAM, "mla_int8: context %d of sequence %d exceeds its %d blocks", ctx, b,
                        c->maxBlocksPerSeq);
        }
        if (c->hasMask && ctx > c->maskLen) {
            return Fail(ERR_INVALID_PARAM, "mla_int8: context %d of sequence %d exceeds the mask's %d positions", ctx, b,
                        c->maskLen);
        }
        if (ctx == 0) {
            continue;
        }
        for (int32_t i = 0; i < nq; ++i) {
            if (qRow > 0x7fffffffLL) {
                return Fail(ERR_INVALID_PARAM, "mla_int8: more than 2^31 query rows");
            }
            if (rows) {
                rows->push_back(Row{b, ctx, static_cast<int32_t>(qRow), 0});
            }
            ++qRow;
        }
    }
    if (qRow > c->numQueryRows) {
        return Fail(ERR_INVALID_PARAM, "mla_int8: the lengths ask for %lld query rows, the tensors hold %d",
                    (long long)qRow, c->numQueryRows);
    }
    return OK;
}

} // namespace mlaint8
} // namespace atbmi

using namespace atbmi;

extern "C" int atbmi_mla_int8_workspace_size(const AtbmiMlaInt8Call *call, uint64_t *bytes)
{
    if (!bytes) {
        return Fail(ERR_INVALID_PARAM, "mla_int8_workspace_size: null result pointer");
    }
    std::vector<mlaint8::Row> rows;
    const int rc = mlaint8::BuildRows(call, &rows);
    if (rc != OK) {
        return rc;
    }
    *bytes = rows.size() * sizeof(mlaint8::Row);
    return OK;
}

extern "C" int atbmi_mla_int8_decode(const AtbmiMlaInt8Call *call, void *workspaceDevice, uint64_t workspaceBytes,
                                     void *stream)
{
    std::vector<mlaint8::Row> rows;
    int rc = mlaint8::BuildRows(call, &rows);
    if (rc != OK) {
        return rc;
    }
    if (rows.empty()) {
        return OK;
    }
    if (!call->query || !call->queryRope || !call->kvCache || !call->kRopeCache || !call->blockTables ||
        !call->qkDescale || !call->pvDescale || !call->out || (call->hasMask && !call->mask)) {
        return Fail(ERR_INVALID_PARAM, "mla_int8: null tensor pointer");
    }
    const size_t bytes = rows.size() * sizeof(mlaint8::Row);
    if (!workspaceDevice || workspaceBytes < bytes) {
        return Fail(ERR_INVALID_PARAM, "mla_int8: workspace of %llu bytes, %llu needed", (unsigned long long)workspaceBytes,
                    (unsigned long long)bytes);
    }
    const int ht = call->numHeads % 16 == 0 ? 16 : 8;
    const int64_t grid = static_cast<int64_t>(rows.size()) * (call->numHeads / ht);
    if (grid > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "mla_int8: %lld workgroups", (long long)grid);
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    rc = UploadTable(rows.data(), bytes, workspaceDevice, s);
    if (rc != OK) {
        return rc;
    }
    mlaint8::Args a{};
    a.q8 = static_cast<const int8_t *>(call->query);
    a.qRope = call->queryRope;
    a.kv8 = static_cast<const int8_t *>(call->kvCache);
    a.kRope = call->kRopeCache;
    a.tables = call->blockTables;
    a.qkDescale = call->qkDescale;
    a.pvDescale = call->pvDescale;
    a.mask = call->hasMask ? call->mask : nullptr;
    a.out = call->out;
    a.lse = call->lse;
    a.rows = static_cast<const mlaint8::Row *>(workspaceDevice);
    a.H = call->numHeads;
    a.maxBlocksPerSeq = call->maxBlocksPerSeq;
    a.maskLen = call->maskLen;
    a.bf16 = call->outDtype == ATBMI_BF16 ? 1 : 0;
    a.qkScale = call->qkScale;
    auto kernel = ht == 16 ? mlaint8::MlaInt8Kernel<16> : mlaint8::MlaInt8Kernel<8>;
    const int ldsBytes = ht == 16 ? mlaint8::Lds<16>::BYTES : mlaint8::Lds<8>::BYTES;
    rc = ConfigureKernelLds(reinterpret_cast<const void *>(kernel), ldsBytes);
    if (rc != OK) {
        return rc;
    }
    kernel<<<static_cast<unsigned>(grid), mlaint8::THREADS, ldsBytes, s>>>(a);
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}
