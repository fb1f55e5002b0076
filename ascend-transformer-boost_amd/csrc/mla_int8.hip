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
// Every integer product is exact (v_mfma_i32_16x16x64_i8; a tile's sums stay below 2^24).
//
// A workgroup of eight waves owns one query row and 16 heads and walks the row's context block by block:
//   load    the block's int8 rows and rotary rows from the NZ layout into row-major LDS tiles;
//   scores  wave w for tokens 16 w .. 16 w + 15: S^T[token, head] = K . Q^T, eight int8 MFMAs over the 512
//           latent channels (K rows from LDS as A, the query resident in registers as B) and two 16-bit MFMAs
//           over the rotary channels;
//   softmax wave w for heads 2 w and 2 w + 1, two tokens a lane; int8 weights P[head][token] go to LDS;
//   values  wave w for channels 64 w .. 64 w + 63: O^T[channel, head] += V^T . P^T, V^T read from the row-major
//           tile by the transposing ds_read_b64_tr_b8 (lane (channel, kg) gets the bytes of 8 consecutive
//           tokens), P^T as 16 consecutive bytes of a head's weights.
// Operand layout of v_mfma_i32_16x16x64_i8 (checked with a probe on the device): lane (n = lane % 16, kg =
// lane / 16) supplies the 16 contraction values 16 kg .. 16 kg + 15 of row n (A) / column n (B) and receives
// D[4 kg + e][n], e = 0 .. 3.
// Four barriers a block, one pass per query row (no split over the context).
#include <vector>
#include "pa_internal.h"
#include "upload_ring.h"

namespace atbmi {
namespace mlaint8 {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int TILE = 128;            // tokens per tile = the block size of the cache
constexpr int DN = 512;              // int8 channels (keys and values)
constexpr int DR = 64;               // rotary channels (16-bit)
constexpr int HT = 16;               // heads per workgroup (the N extent of the MFMA)
constexpr int THREADS = 512;         // eight waves, two a SIMD
constexpr int NWAVES = THREADS / WAVE;
constexpr int K_PITCH = DN + 16;     // bytes; 16-byte reads of 16 consecutive rows touch every bank once
constexpr int R_PITCH = DR * 2 + 16;
constexpr int LDS_K = 0;
constexpr int LDS_R = LDS_K + TILE * K_PITCH;
constexpr int LDS_S = LDS_R + TILE * R_PITCH;          // [HT][TILE] fp32 scores
constexpr int LDS_P = LDS_S + HT * TILE * 4;           // [HT][TILE] int8 weights
constexpr int LDS_STAT = LDS_P + HT * TILE;            // [HT] {keep, value scale, 1 / sum, lse}
constexpr int LDS_BYTES = LDS_STAT + HT * 16;
static_assert(LDS_BYTES <= 160 * 1024 && LDS_R % 16 == 0 && LDS_S % 16 == 0 && LDS_P % 16 == 0, "LDS layout");
static_assert(TILE == NWAVES * 16 && DN == NWAVES * 64 && HT == 2 * NWAVES, "eight waves share a tile this way");

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
    float qkScale;
};

__device__ __forceinline__ float Load16AsFloat(uint32_t bits, bool bf16)
{
    return bf16 ? Bf16ToFloat(static_cast<uint16_t>(bits)) : HalfBitsToFloat(static_cast<uint16_t>(bits));
}

template <bool BF16> __device__ __forceinline__ f32x4 Mma16(u32x4 a, u32x4 b, f32x4 c)
{
    if constexpr (BF16) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b),
                                                       c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c,
                                                      0, 0, 0);
    }
}

template <bool BF16> __global__ __launch_bounds__(THREADS) void MlaInt8Kernel(const Args a)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = tid / WAVE;
    const int n = lane & 15;  // MFMA row (A) / column (B, D) of this lane
    const int kg = lane >> 4; // which 16 contraction values / 4 result rows this lane holds
    const int headTiles = (a.H + HT - 1) / HT;
    const Row row = a.rows[blockIdx.x / headTiles];
    const int h0 = (blockIdx.x % headTiles) * HT;
    const int nh = min(HT, a.H - h0);                 // heads past the last one compute on zeros and store nothing
    const int hn = h0 + min(n, nh - 1);               // a head this lane may read the descale of
    const int32_t *table = a.tables + static_cast<int64_t>(row.tableRow) * a.maxBlocksPerSeq;

    // ---- Q^T as B operands: lane (n, kg) holds q8[head n][64 j + 16 kg .. +16) and qRope[head n][32 m + 8 kg .. +8)
    i32x4 q8[DN / 64];
    u32x4 qr[DR / 32];
    {
        const int64_t rowHead = static_cast<int64_t>(row.qRow) * a.H + hn;
#pragma unroll
        for (int j = 0; j < DN / 64; ++j) {
            q8[j] = *reinterpret_cast<const i32x4 *>(a.q8 + rowHead * DN + j * 64 + kg * 16);
            if (n >= nh) {
                q8[j] = i32x4{0, 0, 0, 0};
            }
        }
#pragma unroll
        for (int m = 0; m < DR / 32; ++m) {
            qr[m] = *reinterpret_cast<const u32x4 *>(reinterpret_cast<const uint16_t *>(a.qRope) + rowHead * DR + m * 32 + kg * 8);
            if (n >= nh) {
                qr[m] = u32x4{0u, 0u, 0u, 0u};
            }
        }
    }
    const float descale = a.qkDescale[hn];
    const uint16_t *maskRow = a.mask ? reinterpret_cast<const uint16_t *>(a.mask) + static_cast<int64_t>(row.qRow) * a.maskLen
                                     : nullptr;
    // softmax: this wave's two heads; the running maximum and sum live in its lanes
    float runMax[2] = {-INFINITY, -INFINITY};
    float runSum[2] = {0.0f, 0.0f};
    // values: channels 64 wave + 16 cs + 4 kg + e of head n
    f32x4 acc[4];
#pragma unroll
    for (int cs = 0; cs < 4; ++cs) {
        acc[cs] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    const int l16 = lane & 15;

    for (int t0 = 0; t0 < row.ctxLen; t0 += TILE) {
        const int64_t blk = table[t0 / TILE];
        __syncthreads(); // everybody has left the tiles of the block before
        // ---- the block, NZ [channels / 32][128][32] int8 and [4][128][16] 16-bit, into row-major tiles
        {
            const u32x4 *src = reinterpret_cast<const u32x4 *>(a.kv8 + blk * (TILE * DN));
#pragma unroll 4
            for (int v = tid; v < TILE * DN / 16; v += THREADS) {
                const int slab = v / (TILE * 2);
                const int r = (v % (TILE * 2)) / 2;
                *reinterpret_cast<u32x4 *>(smem + LDS_K + r * K_PITCH + slab * 32 + (v & 1) * 16) = src[v];
            }
            const u32x4 *srcR = reinterpret_cast<const u32x4 *>(reinterpret_cast<const unsigned char *>(a.kRope) +
                                                                blk * (TILE * DR * 2));
            for (int v = tid; v < TILE * DR * 2 / 16; v += THREADS) {
                const int slab = v / (TILE * 2);
                const int r = (v % (TILE * 2)) / 2;
                *reinterpret_cast<u32x4 *>(smem + LDS_R + r * R_PITCH + slab * 32 + (v & 1) * 16) = srcR[v];
            }
        }
        __syncthreads();
        // ---- scores of tokens 16 wave .. + 15 for the 16 heads
        {
            i32x4 dot = {0, 0, 0, 0};
            const unsigned char *krow = smem + LDS_K + (wave * 16 + n) * K_PITCH + kg * 16;
#pragma unroll
            for (int j = 0; j < DN / 64; ++j) {
                const i32x4 kk = *reinterpret_cast<const i32x4 *>(krow + j * 64);
                dot = __builtin_amdgcn_mfma_i32_16x16x64_i8(kk, q8[j], dot, 0, 0, 0);
            }
            f32x4 rope = {0.0f, 0.0f, 0.0f, 0.0f};
            const unsigned char *rrow = smem + LDS_R + (wave * 16 + n) * R_PITCH + kg * 16;
#pragma unroll
            for (int m = 0; m < DR / 32; ++m) {
                rope = Mma16<BF16>(*reinterpret_cast<const u32x4 *>(rrow + m * 64), qr[m], rope);
            }
            // lane (head n, kg) holds tokens 16 wave + 4 kg + e
            const int tok = t0 + wave * 16 + kg * 4;
            f32x4 sc;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const bool live = tok + e < row.ctxLen;
                const float bias = (maskRow && live) ? Load16AsFloat(maskRow[tok + e], BF16) : 0.0f;
                const float x = (static_cast<float>(dot[e]) * descale + rope[e]) * a.qkScale + bias;
                sc[e] = live ? x : -INFINITY;
            }
            *reinterpret_cast<f32x4 *>(smem + LDS_S + (n * TILE + wave * 16 + kg * 4) * 4) = sc;
        }
        __syncthreads();
        // ---- weights of the tile for heads 2 wave, 2 wave + 1
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int h = 2 * wave + i;
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
                stat[1] = a.pvDescale[h0 + min(h, nh - 1)] * wmax / 127.0f;
            }
        }
        __syncthreads();
        // ---- values: O^T[channel, head] += V^T . P^T for channels 64 wave .. + 63
        {
            const float keep = reinterpret_cast<const float *>(smem + LDS_STAT)[n * 4];
            const float vscale = reinterpret_cast<const float *>(smem + LDS_STAT)[n * 4 + 1];
            // the transposing read hands lane (channel l16, kg) the bytes of tokens r .. r + 7 when lane l16 of the
            // group points at token r + l16 / 2, channels (l16 % 2) * 8 .. + 8
            const unsigned char *vbase = smem + LDS_K + (kg * 16 + (l16 >> 1)) * K_PITCH + wave * 64 + (l16 & 1) * 8;
            const unsigned char *pbase = smem + LDS_P + n * TILE + kg * 16;
#pragma unroll
            for (int cs = 0; cs < 4; ++cs) {
                i32x4 iacc = {0, 0, 0, 0};
#pragma unroll
                for (int hh = 0; hh < TILE / 64; ++hh) {
                    const unsigned char *vp = vbase + hh * 64 * K_PITCH + cs * 16;
                    const i32x2 lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) i32x2 *)(vp));
                    const i32x2 hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
                        (__attribute__((address_space(3))) i32x2 *)(vp + 8 * K_PITCH));
                    const i32x4 pw = *reinterpret_cast<const i32x4 *>(pbase + hh * 64);
                    iacc = __builtin_amdgcn_mfma_i32_16x16x64_i8(i32x4{lo[0], lo[1], hi[0], hi[1]}, pw, iacc, 0, 0, 0);
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    acc[cs][e] = acc[cs][e] * keep + static_cast<float>(iacc[e]) * vscale;
                }
            }
        }
    }
    // ---- the rows: acc / sum, and log(sum) + max
    __syncthreads();
    if (lane == 0) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            float *stat = reinterpret_cast<float *>(smem + LDS_STAT) + (2 * wave + i) * 4;
            stat[2] = runSum[i] > 0.0f ? 1.0f / runSum[i] : 0.0f;
            stat[3] = runSum[i] > 0.0f ? logf(runSum[i]) + runMax[i] : -INFINITY;
        }
    }
    __syncthreads();
    if (n < nh) {
        const float inv = reinterpret_cast<const float *>(smem + LDS_STAT)[n * 4 + 2];
        uint16_t *orow = reinterpret_cast<uint16_t *>(a.out) + (static_cast<int64_t>(row.qRow) * a.H + h0 + n) * DN +
                         wave * 64 + kg * 4;
#pragma unroll
        for (int cs = 0; cs < 4; ++cs) {
            uint16_t bits[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float o = acc[cs][e] * inv;
                bits[e] = BF16 ? FloatToBf16(o) : FloatToHalfBits(o);
            }
            uint2 w;
            w.x = static_cast<uint32_t>(bits[0]) | (static_cast<uint32_t>(bits[1]) << 16);
            w.y = static_cast<uint32_t>(bits[2]) | (static_cast<uint32_t>(bits[3]) << 16);
            *reinterpret_cast<uint2 *>(orow + cs * 16) = w;
        }
    }
    if (a.lse && tid < nh) {
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
    if (c->numHeads <= 0) {
        return Fail(ERR_INVALID_PARAM, "mla_int8: %d heads", c->numHeads);
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
    const int64_t grid = static_cast<int64_t>(rows.size()) * ((call->numHeads + mlaint8::HT - 1) / mlaint8::HT);
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
    a.qkScale = call->qkScale;
    auto kernel = call->outDtype == ATBMI_BF16 ? mlaint8::MlaInt8Kernel<true> : mlaint8::MlaInt8Kernel<false>;
    const int ldsBytes = mlaint8::LDS_BYTES;
    rc = ConfigureKernelLds(reinterpret_cast<const void *>(kernel), ldsBytes);
    if (rc != OK) {
        return rc;
    }
    TimedLaunch timed;
    rc = TimedLaunchBegin(s, &timed);
    if (rc != OK) {
        return rc;
    }
    kernel<<<static_cast<unsigned>(grid), mlaint8::THREADS, ldsBytes, s>>>(a);
    ATBMI_HIP_CHECK(hipGetLastError());
    return TimedLaunchEnd(s, timed);
}
