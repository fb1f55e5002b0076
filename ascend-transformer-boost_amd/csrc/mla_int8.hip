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
// A workgroup of eight waves owns one query row and 32 heads (16 when the call has no more) and walks the
// row's context block by block. The int8 rows of a block go from the cache to LDS without passing through
// registers (global_load_lds_dwordx4), one block ahead of the arithmetic, into one of two 64 KiB buffers; the
// rotary rows, which only the wave that scores their tokens needs, are prefetched into that wave's registers.
//   scores  wave w for tokens 16 w .. 16 w + 15: S^T[token, head] = K . Q^T, eight int8 MFMAs over the 512
//           latent channels (K rows from LDS as A, the query resident in registers as B) and two 16-bit MFMAs
//           over the rotary channels, per tile of 16 heads;
//   softmax 16 (32) lanes a head, 8 (4) tokens a lane; int8 weights P[head][token] go to LDS;
//   values  wave w for channels 64 w .. 64 w + 63: O^T[channel, head] += V^T . P^T, V^T read from the token-major
//           buffer by the transposing ds_read_b64_tr_b8 (lane (channel, kg) gets the bytes of 8 consecutive
//           tokens), P^T as 16 consecutive bytes of a head's weights.
// Operand layout of v_mfma_i32_16x16x64_i8 (checked with a probe on the device): lane (n = lane % 16, kg =
// lane / 16) supplies the 16 contraction values 16 kg .. 16 kg + 15 of row n (A) / column n (B) and receives
// D[4 kg + e][n], e = 0 .. 3.
// Three barriers a block, one pass per query row (no split over the context).
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
constexpr int HT = 16;               // heads per head tile (the N extent of the MFMA)
constexpr int THREADS = 512;         // eight waves, two a SIMD
constexpr int NWAVES = THREADS / WAVE;
// A block in LDS: the 1 KiB pieces of the NZ block ([channels / 32][128 tokens][32 bytes]: piece c = 32 tokens of
// one 32-channel slab) keep their order, and inside a piece the 16-byte halves of the 32 tokens are parted: the
// low halves first, 16 bytes a token, then the high halves; tokens 16 .. 31 of the 32 swap their two groups of
// eight (place = token ^ 8). Sixteen tokens' reads of one half are then 256 contiguous bytes (every bank once),
// and the 32 lanes a transposing read serves together (eight tokens x 16 channels twice, 16 tokens apart) touch
// every bank once as well.
constexpr int K_BYTES = TILE * DN;
constexpr int PIECE = 1024;
constexpr int PIECES_PER_WAVE = K_BYTES / PIECE / NWAVES;
__host__ __device__ constexpr int PlaceOfToken(int t) // among the 32 tokens of a piece; its own inverse
{
    return t ^ ((t & 16) >> 1);
}
constexpr int S_PITCH = (TILE + 4) * 4; // 16 heads' 16-byte writes touch every bank once
constexpr int P_PITCH = TILE + 16;      // likewise for 16 heads' 16-byte reads
template <int NT> struct Lds {
    static constexpr int K = 0;                          // two blocks
    static constexpr int S = 2 * K_BYTES;                // [16 NT] fp32 scores
    static constexpr int P = S + NT * HT * S_PITCH;      // [16 NT] int8 weights
    static constexpr int STAT = P + NT * HT * P_PITCH;   // [16 NT] {keep, value scale, 1 / sum, lse}
    static constexpr int BYTES = STAT + NT * HT * 16;
    static_assert(BYTES <= 160 * 1024 && S % 16 == 0 && P % 16 == 0 && STAT % 16 == 0, "LDS layout");
};
static_assert(TILE == NWAVES * 16 && DN == NWAVES * 64 && PIECES_PER_WAVE == 8,
              "eight waves share a tile this way");

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
    int32_t numRows;
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

// Eight transfers of 16 bytes per lane, cache to LDS without passing through registers: transfer i reads
// base + laneOffset + 1024 i and writes LDS address ldsBase + 1024 i + 16 x lane (the instruction's offset field
// moves both ends, so both bases are given 4096 bytes in). base and ldsBase are wave-uniform. The compiler does
// not count these loads: the kernel waits for them with WaitForLoads.
__device__ __forceinline__ void TransferPiecesToLds(uint32_t ldsBase, const void *base, uint32_t laneOffset)
{
    const uint64_t src = reinterpret_cast<uint64_t>(base) + 4096u;
    const uint64_t srcUniform =
        (static_cast<uint64_t>(__builtin_amdgcn_readfirstlane(static_cast<uint32_t>(src >> 32))) << 32) |
        static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<uint32_t>(src)));
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\t"
                 "global_load_lds_dwordx4 %1, %2 offset:-4096\n\t"
                 "global_load_lds_dwordx4 %1, %2 offset:-3072\n\t"
                 "global_load_lds_dwordx4 %1, %2 offset:-2048\n\t"
                 "global_load_lds_dwordx4 %1, %2 offset:-1024\n\t"
                 "global_load_lds_dwordx4 %1, %2\n\t"
                 "global_load_lds_dwordx4 %1, %2 offset:1024\n\t"
                 "global_load_lds_dwordx4 %1, %2 offset:2048\n\t"
                 "global_load_lds_dwordx4 %1, %2 offset:3072"
                 :
                 : "s"(ldsBase + 4096u), "v"(laneOffset), "s"(srcUniform)
                 : "memory", "m0");
}

__device__ __forceinline__ void WaitForLoads()
{
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
}

// Makes the compiler treat a loaded value as used here, so that the wait it inserts for the load lands here
// (next to WaitForLoads) and not later, behind transfers that were requested in between.
template <typename T> __device__ __forceinline__ void Pin(T &v)
{
    asm volatile("" : "+v"(v));
}

// All-reduce over the 16 lanes of a row (lanes 16 r .. 16 r + 15) by rotations inside the row.
template <int ROR> __device__ __forceinline__ float RowRotate(float x)
{
    const int v = __builtin_bit_cast(int, x);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(v, v, 0x120 + ROR, 0xf, 0xf, true));
}
template <int LANES> __device__ __forceinline__ float GroupMax(float x)
{
    x = fmaxf(x, RowRotate<8>(x));
    x = fmaxf(x, RowRotate<4>(x));
    x = fmaxf(x, RowRotate<2>(x));
    x = fmaxf(x, RowRotate<1>(x));
    if constexpr (LANES == 32) {
        x = fmaxf(x, __shfl_xor(x, 16));
    }
    return x;
}
template <int LANES> __device__ __forceinline__ float GroupSum(float x)
{
    x += RowRotate<8>(x);
    x += RowRotate<4>(x);
    x += RowRotate<2>(x);
    x += RowRotate<1>(x);
    if constexpr (LANES == 32) {
        x += __shfl_xor(x, 16);
    }
    return x;
}

template <bool BF16, int NT>
__global__ __launch_bounds__(THREADS) void MlaInt8Kernel(const Args a)
{
    using L = Lds<NT>;
    constexpr int HW = NT * HT;          // heads of the workgroup
    constexpr int CH = THREADS / HW;     // softmax: lanes a head
    constexpr int TPL = TILE / CH;       // softmax: tokens a lane
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int n = lane & 15;  // MFMA row (A) / column (B, D) of this lane
    const int kg = lane >> 4; // which 16 contraction values / 4 result rows this lane holds
    const int headTiles = (a.H + HW - 1) / HW;
    // workgroups go round the eight XCDs: the head tiles of a row, which read the same cache blocks, take
    // neighbouring places on one XCD and share its L2
    const int work = (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8;
    if (work >= a.numRows * headTiles) {
        return;
    }
    const Row row = a.rows[work / headTiles];
    const int h0 = (work % headTiles) * HW;
    const int nh = min(HW, a.H - h0); // heads past the last one compute on zeros and store nothing
    const int32_t *table = a.tables + static_cast<int64_t>(row.tableRow) * a.maxBlocksPerSeq;
    const int numBlocks = (row.ctxLen + TILE - 1) / TILE;
    const uint32_t ldsBase =
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) unsigned char *)smem));

    // ---- requests for a block: this wave's eight pieces of the int8 rows, and its tokens' rotary rows
    const uint32_t pieceLane = PlaceOfToken(lane & 31) * 32 + (lane >> 5) * 16; // place lane % 32, half lane / 32
    auto requestBlock = [&](int64_t blk, int buf) {
        const unsigned char *src =
            reinterpret_cast<const unsigned char *>(a.kv8) + blk * K_BYTES + wave * (PIECES_PER_WAVE * PIECE);
        const uint32_t dst = ldsBase + L::K + buf * K_BYTES + wave * (PIECES_PER_WAVE * PIECE);
        TransferPiecesToLds(__builtin_amdgcn_readfirstlane(dst), src, pieceLane);
    };
    // lane (token n of the wave's 16, kg): rotary channels 32 m + 8 kg .. + 8, NZ [4][128][16]
    const int ropeLane = (kg >> 1) * (TILE * 32) + (wave * 16 + n) * 32 + (kg & 1) * 16;
    auto loadRope = [&](int64_t blk, u32x4(&r)[DR / 32]) {
        const unsigned char *src = reinterpret_cast<const unsigned char *>(a.kRope) + blk * (TILE * DR * 2) + ropeLane;
#pragma unroll
        for (int m = 0; m < DR / 32; ++m) {
            r[m] = *reinterpret_cast<const u32x4 *>(src + m * (2 * TILE * 32));
        }
    };
    u32x4 ropeNext[DR / 32] = {};
    if (numBlocks > 0) {
        const int64_t blk = table[0];
        loadRope(blk, ropeNext);
        requestBlock(blk, 0);
    }

    // ---- Q^T as B operands: lane (n, kg) holds q8[head n][64 j + 16 kg .. +16) and qRope[head n][32 m + 8 kg .. +8)
    i32x4 q8[NT][DN / 64];
    u32x4 qr[NT][DR / 32];
    float descale[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const bool live = nt * HT + n < nh;
        const int hn = h0 + min(nt * HT + n, nh - 1);
        const int64_t rowHead = static_cast<int64_t>(row.qRow) * a.H + hn;
#pragma unroll
        for (int j = 0; j < DN / 64; ++j) {
            q8[nt][j] = *reinterpret_cast<const i32x4 *>(a.q8 + rowHead * DN + j * 64 + kg * 16);
            if (!live) {
                q8[nt][j] = i32x4{0, 0, 0, 0};
            }
        }
#pragma unroll
        for (int m = 0; m < DR / 32; ++m) {
            qr[nt][m] = *reinterpret_cast<const u32x4 *>(reinterpret_cast<const uint16_t *>(a.qRope) + rowHead * DR +
                                                          m * 32 + kg * 8);
            if (!live) {
                qr[nt][m] = u32x4{0u, 0u, 0u, 0u};
            }
        }
        descale[nt] = a.qkDescale[hn];
    }
    const uint16_t *maskRow = a.mask ? reinterpret_cast<const uint16_t *>(a.mask) + static_cast<int64_t>(row.qRow) * a.maskLen
                                     : nullptr;
    // softmax: lane (head tid / CH, tokens 4 (tid % CH + CH k) .. + 4 for k < TPL / 4); a head's lanes all hold its
    // running maximum and sum
    const int smHead = tid / CH;
    const int smTok = (tid % CH) * 4;
    const float smPvDescale = a.pvDescale[h0 + min(smHead, nh - 1)];
    float runMax = -INFINITY;
    float runSum = 0.0f;
    // values: channels 64 wave + 16 cs + 4 kg + e of head 16 nt + n
    f32x4 acc[NT][4];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
        for (int cs = 0; cs < 4; ++cs) {
            acc[nt][cs] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
    }
    // byte offsets into a block in LDS
    const int scoreLane = (kg >> 1) * 4096 + (wave >> 1) * PIECE + (kg & 1) * 512 + PlaceOfToken((wave & 1) * 16 + n) * 16;
    // the transposing read hands lane (channel n, kg) the bytes of tokens r .. r + 7 when lane n of the group
    // points at token r + n / 2, channels (n % 2) * 8 .. + 8
    const int valueLane = wave * 8192 + (kg >> 1) * PIECE + PlaceOfToken((kg & 1) * 16 + (n >> 1)) * 16 + (n & 1) * 8;
    const int valueHigh = (kg & 1) ? -128 : 128; // to the tokens eight further on

    for (int i = 0; i < numBlocks; ++i) {
        const int t0 = i * TILE;
        const int tok = t0 + wave * 16 + kg * 4; // scores: this lane's four tokens
        uint32_t maskBits[4] = {0u, 0u, 0u, 0u};
        if (maskRow) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                maskBits[e] = maskRow[min(tok + e, row.ctxLen - 1)];
            }
        }
        const bool more = i + 1 < numBlocks;
        const int64_t nextBlk = more ? table[i + 1] : 0;
        WaitForLoads(); // this wave's pieces of block i are in LDS, its rotary rows and mask values in registers
        u32x4 rope[DR / 32];
#pragma unroll
        for (int m = 0; m < DR / 32; ++m) {
            Pin(ropeNext[m]);
            rope[m] = ropeNext[m];
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            Pin(maskBits[e]);
        }
        __syncthreads(); // block i is complete; everybody has left block i - 1, the scores and the weights
        if (more) {
            loadRope(nextBlk, ropeNext);
            requestBlock(nextBlk, (i + 1) & 1);
        }
        const unsigned char *kbuf = smem + L::K + (i & 1) * K_BYTES;
        // ---- scores of tokens 16 wave .. + 15
        {
            i32x4 kk[DN / 64];
#pragma unroll
            for (int j = 0; j < DN / 64; ++j) {
                kk[j] = *reinterpret_cast<const i32x4 *>(kbuf + scoreLane + j * 8192);
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                i32x4 dot = {0, 0, 0, 0};
#pragma unroll
                for (int j = 0; j < DN / 64; ++j) {
                    dot = __builtin_amdgcn_mfma_i32_16x16x64_i8(kk[j], q8[nt][j], dot, 0, 0, 0);
                }
                f32x4 rdot = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int m = 0; m < DR / 32; ++m) {
                    rdot = Mma16<BF16>(rope[m], qr[nt][m], rdot);
                }
                f32x4 sc;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const bool live = tok + e < row.ctxLen;
                    const float bias = maskRow ? Load16AsFloat(maskBits[e], BF16) : 0.0f;
                    const float x = (static_cast<float>(dot[e]) * descale[nt] + rdot[e]) * a.qkScale + bias;
                    sc[e] = live ? x : -INFINITY;
                }
                *reinterpret_cast<f32x4 *>(smem + L::S + (nt * HT + n) * S_PITCH + (wave * 16 + kg * 4) * 4) = sc;
            }
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
            tileMax = GroupMax<CH>(tileMax);
            const float newMax = fmaxf(runMax, tileMax);
            const bool any = newMax > -INFINITY; // (a mask of -inf can hide everything seen so far)
            float sum = 0.0f, wmax = 0.0f;
#pragma unroll
            for (int k = 0; k < TPL; ++k) {
                w[k] = any ? __expf(w[k] - newMax) : 0.0f;
                sum += w[k];
                wmax = fmaxf(wmax, w[k]);
            }
            sum = GroupSum<CH>(sum);
            wmax = GroupMax<CH>(wmax);
            const float keep = (any && runMax > -INFINITY) ? __expf(runMax - newMax) : 0.0f;
            runSum = runSum * keep + sum;
            runMax = newMax;
            // rint(fp16(w / step)), 0 .. 127. The quotient by a multiplication with 1 / step and one fused
            // correction (the division's own sequence without its rescaling); a step too small for that takes
            // the division.
            const float step = wmax / 127.0f;
            uint32_t packed[TPL / 4] = {};
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
            unsigned char *prow = smem + L::P + smHead * P_PITCH + smTok;
#pragma unroll
            for (int k = 0; k < TPL / 4; ++k) {
                *reinterpret_cast<uint32_t *>(prow + k * CH * 4) = packed[k];
            }
            if (tid % CH == 0) {
                float *stat = reinterpret_cast<float *>(smem + L::STAT) + smHead * 4;
                stat[0] = keep;
                stat[1] = smPvDescale * wmax / 127.0f;
            }
        }
        __syncthreads();
        // ---- values: O^T[channel, head] += V^T . P^T for channels 64 wave .. + 63
        {
            float keep[NT], vscale[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const float *stat = reinterpret_cast<const float *>(smem + L::STAT) + (nt * HT + n) * 4;
                keep[nt] = stat[0];
                vscale[nt] = stat[1];
            }
            i32x4 pw[NT][TILE / 64];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
                for (int hh = 0; hh < TILE / 64; ++hh) {
                    pw[nt][hh] = *reinterpret_cast<const i32x4 *>(smem + L::P + (nt * HT + n) * P_PITCH + hh * 64 + kg * 16);
                }
            }
#pragma unroll
            for (int cs = 0; cs < 4; ++cs) {
                i32x4 vt[TILE / 64];
#pragma unroll
                for (int hh = 0; hh < TILE / 64; ++hh) {
                    const unsigned char *vp = kbuf + valueLane + (cs >> 1) * 4096 + (cs & 1) * 512 + hh * 2048;
                    const i32x2 lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) i32x2 *)(vp));
                    const i32x2 hi =
                        __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) i32x2 *)(vp + valueHigh));
                    vt[hh] = i32x4{lo[0], lo[1], hi[0], hi[1]};
                }
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    i32x4 iacc = {0, 0, 0, 0};
#pragma unroll
                    for (int hh = 0; hh < TILE / 64; ++hh) {
                        iacc = __builtin_amdgcn_mfma_i32_16x16x64_i8(vt[hh], pw[nt][hh], iacc, 0, 0, 0);
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        acc[nt][cs][e] = acc[nt][cs][e] * keep[nt] + static_cast<float>(iacc[e]) * vscale[nt];
                    }
                }
            }
        }
    }
    // ---- the rows: acc / sum, and log(sum) + max
    __syncthreads();
    if (tid % CH == 0) {
        float *stat = reinterpret_cast<float *>(smem + L::STAT) + smHead * 4;
        stat[2] = runSum > 0.0f ? 1.0f / runSum : 0.0f;
        stat[3] = runSum > 0.0f ? logf(runSum) + runMax : -INFINITY;
    }
    __syncthreads();
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        if (nt * HT + n < nh) {
            const float inv = reinterpret_cast<const float *>(smem + L::STAT)[(nt * HT + n) * 4 + 2];
            uint16_t *orow = reinterpret_cast<uint16_t *>(a.out) +
                             (static_cast<int64_t>(row.qRow) * a.H + h0 + nt * HT + n) * DN + wave * 64 + kg * 4;
#pragma unroll
            for (int cs = 0; cs < 4; ++cs) {
                uint16_t bits[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float o = acc[nt][cs][e] * inv;
                    bits[e] = BF16 ? FloatToBf16(o) : FloatToHalfBits(o);
                }
                uint2 w;
                w.x = static_cast<uint32_t>(bits[0]) | (static_cast<uint32_t>(bits[1]) << 16);
                w.y = static_cast<uint32_t>(bits[2]) | (static_cast<uint32_t>(bits[3]) << 16);
                *reinterpret_cast<uint2 *>(orow + cs * 16) = w;
            }
        }
    }
    if (a.lse && tid < nh) {
        a.lse[static_cast<int64_t>(row.qRow) * a.H + h0 + tid] = reinterpret_cast<const float *>(smem + L::STAT)[tid * 4 + 3];
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
        const bool causal = c->causalRows && (!c->hostCausalUse || c->hostCausalUse[b] != 0);
        if (causal && ctx > 0 && nq > ctx) {
            return Fail(ERR_INVALID_PARAM, "mla_int8: sequence %d has %d query tokens but a context of %d", b, nq, ctx);
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
            // an empty context still owns its query rows (nothing is written to their outputs): the reference's
            // tiling moves on by qSeqLen whatever kvSeqLen is (tiling/mla_tiling.cpp:146-149)
            qRow += nq;
            continue;
        }
        for (int32_t i = 0; i < nq; ++i) {
            if (qRow > 0x7fffffffLL) {
                return Fail(ERR_INVALID_PARAM, "mla_int8: more than 2^31 query rows");
            }
            if (rows) {
                rows->push_back(Row{b, causal ? ctx - nq + i + 1 : ctx, static_cast<int32_t>(qRow), 0});
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
    const int nt = call->numHeads > mlaint8::HT ? 2 : 1; // head tiles of 16 a workgroup
    const int headsPerWg = nt * mlaint8::HT;
    const int64_t grid = (static_cast<int64_t>(rows.size()) * ((call->numHeads + headsPerWg - 1) / headsPerWg) + 7) / 8 * 8;
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
    a.numRows = static_cast<int32_t>(rows.size());
    a.maxBlocksPerSeq = call->maxBlocksPerSeq;
    a.maskLen = call->maskLen;
    a.qkScale = call->qkScale;
    const bool bf16 = call->outDtype == ATBMI_BF16;
    auto kernel = nt == 2 ? (bf16 ? mlaint8::MlaInt8Kernel<true, 2> : mlaint8::MlaInt8Kernel<false, 2>)
                          : (bf16 ? mlaint8::MlaInt8Kernel<true, 1> : mlaint8::MlaInt8Kernel<false, 1>);
    const int ldsBytes = nt == 2 ? mlaint8::Lds<2>::BYTES : mlaint8::Lds<1>::BYTES;
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
    rc = TimedLaunchKernelDone(s, timed);
    return rc != OK ? rc : TimedLaunchEnd(s, timed, false);
}
