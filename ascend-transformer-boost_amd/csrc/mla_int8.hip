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
// registers (global_load_lds_dwordx4) into one of two 64 KiB buffers; the rotary rows, which only the wave that
// scores their tokens needs, are prefetched into that wave's registers.
//   scores  wave w for tokens 16 w .. 16 w + 15: S^T[token, head] = K . Q^T, eight int8 MFMAs over the 512
//           latent channels (K rows from LDS as A, the query resident in registers as B) and two 16-bit MFMAs
//           over the rotary channels, per tile of 16 heads. The scores stay in the lanes the MFMA left them in
//           (lane (head n, kg): tokens 16 w + 4 kg .. + 3), in units of log 2;
//   softmax the waves exchange only the largest score each has for a head (8 floats a head through LDS); every
//           lane then makes the weights of its own four tokens, keeps its own share of the running sum (the
//           shares are added once, at the end of the row) and writes four int8 weights P[head][token] to LDS;
//   values  wave w for channels 64 w .. 64 w + 63: O^T[channel, head] += V^T . P^T, V^T read from the token-major
//           buffer by the transposing ds_read_b64_tr_b8 (lane (channel, kg) gets the bytes of 8 consecutive
//           tokens), P^T as 16 consecutive bytes of a head's weights. The accumulators are kept in units of the
//           last tile's step: acc = acc x (keep x previous step / step) + int32 sum, two vector instructions a
//           value, and pvDescale x step is applied with 1 / sum when the row is written.
// Two barriers a block: [values of block i - 1, scores of block i] | [weights of block i, V^T of block i into
// registers]. A wave asks for its eight pieces of block i + 1 (the channels only it reads for the values) during
// the first span, as soon as it holds V^T of block i - 1 in registers, one piece at a time between its matrix
// instructions, and waits for them before the second barrier: the path from a compute unit to its cache takes
// one wave's 1 KiB request in about 16 cycles, and a wave that finds the path full stalls with all it has to do.
// The kernel is bound by the vector instructions of a workgroup (about 230 a wave and block, four cycles each,
// two waves a SIMD), not by HBM or the matrix pipe, so the code is written to spend few of them: no pass that
// quiets NaNs around max, rint(fp16(x)) as one packed fp16 addition of 1024 for two weights, tokens past the
// row's end masked only in its last block, the mask a template parameter.
// Operand layout of v_mfma_i32_16x16x64_i8 (checked with a probe on the device): lane (n = lane % 16, kg =
// lane / 16) supplies the 16 contraction values 16 kg .. 16 kg + 15 of row n (A) / column n (B) and receives
// D[4 kg + e][n], e = 0 .. 3.
// One pass per query row when the call has workgroups enough for the chip; a call with few heads cuts every row's
// blocks into up to four equal pieces, each a workgroup's, and MlaInt8MergeKernel joins them (SplitFor).
#include <algorithm>
#include <type_traits>
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
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

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
constexpr int P_PITCH = TILE + 16;      // 16 heads' 16-byte reads touch every bank once
template <int NT> struct Lds {
    static constexpr int K = 0;                            // two blocks
    static constexpr int P = 2 * K_BYTES;                  // [16 NT][tokens] int8 weights
    static constexpr int MAXB = P + NT * HT * P_PITCH;     // [16 NT][waves] fp32: the waves' largest scores of a tile
    static constexpr int BYTES = MAXB + NT * HT * NWAVES * 4;
    static_assert(BYTES <= 160 * 1024 && P % 16 == 0 && MAXB % 16 == 0, "LDS layout");
};
static_assert(TILE == NWAVES * 16 && DN == NWAVES * 64 && PIECES_PER_WAVE == 8,
              "eight waves share a tile this way");

// One query row, or one of the equal pieces its context is cut into (Args::pieces > 1, piece `piece` of every row
// in turn): its sequence's block-table row and context length, the row of query / out / mask.
struct Row {
    int32_t tableRow;
    int32_t ctxLen;
    int32_t qRow;
    int32_t piece;
};
constexpr int MAX_PIECES = 4;

constexpr int INLINE_ROWS = 128; // calls with up to this many query rows carry them in the kernel arguments

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
    const Row *rows; // null: inlineRows
    void *partO;     // pieces > 1: [entries][H][512] rows of the pieces, each normalised on its own, in the type of out
    float *partLse;  // pieces > 1: [entries][H] their base-2 log-sum-exps (-inf: a piece without tokens)
    int32_t pieces;  // pieces a row's blocks are cut into (1: none; the kernel then writes out and lse itself)
    int32_t H;
    int32_t numRows;
    int32_t maxBlocksPerSeq;
    int32_t maskLen;
    float qkScale;
    Row inlineRows[INLINE_ROWS];
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

// One transfer of 16 bytes per lane, cache to LDS without passing through registers: lane l's 16 bytes at
// base + laneOffset + OFFSET go to LDS address ldsBase + OFFSET + 16 l (the instruction's offset field moves both
// ends). base and ldsBase are wave-uniform. With WAIT the LDS reads this wave has asked for are waited for first:
// the transfer may land where they read. The compiler does not count these loads: the kernel waits for them with
// WaitForLoads. A wave asks for one piece at a time, between pieces of arithmetic: the path from the compute unit
// to its cache takes a wave's request for 1 KiB in about 16 cycles, and a wave whose request finds that path full
// waits with everything else it has to do. The requests carry the non-temporal hint: a cache row is read once a call.
template <int OFFSET, bool WAIT>
__device__ __forceinline__ void TransferPieceToLds(uint32_t ldsBase, const unsigned char *base, uint32_t laneOffset)
{
    static_assert(OFFSET >= -4096 && OFFSET < 4096, "13-bit offset field");
    if constexpr (WAIT) {
        asm volatile("s_mov_b32 m0, %0\n\ts_waitcnt lgkmcnt(0)\n\tglobal_load_lds_dwordx4 %1, %2 offset:%3 nt"
                     :
                     : "s"(ldsBase), "v"(laneOffset), "s"(base), "n"(OFFSET)
                     : "memory", "m0");
    } else {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:%3 nt"
                     :
                     : "s"(ldsBase), "v"(laneOffset), "s"(base), "n"(OFFSET)
                     : "memory", "m0");
    }
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

// max without the pass that quiets signalling NaNs (scores are finite or -inf). The compiler does not look into the
// statement when it spaces instructions for the hardware: an operand must not be the result of a transcendental
// instruction (v_exp_f32, v_rcp_f32), which a reader has to follow at a distance.
__device__ __forceinline__ float Max(float a, float b)
{
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}
__device__ __forceinline__ float Max3(float a, float b, float c)
{
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

// Largest / sum of the values lanes n, n + 16, n + 32 and n + 48 hold, in all four of them: the rows of 16 lanes
// change places pairwise (rows 1 and 2, then the halves of the wave).
__device__ __forceinline__ float RowsMax(float x)
{
    float y = x;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1\n\tv_max_f32 %0, %0, %1\n\tv_mov_b32 %1, %0\n\t"
                 "s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1\n\tv_max_f32 %0, %0, %1"
                 : "+v"(x), "+v"(y));
    return x;
}
__device__ __forceinline__ float RowsSum(float x)
{
    float y = x;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\ts_nop 1\n\tv_add_f32 %0, %0, %1\n\tv_mov_b32 %1, %0\n\t"
                 "s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1\n\tv_add_f32 %0, %0, %1"
                 : "+v"(x), "+v"(y));
    return x;
}

template <bool BF16, int NT, bool MASK>
__global__ __launch_bounds__(THREADS) void MlaInt8Kernel(const Args a)
{
    using L = Lds<NT>;
    constexpr int HW = NT * HT; // heads of the workgroup
    constexpr float LOG2E = 1.44269504088896f;
    constexpr float LN2 = 0.693147180559945f;
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
    const int entry = work / headTiles;
    const Row row = a.rows ? a.rows[entry] : a.inlineRows[entry];
    const int h0 = (work % headTiles) * HW;
    const int nh = min(HW, a.H - h0); // heads past the last one compute on zeros and store nothing
    // this workgroup's blocks of the row: all of them, or piece `row.piece` of a.pieces equal shares
    const int allBlocks = (row.ctxLen + TILE - 1) / TILE;
    const int firstBlock = a.pieces > 1 ? allBlocks * row.piece / a.pieces : 0;
    const int numBlocks = (a.pieces > 1 ? allBlocks * (row.piece + 1) / a.pieces : allBlocks) - firstBlock;
    if (numBlocks <= 0) { // (a row with fewer blocks than pieces)
        if (tid < nh) {
            a.partLse[static_cast<int64_t>(entry) * a.H + h0 + tid] = -INFINITY;
        }
        return;
    }
    const int32_t *table = a.tables + static_cast<int64_t>(row.tableRow) * a.maxBlocksPerSeq + firstBlock;
    const uint32_t ldsBase =
        static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) unsigned char *)smem));

    // ---- requests for a block: this wave's eight pieces of the int8 rows (channels 64 wave .. + 63 of all 128
    // tokens: what this wave, and only this wave, reads for the values) and its tokens' rotary rows and mask values
    const uint32_t pieceLane = PlaceOfToken(lane & 31) * 32 + (lane >> 5) * 16; // place lane % 32, half lane / 32
    // (source and destination of a block's pieces are given 4096 bytes into this wave's eight, so that the offset
    // field reaches all of them)
    auto sourceOf = [&](int32_t blk) {
        return reinterpret_cast<const unsigned char *>(a.kv8) +
               static_cast<int64_t>(__builtin_amdgcn_readfirstlane(blk)) * K_BYTES + wave * (PIECES_PER_WAVE * PIECE) + 4096;
    };
    auto placeOf = [&](int buf) {
        return static_cast<uint32_t>(
            __builtin_amdgcn_readfirstlane(ldsBase + L::K + buf * K_BYTES + wave * (PIECES_PER_WAVE * PIECE) + 4096));
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
    const uint16_t *maskRow = reinterpret_cast<const uint16_t *>(a.mask) + static_cast<int64_t>(row.qRow) * a.maskLen;
    auto loadMask = [&](int block, uint32_t(&bits)[4]) { // this lane's four tokens of the block
        if constexpr (MASK) {
            const int tok = (firstBlock + block) * TILE + wave * 16 + kg * 4;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                bits[e] = maskRow[min(tok + e, row.ctxLen - 1)];
            }
        }
    };
    u32x4 ropeNext[DR / 32] = {};
    uint32_t maskNext[4] = {0u, 0u, 0u, 0u};
    int32_t nextId; // id of the block after the one being scored, asked for a block ahead
    int32_t firstId = table[0]; // (asked for before the query, used after it: the two answers travel together)

    // ---- Q^T as B operands: lane (n, kg) holds q8[head n][64 j + 16 kg .. +16) and qRope[head n][32 m + 8 kg .. +8)
    i32x4 q8[NT][DN / 64];
    u32x4 qr[NT][DR / 32];
    float descale[NT], pvDescale[NT];
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
        pvDescale[nt] = a.pvDescale[hn];
    }
    {
        Pin(firstId);
        const int64_t blk = firstId;
        loadRope(blk, ropeNext);
        loadMask(0, maskNext);
        const unsigned char *src = sourceOf(firstId);
        const uint32_t dst = placeOf(0);
        TransferPieceToLds<-4096, false>(dst, src, pieceLane);
        TransferPieceToLds<-3072, false>(dst, src, pieceLane);
        TransferPieceToLds<-2048, false>(dst, src, pieceLane);
        TransferPieceToLds<-1024, false>(dst, src, pieceLane);
        TransferPieceToLds<0, false>(dst, src, pieceLane);
        TransferPieceToLds<1024, false>(dst, src, pieceLane);
        TransferPieceToLds<2048, false>(dst, src, pieceLane);
        TransferPieceToLds<3072, false>(dst, src, pieceLane);
        nextId = table[min(1, numBlocks - 1)];
    }

    const float scale2 = a.qkScale * LOG2E; // scores are kept in units of log 2: the weights are powers of two
    // Softmax state of head 16 nt + n, the same in all lanes and waves that hold it except sumPart: the running
    // maximum, this lane's share of the running sum (its four tokens of every tile), and the unit the accumulators
    // are in: acc x pvDescale x unitStep are the weighted values.
    float runMax[NT], sumPart[NT], unitStep[NT], ratio[NT];
    // values: channels 64 wave + 16 cs + 4 kg + e of head 16 nt + n
    f32x4 acc[NT][4];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        runMax[nt] = -INFINITY;
        sumPart[nt] = 0.0f;
        unitStep[nt] = 0.0f;
        ratio[nt] = 0.0f;
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
    float *maxRow[NT]; // the eight waves' entries of head 16 nt + n
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        maxRow[nt] = reinterpret_cast<float *>(smem + L::MAXB) + (nt * HT + n) * NWAVES;
    }

    // V^T of this wave's 64 channels of the block in vbuf: [channel tile][token half], the two 8-byte halves of every
    // A operand
    auto readValues = [&](const unsigned char *vbuf, i32x2(&vlo)[4][TILE / 64], i32x2(&vhi)[4][TILE / 64]) {
#pragma unroll
        for (int cs = 0; cs < 4; ++cs) {
#pragma unroll
            for (int hh = 0; hh < TILE / 64; ++hh) {
                const unsigned char *vp = vbuf + valueLane + (cs >> 1) * 4096 + (cs & 1) * 512 + hh * 2048;
                vlo[cs][hh] = __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) i32x2 *)(vp));
                vhi[cs][hh] =
                    __builtin_amdgcn_ds_read_tr8_b64_v2i32((__attribute__((address_space(3))) i32x2 *)(vp + valueHigh));
            }
        }
    };
    // O^T[channel, head] += V^T . P^T for channel tile cs, with the weights pw
    auto values = [&](int cs, const i32x2(&vlo)[4][TILE / 64], const i32x2(&vhi)[4][TILE / 64],
                      const i32x4(&pw)[NT][TILE / 64]) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            i32x4 iacc = {0, 0, 0, 0};
#pragma unroll
            for (int hh = 0; hh < TILE / 64; ++hh) {
                const i32x4 vt = {vlo[cs][hh][0], vlo[cs][hh][1], vhi[cs][hh][0], vhi[cs][hh][1]};
                iacc = __builtin_amdgcn_mfma_i32_16x16x64_i8(vt, pw[nt][hh], iacc, 0, 0, 0);
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                acc[nt][cs][e] = __builtin_fmaf(acc[nt][cs][e], ratio[nt], static_cast<float>(iacc[e]));
            }
        }
    };
    auto loadWeights = [&](i32x4(&pw)[NT][TILE / 64]) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
            for (int hh = 0; hh < TILE / 64; ++hh) {
                pw[nt][hh] = *reinterpret_cast<const i32x4 *>(smem + L::P + (nt * HT + n) * P_PITCH + hh * 64 + kg * 16);
            }
        }
    };

    i32x2 vlo[4][TILE / 64], vhi[4][TILE / 64]; // V^T of the block whose weights are being made, read while they are made
    WaitForLoads();
    __syncthreads(); // block 0 is complete
    auto iteration = [&](int i, auto firstTag, auto moreTag) __attribute__((always_inline)) {
        constexpr bool FIRST = decltype(firstTag)::value;
        constexpr bool MORE = decltype(moreTag)::value;
        const unsigned char *kbuf = smem + L::K + (i & 1) * K_BYTES;
        u32x4 rope[DR / 32];
        uint32_t maskBits[4];
#pragma unroll
        for (int m = 0; m < DR / 32; ++m) {
            Pin(ropeNext[m]);
            rope[m] = ropeNext[m];
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            Pin(maskNext[e]);
            maskBits[e] = maskNext[e];
        }
        Pin(nextId);
        const int64_t nextBlk = nextId;
        const unsigned char *src = sourceOf(nextId);
        const uint32_t dst = placeOf((i + 1) & 1);
        // ---- the values of block i - 1, whose V^T this wave holds in registers: its channels of block i + 1 may take
        // their place in LDS (nobody else reads them before the next barrier but one)
        if constexpr (!FIRST) {
            i32x4 pw[NT][TILE / 64];
            loadWeights(pw);
            values(0, vlo, vhi, pw);
            values(1, vlo, vhi, pw);
            if constexpr (MORE) {
                TransferPieceToLds<-4096, true>(dst, src, pieceLane); // (all reads of the block have arrived)
            }
            values(2, vlo, vhi, pw);
            if constexpr (MORE) {
                TransferPieceToLds<-3072, false>(dst, src, pieceLane);
            }
            values(3, vlo, vhi, pw);
            if constexpr (MORE) {
                TransferPieceToLds<-2048, false>(dst, src, pieceLane);
            }
        } else if constexpr (MORE) {
            TransferPieceToLds<-4096, false>(dst, src, pieceLane);
            TransferPieceToLds<-3072, false>(dst, src, pieceLane);
            TransferPieceToLds<-2048, false>(dst, src, pieceLane);
        }
        if constexpr (MORE) {
            loadRope(nextBlk, ropeNext);
            loadMask(i + 1, maskNext);
            nextId = table[min(i + 2, numBlocks - 1)];
        }
        // ---- scores of tokens 16 wave .. + 15, in units of log 2
        float x2[NT][4];
        {
            const int tok = (firstBlock + i) * TILE + wave * 16 + kg * 4; // this lane's four tokens
            // every piece of the rows serves all head tiles as it arrives
            i32x4 dots[NT];
            f32x4 rdots[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                dots[nt] = i32x4{0, 0, 0, 0};
                rdots[nt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int m = 0; m < DR / 32; ++m) {
                    rdots[nt] = Mma16<BF16>(rope[m], qr[nt][m], rdots[nt]);
                }
            }
#pragma unroll
            for (int j = 0; j < DN / 64; ++j) {
                const i32x4 kk = *reinterpret_cast<const i32x4 *>(kbuf + scoreLane + j * 8192);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    dots[nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(kk, q8[nt][j], dots[nt], 0, 0, 0);
                }
            }
            if constexpr (MORE) {
                TransferPieceToLds<-1024, false>(dst, src, pieceLane);
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const i32x4 dot = dots[nt];
                const f32x4 rdot = rdots[nt];
                if constexpr (MORE) {
                    if (nt == 0) {
                        TransferPieceToLds<0, false>(dst, src, pieceLane);
                        if constexpr (NT == 1) {
                            TransferPieceToLds<2048, false>(dst, src, pieceLane);
                        }
                    } else {
                        TransferPieceToLds<2048, false>(dst, src, pieceLane);
                    }
                }
                float tileMax;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float x = __builtin_fmaf(static_cast<float>(dot[e]), descale[nt], rdot[e]) * scale2;
                    if constexpr (MASK) {
                        x = __builtin_fmaf(Load16AsFloat(maskBits[e], BF16), LOG2E, x);
                    }
                    // (only the last block of a row has tokens past its end)
                    x2[nt][e] = (MORE || tok + e < row.ctxLen) ? x : -INFINITY;
                }
                tileMax = RowsMax(Max(Max(x2[nt][0], x2[nt][1]), Max(x2[nt][2], x2[nt][3])));
                maxRow[nt][wave] = tileMax; // (the four lanes that hold a head all write its value)
                if constexpr (MORE) {
                    if (nt == 0) {
                        TransferPieceToLds<1024, false>(dst, src, pieceLane);
                        if constexpr (NT == 1) {
                            TransferPieceToLds<3072, false>(dst, src, pieceLane);
                        }
                    } else {
                        TransferPieceToLds<3072, false>(dst, src, pieceLane);
                    }
                }
            }
        }
        __syncthreads(); // every wave's largest scores of block i are there; everybody has left the weights of block i - 1
        readValues(kbuf, vlo, vhi); // (for the values of this block, after the next barrier)
        // ---- weights of the tile: this lane's four tokens of head 16 nt + n
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const f32x4 m0 = *reinterpret_cast<const f32x4 *>(maxRow[nt]);
            const f32x4 m1 = *reinterpret_cast<const f32x4 *>(maxRow[nt] + 4);
            const float tileMax = Max(Max3(m0[0], m0[1], m0[2]), Max3(Max3(m0[3], m1[0], m1[1]), m1[2], m1[3]));
            // the reference point of the weights: the largest score so far (a mask of -inf can hide everything seen so
            // far: the largest finite number below zero then stands in, and every weight is 0)
            const float ref = Max3(runMax[nt], tileMax, -3.402823466e38f);
            const float keep = __builtin_amdgcn_exp2f(runMax[nt] - ref);
            runMax[nt] = Max(runMax[nt], tileMax);
            // int8 weights rint(fp16(w / step)), step = wmax / 127, but no finer than 2^-40 / 127: a tile whose largest
            // weight is below 2^-40 of the largest so far (or that is hidden altogether) contributes less than a float
            // accumulator notices, and is quantised with that step instead of its own
            const float wmax = __builtin_amdgcn_exp2f(Max(tileMax - ref, -40.0f)); // the largest weight of the tile
            const float step = wmax * (1.0f / 127.0f);
            const float perStep = __builtin_amdgcn_rcpf(step);
            float w[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                w[e] = __builtin_amdgcn_exp2f(x2[nt][e] - ref);
            }
            const float sum = (w[0] + w[1]) + (w[2] + w[3]);
            // fp16(w / step) + 1024 in fp16 is 1024 + rint(fp16(w / step)): the integer is the low byte of the half
            const f16x2 k1024 = {static_cast<_Float16>(1024.0f), static_cast<_Float16>(1024.0f)};
            const f16x2 q01 = f16x2{static_cast<_Float16>(w[0] * perStep), static_cast<_Float16>(w[1] * perStep)} + k1024;
            const f16x2 q23 = f16x2{static_cast<_Float16>(w[2] * perStep), static_cast<_Float16>(w[3] * perStep)} + k1024;
            const uint32_t packed = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, q23), __builtin_bit_cast(uint32_t, q01),
                                                          0x06040200u);
            *reinterpret_cast<uint32_t *>(smem + L::P + (nt * HT + n) * P_PITCH + wave * 16 + kg * 4) = packed;
            sumPart[nt] = __builtin_fmaf(sumPart[nt], keep, sum);
            // the accumulators change their unit to this tile's step
            ratio[nt] = keep * unitStep[nt] * perStep;
            unitStep[nt] = step;
        }
        if constexpr (MORE) {
            WaitForLoads(); // this wave's pieces of block i + 1 are in LDS, its rotary rows and mask values in registers
        }
        __syncthreads(); // the weights of block i are there; block i + 1 is complete
    };
    using Yes = std::true_type;
    using No = std::false_type;
    if (numBlocks == 1) {
        iteration(0, Yes{}, No{});
    } else {
        iteration(0, Yes{}, Yes{});
        for (int i = 1; i < numBlocks - 1; ++i) {
            iteration(i, No{}, Yes{});
        }
        iteration(numBlocks - 1, No{}, No{});
    }
    // ---- the values of the last block
    {
        i32x4 pw[NT][TILE / 64];
        loadWeights(pw);
        values(0, vlo, vhi, pw);
        values(1, vlo, vhi, pw);
        values(2, vlo, vhi, pw);
        values(3, vlo, vhi, pw);
    }
    // ---- the rows: acc x unit / sum, and log(sum) + max
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const float s = RowsSum(sumPart[nt]);
        if (kg == 0) {
            maxRow[nt][wave] = s; // (the largest scores were last read before the loop's last barrier)
        }
    }
    __syncthreads();
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const f32x4 s0 = *reinterpret_cast<const f32x4 *>(maxRow[nt]);
        const f32x4 s1 = *reinterpret_cast<const f32x4 *>(maxRow[nt] + 4);
        const float total = ((s0[0] + s0[1]) + (s0[2] + s0[3])) + ((s1[0] + s1[1]) + (s1[2] + s1[3]));
        if (nt * HT + n < nh) {
            const float inv = total > 0.0f ? pvDescale[nt] * unitStep[nt] / total : 0.0f;
            // the row itself, or this piece's share of it for the merge kernel
            const int64_t rowHead = a.pieces > 1 ? static_cast<int64_t>(entry) * a.H + h0 + nt * HT + n
                                                 : static_cast<int64_t>(row.qRow) * a.H + h0 + nt * HT + n;
            uint16_t *orow = reinterpret_cast<uint16_t *>(a.pieces > 1 ? a.partO : a.out) + rowHead * DN + wave * 64 + kg * 4;
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
            if (wave == 0 && kg == 0) {
                if (a.pieces > 1) {
                    a.partLse[rowHead] = total > 0.0f ? __log2f(total) + runMax[nt] : -INFINITY;
                } else if (a.lse) {
                    a.lse[rowHead] = total > 0.0f ? logf(total) + runMax[nt] * LN2 : -INFINITY;
                }
            }
        }
    }
}

// Joins the pieces of every row: one wave per (row, head), eight channels a lane. A piece weighs 2^(its log-sum-exp
// less the largest of the row's).
constexpr int MERGE_THREADS = 256;
template <bool BF16> __global__ __launch_bounds__(MERGE_THREADS) void MlaInt8MergeKernel(const Args a)
{
    constexpr float LN2 = 0.693147180559945f;
    const int lane = threadIdx.x % WAVE;
    const int64_t pair = static_cast<int64_t>(blockIdx.x) * (MERGE_THREADS / WAVE) + threadIdx.x / WAVE;
    const int rowIdx = static_cast<int>(pair / a.H);
    const int head = static_cast<int>(pair % a.H);
    if (rowIdx >= a.numRows / a.pieces) {
        return;
    }
    const int entry0 = rowIdx * a.pieces;
    const Row row = a.rows ? a.rows[entry0] : a.inlineRows[entry0];
    float lse[MAX_PIECES];
    float top = -INFINITY;
    for (int p = 0; p < a.pieces; ++p) {
        lse[p] = a.partLse[static_cast<int64_t>(entry0 + p) * a.H + head];
        top = fmaxf(top, lse[p]);
    }
    float acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    float sum = 0.0f;
    for (int p = 0; p < a.pieces; ++p) {
        if (lse[p] == -INFINITY) {
            continue; // (nothing was written for a piece without tokens)
        }
        const float w = exp2f(lse[p] - top);
        sum += w;
        const uint4 raw = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(a.partO) +
                                                           (static_cast<int64_t>(entry0 + p) * a.H + head) * DN + lane * 8);
        const uint32_t words[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            acc[2 * k] += w * Load16AsFloat(words[k] & 0xffffu, BF16);
            acc[2 * k + 1] += w * Load16AsFloat(words[k] >> 16, BF16);
        }
    }
    const float inv = sum > 0.0f ? 1.0f / sum : 0.0f;
    uint32_t packed[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float lo = acc[2 * k] * inv, hi = acc[2 * k + 1] * inv;
        packed[k] = static_cast<uint32_t>(BF16 ? FloatToBf16(lo) : FloatToHalfBits(lo)) |
                    (static_cast<uint32_t>(BF16 ? FloatToBf16(hi) : FloatToHalfBits(hi)) << 16);
    }
    const int64_t rowHead = static_cast<int64_t>(row.qRow) * a.H + head;
    *reinterpret_cast<uint4 *>(reinterpret_cast<uint16_t *>(a.out) + rowHead * DN + lane * 8) =
        uint4{packed[0], packed[1], packed[2], packed[3]};
    if (a.lse && lane == 0) {
        a.lse[rowHead] = sum > 0.0f ? (top + log2f(sum)) * LN2 : -INFINITY;
    }
}

// How a call is dealt to the chip: head tiles of 16 a workgroup (one or two) and the equal pieces every row's blocks
// are cut into (one to four). A call lasts as long as its longest workgroup, and one workgroup runs on a CU at a
// time. Two head tiles share a block's rows in LDS and take 1.5 times one tile's time a block; pieces fill CUs that
// would idle, at the price of the merge kernel (3 to 5 us) and of a workgroup's fixed cost. Measured at batch 64,
// contexts of 2 048 to 4 096 tokens: 128 heads are fastest as two tiles and whole rows (65 us), 64 heads as two
// tiles and two pieces (44 us against 48 as whole rows of one tile), 32 heads as one tile and two pieces (36 us
// against 47), 16 heads as one tile and four pieces (32 us against 47). The rule below gives those: one tile when at
// least two pieces of it fit the chip, as many pieces as fit (of at least four blocks in the longest row).
struct Split {
    int headTiles;
    int pieces;
};
Split SplitFor(const AtbmiMlaInt8Call *c, const std::vector<Row> &rows)
{
    const int64_t cus = DeviceComputeUnits();
    const int64_t tilesOfOne = static_cast<int64_t>(rows.size()) * ((c->numHeads + HT - 1) / HT);
    const int64_t tilesOfTwo = static_cast<int64_t>(rows.size()) * ((c->numHeads + 2 * HT - 1) / (2 * HT));
    Split split{1, 1};
    if (tilesOfOne == 0) {
        return split;
    }
    split.headTiles = (c->numHeads > HT && 2 * tilesOfOne > cus) ? 2 : 1;
    int32_t longest = 0;
    for (const Row &r : rows) {
        longest = std::max(longest, (r.ctxLen + TILE - 1) / TILE);
    }
    const int64_t workgroups = split.headTiles == 2 ? tilesOfTwo : tilesOfOne;
    int pieces = static_cast<int>(std::min<int64_t>(MAX_PIECES, cus / workgroups));
    while (pieces > 1 && longest < 4 * pieces) {
        --pieces;
    }
    split.pieces = std::max(pieces, 1);
    return split;
}

// Bytes of the workspace's parts: the table of rows (entries x 16, to a multiple of 256), the pieces' rows and
// their log-sum-exps (none when the rows are whole).
struct WorkspaceLayout {
    size_t table, partO, partLse;
    size_t Total() const { return table + partO + partLse; }
};
WorkspaceLayout LayoutFor(const AtbmiMlaInt8Call *c, size_t rowCount, int pieces)
{
    const size_t entries = rowCount * static_cast<size_t>(pieces);
    WorkspaceLayout l{};
    l.table = (entries * sizeof(Row) + 255) / 256 * 256;
    if (pieces > 1) {
        l.partO = entries * static_cast<size_t>(c->numHeads) * DN * sizeof(uint16_t);
        l.partLse = (entries * static_cast<size_t>(c->numHeads) * sizeof(float) + 255) / 256 * 256;
    }
    return l;
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
    *bytes = mlaint8::LayoutFor(call, rows.size(), mlaint8::SplitFor(call, rows).pieces).Total();
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
    const mlaint8::Split split = mlaint8::SplitFor(call, rows);
    const int pieces = split.pieces;
    const mlaint8::WorkspaceLayout layout = mlaint8::LayoutFor(call, rows.size(), pieces);
    const size_t bytes = layout.Total();
    if (pieces > 1) { // every row once per piece, a row's pieces next to each other
        std::vector<mlaint8::Row> entries;
        entries.reserve(rows.size() * pieces);
        for (const mlaint8::Row &r : rows) {
            for (int p = 0; p < pieces; ++p) {
                entries.push_back(mlaint8::Row{r.tableRow, r.ctxLen, r.qRow, p});
            }
        }
        rows.swap(entries);
    }
    if (!workspaceDevice || workspaceBytes < bytes) {
        return Fail(ERR_INVALID_PARAM, "mla_int8: workspace of %llu bytes, %llu needed", (unsigned long long)workspaceBytes,
                    (unsigned long long)bytes);
    }
    const int nt = split.headTiles;
    const int headsPerWg = nt * mlaint8::HT;
    const int64_t grid = (static_cast<int64_t>(rows.size()) * ((call->numHeads + headsPerWg - 1) / headsPerWg) + 7) / 8 * 8;
    if (grid > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "mla_int8: %lld workgroups", (long long)grid);
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool inlineRows = rows.size() <= static_cast<size_t>(mlaint8::INLINE_ROWS);
    if (!inlineRows) {
        rc = UploadTable(rows.data(), rows.size() * sizeof(mlaint8::Row), workspaceDevice, s);
        if (rc != OK) {
            return rc;
        }
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
    a.rows = inlineRows ? nullptr : static_cast<const mlaint8::Row *>(workspaceDevice);
    if (inlineRows) {
        std::copy(rows.begin(), rows.end(), a.inlineRows);
    }
    a.partO = pieces > 1 ? static_cast<unsigned char *>(workspaceDevice) + layout.table : nullptr;
    a.partLse = pieces > 1 ? reinterpret_cast<float *>(static_cast<unsigned char *>(workspaceDevice) + layout.table + layout.partO)
                           : nullptr;
    a.pieces = pieces;
    a.H = call->numHeads;
    a.numRows = static_cast<int32_t>(rows.size());
    a.maxBlocksPerSeq = call->maxBlocksPerSeq;
    a.maskLen = call->maskLen;
    a.qkScale = call->qkScale;
    const bool bf16 = call->outDtype == ATBMI_BF16;
    using Kernel = void (*)(const mlaint8::Args);
    static const Kernel kernels[2][2][2] = {
        {{mlaint8::MlaInt8Kernel<false, 1, false>, mlaint8::MlaInt8Kernel<false, 1, true>},
         {mlaint8::MlaInt8Kernel<false, 2, false>, mlaint8::MlaInt8Kernel<false, 2, true>}},
        {{mlaint8::MlaInt8Kernel<true, 1, false>, mlaint8::MlaInt8Kernel<true, 1, true>},
         {mlaint8::MlaInt8Kernel<true, 2, false>, mlaint8::MlaInt8Kernel<true, 2, true>}}};
    const Kernel kernel = kernels[bf16 ? 1 : 0][nt - 1][call->hasMask ? 1 : 0];
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
    if (rc != OK) {
        return rc;
    }
    if (pieces > 1) {
        const int64_t pairs = static_cast<int64_t>(rows.size() / pieces) * call->numHeads;
        const int perGroup = mlaint8::MERGE_THREADS / WAVE;
        const unsigned mergeGrid = static_cast<unsigned>((pairs + perGroup - 1) / perGroup);
        if (bf16) {
            mlaint8::MlaInt8MergeKernel<true><<<mergeGrid, mlaint8::MERGE_THREADS, 0, s>>>(a);
        } else {
            mlaint8::MlaInt8MergeKernel<false><<<mergeGrid, mlaint8::MERGE_THREADS, 0, s>>>(a);
        }
        ATBMI_HIP_CHECK(hipGetLastError());
    }
    return TimedLaunchEnd(s, timed, pieces > 1);
}
