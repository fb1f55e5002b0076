// Prefill attention of MultiLatentAttention (calcType PREFILL) for gfx950: variable-length flash attention
// with 128 + 64 key channels and 128 value channels per head (reference operator
// src/ops/ops_infer/multi_latent_attention/multi_latent_attention_ops_runner_prefill.cpp, device kernels
// src/kernels/mixkernels/multi_latent_attention/op_kernel/mla_prefill*.cce).
//
// A workgroup owns 128 consecutive queries of one sequence and one head: four waves of 32 queries each
// walk the keys the block may see in 32-token steps over tiles that the workgroup stages in LDS once.
//   HBM -> LDS         : global_load_lds_dwordx4, no staging registers: wave w moves rows 8 w .. 8 w + 7 of
//                        the K tile (128 + 64 channels from two tensors) and of the V tile with seven
//                        transfers; three tile buffers, the tile two steps ahead is requested before this
//                        step's arithmetic (a step is shorter than a round trip to L2 or HBM), one barrier
//                        per step;
//   S^T = K . Q^T      : v_mfma_f32_32x32x16, K from LDS as A (ds_read_b128), Q^T resident in registers as B;
//                        lane (n, kh) then holds 16 tokens of query n: 8 (e / 4) + 4 kh + e % 4;
//   softmax            : base 2, online; the row maximum needs one exchange between lanes n and n + 32;
//   O^T += V^T . P^T   : the score registers are the B operand as they stand (k index 8 kh + e of the
//                        half-step kb is token 16 kb + 8 (e / 4) + 4 kh + e % 4), V^T comes from the
//                        row-major tile through the transposing ds_read_b64_tr_b16.
// Steps that a mask hides completely are not visited (causal: keys past the block's last query; window:
// keys before the first query's window); inside a visited step hidden scores are -inf. Tile rows past the
// end of a sequence repeat its last row: their scores are hidden and their value rows finite.
//
// The transfers are inline assembly, so the compiler neither sees their LDS writes nor counts them: every
// wait for them is written out (vmcnt counts loads in issue order; the loop issues no other load), and the
// barrier that follows a wait makes the landed rows of all four waves visible to all.
#include <algorithm>
#include <vector>
#include "pa_internal.h"
#include "upload_ring.h"

namespace atbmi {
namespace prefill {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int DN = 128;               // channels of query / key
constexpr int DR = 64;                // channels of queryRope / keyRope
constexpr int D = DN + DR;
constexpr int DV = 128;
constexpr int QW = 32;                // queries per wave
constexpr int NWAVES = 4;
constexpr int QB = QW * NWAVES;       // queries per workgroup
constexpr int STEP = 32;              // keys per step
constexpr int K_PITCH = D * 2 + 16;   // 400 bytes: 16 lanes x 16 bytes of one operand read touch every bank once
constexpr int V_PITCH = DV * 2 + 64;  // 320 bytes: four rows x 64 bytes of one transposing read likewise
constexpr int K_TILE = STEP * K_PITCH;
constexpr int V_TILE = STEP * V_PITCH;
constexpr int BUF = K_TILE + V_TILE;
constexpr int NBUF = 3;
constexpr int LDS_BYTES = NBUF * BUF;
// A transfer fills 64 consecutive 16-byte slots of LDS, one per lane. A wave's 8 rows are 200 slots of the K
// tile (25 a row, the last one padding) and 160 of the V tile (20 a row, four of them padding).
constexpr int ROWS_PER_WAVE = STEP / NWAVES;
constexpr int K_SLOTS = K_PITCH / 16;
constexpr int V_SLOTS = V_PITCH / 16;
constexpr int K_DMA = (ROWS_PER_WAVE * K_SLOTS + WAVE - 1) / WAVE;
constexpr int V_DMA = (ROWS_PER_WAVE * V_SLOTS + WAVE - 1) / WAVE;
constexpr int DMA_PER_TILE = K_DMA + V_DMA;
static_assert(K_DMA == 4 && V_DMA == 3 && LDS_BYTES == 69120, "the waits below count seven transfers a tile");

// One block of queries: rows [qRow0, qRow0 + nQ) of the query tensors, positions [qPos0, qPos0 + nQ) of
// a sequence whose keys are rows [kRow0, kRow0 + kvLen) of the key / value tensors.
struct Item {
    int32_t qRow0;
    int32_t nQ;
    int32_t kRow0;
    int32_t kvLen;
    int32_t qPos0;
    int32_t pad[3];
};

struct Args {
    const void *q;
    const void *qRope;
    const void *k;
    const void *kRope;
    const void *v;
    void *out;
    const Item *items;
    int32_t numItems;
    int32_t H;
    int32_t G;
    int32_t group;   // H / G
    int32_t mask;    // AtbmiMlaPrefillMask
    int32_t window;
    float scale2;    // qkScale * log2(e)
};

template <bool BF16> __device__ __forceinline__ f32x16 Mma(u32x4 a, u32x4 b, f32x16 c)
{
    if constexpr (BF16) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b),
                                                       c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c,
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

__device__ __forceinline__ float Exp2(float x)
{
    return __builtin_amdgcn_exp2f(x);
}

// 16 bytes per active lane from `src` to LDS address ldsBase + 16 x lane (ldsBase wave-uniform).
__device__ __forceinline__ void TransferToLds(uint32_t ldsBase, const void *src)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 :
                 : "s"(ldsBase), "v"(src)
                 : "memory", "m0");
}

template <bool BF16>
__global__ __launch_bounds__(NWAVES *WAVE) __attribute__((amdgpu_waves_per_eu(2, 2))) void MlaPrefillKernel(const Args a)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int n = lane & 31;  // query column of this lane
    const int kh = lane >> 5; // which half of an MFMA's contraction values this lane holds
    // Workgroups go to the 8 XCDs round-robin, and every XCD has an L2 of its own: XCD x takes the x-th
    // eighth of the work list, which runs head by head, sequence by sequence, query block by query block, so
    // that the blocks of one (sequence, head) pair, which read the same keys, run side by side on one XCD.
    const int chunk = gridDim.x / 8;
    const int work = (blockIdx.x % 8) * chunk + blockIdx.x / 8;
    if (work >= a.numItems * a.H) {
        return;
    }
    const int h = work / a.numItems;
    const Item it = a.items[work % a.numItems];
    const int g = h / a.group;

    const int qLocal = wave * QW + n;
    const bool qValid = qLocal < it.nQ;
    const int qPos = it.qPos0 + qLocal;
    const bool waveHasWork = wave * QW < it.nQ;
    const int qFirstW = it.qPos0 + wave * QW;                       // first and last query position of this wave
    const int qLastW = it.qPos0 + min(it.nQ, wave * QW + QW) - 1;

    // ---- the keys this block visits
    int tBegin = 0;
    int tEnd = it.kvLen;
    if (a.mask != ATBMI_MLA_PREFILL_MASK_NONE) {
        tEnd = min(tEnd, it.qPos0 + it.nQ);
    }
    if (a.mask == ATBMI_MLA_PREFILL_MASK_WINDOW) {
        tBegin = max(0, it.qPos0 - a.window + 1) & ~(STEP - 1);
    }
    const int numTiles = tEnd > tBegin ? (tEnd - tBegin + STEP - 1) / STEP : 0;

    // ---- sources of this lane's slot in each of the wave's seven transfers: the address of its piece in
    // row 0 of the tensor, the bytes between rows of that tensor, and the slot's row inside the wave's eight
    const unsigned char *srcBase[DMA_PER_TILE];
    uint32_t srcStride[DMA_PER_TILE];
    uint32_t srcRows = 0; // 3 bits per transfer
#pragma unroll
    for (int i = 0; i < K_DMA; ++i) {
        const int slot = min(i * WAVE + lane, ROWS_PER_WAVE * K_SLOTS - 1);
        const int row = slot / K_SLOTS;
        const int piece = min(slot % K_SLOTS, D / 8 - 1);
        const bool rope = piece >= DN / 8;
        srcBase[i] = rope ? reinterpret_cast<const unsigned char *>(a.kRope) + (g * DR + (piece - DN / 8) * 8) * 2
                          : reinterpret_cast<const unsigned char *>(a.k) + (g * DN + piece * 8) * 2;
        srcStride[i] = static_cast<uint32_t>(a.G) * (rope ? DR * 2 : DN * 2);
        srcRows |= static_cast<uint32_t>(row) << (3 * i);
    }
#pragma unroll
    for (int i = 0; i < V_DMA; ++i) {
        const int slot = min(i * WAVE + lane, ROWS_PER_WAVE * V_SLOTS - 1);
        const int row = slot / V_SLOTS;
        const int piece = min(slot % V_SLOTS, DV / 8 - 1);
        srcBase[K_DMA + i] = reinterpret_cast<const unsigned char *>(a.v) + (g * DV + piece * 8) * 2;
        srcStride[K_DMA + i] = static_cast<uint32_t>(a.G) * (DV * 2);
        srcRows |= static_cast<uint32_t>(row) << (3 * (K_DMA + i));
    }
    const uint32_t ldsBase = static_cast<uint32_t>(
        reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) unsigned char *)smem));
    const uint32_t ldsWaveK = ldsBase + wave * (ROWS_PER_WAVE * K_PITCH);
    const uint32_t ldsWaveV = ldsBase + K_TILE + wave * (ROWS_PER_WAVE * V_PITCH);
    // Tiles are requested in order: a cursor per transfer walks this lane's source row from tile to tile, and only
    // a tile that reaches past the last key computes (and clamps) its rows anew.
    const unsigned char *cursor[DMA_PER_TILE];
#pragma unroll
    for (int i = 0; i < DMA_PER_TILE; ++i) {
        const int row = tBegin + wave * ROWS_PER_WAVE + static_cast<int>((srcRows >> (3 * i)) & 7u);
        cursor[i] = srcBase[i] + static_cast<uint64_t>(it.kRow0 + row) * srcStride[i];
    }
    // Requests this wave's rows of the tile at key t into tile buffer `buf`: seven transfers, always.
    auto requestTile = [&](int t, int buf) {
        const int row0 = t + wave * ROWS_PER_WAVE;
        const bool whole = t + STEP <= it.kvLen;
#pragma unroll
        for (int i = 0; i < DMA_PER_TILE; ++i) {
            const unsigned char *src = cursor[i];
            if (!whole) {
                const int row = min(row0 + static_cast<int>((srcRows >> (3 * i)) & 7u), it.kvLen - 1);
                src = srcBase[i] + static_cast<uint64_t>(it.kRow0 + row) * srcStride[i];
            }
            cursor[i] += STEP * srcStride[i];
            const bool isK = i < K_DMA;
            const int j = isK ? i : i - K_DMA;
            const uint32_t dst = (isK ? ldsWaveK : ldsWaveV) + static_cast<uint32_t>(buf * BUF + j * (WAVE * 16));
            const int slots = isK ? ROWS_PER_WAVE * K_SLOTS : ROWS_PER_WAVE * V_SLOTS;
            if (j * WAVE + lane < slots) {
                TransferToLds(__builtin_amdgcn_readfirstlane(dst), src);
            }
        }
    };
    if (numTiles > 0) {
        requestTile(tBegin, 0);
    }
    if (numTiles > 1) {
        requestTile(tBegin + STEP, 1);
    }

    // ---- Q^T as B operand: lane (n, kh) holds q[n][16 j + 8 kh .. +8) for the 12 pieces j
    u32x4 qreg[D / 16];
    {
        const int64_t rowHead = (static_cast<int64_t>(it.qRow0) + (qValid ? qLocal : 0)) * a.H + h;
        const uint16_t *qn = reinterpret_cast<const uint16_t *>(a.q) + rowHead * DN + kh * 8;
        const uint16_t *qr = reinterpret_cast<const uint16_t *>(a.qRope) + rowHead * DR + kh * 8;
#pragma unroll
        for (int j = 0; j < D / 16; ++j) {
            qreg[j] = *reinterpret_cast<const u32x4 *>(j < DN / 16 ? qn + 16 * j : qr + 16 * (j - DN / 16));
            if (!qValid) {
                qreg[j] = u32x4{0u, 0u, 0u, 0u};
            }
        }
    }

    float m = -INFINITY; // running maximum of query n, base-2 exponent units
    float l = 0.0f;      // this lane's share of the running denominator
    f32x16 acc[DV / 32];
#pragma unroll
    for (int i = 0; i < DV / 32; ++i) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            acc[i][e] = 0.0f;
        }
    }

    const int l16 = lane & 15;
    const int kOperand = n * K_PITCH + kh * 16;
    const int vOperand = K_TILE + (4 * kh + (l16 >> 2)) * V_PITCH + (((lane >> 4) & 1) * 16 + (l16 & 3) * 4) * 2;

    constexpr float SLACK = 8.0f;
    auto computeStep = [&](int t, const unsigned char *buf) {
        f32x16 s;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            s[e] = 0.0f;
        }
        // K operands are requested four pieces ahead of the MFMA that takes them
        constexpr int AHEAD = 4;
        u32x4 kk[AHEAD];
#pragma unroll
        for (int j = 0; j < AHEAD; ++j) {
            kk[j] = *reinterpret_cast<const u32x4 *>(buf + kOperand + j * 32);
        }
#pragma unroll
        for (int j = 0; j < D / 16; ++j) {
            s = Mma<BF16>(kk[j % AHEAD], qreg[j], s);
            if (j + AHEAD < D / 16) {
                kk[j % AHEAD] = *reinterpret_cast<const u32x4 *>(buf + kOperand + (j + AHEAD) * 32);
            }
        }
        // keep that order: four reads, then one MFMA and one read in turn (the scheduler would otherwise
        // hold only two reads in flight and wait for each pair)
        __builtin_amdgcn_sched_group_barrier(0x100, AHEAD, 0);
#pragma unroll
        for (int j = 0; j + AHEAD < D / 16; ++j) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, AHEAD, 0);
        // every key of the step visible to every query of the wave: no comparisons
        const bool open = t + STEP <= it.kvLen &&
                          (a.mask == ATBMI_MLA_PREFILL_MASK_NONE ||
                           (t + STEP - 1 <= qFirstW &&
                            (a.mask != ATBMI_MLA_PREFILL_MASK_WINDOW || t > qLastW - a.window)));
        if (!open) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int tok = t + 8 * (e >> 2) + 4 * kh + (e & 3);
                bool hidden = tok >= it.kvLen;
                if (a.mask != ATBMI_MLA_PREFILL_MASK_NONE) {
                    hidden = hidden || tok > qPos;
                }
                if (a.mask == ATBMI_MLA_PREFILL_MASK_WINDOW) {
                    hidden = hidden || tok <= qPos - a.window;
                }
                s[e] = hidden ? -INFINITY : s[e];
            }
        }
        // the maximum is taken over the raw scores (the scale is positive) and the scale multiplies inside the
        // exponent's fused multiply-add
        float mLoc = fmaxf(fmaxf(s[0], s[1]), s[2]);
#pragma unroll
        for (int e = 3; e < 15; e += 2) {
            mLoc = fmaxf(fmaxf(mLoc, s[e]), s[e + 1]);
        }
        mLoc = fmaxf(mLoc, s[15]);
        mLoc = fmaxf(mLoc, __shfl_xor(mLoc, 32)) * a.scale2;
        // The reference point of the exponents moves only when the step's maximum is more than 2^SLACK above
        // it: weights may then reach 2^SLACK, which the 16-bit P and the fp32 sums hold with the same relative
        // precision, and the 64 accumulators are rescaled on a few steps instead of most.
        const float mNew = mLoc > m + SLACK ? mLoc : m; // (m = -inf: the first visible key sets it)
        const float mRef = mNew == -INFINITY ? 0.0f : mNew; // nothing visible so far: every weight is 0
        const float corr = Exp2(m - mRef);
        m = mNew;
        float sum = 0.0f;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            s[e] = Exp2(__builtin_fmaf(s[e], a.scale2, -mRef));
            sum += s[e];
        }
        l = l * corr + sum;
        if (__any(corr != 1.0f)) {
#pragma unroll
            for (int i = 0; i < DV / 32; ++i) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    acc[i][e] *= corr;
                }
            }
        }
        u32x4 pop[2]; // P^T as B operand of the two half-steps
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                pop[kb][w] = Pack2<BF16>(s[8 * kb + 2 * w], s[8 * kb + 2 * w + 1]);
            }
        }
        auto readV = [&](int idx) -> u32x4 { // V^T operand of output tile idx / 2, half-step idx % 2
            const unsigned char *vp = buf + vOperand + (idx & 1) * 16 * V_PITCH + (idx >> 1) * 64;
            const i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4 *)(vp));
            const i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) i16x4 *)(vp + 8 * V_PITCH));
            const u32x2 lo2 = __builtin_bit_cast(u32x2, lo);
            const u32x2 hi2 = __builtin_bit_cast(u32x2, hi);
            return u32x4{lo2[0], lo2[1], hi2[0], hi2[1]};
        };
        constexpr int NV = 2 * (DV / 32);
        u32x4 vv[AHEAD];
#pragma unroll
        for (int i = 0; i < AHEAD; ++i) {
            vv[i] = readV(i);
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            acc[i >> 1] = Mma<BF16>(vv[i % AHEAD], pop[i & 1], acc[i >> 1]);
            if (i + AHEAD < NV) {
                vv[i % AHEAD] = readV(i + AHEAD);
            }
        }
    };

    int buf = 0;
    for (int i = 0; i < numTiles; ++i) {
        const int t = tBegin + i * STEP;
        // this wave's rows of tile i have landed (the transfers of tile i + 1 may still be on their way) ...
        if (i + 1 < numTiles) {
            asm volatile("s_waitcnt vmcnt(7)" ::: "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        // ... and so have everybody else's, and everybody has left tile i - 1, whose buffer tile i + 2 takes
        __syncthreads();
        if (i + 2 < numTiles) {
            requestTile(t + 2 * STEP, buf == 0 ? 2 : buf - 1);
        }
        // a wave skips the steps that its own queries cannot see
        bool visit = waveHasWork;
        if (a.mask != ATBMI_MLA_PREFILL_MASK_NONE) {
            visit = visit && t <= qLastW;
        }
        if (a.mask == ATBMI_MLA_PREFILL_MASK_WINDOW) {
            visit = visit && t + STEP - 1 > qFirstW - a.window;
        }
        if (visit) {
            computeStep(t, smem + buf * BUF);
        }
        buf = buf == NBUF - 1 ? 0 : buf + 1;
    }

    // ---- out[q][h][32 i + 8 r + 4 kh .. +4) = acc / l
    l += __shfl_xor(l, 32);
    const float inv = l > 0.0f ? 1.0f / l : 0.0f; // a query that sees no key yields zeros
    if (qValid) {
        uint16_t *orow = reinterpret_cast<uint16_t *>(a.out) +
                         ((static_cast<int64_t>(it.qRow0) + qLocal) * a.H + h) * DV + 4 * kh;
#pragma unroll
        for (int i = 0; i < DV / 32; ++i) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                u32x2 w;
                w[0] = Pack2<BF16>(acc[i][4 * r] * inv, acc[i][4 * r + 1] * inv);
                w[1] = Pack2<BF16>(acc[i][4 * r + 2] * inv, acc[i][4 * r + 3] * inv);
                *reinterpret_cast<u32x2 *>(orow + 32 * i + 8 * r) = w;
            }
        }
    }
}

// Checks the call and lists its query blocks.
int BuildItems(const AtbmiMlaPrefillCall *c, std::vector<Item> *items)
{
    if (!c || !c->hostQLens || !c->hostKvLens) {
        return Fail(ERR_INVALID_PARAM, "mla_prefill: null call or length arrays");
    }
    if (c->dtype != ATBMI_F16 && c->dtype != ATBMI_BF16) {
        return Fail(ERR_INVALID_PARAM, "mla_prefill: dtype %d (fp16 or bf16)", c->dtype);
    }
    if (c->numHeads <= 0 || c->numKvHeads <= 0 || c->numHeads % c->numKvHeads != 0) {
        return Fail(ERR_INVALID_PARAM, "mla_prefill: %d heads over %d KV heads", c->numHeads, c->numKvHeads);
    }
    if (c->mask < ATBMI_MLA_PREFILL_MASK_NONE || c->mask > ATBMI_MLA_PREFILL_MASK_WINDOW) {
        return Fail(ERR_INVALID_PARAM, "mla_prefill: mask %d", c->mask);
    }
    if (c->mask == ATBMI_MLA_PREFILL_MASK_WINDOW && c->windowSize <= 0) {
        return Fail(ERR_INVALID_PARAM, "mla_prefill: a window mask needs windowSize > 0, got %d", c->windowSize);
    }
    if (c->batch < 0 || c->kvPaddedRows < 0 || !(c->qkScale > 0.0f)) {
        return Fail(ERR_INVALID_PARAM, "mla_prefill: batch %d, kvPaddedRows %lld, qkScale %g", c->batch,
                    (long long)c->kvPaddedRows, c->qkScale);
    }
    int64_t qRow = 0, kRow = 0;
    for (int32_t b = 0; b < c->batch; ++b) {
        const int32_t nq = c->hostQLens[b];
        const int32_t nk = c->hostKvLens[b];
        if (nq < 0 || nk < 0) {
            return Fail(ERR_INVALID_PARAM, "mla_prefill: sequence %d has lengths %d / %d", b, nq, nk);
        }
        if (c->mask != ATBMI_MLA_PREFILL_MASK_NONE && nq != nk) {
            return Fail(ERR_INVALID_PARAM, "mla_prefill: with a mask, query and key lengths must agree (sequence %d: %d / %d)",
                        b, nq, nk);
        }
        if (c->kvPaddedRows > 0) {
            if (nk > c->kvPaddedRows) {
                return Fail(ERR_INVALID_PARAM, "mla_prefill: sequence %d has %d keys in %lld padded rows", b, nk,
                            (long long)c->kvPaddedRows);
            }
            kRow = static_cast<int64_t>(b) * c->kvPaddedRows;
        }
        if (qRow + nq > 0x7fffffffLL || kRow + nk > 0x7fffffffLL) {
            return Fail(ERR_INVALID_PARAM, "mla_prefill: more than 2^31 rows");
        }
        // the blocks of a sequence follow each other, the one that walks the most keys (under a mask: the
        // last one) first
        for (int32_t q0 = (nq - 1) / QB * QB; nq > 0 && q0 >= 0; q0 -= QB) {
            Item it{};
            it.qRow0 = static_cast<int32_t>(qRow + q0);
            it.nQ = nq - q0 < QB ? nq - q0 : QB;
            it.kRow0 = static_cast<int32_t>(kRow);
            it.kvLen = nk;
            it.qPos0 = q0;
            if (items) {
                items->push_back(it);
            }
        }
        qRow += nq;
        kRow += nk;
    }
    return OK;
}

} // namespace prefill
} // namespace atbmi

using namespace atbmi;

extern "C" int atbmi_mla_prefill_workspace_size(const AtbmiMlaPrefillCall *call, uint64_t *bytes)
{
    if (!bytes) {
        return Fail(ERR_INVALID_PARAM, "mla_prefill_workspace_size: null result pointer");
    }
    std::vector<prefill::Item> items;
    const int rc = prefill::BuildItems(call, &items);
    if (rc != OK) {
        return rc;
    }
    *bytes = items.size() * sizeof(prefill::Item);
    return OK;
}

extern "C" int atbmi_mla_prefill(const AtbmiMlaPrefillCall *call, void *workspaceDevice, uint64_t workspaceBytes,
                                 void *stream)
{
    std::vector<prefill::Item> items;
    int rc = prefill::BuildItems(call, &items);
    if (rc != OK) {
        return rc;
    }
    if (items.empty()) {
        return OK;
    }
    if (!call->query || !call->queryRope || !call->key || !call->keyRope || !call->value || !call->out) {
        return Fail(ERR_INVALID_PARAM, "mla_prefill: null tensor pointer");
    }
    const size_t bytes = items.size() * sizeof(prefill::Item);
    if (!workspaceDevice || workspaceBytes < bytes) {
        return Fail(ERR_INVALID_PARAM, "mla_prefill: workspace of %llu bytes, %llu needed",
                    (unsigned long long)workspaceBytes, (unsigned long long)bytes);
    }
    const int64_t grid = (static_cast<int64_t>(items.size()) * call->numHeads + 7) / 8 * 8;
    if (grid > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "mla_prefill: %lld workgroups", (long long)grid);
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    rc = UploadTable(items.data(), bytes, workspaceDevice, s);
    if (rc != OK) {
        return rc;
    }
    prefill::Args a{};
    a.q = call->query;
    a.qRope = call->queryRope;
    a.k = call->key;
    a.kRope = call->keyRope;
    a.v = call->value;
    a.out = call->out;
    a.items = static_cast<const prefill::Item *>(workspaceDevice);
    a.numItems = static_cast<int32_t>(items.size());
    a.H = call->numHeads;
    a.G = call->numKvHeads;
    a.group = call->numHeads / call->numKvHeads;
    a.mask = call->mask;
    a.window = call->windowSize;
    a.scale2 = call->qkScale * 1.4426950408889634f;
    auto kernel = call->dtype == ATBMI_BF16 ? prefill::MlaPrefillKernel<true> : prefill::MlaPrefillKernel<false>;
    rc = ConfigureKernelLds(reinterpret_cast<const void *>(kernel), prefill::LDS_BYTES);
    if (rc != OK) {
        return rc;
    }
    kernel<<<static_cast<unsigned>(grid), prefill::NWAVES * WAVE, prefill::LDS_BYTES, s>>>(a);
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}
