// Decode attention over the combined MLA cache (key row 576 channels, value =
// its first 512) for 128 query heads per workgroup, gfx950 (MI355X).
//
// Why a kernel of its own: at 576/512 channels the arithmetic intensity is
// 128 heads x 2 flop per cache byte-pair, close to the machine's ridge, and the
// bound is no longer HBM but how fast the latent tile can be fed from LDS into
// the matrix cores. What matters then is how many query heads share one LDS
// operand read, and that a single wave per SIMD (all the registers: the 32-head
// accumulators alone are 256 of them) keeps its matrix pipe busy. Hence:
//   - v_mfma_f32_32x32x16: 32 query heads per wave, so every K / V^T operand
//     read from LDS feeds 32 heads, and one wave issuing these 8-pass
//     instructions back to back saturates its SIMD's matrix pipe (16x16x32
//     from a single wave reaches two thirds of that).
//   - 4 waves x 32 heads = all 128 heads of one token range in one workgroup:
//     the latent tile is fetched from HBM once and staged once.
//   - HBM -> LDS directly (global_load_lds_dwordx4), no staging registers, no
//     LDS store instructions. Three tile buffers: while a step computes on
//     one, the next tile has landed or is landing in the second and the
//     transfers of the tile after it are issued into the third, a few MFMAs
//     apart. Each wave stages 8 of the 32 rows into its own region of the
//     tile; rows keep the cache's order at a pitch of 1168 bytes (292 dwords
//     = 36 mod 64 banks) and odd regions start half the banks further, which
//     makes both the 32-row operand reads and the transposing reads
//     conflict-free.
//
// Layouts (lane = 32 kh + n):
//   S^T = K . Q^T   A = K tile: lane reads token row n, channels 16 j + 8 kh .. +8 (ds_read_b128)
//                   B = Q^T in registers: head n, same channels; 36 k-steps
//                   accumulator element e of lane (n, kh): token 8 (e/4) + 4 kh + e%4, head n
//   O^T += V^T.P^T  contraction over 16 tokens per MFMA, two per 32-token step (kb = 0, 1). The k index
//                   8 kh + e stands for token 16 kb + 8 (e/4) + 4 kh + e%4, which is exactly the token of
//                   accumulator element 8 kb + e: P goes from the softmax into the B operand without
//                   leaving its lane. V^T (A operand, channel 32 i + n) is read with two transposing
//                   ds_read_b64_tr_b16 per MFMA, each lane pointing at the token row the permutation asks for.
//
// The plan is the "stream" plan of the 16-bit kernels with one wave range per
// workgroup: ranges that cross a sequence boundary finish one row and start
// the next, rows spanning several ranges leave partials for the merge kernel.
#ifndef ATBMI_PA_MLA_KERNEL_H
#define ATBMI_PA_MLA_KERNEL_H
#include <type_traits>
#include "pa_mfma_kernel.h"

namespace atbmi {
namespace mla {

using mfma::f16x8;
using mfma::bf16x8;
using mfma::i16x4;
using mfma::u32x2;
using mfma::u32x4;
using mfma::f32x4;
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int D = 576;
constexpr int DV = 512;
constexpr int STEP = PA_MFMA_STEP;           // tokens per step
constexpr int NW = PA_MLA_WAVES;             // waves per workgroup
constexpr int HPW = PA_MLA_HEADS_PER_WG / NW; // query heads per wave (the N extent of the 32x32 tile)
constexpr int PITCH = D * 2 + 16;            // tile row pitch in bytes
constexpr int ROWS_PER_WAVE = STEP / NW;     // tile rows each wave stages: one region of the tile
constexpr int CHUNKS = (ROWS_PER_WAVE * PITCH + 1023) / 1024; // 1 KB transfer instructions per wave and step
// A region is written by whole-wave transfers only (no lane is ever masked off): CHUNKS KB, of which the
// 8 rows use 9344 bytes and the rest is padding; 128 more bytes shift odd regions by half the LDS banks, so
// that the 16 rows a quarter-wave reads together (two regions) fall on 16 different bank groups.
constexpr int REGION = CHUNKS * 1024 + 128;
constexpr int TILE_BYTES = NW * REGION;
constexpr int SLOTS_PER_ROW = PITCH / 16;    // 16-byte slots per tile row, the last one padding
constexpr int WAVE_SLOTS = ROWS_PER_WAVE * SLOTS_PER_ROW;
// LDS byte offset of tile row `row`
__device__ __forceinline__ constexpr int RowOffset(int row)
{
    return (row / ROWS_PER_WAVE) * REGION + (row % ROWS_PER_WAVE) * PITCH;
}
constexpr int NQ = D / 16;                   // QK MFMAs per step
constexpr int NO = DV / 32;                  // output tiles of 32 channels
constexpr int KD = 5;                        // K operands in flight ahead of the MFMA that uses them
constexpr int VD = 5;                        // V^T operands in flight
constexpr int QK_PER_TRANSFER = NQ / (CHUNKS / 2);          // QK MFMAs between transfers
constexpr int PV_PER_TRANSFER = 2 * NO / (CHUNKS - CHUNKS / 2); // PV MFMAs between transfers
constexpr int BLK_IDS = 1024;                // block ids of a segment held in LDS at a time
static_assert(HPW == 32 && STEP == 32 && ROWS_PER_WAVE == 8, "built around the 32x32x16 tile");

// The three MFMA forms the kernel uses, written as assembly so that the register file is split the one
// way that fits: the 16 output accumulators are the 256 AGPRs, everything else (Q, scores, operands)
// lives in the 256 VGPRs. Left to the register allocator the two halves get mixed and the loop spills.
// The compiler cannot see the latency of these instructions: MmaFence() must separate the last of a
// chain from the first ordinary instruction that reads the chain's result, and MmaOperandFence() an
// ordinary instruction that writes an operand from the MFMA that reads it (the forms that start a
// chain carry that wait themselves).
#define ATBMI_MFMA32(type) "v_mfma_f32_32x32x16_" type " %0, %1, %2, "
template <bool BF16> __device__ __forceinline__ void MmaScoreFirst(f32x16 &s, u32x4 a, u32x4 b)
{
    if constexpr (BF16) {
        asm volatile("s_nop 15\n\t" ATBMI_MFMA32("bf16") "0" : "=v"(s) : "v"(a), "v"(b));
    } else {
        asm volatile("s_nop 15\n\t" ATBMI_MFMA32("f16") "0" : "=v"(s) : "v"(a), "v"(b));
    }
}
template <bool BF16> __device__ __forceinline__ void MmaScore(f32x16 &s, u32x4 a, u32x4 b)
{
    if constexpr (BF16) {
        asm volatile(ATBMI_MFMA32("bf16") "%0" : "+v"(s) : "v"(a), "v"(b));
    } else {
        asm volatile(ATBMI_MFMA32("f16") "%0" : "+v"(s) : "v"(a), "v"(b));
    }
}
template <bool BF16> __device__ __forceinline__ void MmaOut(f32x16 &acc, u32x4 a, u32x4 b)
{
    if constexpr (BF16) {
        asm volatile(ATBMI_MFMA32("bf16") "%0" : "+a"(acc) : "v"(a), "v"(b));
    } else {
        asm volatile(ATBMI_MFMA32("f16") "%0" : "+a"(acc) : "v"(a), "v"(b));
    }
}
// acc = 0 (a product of zero operands), without staging 256 zeros in VGPRs.
template <bool BF16> __device__ __forceinline__ void MmaOutZero(f32x16 &acc)
{
    const u32x4 z = {0u, 0u, 0u, 0u};
    if constexpr (BF16) {
        asm volatile("s_nop 15\n\t" ATBMI_MFMA32("bf16") "0" : "=a"(acc) : "v"(z), "v"(z));
    } else {
        asm volatile("s_nop 15\n\t" ATBMI_MFMA32("f16") "0" : "=a"(acc) : "v"(z), "v"(z));
    }
}
#undef ATBMI_MFMA32
__device__ __forceinline__ void MmaOperandFence(u32x4 &b0, u32x4 &b1)
{
    // the operands pass through the statement, so the compiler cannot move their last write below it
    asm volatile("s_nop 15" : "+v"(b0), "+v"(b1));
}
// 18 idle cycles: more than the wait an 8-pass MFMA result needs before another unit may read it.
__device__ __forceinline__ void MmaFence(f32x16 &v)
{
    asm volatile("s_nop 15\n\ts_nop 1" : "+v"(v));
}
__device__ __forceinline__ void MmaFenceOut(f32x16 (&acc)[NO])
{
    static_assert(NO == 16, "operand list below");
    asm volatile("s_nop 15\n\ts_nop 1"
                 : "+a"(acc[0]), "+a"(acc[1]), "+a"(acc[2]), "+a"(acc[3]), "+a"(acc[4]), "+a"(acc[5]), "+a"(acc[6]),
                   "+a"(acc[7]), "+a"(acc[8]), "+a"(acc[9]), "+a"(acc[10]), "+a"(acc[11]), "+a"(acc[12]),
                   "+a"(acc[13]), "+a"(acc[14]), "+a"(acc[15]));
}

// HBM -> LDS transfers that pass through no register. DmaBase sets the LDS base (register M0) for a run
// of them; DmaPieceAt then moves, for every lane, 16 bytes from src + OFFSET to LDS base + OFFSET +
// 16 * lane (the instruction's immediate offset, -4096 .. 4095, moves both addresses). The compiler
// neither sees the transfers nor knows that M0 is in use: no code of its own between DmaBase and the
// last DmaPieceAt of a run may use M0 (nothing this kernel is compiled to does), and DmaWait() or a
// counted wait must come before the barrier that publishes a tile.
__device__ __forceinline__ void DmaBase(uint32_t ldsBase)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0" : : "s"(ldsBase) : "memory");
}
template <int OFFSET> __device__ __forceinline__ void DmaPieceAt(const void *src)
{
    asm volatile("global_load_lds_dwordx4 %0, off offset:%1" : : "v"(src), "n"(OFFSET) : "memory");
}

__device__ __forceinline__ void DmaWait()
{
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// SPLIT: the last 64 channels of every latent row live in a cache of their own (a.kRope), those of every
// query row in a.qRope; a.kc and a.q then hold 512-channel rows.
template <bool BF16, bool SPLIT>
__global__ __launch_bounds__(NW *WAVE) void PaMlaWideKernel(const PaArgs a, const PaStreamPlan p)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int lane = threadIdx.x % WAVE;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int n = lane & 31; // head (B operand / accumulator column); token or channel (A operand row)
    const int kh = lane >> 5; // which 8 of the 16 contraction values this lane holds
    const bool qBf16 = a.qIsBf16 != 0;

    // Workgroup -> (token range, group of 128 heads): the groups of one range sit 8 ids apart (same XCD).
    const int octet = blockIdx.x / (8 * p.headGroups);
    const int within = blockIdx.x % (8 * p.headGroups);
    const int hgIdx = within / 8;
    const int wr = octet * 8 + within % 8;
    if (wr >= p.numWgRanges) {
        return;
    }
    const int s0 = PaRangeBegin(wr, p.totalSteps, p.numWaveRanges);
    const int s1 = PaRangeBegin(wr + 1, p.totalSteps, p.numWaveRanges);
    if (s0 >= s1) {
        return;
    }
    const int h0 = hgIdx * PA_MLA_HEADS_PER_WG + wave * HPW;

    const uint32_t ldsBase = static_cast<uint32_t>(
        reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) unsigned char *)smem));
    const unsigned char *kcBase = reinterpret_cast<const unsigned char *>(a.kc);
    const int64_t rowBytes = a.kRowStride * 2;
    const unsigned char *krBase = reinterpret_cast<const unsigned char *>(a.kRope);
    const int64_t ropeRowBytes = a.ropeRowStride * 2;
    constexpr int NOPE_PIECES = DV * 2 / 16; // 16-byte pieces of a latent row ahead of its rope channels
    constexpr float LOG2E = 1.4426950408889634f;
    const float scale2 = a.qkScale * LOG2E;

    // The plan is the same for every lane: say so, and the loop control below runs on the scalar unit.
    auto uniform = [](int v) { return __builtin_amdgcn_readfirstlane(v); };
    int seqIdx = uniform(p.firstSeq ? p.firstSeq[wr] : p.inlineFirst[wr]);
    while (uniform(mfma::PlanSeq(p, seqIdx + 1).stepBegin) <= s0) {
        ++seqIdx;
    }

    for (; seqIdx < p.numSeqs; ++seqIdx) {
        PaSeq sq = mfma::PlanSeq(p, seqIdx);
        sq.tableRow = uniform(sq.tableRow);
        sq.ctxLen = uniform(sq.ctxLen);
        sq.stepBegin = uniform(sq.stepBegin);
        if (sq.stepBegin >= s1) {
            break;
        }
        const int seqEnd = uniform(mfma::PlanSeq(p, seqIdx + 1).stepBegin);
        const int segBegin = max(s0, sq.stepBegin);
        const int segEnd = min(s1, seqEnd);
        const int tokBegin = (segBegin - sq.stepBegin) * STEP;
        const int tokEnd = min(sq.ctxLen, (segEnd - sq.stepBegin) * STEP);
        const bool complete = segBegin == sq.stepBegin && segEnd == seqEnd;
        const int qRow = uniform(sq.qRow); // (128 heads fill the tile: a pass never holds a second query token)

        // ---- block ids of this segment sit in LDS (BLK_IDS at a time) and are read one tile ahead of
        // their use: the step loop then holds no memory instruction of the compiler's whose wait would
        // also wait for the tile transfers in flight (vector loads), or stall every LDS wait behind an
        // HBM round trip (scalar loads return out of order).
        const int32_t *table = a.tables + static_cast<int64_t>(sq.tableRow) * a.maxBlocksPerSeq;
        const int lastBlk = (tokEnd - 1) / a.blockSize; // entries past this one are never read
        int curBlk = tokBegin / a.blockSize;            // cursor: the next 16-token sub-tile to look up
        int curOff = tokBegin % a.blockSize;
        int idBase = curBlk;                            // block index of blkIds[0]
        int32_t *blkIds = reinterpret_cast<int32_t *>(smem + 3 * TILE_BYTES);
        auto fillIds = [&]() { // all waves together
            __syncthreads(); // nobody still reads the old ids
            for (int i = threadIdx.x; i < BLK_IDS && idBase + i <= lastBlk; i += NW * WAVE) {
                blkIds[i] = table[idBase + i];
            }
            __syncthreads();
        };
        fillIds();
        int pendBlk[2]; // (still in flight from LDS) block ids of the two sub-tiles of the next tile
        int pendOff[2]; // and the row offsets inside those blocks
        auto lookAhead = [&]() {
#pragma unroll
            for (int sub = 0; sub < 2; ++sub) {
                const int blkIdx = min(curBlk, lastBlk);
                if (blkIdx >= idBase + BLK_IDS) {
                    idBase = blkIdx;
                    fillIds();
                }
                pendBlk[sub] = blkIds[blkIdx - idBase];
                pendOff[sub] = curOff;
                curOff += 16;
                if (curOff >= a.blockSize) {
                    curOff = 0;
                    ++curBlk;
                }
            }
        };
        lookAhead();

        // Transfer of the 32 latent rows at token t into the tile at LDS address tileAddr: prepare() once,
        // then transfer(0 .. CHUNKS-1), exactly CHUNKS instructions per wave whatever the tile (the waits
        // below count them). Wave w moves tile rows 8w .. 8w+7; the rows of a 16-token sub-tile are
        // consecutive cache rows (a sub-tile never straddles cache blocks). Tile rows at or past the end
        // of the segment get a copy of its last row: they only have to be finite, their weights are
        // exact zeros. Lane l of transfer i fills slot 64 i + l of the wave's region; slots that hold no
        // data (the padding slot of each row, everything past the 8 rows) fetch a neighbour's piece, so
        // every lane of every transfer is active and reads valid memory.
        const unsigned char *stSub0 = nullptr, *stSub1 = nullptr;
        const unsigned char *stRope0 = nullptr, *stRope1 = nullptr; // SPLIT: the same rows of the rope cache
        int stLastRow = 0;
        uint32_t stDst = 0;
        auto prepare = [&](int t, uint32_t tileAddr) {
            const int64_t row0 = static_cast<int64_t>(__builtin_amdgcn_readfirstlane(pendBlk[0])) * a.blockSize + pendOff[0];
            const int64_t row1 = static_cast<int64_t>(__builtin_amdgcn_readfirstlane(pendBlk[1])) * a.blockSize + pendOff[1];
            stSub0 = kcBase + row0 * rowBytes;
            stSub1 = kcBase + row1 * rowBytes;
            if constexpr (SPLIT) {
                stRope0 = krBase + row0 * ropeRowBytes;
                stRope1 = krBase + row1 * ropeRowBytes;
            }
            lookAhead();
            stLastRow = min(tokEnd - 1 - t, STEP - 1);
            stDst = tileAddr + static_cast<uint32_t>(wave * REGION);
        };
        // Transfers 0 .. 7 go through one setting of the LDS base (the middle of their 8 KB), 8 and 9
        // through a second one.
        auto transfer = [&](auto index) {
            constexpr int i = decltype(index)::value;
            int ln = lane;
            if constexpr (SPLIT) {
                // rederive the slot from the lane id at every transfer: hoisted out of the loop, the
                // per-lane row, piece and cache choice of ten transfers would not fit the registers
                asm volatile("" : "+v"(ln));
            }
            int slot = i * WAVE + ln;
            slot = slot < WAVE_SLOTS ? slot : slot - WAVE_SLOTS;
            const int rowIn = slot / SLOTS_PER_ROW;
            const int col = min(slot - rowIn * SLOTS_PER_ROW, SLOTS_PER_ROW - 2);
            const int row = min(ROWS_PER_WAVE * wave + rowIn, stLastRow);
            const unsigned char *src = ((row >> 4) ? stSub1 : stSub0) +
                                       static_cast<uint32_t>(row & 15) * static_cast<uint32_t>(rowBytes) + col * 16;
            if constexpr (SPLIT) {
                if (col >= NOPE_PIECES) {
                    src = ((row >> 4) ? stRope1 : stRope0) +
                          static_cast<uint32_t>(row & 15) * static_cast<uint32_t>(ropeRowBytes) + (col - NOPE_PIECES) * 16;
                }
            }
            if constexpr (i == 0) {
                DmaBase(stDst + 4096);
            }
            if constexpr (i == 8) {
                DmaBase(stDst + 8192);
            }
            constexpr int imm = i < 8 ? (i - 4) * 1024 : (i - 8) * 1024;
            DmaPieceAt<imm>(src - imm);
        };
        auto transferAll = [&]() {
            transfer(std::integral_constant<int, 0>{});
            transfer(std::integral_constant<int, 1>{});
            transfer(std::integral_constant<int, 2>{});
            transfer(std::integral_constant<int, 3>{});
            transfer(std::integral_constant<int, 4>{});
            transfer(std::integral_constant<int, 5>{});
            transfer(std::integral_constant<int, 6>{});
            transfer(std::integral_constant<int, 7>{});
            transfer(std::integral_constant<int, 8>{});
            transfer(std::integral_constant<int, 9>{});
        };
        static_assert(CHUNKS == 10, "transfer schedule");

        // The first two tiles are on their way while Q is fetched; from then on the transfers of the tile
        // two steps ahead are issued during each step, one every few MFMAs.
        prepare(tokBegin, ldsBase);
        transferAll();
        if (tokBegin + STEP < tokEnd) {
            prepare(tokBegin + STEP, ldsBase + TILE_BYTES);
            transferAll();
        }

        // ---- Q^T as B operand: lane (n, kh) holds q[h0+n][16 j + 8 kh .. +8) for j < NQ
        u32x4 qreg[NQ];
        {
            const int64_t qh = static_cast<int64_t>(qRow) * a.H + h0 + n;
            const uint16_t *qrow = reinterpret_cast<const uint16_t *>(a.q) + qh * (SPLIT ? DV : D) + kh * 8;
            const uint16_t *qrope = reinterpret_cast<const uint16_t *>(a.qRope) + qh * (D - DV) - DV + kh * 8;
#pragma unroll
            for (int j = 0; j < NQ; ++j) {
                qreg[j] = mfma::LoadGlobal16((SPLIT && j * 16 >= DV ? qrope : qrow) + j * 16);
            }
        }

        float m = -INFINITY; // running maximum of head n, base-2 exponent units
        float lsum = 0.0f;   // this lane's share (its 16 tokens of every step) of the denominator of head n
        f32x16 acc[NO];
#pragma unroll
        for (int i = 0; i < NO; ++i) {
            MmaOutZero<BF16>(acc[i]); // zeros written by the matrix core, straight into the AGPRs
        }

        DmaWait();
        // Touch Q here so that the compiler's own wait for the Q loads lands before the loop and not,
        // counting down, inside it, where it would also wait for the tile transfers in flight.
#pragma unroll
        for (int j = 0; j < NQ; ++j) {
            asm volatile("" : "+v"(qreg[j]));
        }
        __syncthreads();

        int buf = 0;
        for (int t = tokBegin; t < tokEnd; t += STEP) {
            const unsigned char *tile = smem + buf * TILE_BYTES;
            // Operand read offsets inside the tile, rederived from the lane id every step (two
            // instructions each) rather than kept live across the whole kernel.
            int ln = lane;
            asm volatile("" : "+v"(ln));
            const int kOff = RowOffset(ln & 31) + (ln >> 5) * 16;
            const int vOff = (4 * (ln >> 5) + ((ln >> 2) & 3)) * PITCH + (16 * ((ln >> 4) & 1) + 4 * (ln & 3)) * 2;

            const bool fetch = t + 2 * STEP < tokEnd; // a tile two steps ahead exists: fetch it during this step
            if (fetch) {
                prepare(t + 2 * STEP, ldsBase + (buf == 0 ? 2 : buf - 1) * TILE_BYTES);
            }

            // ---- S^T = K . Q^T, operands fetched KD MFMAs ahead
            f32x16 s;
            {
                const unsigned char *krow = tile + kOff;
                u32x4 kop[KD + 1];
#pragma unroll
                for (int j = 0; j < KD; ++j) {
                    kop[j] = *reinterpret_cast<const u32x4 *>(krow + j * 32);
                }
#pragma unroll
                for (int j = 0; j < NQ; ++j) {
                    if (j + KD < NQ) {
                        kop[(j + KD) % (KD + 1)] = *reinterpret_cast<const u32x4 *>(krow + (j + KD) * 32);
                    }
                    if (j == 0) {
                        MmaScoreFirst<BF16>(s, kop[0], qreg[0]);
                    } else {
                        MmaScore<BF16>(s, kop[j % (KD + 1)], qreg[j]);
                    }
                    if (j % QK_PER_TRANSFER == QK_PER_TRANSFER / 2 && j / QK_PER_TRANSFER < CHUNKS / 2 && fetch) {
                        switch (j / QK_PER_TRANSFER) {
                            case 0: transfer(std::integral_constant<int, 0>{}); break;
                            case 1: transfer(std::integral_constant<int, 1>{}); break;
                            case 2: transfer(std::integral_constant<int, 2>{}); break;
                            case 3: transfer(std::integral_constant<int, 3>{}); break;
                            default: transfer(std::integral_constant<int, 4>{}); break;
                        }
                    }
                }
                MmaFence(s);
            }

            // ---- online softmax in base 2; element e is token t + 8 (e/4) + 4 kh + e%4 of head n
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                s[e] *= scale2;
            }
            if (t + STEP > tokEnd) { // last step of the segment: mask the tokens past its end
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int tok = t + 8 * (e >> 2) + 4 * kh + (e & 3);
                    s[e] = tok < tokEnd ? s[e] : -INFINITY;
                }
            }
            float mloc = fmaxf(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])), fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7])));
            mloc = fmaxf(mloc, fmaxf(fmaxf(fmaxf(s[8], s[9]), fmaxf(s[10], s[11])),
                                     fmaxf(fmaxf(s[12], s[13]), fmaxf(s[14], s[15]))));
            mloc = fmaxf(mloc, __shfl_xor(mloc, 32, WAVE));
            // The reference point of the exponentials only has to stay within 2^RESCALE_SLACK of the true
            // running maximum (weights then reach at most 2^RESCALE_SLACK, harmless in fp32 accumulators
            // and in the 16-bit P); numerator and denominator share it, so the result is the same. Moving
            // it means a pass over all 256 accumulator registers, which this makes rare. mloc is finite:
            // every step holds at least one valid token.
            constexpr float RESCALE_SLACK = 8.0f;
            if (__builtin_amdgcn_ballot_w64(mloc > m + RESCALE_SLACK) != 0) {
                const float mNew = fmaxf(m, mloc);
                const float corr = mfma::Exp2(m - mNew);
                m = mNew;
                lsum *= corr;
                if (t != tokBegin) { // (the first step starts from zeros)
                    MmaFenceOut(acc);
#pragma unroll
                    for (int i = 0; i < NO; ++i) { // one tile at a time through the VGPRs
                        acc[i] *= corr;
                        asm volatile("" : "+a"(acc[i])); // back into its AGPRs before the next tile is touched
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
            u32x4 pop[2]; // P^T as B operand of the two 16-token contractions
#pragma unroll
            for (int e = 0; e < 16; e += 2) {
                const uint32_t pair = mfma::Pack2<BF16>(mfma::Exp2(s[e] - m), mfma::Exp2(s[e + 1] - m));
                pop[e >> 3][(e >> 1) & 3] = pair;
                // the denominator adds up the rounded weights, the ones that multiply V
                lsum += mfma::Unpack(pair, 0, BF16) + mfma::Unpack(pair, 1, BF16);
            }

            // ---- O^T += V^T . P^T, operands fetched VD MFMAs ahead
            {
                const unsigned char *vrow = tile + vOff;
                auto readV = [&](int idx) -> u32x4 { // idx = 2 * channel tile + kb
                    const unsigned char *ptr = vrow + (idx >> 1) * 64 + (idx & 1) * RowOffset(16);
                    const u32x2 lo = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (__attribute__((address_space(3))) i16x4 *)(ptr)));
                    const u32x2 hi = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (__attribute__((address_space(3))) i16x4 *)(ptr + RowOffset(8))));
                    return u32x4{lo[0], lo[1], hi[0], hi[1]};
                };
                u32x4 vop[VD + 1];
#pragma unroll
                for (int i = 0; i < VD; ++i) {
                    vop[i] = readV(i);
                }
                MmaOperandFence(pop[0], pop[1]); // P was packed by ordinary instructions just above
#pragma unroll
                for (int i = 0; i < 2 * NO; ++i) {
                    if (i + VD < 2 * NO) {
                        vop[(i + VD) % (VD + 1)] = readV(i + VD);
                    }
                    MmaOut<BF16>(acc[i >> 1], vop[i % (VD + 1)], pop[i & 1]);
                    if (i % PV_PER_TRANSFER == PV_PER_TRANSFER / 2 && i / PV_PER_TRANSFER < CHUNKS - CHUNKS / 2 && fetch) {
                        switch (i / PV_PER_TRANSFER) {
                            case 0: transfer(std::integral_constant<int, 5>{}); break;
                            case 1: transfer(std::integral_constant<int, 6>{}); break;
                            case 2: transfer(std::integral_constant<int, 7>{}); break;
                            case 3: transfer(std::integral_constant<int, 8>{}); break;
                            default: transfer(std::integral_constant<int, 9>{}); break;
                        }
                    }
                }
            }

            // Transfers in flight, oldest first: the next step's tile (started during the previous step),
            // then the one started during this step. The first must be in (for this wave's pieces; the
            // barrier makes it everyone's), the second may stay in flight. After the barrier this step's
            // buffer is free for the tile the next step will start to fetch.
            if (fetch) {
                asm volatile("s_waitcnt vmcnt(%0)" : : "n"(CHUNKS) : "memory");
            } else {
                DmaWait();
            }
            __syncthreads();
            buf = buf == 2 ? 0 : buf + 1;
        }

        // ---- finish the row (or this range's share of it)
        MmaFenceOut(acc);
        const float l = lsum + __shfl_xor(lsum, 32, WAVE);
        const float inv = 1.0f / l;
        const int h = h0 + n;
        if (complete) {
            uint16_t *orow = reinterpret_cast<uint16_t *>(a.out) + (static_cast<int64_t>(qRow) * a.H + h) * DV;
#pragma unroll
            for (int i = 0; i < NO; ++i) {
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    const int d = 32 * i + 8 * r4 + 4 * kh;
                    u32x2 packed;
                    if (qBf16) {
                        packed[0] = mfma::Pack2<true>(acc[i][4 * r4] * inv, acc[i][4 * r4 + 1] * inv);
                        packed[1] = mfma::Pack2<true>(acc[i][4 * r4 + 2] * inv, acc[i][4 * r4 + 3] * inv);
                    } else {
                        packed[0] = mfma::Pack2<false>(acc[i][4 * r4] * inv, acc[i][4 * r4 + 1] * inv);
                        packed[1] = mfma::Pack2<false>(acc[i][4 * r4 + 2] * inv, acc[i][4 * r4 + 3] * inv);
                    }
                    *reinterpret_cast<u32x2 *>(orow + d) = packed;
                }
                __builtin_amdgcn_sched_barrier(0); // one tile at a time through the VGPRs
            }
            if (a.lse && kh == 0) {
                Store16(a.lse, static_cast<int64_t>(qRow) * a.H + h, (m + log2f(l)) * 0.6931471805599453f, qBf16);
            }
        } else {
            const int slot = 2 * wr + (segBegin == s0 ? 0 : 1);
            const int64_t ph = static_cast<int64_t>(slot) * a.H + h;
#pragma unroll
            for (int i = 0; i < NO; ++i) {
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    const f32x4 v = {acc[i][4 * r4] * inv, acc[i][4 * r4 + 1] * inv, acc[i][4 * r4 + 2] * inv,
                                     acc[i][4 * r4 + 3] * inv};
                    *reinterpret_cast<f32x4 *>(a.partO + ph * DV + 32 * i + 8 * r4 + 4 * kh) = v;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (kh == 0) {
                a.partLse[ph] = m + log2f(l);
            }
        }
    }
}

template <bool BF16, bool SPLIT> int LaunchWide(const PaArgs &args, const PaStreamPlan &plan, hipStream_t stream)
{
    auto kernel = PaMlaWideKernel<BF16, SPLIT>;
    constexpr int lds = 3 * TILE_BYTES + BLK_IDS * 4;
    static bool configured = false; // one attribute call per instantiation and process
    if (!configured) {
        ATBMI_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                            hipFuncAttributeMaxDynamicSharedMemorySize, lds));
        configured = true;
    }
    if (plan.tokenSlices != 1 || plan.numWaveRanges != plan.numWgRanges ||
        plan.headGroups * PA_MLA_HEADS_PER_WG != args.H || args.G != 1 || args.D != D || args.Dv != DV ||
        args.ropeDim != (SPLIT ? D - DV : 0)) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: plan or shape does not fit the 128-head MLA kernel");
    }
    const int64_t grid = (static_cast<int64_t>(plan.numWgRanges) + 7) / 8 * 8 * plan.headGroups;
    if (grid <= 0 || grid > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: grid of %lld workgroups is out of range", (long long)grid);
    }
    kernel<<<static_cast<unsigned>(grid), NW * WAVE, lds, stream>>>(args, plan);
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}

} // namespace mla
} // namespace atbmi
#endif
