// Decode attention over the combined MLA cache (key row 576 channels, value = its first 512), 128 query
// heads per workgroup, with every register of the step loop assigned by hand (gfx950 assembly).
//
// One wave per SIMD owns 32 heads: their 32 x 512 fp32 outputs are the 256 accumulation registers, their
// 32 x 576 query the upper 144 vector registers. The step loop is software-pipelined so that the matrix
// pipe does not wait for the vector unit:
//     step i:   S(i+1) = K(i+1) . Q^T   (36 MFMAs)   with the softmax of S(i) between them
//               O     += V(i)^T . P(i)^T (32 MFMAs)  with the HBM -> LDS transfers of tile i+3 between them
// Four tile buffers: PV reads tile i, QK tile i+1, tile i+2 has landed or is landing, tile i+3 is being
// requested. A register allocator does not hold this working set (it spills the query or moves the
// accumulators through scratch), so the loop is one asm statement; the C++ around it only walks the plan
// and hands over wave-uniform values.
//
// Operand layouts are those of v_mfma_f32_32x32x16 (lane = 32 kh + n):
//   S^T = K . Q^T   A = K tile: lane reads token row n, channels 16 j + 8 kh .. +8 (ds_read_b128)
//                   B = Q^T: head n, same channels; element e of the result is token 8 (e/4) + 4 kh + e%4
//   O^T += V^T.P^T  contraction over 16 tokens per MFMA (kb = 0, 1); the k index 8 kh + e stands for token
//                   16 kb + 8 (e/4) + 4 kh + e%4, the token of score element 8 kb + e, so P never leaves its
//                   lane; V^T (channel 32 i + n) comes from two transposing ds_read_b64_tr_b16.
//
// Tile in LDS: the 32 token rows at a pitch of 1168 bytes; wave w stages rows 8 w .. 8 w + 7 with ten
// global_load_lds_dwordx4 (the last one on 8 lanes). 37 376 bytes a tile, four tiles.
//
// Hazards the assembler does not check and the code keeps by construction:
//   - a result of an MFMA is read by the vector unit no sooner than 18 wait states after the MFMA was
//     issued (S: a whole PV phase lies between; accumulators: s_nop before the epilogue / the rescale runs
//     ten QK MFMAs after the last PV MFMA);
//   - an operand register of the K / V^T rings is rewritten by an LDS read issued after the MFMA that read
//     it last, and LDS latency exceeds the MFMA's operand fetch;
//   - counted lgkmcnt waits only ever count LDS instructions (no scalar loads anywhere in the loop);
//   - M0 (LDS base of the transfers) is only written when no LDS read of the wave is in flight.
//
// MASK builds add a bias per (query row, token) to the scaled scores: the 32 values of a tile come through four
// buffer loads a lane (a descriptor over the mask row: what lies past its end reads as zero), asked for one step
// ahead, in front of that step's tile transfers, so that the step's own wait for the transfers covers them.
#ifndef ATBMI_PA_MLA_KERNEL_H
#define ATBMI_PA_MLA_KERNEL_H
#include "pa_mfma_kernel.h"

namespace atbmi {
namespace mla {

constexpr int D = 576;
constexpr int DV = 512;
constexpr int STEP = PA_MFMA_STEP;
constexpr int NW = PA_MLA_WAVES;
constexpr int HPW = PA_MLA_HEADS_PER_WG / NW;
constexpr int PITCH = D * 2 + 16;
constexpr int TILE_BYTES = 32 * PITCH;
constexpr int NBUF = 4;
constexpr int LDS_BYTES = NBUF * TILE_BYTES;
static_assert(PITCH == 1168 && TILE_BYTES == 37376 && HPW == 32 && STEP == 32, "constants repeated in the assembly");

#define ATBMI_REGS_0_99(X) X"0", X"1", X"2", X"3", X"4", X"5", X"6", X"7", X"8", X"9", X"10", X"11", X"12", X"13", X"14", X"15", \
    X"16", X"17", X"18", X"19", X"20", X"21", X"22", X"23", X"24", X"25", X"26", X"27", X"28", X"29", X"30", X"31", X"32", X"33", \
    X"34", X"35", X"36", X"37", X"38", X"39", X"40", X"41", X"42", X"43", X"44", X"45", X"46", X"47", X"48", X"49", X"50", X"51", \
    X"52", X"53", X"54", X"55", X"56", X"57", X"58", X"59", X"60", X"61", X"62", X"63", X"64", X"65", X"66", X"67", X"68", X"69", \
    X"70", X"71", X"72", X"73", X"74", X"75", X"76", X"77", X"78", X"79", X"80", X"81", X"82", X"83", X"84", X"85", X"86", X"87", \
    X"88", X"89", X"90", X"91", X"92", X"93", X"94", X"95", X"96", X"97", X"98", X"99"
#define ATBMI_REGS_100_111(X) X"100", X"101", X"102", X"103", X"104", X"105", X"106", X"107", X"108", X"109", X"110", X"111"
#define ATBMI_REGS_112_255(X) X"112", X"113", X"114", X"115", X"116", X"117", X"118", X"119", X"120", X"121", X"122", X"123", \
    X"124", X"125", X"126", X"127", X"128", X"129", X"130", X"131", X"132", X"133", X"134", X"135", X"136", X"137", X"138", X"139", \
    X"140", X"141", X"142", X"143", X"144", X"145", X"146", X"147", X"148", X"149", X"150", X"151", X"152", X"153", X"154", X"155", \
    X"156", X"157", X"158", X"159", X"160", X"161", X"162", X"163", X"164", X"165", X"166", X"167", X"168", X"169", X"170", X"171", \
    X"172", X"173", X"174", X"175", X"176", X"177", X"178", X"179", X"180", X"181", X"182", X"183", X"184", X"185", X"186", X"187", \
    X"188", X"189", X"190", X"191", X"192", X"193", X"194", X"195", X"196", X"197", X"198", X"199", X"200", X"201", X"202", X"203", \
    X"204", X"205", X"206", X"207", X"208", X"209", X"210", X"211", X"212", X"213", X"214", X"215", X"216", X"217", X"218", X"219", \
    X"220", X"221", X"222", X"223", X"224", X"225", X"226", X"227", X"228", X"229", X"230", X"231", X"232", X"233", X"234", X"235", \
    X"236", X"237", X"238", X"239", X"240", X"241", X"242", X"243", X"244", X"245", X"246", X"247", X"248", X"249", X"250", X"251", \
    X"252", X"253", X"254", X"255"
#define ATBMI_SREGS_36_69(X) X"36", X"37", X"38", X"39", X"40", X"41", X"42", X"43", X"44", X"45", X"46", X"47", X"48", X"49", X"50", \
    X"51", X"52", X"53", X"54", X"55", X"56", X"57", X"58", X"59", X"60", X"61", X"62", X"63", X"64", X"65", X"66", X"67", X"68", X"69"

// Wave-uniform description of one segment: the part of a sequence's context that one workgroup range
// holds, for the 32 heads of one wave.
struct Segment {
    const void *cache;    // key cache
    const int32_t *table; // block ids of the sequence
    const void *q;        // q[qRow][h0]: the first of this wave's 32 heads
    const void *qRope;    // split layout: the last 64 channels of the same rows
    const void *ropeCache; // split layout: the last 64 channels of the cache rows
    void *out;            // out[qRow][h0] (complete) or partO[slot][h0], both in the query's type
    void *lse;            // lse[qRow][h0] (complete; may be null) or partLse[slot][h0]
    uint32_t rowBytes;    // bytes between consecutive cache rows
    uint32_t ropeRowBytes; // ... of the rope cache
    uint32_t blockShift;  // log2 of the block size
    uint32_t tokBegin;    // multiple of 32
    uint32_t tokEnd;      // > tokBegin
    uint32_t complete;    // 1: the segment is the whole row, write the final output
    uint32_t heads;       // how many of the wave's 32 heads the call has (0: none; q then points at any valid row)
    const void *mask;     // MASK builds: the mask row of the pass's first query token (16-bit values of the query's
                          // type, 4-byte aligned)
    uint32_t maskBytes;   // ... bytes from there to the end of its last token's row, rounded up to 4
    uint32_t maskTokenBytes; // ... bytes between the rows of consecutive query tokens of the pass
    uint32_t realHeads;   // heads of the call: lane v of the pass (its 32 wave + n-th row) is token v / realHeads
};

// One segment from start to finish: stages the first tiles, loads Q, runs the pipelined step loop, writes
// the (partial) row. All four waves of a workgroup call it with the same token range and block table.
template <bool BF16, bool SPLIT, bool NZ, bool MASK>
__device__ __forceinline__ void RunSegment(const Segment &sg, uint32_t ldsBase, uint32_t wave, float scale2)
{
    // Every input is wave-uniform; saying so value by value keeps each of them in scalar registers, which
    // is where the statement's "s" operands must be.
    auto uni = [](uint32_t v) { return static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(v))); };
    auto uni64 = [&](const void *ptr) {
        const uint64_t v = reinterpret_cast<uintptr_t>(ptr);
        return (static_cast<uint64_t>(uni(static_cast<uint32_t>(v >> 32))) << 32) | uni(static_cast<uint32_t>(v));
    };
    const uint64_t cache = uni64(sg.cache);
    const uint32_t cacheLo = static_cast<uint32_t>(cache);
    const uint32_t cacheHi = static_cast<uint32_t>(cache >> 32);
    const uint64_t table = uni64(sg.table), q = uni64(sg.q), out = uni64(sg.out), lse = uni64(sg.lse);
    const uint64_t qRope = uni64(sg.qRope), rope = uni64(sg.ropeCache);
    const uint32_t ropeLo = static_cast<uint32_t>(rope), ropeHi = static_cast<uint32_t>(rope >> 32);
    const uint32_t ropeRowBytes = uni(sg.ropeRowBytes);
    const uint32_t rowBytes = uni(sg.rowBytes), blockShift = uni(sg.blockShift), tokBegin = uni(sg.tokBegin);
    const uint32_t tokEnd = uni(sg.tokEnd), complete = uni(sg.complete);
    const uint32_t heads = uni(sg.heads), lastHead = uni(sg.heads > 0 ? sg.heads - 1 : 0);
    const uint64_t mask = uni64(sg.mask);
    const uint32_t maskLo = static_cast<uint32_t>(mask), maskHi = static_cast<uint32_t>(mask >> 32) & 0xffffu;
    const uint32_t maskBytes = uni(sg.maskBytes), maskTokenBytes = uni(sg.maskTokenBytes), realHeads = uni(sg.realHeads);
    ldsBase = uni(ldsBase);
    wave = uni(wave);
    scale2 = __builtin_bit_cast(float, uni(__builtin_bit_cast(uint32_t, scale2)));
    asm volatile(R"ASM(
    // ---------------------------------------------------------------- register map
    // v[0:15] S_A   v[16:31] S_B           scores of two consecutive steps
    // v[32:47] K operand ring (4 x 4)      v[48:63] V^T operand ring (4 x 4)
    // v[64:71] P operands (kb 0: 64..67, kb 1: 68..71)
    // v[72:81] per-lane source offsets of the ten tile transfers
    // v82 m   v83 lsum   v84 mloc   v85 corr   v86 ds_bpermute address of lane ^ 32   v87 4 kh
    // v[88:93] temporaries   v94 K operand address of the QK tile   v95 V^T operand address of the PV tile
    // v96 K operand address in buffer 0   v97 V^T operand address in buffer 0
    // v98 block ids (lane k: block s42 + k)   v99 row (less 8 wave) of each transfer's slot, 3 bits each
    // v[112:255] Q, piece j in v[112+4j : 115+4j];   a[16 i : 16 i + 15] output tile i
    // s36 token of the PV tile   s37 end of the segment   s38 / s39 / s41 buffer offset of the PV / QK / fetched tile
    // s40 steps done   s42 first block index in v98   s43 last block index   s44 8 wave   s45 block size - 1
    // s[46:55] temporaries   s[56:57] transfer source base   s58 LDS address of this wave's rows in buffer 0
    // s59 token of the tile to fetch   s[60:61] saved exec   s62 rows of this wave inside the segment
    .set BF16, %[bf16]
    .set SPLIT, %[split]
    .set NZ, %[nz]
    .set MASK, %[mask_on]
    // MASK: v[100:107] the mask values of the tile whose softmax comes next (16-bit pairs: register 2 g + h holds
    // tokens 8 g + 4 kh + 2 h, + 1 of the tile); v108 the lane's byte offset into the mask rows (its query token's
    // row, 8 kh); s[68:71] the buffer descriptor of the mask rows of the pass.
    // the four loads of the mask values of the tile at token \tok (a scalar register)
    .macro MASK_LOAD tok
      .if MASK
        s_lshl_b32 s46, \tok, 1
        v_add_u32 v88, s46, v108             // byte of token tok + 4 kh in the lane's row
        .irp g,0,1,2,3
          buffer_load_dwordx2 v[100+2*\g:101+2*\g], v88, s[68:71], 0 offen offset:16*\g
        .endr
      .endif
    .endm
    // SPLIT: the last 64 channels of every cache row come from a cache of their own (rows of 128 bytes) and
    // those of every query row from a tensor of their own. A transfer then takes its lanes from two sources:
    // lanes whose slot (64 i + lane, 73 slots a row, the last one padding) holds one of the first 64 pieces
    // of a row, and lanes whose slot holds piece 64 .. 71 (or the padding). The lane masks of both kinds:
    .set NOPE_LO_0, 0xffffffff
    .set NOPE_HI_0, 0xffffffff
    .set ROPE_LO_0, 0x00000000
    .set ROPE_HI_0, 0x00000000
    .set NOPE_LO_1, 0xfffffe00
    .set NOPE_HI_1, 0xffffffff
    .set ROPE_LO_1, 0x000001ff
    .set ROPE_HI_1, 0x00000000
    .set NOPE_LO_2, 0xfffc01ff
    .set NOPE_HI_2, 0xffffffff
    .set ROPE_LO_2, 0x0003fe00
    .set ROPE_HI_2, 0x00000000
    .set NOPE_LO_3, 0xf803ffff
    .set NOPE_HI_3, 0xffffffff
    .set ROPE_LO_3, 0x07fc0000
    .set ROPE_HI_3, 0x00000000
    .set NOPE_LO_4, 0x07ffffff
    .set NOPE_HI_4, 0xfffffff0
    .set ROPE_LO_4, 0xf8000000
    .set ROPE_HI_4, 0x0000000f
    .set NOPE_LO_5, 0xffffffff
    .set NOPE_HI_5, 0xffffe00f
    .set ROPE_LO_5, 0x00000000
    .set ROPE_HI_5, 0x00001ff0
    .set NOPE_LO_6, 0xffffffff
    .set NOPE_HI_6, 0xffc01fff
    .set ROPE_LO_6, 0x00000000
    .set ROPE_HI_6, 0x003fe000
    .set NOPE_LO_7, 0xffffffff
    .set NOPE_HI_7, 0x803fffff
    .set ROPE_LO_7, 0x00000000
    .set ROPE_HI_7, 0x7fc00000
    .set NOPE_LO_8, 0xffffffff
    .set NOPE_HI_8, 0x7fffffff
    .set ROPE_LO_8, 0x00000000
    .set ROPE_HI_8, 0x80000000
    .set NOPE_LO_9, 0x00000000
    .set NOPE_HI_9, 0x00000000
    .set ROPE_LO_9, 0x000000ff
    .set ROPE_HI_9, 0x00000000
    .if SPLIT
      .set NDMA, 18                       // transfer instructions of a tile (empty lane masks issue none)
    .else
      .set NDMA, 10
    .endif
    .set PITCH, 1168
    .set ROW8, 9344
    .set ROW16, 18688
    .set REGION, 9344
    .set TILE, 37376

    .macro LDK slot, j
      ds_read_b128 v[32+4*(\slot):35+4*(\slot)], v94 offset:32*(\j)
    .endm
    .macro LDV slot, idx
      ds_read_b64_tr_b16 v[48+4*(\slot):49+4*(\slot)], v95 offset:((\idx)/2)*64+((\idx)%%2)*ROW16
      ds_read_b64_tr_b16 v[50+4*(\slot):51+4*(\slot)], v95 offset:((\idx)/2)*64+((\idx)%%2)*ROW16+ROW8
    .endm

    // ---- softmax slice k (k = the QK slot it rides on) of the scores at v[SO : SO+15]; P goes to v[64:71]
    .macro SM_SLICE k, SO
      .if \k == 0
        .if MASK
          // scores <- scores x scale + mask x log2(e): the softmax below then works on scaled scores
          .irp p,0,1,2,3,4,5,6,7
            .if BF16
              v_lshlrev_b32 v88, 16, v[100+\p]
              v_and_b32 v89, 0xffff0000, v[100+\p]
            .else
              v_lshrrev_b32 v89, 16, v[100+\p]
              v_cvt_f32_f16 v88, v[100+\p]
              v_cvt_f32_f16 v89, v89
            .endif
            v_mul_f32 v88, 0x3fb8aa3b, v88
            v_mul_f32 v89, 0x3fb8aa3b, v89
            v_fma_f32 v[\SO+4*(\p/2)+2*(\p%%2)], v[\SO+4*(\p/2)+2*(\p%%2)], %[scale], v88
            v_fma_f32 v[\SO+4*(\p/2)+2*(\p%%2)+1], v[\SO+4*(\p/2)+2*(\p%%2)+1], %[scale], v89
          .endr
        .endif
        v_max3_f32 v84, v[\SO+0], v[\SO+1], v[\SO+2]
      .elseif \k == 1
        v_max3_f32 v88, v[\SO+3], v[\SO+4], v[\SO+5]
      .elseif \k == 2
        v_max3_f32 v89, v[\SO+6], v[\SO+7], v[\SO+8]
      .elseif \k == 3
        v_max3_f32 v90, v[\SO+9], v[\SO+10], v[\SO+11]
      .elseif \k == 4
        v_max3_f32 v91, v[\SO+12], v[\SO+13], v[\SO+14]
      .elseif \k == 5
        v_max3_f32 v84, v84, v88, v89
        v_max3_f32 v90, v90, v91, v[\SO+15]
      .elseif \k == 6
        v_max_f32 v84, v84, v90
        s_nop 0
        ds_bpermute_b32 v88, v86, v84
      .elseif \k == 10
        // (the exchange was issued before K piece 10 was requested: the wait for that piece covers it)
        v_max_f32 v84, v84, v88
        .if !MASK
          v_mul_f32 v84, %[scale], v84
        .endif
        v_add_f32 v89, 0x41000000, v82
        v_cmp_gt_f32 vcc, v84, v89
        s_cbranch_vccz 10f
        // some head's maximum grew by more than 2^8: move the reference point of the exponentials
        v_max_f32 v89, v82, v84
        v_sub_f32 v90, v82, v89
        v_exp_f32 v85, v90
        v_mov_b32 v82, v89
        s_nop 1
        v_mul_f32 v83, v83, v85
        s_cmp_eq_u32 s40, 0
        s_cbranch_scc1 10f               // first step: the accumulators are still zero
        .irp r,0,1,2,3,4,5,6,7,8,9,10,11,12,13,14,15
          .irp c,0,1,2,3,4,5,6,7,8,9,10,11,12,13,14,15
            v_accvgpr_read_b32 v90, a[16*\r+\c]
            s_nop 0
            v_mul_f32 v90, v90, v85
            s_nop 0
            v_accvgpr_write_b32 a[16*\r+\c], v90
          .endr
        .endr
        10:
      .elseif (\k >= 11) && (\k <= 26)
        .if MASK
          v_sub_f32 v[88+(\k%%2)], v[\SO+\k-11], v82
        .else
          v_fma_f32 v[88+(\k%%2)], v[\SO+\k-11], %[scale], -v82
        .endif
        s_nop 0
        v_exp_f32 v[\SO+\k-11], v[88+(\k%%2)]
      .elseif (\k >= 27) && (\k <= 34)
        .if BF16
          v_cvt_pk_bf16_f32 v[64+\k-27], v[\SO+2*(\k-27)], v[\SO+2*(\k-27)+1]
          s_nop 0
          v_lshlrev_b32 v90, 16, v[64+\k-27]
          v_and_b32 v91, 0xffff0000, v[64+\k-27]
        .else
          v_cvt_f16_f32 v90, v[\SO+2*(\k-27)]
          v_cvt_f16_f32 v91, v[\SO+2*(\k-27)+1]
          s_nop 0
          v_pack_b32_f16 v[64+\k-27], v90, v91
          v_cvt_f32_f16 v90, v90
          v_cvt_f32_f16 v91, v91
        .endif
        // the denominator adds up the rounded weights, the ones that multiply V
        v_add_f32 v83, v83, v90
        v_add_f32 v83, v83, v91
      .endif
    .endm

    // ---- QK slot j: S_new (v[SN : SN+15]) += K piece j . Q piece j; with SO >= 0 softmax slice j of S_old rides along
    .macro QK_SLOT j, SN, SO
      .if \j + 3 < 36
        LDK ((\j+3)%%4), (\j+3)
      .endif
      .if \j >= 33
        s_waitcnt lgkmcnt(35-\j)
      .elseif (\SO >= 0) && (\j >= 7) && (\j <= 9)
        s_waitcnt lgkmcnt(4)
      .else
        s_waitcnt lgkmcnt(3)
      .endif
      .if \j == 0
        .if BF16
          v_mfma_f32_32x32x16_bf16 v[\SN:\SN+15], v[32+4*(\j%%4):35+4*(\j%%4)], v[112+4*\j:115+4*\j], 0
        .else
          v_mfma_f32_32x32x16_f16 v[\SN:\SN+15], v[32+4*(\j%%4):35+4*(\j%%4)], v[112+4*\j:115+4*\j], 0
        .endif
      .else
        .if BF16
          v_mfma_f32_32x32x16_bf16 v[\SN:\SN+15], v[32+4*(\j%%4):35+4*(\j%%4)], v[112+4*\j:115+4*\j], v[\SN:\SN+15]
        .else
          v_mfma_f32_32x32x16_f16 v[\SN:\SN+15], v[32+4*(\j%%4):35+4*(\j%%4)], v[112+4*\j:115+4*\j], v[\SN:\SN+15]
        .endif
      .endif
      .if \SO >= 0
        SM_SLICE \j, \SO
      .endif
    .endm
    .macro QK_PHASE SN, SO
      LDK 0, 0
      LDK 1, 1
      LDK 2, 2
      .irp j,0,1,2,3,4,5,6,7,8,9,10,11,12,13,14,15,16,17,18,19,20,21,22,23,24,25,26,27,28,29,30,31,32,33,34,35
        QK_SLOT \j, \SN, \SO
      .endr
    .endm

    // ---- softmax of the scores at v[SO : SO+15] on its own: the last step of a segment, whose tokens at or
    // past the end of the segment get a score of -inf
    .macro SM_ALONE SO
      s_sub_u32 s46, s37, s36              // tokens of this tile inside the segment
      s_cmp_ge_u32 s46, 32
      s_cbranch_scc1 11f
      v_mov_b32 v88, 0xff800000
      .irp e,0,1,2,3,4,5,6,7,8,9,10,11,12,13,14,15
        s_sub_i32 s47, s46, 8*(\e/4)+(\e%%4)
        v_cmp_gt_i32 vcc, s47, v87
        s_nop 1
        v_cndmask_b32 v[\SO+\e], v88, v[\SO+\e], vcc
      .endr
      11:
      .irp k,0,1,2,3,4,5,6
        SM_SLICE \k, \SO
      .endr
      s_waitcnt lgkmcnt(0)
      .irp k,10,11,12,13,14,15,16,17,18,19,20,21,22,23,24,25,26,27,28,29,30,31,32,33,34
        SM_SLICE \k, \SO
      .endr
    .endm

    // ---- source of the transfers of the tile at token s59 for this wave: s[56:57] = address of the cache row
    // of token s59 + 8 wave, less 4096; s62 = tile rows of this wave that lie inside the segment (<= 0: none).
    // Refills the block ids when the row's block is past the 64 held (waits for everything in flight then).
    .macro DMA_PREP
      s_add_u32 s46, s59, s44              // token of this wave's first row
      s_sub_i32 s62, s37, s46              // rows left from there
      s_lshr_b32 s47, s46, %[bshift]
      s_min_u32 s47, s47, s43              // (a wave wholly past the end looks at the last block; it moves nothing)
      s_sub_u32 s48, s47, s42
      s_cmp_lt_u32 s48, 64
      s_cbranch_scc1 12f
      s_mov_b32 s42, s47
      v_mbcnt_lo_u32_b32 v88, -1, 0
      v_mbcnt_hi_u32_b32 v88, -1, v88
      v_add_u32 v88, s42, v88
      v_min_u32 v88, s43, v88
      v_lshlrev_b32 v88, 2, v88
      global_load_dword v98, v88, %[table]
      s_waitcnt vmcnt(0)
      s_mov_b32 s48, 0
      12:
      s_nop 0
      v_readlane_b32 s49, v98, s48         // block id
      s_and_b32 s50, s46, s45              // row inside the block
      s_nop 3
      .if NZ
        // fractal-NZ blocks: slabs of (block size) x 16 channels, 32 channel slabs in the latent cache and
        // 4 in the rope cache; a token's 32 bytes of a slab follow those of the token before
        s_lshl_b32 s50, s50, 5
        s_add_u32 s52, %[bshift], 10
        s_mov_b32 s56, s49
        s_mov_b32 s57, 0
        s_lshl_b64 s[56:57], s[56:57], s52 // block id x block size x 1024 bytes
        s_add_u32 s56, s56, s50
        s_addc_u32 s57, s57, 0
        s_add_u32 s56, s56, %[cache_lo]
        s_addc_u32 s57, s57, %[cache_hi]
        s_sub_u32 s56, s56, 4096
        s_subb_u32 s57, s57, 0
        s_add_u32 s52, %[bshift], 7
        s_mov_b32 s64, s49
        s_mov_b32 s65, 0
        s_lshl_b64 s[64:65], s[64:65], s52 // block id x block size x 128 bytes
        s_add_u32 s64, s64, s50
        s_addc_u32 s65, s65, 0
        s_add_u32 s64, s64, %[rope_lo]
        s_addc_u32 s65, s65, %[rope_hi]
        s_sub_u32 s64, s64, 4096
        s_subb_u32 s65, s65, 0
      .else
      s_lshl_b32 s49, s49, %[bshift]
      s_add_u32 s49, s49, s50              // cache row
      s_mul_i32 s56, s49, %[rowbytes]
      s_mul_hi_u32 s57, s49, %[rowbytes]
      s_add_u32 s56, s56, %[cache_lo]
      s_addc_u32 s57, s57, %[cache_hi]
      s_sub_u32 s56, s56, 4096
      s_subb_u32 s57, s57, 0
      .if SPLIT
        s_mul_i32 s64, s49, %[roperowbytes]
        s_mul_hi_u32 s65, s49, %[roperowbytes]
        s_add_u32 s64, s64, %[rope_lo]
        s_addc_u32 s65, s65, %[rope_hi]
        s_sub_u32 s64, s64, 4096
        s_subb_u32 s65, s65, 0
      .endif
      .endif
    .endm
    // the instruction of transfer i from the source base in s[base : base+1]; M0 = region + 4096 for i < 8,
    // region + 8192 after
    // (non-temporal: a cache row is read once a step; the hint is worth a twentieth of the stream from HBM)
    .macro DMA_LOAD i, base
      .if \i < 8
        global_load_lds_dwordx4 v[72+\i], s[\base:\base+1] offset:(\i-4)*1024 nt
      .else
        global_load_lds_dwordx4 v[72+\i], s[\base:\base+1] offset:(\i-8)*1024 nt
      .endif
    .endm
    // transfer i of a tile whose rows all lie inside the segment
    .macro DMA_ONE i
      .if SPLIT
        .if (NOPE_LO_\i != 0) || (NOPE_HI_\i != 0)
          s_mov_b32 exec_lo, NOPE_LO_\i
          s_mov_b32 exec_hi, NOPE_HI_\i
          DMA_LOAD \i, 56
        .endif
        .if (ROPE_LO_\i != 0) || (ROPE_HI_\i != 0)
          s_mov_b32 exec_lo, ROPE_LO_\i
          s_mov_b32 exec_hi, ROPE_HI_\i
          DMA_LOAD \i, 64
        .endif
        s_mov_b64 exec, -1
      .else
        .if \i == 9
          s_mov_b64 exec, 0xff
        .endif
        DMA_LOAD \i, 56
        .if \i == 9
          s_mov_b64 exec, -1
        .endif
      .endif
    .endm
    // all ten transfers of a tile in a row, into the buffer at offset s41; slots of rows past the segment's
    // end (s62 rows are inside) are filled with zeros instead. Not while LDS reads are being counted.
    .macro DMA_ANY
      s_add_u32 s53, s58, s41
      s_mov_b64 s[60:61], exec
      v_mov_b32 v88, 0
      v_mov_b32 v89, 0
      v_mov_b32 v90, 0
      v_mov_b32 v91, 0
      v_mbcnt_lo_u32_b32 v92, -1, 0
      v_mbcnt_hi_u32_b32 v92, -1, v92
      v_lshlrev_b32 v92, 4, v92
      v_add_u32 v92, s53, v92              // LDS address of this lane's slot in transfer 0
      .irp i,0,1,2,3,4,5,6,7,8,9
        .if \i == 0
          s_add_u32 s54, s53, 4096
          s_mov_b32 m0, s54
        .elseif \i == 8
          s_add_u32 s54, s53, 8192
          s_mov_b32 m0, s54
        .endif
        v_bfe_u32 v93, v99, 3*\i, 3
        v_cmp_gt_i32 vcc, s62, v93         // the row of this slot lies inside the segment
        s_nop 1
        .if SPLIT
          .if (NOPE_LO_\i != 0) || (NOPE_HI_\i != 0)
            s_and_b32 exec_lo, vcc_lo, NOPE_LO_\i
            s_and_b32 exec_hi, vcc_hi, NOPE_HI_\i
            DMA_LOAD \i, 56
          .endif
          .if (ROPE_LO_\i != 0) || (ROPE_HI_\i != 0)
            s_and_b32 exec_lo, vcc_lo, ROPE_LO_\i
            s_and_b32 exec_hi, vcc_hi, ROPE_HI_\i
            DMA_LOAD \i, 64
          .endif
        .else
          .if \i == 9
            s_and_b64 vcc, vcc, 0xff
          .endif
          s_mov_b64 exec, vcc
          DMA_LOAD \i, 56
        .endif
        .if \i == 9
          s_andn2_b64 exec, 0xff, vcc
        .else
          s_andn2_b64 exec, s[60:61], vcc
        .endif
        ds_write_b128 v92, v[88:91] offset:1024*\i
        s_mov_b64 exec, s[60:61]
      .endr
    .endm

    // ---- PV slot i: O tile i/2 += V^T piece i . P (kb = i mod 2); with DMA transfers of the fetched tile ride along
    .macro PV_SLOT i, DMA
      .if \i + 3 < 32
        LDV ((\i+3)%%4), (\i+3)
      .endif
      .if \i >= 29
        s_waitcnt lgkmcnt(2*(31-\i))
      .else
        s_waitcnt lgkmcnt(6)
      .endif
      .if BF16
        v_mfma_f32_32x32x16_bf16 a[16*(\i/2):16*(\i/2)+15], v[48+4*(\i%%4):51+4*(\i%%4)], v[64+4*(\i%%2):67+4*(\i%%2)], a[16*(\i/2):16*(\i/2)+15]
      .else
        v_mfma_f32_32x32x16_f16 a[16*(\i/2):16*(\i/2)+15], v[48+4*(\i%%4):51+4*(\i%%4)], v[64+4*(\i%%2):67+4*(\i%%2)], a[16*(\i/2):16*(\i/2)+15]
      .endif
      .if \DMA
        .if \i == 1
          DMA_ONE 0
        .elseif \i == 5
          DMA_ONE 1
        .elseif \i == 9
          DMA_ONE 2
        .elseif \i == 13
          DMA_ONE 3
        .elseif \i == 17
          DMA_ONE 4
        .elseif \i == 21
          DMA_ONE 5
        .elseif \i == 25
          DMA_ONE 6
        .elseif \i == 29
          DMA_ONE 7
        .endif
      .endif
    .endm
    .macro PV_PHASE DMA
      .if MASK
        s_add_u32 s47, s36, 32
        MASK_LOAD s47                      // of the tile whose softmax rides on the next step's QK phase
      .endif
      .if \DMA
        // both LDS bases are set while none of the wave's LDS reads is in flight
        s_add_u32 s53, s58, s41
        s_add_u32 s54, s53, 8192
        s_mov_b32 m0, s54
        s_nop 0
        DMA_ONE 8
        DMA_ONE 9
        s_add_u32 s54, s53, 4096
        s_mov_b32 m0, s54
      .endif
      LDV 0, 0
      LDV 1, 1
      LDV 2, 2
      s_nop 7
      .irp i,0,1,2,3,4,5,6,7,8,9,10,11,12,13,14,15,16,17,18,19,20,21,22,23,24,25,26,27,28,29,30,31
        PV_SLOT \i, \DMA
      .endr
    .endm

    // ---- one step: QK of the next tile into S_new with the softmax of S_old riding along, then PV of
    // this tile; leaves to \tail when this tile is the segment's last
    .macro BODY SN, SO, tail
      s_add_u32 s46, s36, 32
      s_cmp_ge_u32 s46, s37
      s_cbranch_scc1 \tail
      v_add_u32 v94, s39, v96
      v_add_u32 v95, s38, v97
      s_add_u32 s46, s59, 32
      s_cmp_le_u32 s46, s37
      s_cbranch_scc0 5f
      // a whole tile three steps ahead: its transfers ride along
      DMA_PREP
      s_cmp_eq_u32 %[nh], 0
      s_cbranch_scc1 20f
      QK_PHASE \SN, \SO
      PV_PHASE 1
      s_branch 21f
      20:
      // a wave without heads only moves its rows of the tile
      s_add_u32 s53, s58, s41
      s_add_u32 s54, s53, 8192
      s_mov_b32 m0, s54
      s_nop 0
      DMA_ONE 8
      DMA_ONE 9
      s_add_u32 s54, s53, 4096
      s_mov_b32 m0, s54
      s_nop 0
      .irp i,0,1,2,3,4,5,6,7
        DMA_ONE \i
      .endr
      21:
      s_waitcnt vmcnt(NDMA)                // all but the tile just requested have landed
      s_branch 6f
      5:
      s_cmp_eq_u32 %[nh], 0
      s_cbranch_scc1 22f
      QK_PHASE \SN, \SO
      PV_PHASE 0
      22:
      s_cmp_lt_u32 s59, s37
      s_cbranch_scc0 7f
      DMA_PREP                             // the segment's last, partial tile
      DMA_ANY
      7:
      s_waitcnt vmcnt(0) lgkmcnt(0)
      6:
      s_barrier
      s_mov_b32 s38, s39
      s_add_u32 s39, s39, TILE
      s_cmp_eq_u32 s39, 4*TILE
      s_cselect_b32 s39, 0, s39
      s_add_u32 s41, s41, TILE
      s_cmp_eq_u32 s41, 4*TILE
      s_cselect_b32 s41, 0, s41
      s_add_u32 s36, s36, 32
      s_add_u32 s59, s59, 32
      s_add_u32 s40, s40, 1
    .endm

    // ================================================================ the segment
    s_barrier                              // every wave has left the tiles of the segment before
    // ---- lane constants
    v_mbcnt_lo_u32_b32 v88, -1, 0
    v_mbcnt_hi_u32_b32 v88, -1, v88        // lane
    v_and_b32 v89, 31, v88                 // n
    v_lshrrev_b32 v90, 5, v88              // kh
    v_mul_u32_u24 v96, PITCH, v89
    v_lshl_add_u32 v96, v90, 4, v96
    v_add_u32 v96, %[lds], v96             // K operand: row n, 16 bytes per kh
    v_bfe_u32 v91, v88, 2, 2
    v_lshl_add_u32 v91, v90, 2, v91        // 4 kh + (lane / 4) mod 4
    v_mul_u32_u24 v97, PITCH, v91
    v_bfe_u32 v91, v88, 4, 1
    v_lshlrev_b32 v91, 5, v91
    v_and_b32 v92, 3, v88
    v_lshlrev_b32 v92, 3, v92
    v_add3_u32 v97, v97, v91, v92
    v_add_u32 v97, %[lds], v97             // V^T operand
    v_xor_b32 v86, 32, v88
    v_lshlrev_b32 v86, 2, v86
    v_lshlrev_b32 v87, 2, v90
    v_mov_b32 v99, 0
    .irp i,0,1,2,3,4,5,6,7,8,9
      // slot 64 i + lane of this wave's rows: row = slot / 73, piece = min(slot mod 73, 71)
      v_add_u32 v91, 64*\i, v88
      v_mul_u32_u24 v92, 449, v91
      v_lshrrev_b32 v92, 15, v92
      v_mul_u32_u24 v93, 73, v92
      v_sub_u32 v93, v91, v93
      v_min_u32 v93, 71, v93
      .if NZ
        // piece p of tile row r: r x 32 + (p / 2) x 32 x block size + (p mod 2) x 16 past the token of the
        // tile's first row; pieces 64 .. 71 the same with p - 64, in the rope cache
        v_cmp_lt_u32 vcc, 63, v93
        v_add_u32 v95, -64, v93
        s_nop 1
        v_cndmask_b32 v94, v93, v95, vcc
        v_lshrrev_b32 v95, 1, v94
        v_and_b32 v94, 1, v94
        v_lshlrev_b32 v94, 4, v94
        s_add_u32 s46, %[bshift], 5
        v_lshlrev_b32 v95, s46, v95
        v_lshl_add_u32 v91, v92, 5, v94
        v_add_u32 v91, v91, v95
      .else
      v_mul_lo_u32 v91, v92, %[rowbytes]
      v_lshl_add_u32 v91, v93, 4, v91
      .endif
      .if SPLIT && !NZ
        // pieces 64 .. 71 of a row: piece - 64 of the same row of the rope cache
        v_mul_lo_u32 v94, v92, %[roperowbytes]
        v_add_u32 v95, -64, v93
        v_lshl_add_u32 v94, v95, 4, v94
        v_cmp_lt_u32 vcc, 63, v93
        s_nop 1
        v_cndmask_b32 v91, v91, v94, vcc
      .endif
      .if \i < 8
        v_add_u32 v[72+\i], 8192-1024*\i, v91
      .else
        v_add_u32 v[72+\i], 4096-1024*(\i-8), v91
      .endif
      v_and_b32 v92, 7, v92
      v_lshl_or_b32 v99, v92, 3*\i, v99
    .endr
    .if MASK
      // the lane's query token: row v = 32 wave + n of the pass belongs to token v / heads (at most 8 tokens a pass)
      s_lshl_b32 s46, %[wave], 5
      v_add_u32 v91, s46, v89
      v_mov_b32 v92, 0
      .irp k,1,2,3,4,5,6,7
        s_mul_i32 s47, %[real_heads], \k
        v_cmp_le_u32 vcc, s47, v91
        s_nop 1
        v_addc_co_u32 v92, vcc, 0, v92, vcc
      .endr
      v_mul_lo_u32 v108, v92, %[mask_token_bytes]
      v_lshl_add_u32 v108, v87, 1, v108
      s_mov_b32 s68, %[mask_lo]
      s_mov_b32 s69, %[mask_hi]              // (stride 0: a raw buffer)
      s_mov_b32 s70, %[mask_bytes]
      s_mov_b32 s71, 0x00020000
    .endif
    // ---- segment state
    s_mov_b32 s36, %[tokbegin]
    s_mov_b32 s37, %[tokend]
    s_mov_b32 s38, 0
    s_mov_b32 s39, TILE
    s_mov_b32 s40, 0
    s_sub_u32 s43, s37, 1
    s_lshr_b32 s43, s43, %[bshift]
    s_lshl_b32 s44, %[wave], 3
    s_lshl_b32 s45, 1, %[bshift]
    s_sub_u32 s45, s45, 1
    s_mul_i32 s58, %[wave], REGION
    s_add_u32 s58, s58, %[lds]
    // ---- the block ids of this wave's first rows, then Q behind them: the ids are back (and the tile
    // transfers can start) while Q is still on its way
    s_add_u32 s46, s36, s44
    s_lshr_b32 s42, s46, %[bshift]
    s_min_u32 s42, s42, s43
    v_add_u32 v91, s42, v88
    v_min_u32 v91, s43, v91
    v_lshlrev_b32 v91, 2, v91
    global_load_dword v98, v91, %[table]
    // ---- Q: lane (n, kh) holds q[h0 + n][16 j + 8 kh .. +8) for the 36 pieces j; a wave with fewer than 32 heads
    // repeats its last one in the lanes past it (their rows are computed and not stored)
    v_min_u32 v93, %[qlast], v89
    .if SPLIT
      v_lshlrev_b32 v88, 10, v93
      v_lshl_add_u32 v88, v90, 4, v88      // rows of 512 channels
      v_lshlrev_b32 v91, 7, v93
      v_lshl_add_u32 v91, v90, 4, v91      // rows of 64 channels
      .irp j,0,1,2,3,4,5,6,7,8,9,10,11,12,13,14,15,16,17,18,19,20,21,22,23,24,25,26,27,28,29,30,31
        global_load_dwordx4 v[112+4*\j:115+4*\j], v88, %[q] offset:32*\j
      .endr
      .irp j,32,33,34,35
        global_load_dwordx4 v[112+4*\j:115+4*\j], v91, %[qrope] offset:32*(\j-32)
      .endr
    .else
      v_mul_u32_u24 v88, 1152, v93
      v_lshl_add_u32 v88, v90, 4, v88
      .irp j,0,1,2,3,4,5,6,7,8,9,10,11,12,13,14,15,16,17,18,19,20,21,22,23,24,25,26,27,28,29,30,31,32,33,34,35
        global_load_dwordx4 v[112+4*\j:115+4*\j], v88, %[q] offset:32*\j
      .endr
    .endif
    s_waitcnt vmcnt(36)
    // ---- the first three tiles
    s_mov_b32 s59, s36
    s_mov_b32 s41, 0
    DMA_PREP
    DMA_ANY
    s_add_u32 s59, s59, 32
    s_mov_b32 s41, TILE
    s_cmp_lt_u32 s59, s37
    s_cbranch_scc0 8f
    DMA_PREP
    DMA_ANY
    8:
    s_add_u32 s59, s59, 32
    s_mov_b32 s41, 2*TILE
    s_cmp_lt_u32 s59, s37
    s_cbranch_scc0 9f
    DMA_PREP
    DMA_ANY
    9:
    s_add_u32 s59, s59, 32
    s_mov_b32 s41, 3*TILE
    // ---- O = 0, written by the matrix pipe itself
    v_mov_b32 v64, 0
    v_mov_b32 v65, 0
    v_mov_b32 v66, 0
    v_mov_b32 v67, 0
    s_nop 4
    .irp i,0,1,2,3,4,5,6,7,8,9,10,11,12,13,14,15
      .if BF16
        v_mfma_f32_32x32x16_bf16 a[16*\i:16*\i+15], v[64:67], v[64:67], 0
      .else
        v_mfma_f32_32x32x16_f16 a[16*\i:16*\i+15], v[64:67], v[64:67], 0
      .endif
    .endr
    .if MASK
      v_mov_b32 v82, 0xf149f2ca            // -1e30: a tile that the mask hides altogether leaves -inf - m = -inf, not NaN
      MASK_LOAD s36
    .else
      v_mov_b32 v82, 0xff800000
    .endif
    v_mov_b32 v83, 0
    s_waitcnt vmcnt(0) lgkmcnt(0)
    s_barrier
    // ---- scores of the first tile
    v_add_u32 v94, s38, v96
    s_cmp_eq_u32 %[nh], 0
    s_cbranch_scc1 1f
    QK_PHASE 0, -1
    s_nop 15
    s_nop 1
    1:
    BODY 16, 0, 2f
    BODY 0, 16, 3f
    s_branch 1b
    2:
    s_cmp_eq_u32 %[nh], 0
    s_cbranch_scc1 4f
    v_add_u32 v95, s38, v97
    SM_ALONE 0
    PV_PHASE 0
    s_branch 4f
    3:
    s_cmp_eq_u32 %[nh], 0
    s_cbranch_scc1 4f
    v_add_u32 v95, s38, v97
    SM_ALONE 16
    PV_PHASE 0
    4:
    // ================================================================ the row, or this range's share of it
    s_nop 15
    s_nop 1
    ds_bpermute_b32 v88, v86, v83
    v_mbcnt_lo_u32_b32 v92, -1, 0
    v_mbcnt_hi_u32_b32 v92, -1, v92        // lane
    v_and_b32 v89, 31, v92                 // n
    v_lshrrev_b32 v90, 5, v92              // kh
    s_waitcnt lgkmcnt(0)
    v_add_f32 v83, v83, v88                // l: both halves of the head's tokens
    s_nop 0
    v_rcp_f32 v84, v83
    v_log_f32 v85, v83
    s_nop 1
    v_add_f32 v85, v85, v82                // log2 of the sum of 2^score
    .if MASK
      v_cmp_lt_f32 vcc, 0, v83             // a row that the mask hides altogether: zeros, log-sum-exp -inf
      s_nop 1
      v_cndmask_b32 v84, 0, v84, vcc
      v_mov_b32 v88, 0xff800000
      s_nop 0
      v_cndmask_b32 v85, v88, v85, vcc
    .endif
    // ---- the rows in the query's type, out[h0 + n][0 .. 512) (a partial row has the same form). A lane holds
    // four channels at a time (32 i + 8 r + 4 kh ..): stored from there, a row would reach memory in 64 pieces of
    // 16 bytes. The rows go through LDS instead (the tile buffers are idle now: buffer `wave` holds this wave's
    // 32 rows at a pitch of 1040 bytes) and leave as whole rows, 1 KiB an instruction.
    s_barrier                                // every wave has left the tiles
    s_movk_i32 s46, 1040
    s_mul_i32 s48, %[wave], TILE
    s_add_u32 s48, s48, %[lds]               // this wave's staging rows
    v_mul_u32_u24 v91, s46, v89
    v_lshl_add_u32 v91, v90, 3, v91
    v_add_u32 v91, s48, v91                  // row n, byte 8 kh
    .irp i,0,1,2,3,4,5,6,7,8,9,10,11,12,13,14,15
      .irp c,0,1,2,3,4,5,6,7,8,9,10,11,12,13,14,15
        v_accvgpr_read_b32 v[16*(\i%%2)+\c], a[16*\i+\c]
      .endr
      .irp c,0,1,2,3,4,5,6,7,8,9,10,11,12,13,14,15
        v_mul_f32 v[16*(\i%%2)+\c], v[16*(\i%%2)+\c], v84
      .endr
      .irp p,0,1,2,3,4,5,6,7
        .if BF16
          v_cvt_pk_bf16_f32 v[32+8*(\i%%2)+\p], v[16*(\i%%2)+2*\p], v[16*(\i%%2)+2*\p+1]
        .else
          v_cvt_f16_f32 v[16*(\i%%2)+2*\p], v[16*(\i%%2)+2*\p]
          v_cvt_f16_f32 v[16*(\i%%2)+2*\p+1], v[16*(\i%%2)+2*\p+1]
          s_nop 0
          v_pack_b32_f16 v[32+8*(\i%%2)+\p], v[16*(\i%%2)+2*\p], v[16*(\i%%2)+2*\p+1]
        .endif
      .endr
      s_nop 1
      .irp r,0,1,2,3
        ds_write_b64 v91, v[32+8*(\i%%2)+2*\r:33+8*(\i%%2)+2*\r] offset:(32*\i+8*\r)*2
      .endr
    .endr
    v_lshlrev_b32 v92, 4, v92                // 16 lane: this lane's piece of every row
    v_add_u32 v93, s48, v92
    s_mov_b64 s[50:51], %[out]
    s_waitcnt lgkmcnt(0)
    .irp b,0,1,2,3
      .irp k,0,1,2,3,4,5,6,7
        ds_read_b128 v[4*\k:4*\k+3], v93 offset:(8*\b+\k)*1040
      .endr
      s_waitcnt lgkmcnt(0)
      .irp k,0,1,2,3
        s_cmp_gt_u32 %[nh], 8*\b+\k          // (row 8 b + k belongs to a head of the call)
        s_cselect_b64 exec, -1, 0
        s_nop 1
        global_store_dwordx4 v92, v[4*\k:4*\k+3], s[50:51] offset:1024*\k
      .endr
      s_add_u32 s50, s50, 4096
      s_addc_u32 s51, s51, 0
      .irp k,4,5,6,7
        s_cmp_gt_u32 %[nh], 8*\b+\k
        s_cselect_b64 exec, -1, 0
        s_nop 1
        global_store_dwordx4 v92, v[4*\k:4*\k+3], s[50:51] offset:1024*(\k-4)
      .endr
      s_add_u32 s50, s50, 4096
      s_addc_u32 s51, s51, 0
      s_mov_b64 exec, -1
    .endr
    s_barrier                                // the next segment's transfers may take the buffers
    s_mov_b64 s[60:61], exec
    s_cmp_eq_u32 %[complete], 0
    s_cbranch_scc1 13f
    s_cmp_eq_u64 %[lse], 0
    s_cbranch_scc1 14f
    // natural-log log-sum-exp of the row, by the kh = 0 lanes
    v_mul_f32 v85, 0x3f317218, v85
    v_lshlrev_b32 v91, 1, v89
    .if BF16
      v_cvt_pk_bf16_f32 v85, v85, v85
    .else
      v_cvt_f16_f32 v85, v85
    .endif
    s_bfm_b64 exec, %[nh], 0                 // lanes 0 .. heads - 1
    s_nop 1
    global_store_short v91, v85, %[lse]
    s_mov_b64 exec, s[60:61]
    s_branch 14f
    13:
    // partial row: its base-2 log-sum-exp, fp32
    v_lshlrev_b32 v91, 2, v89
    s_bfm_b64 exec, %[nh], 0
    s_nop 1
    global_store_dword v91, v85, %[lse]
    s_mov_b64 exec, s[60:61]
    14:
    .if MASK
      s_waitcnt vmcnt(0)                   // (the last step asked for mask values nobody reads: none may land later)
    .endif
    .purgem MASK_LOAD
    .purgem LDK
    .purgem LDV
    .purgem SM_SLICE
    .purgem QK_SLOT
    .purgem QK_PHASE
    .purgem SM_ALONE
    .purgem DMA_PREP
    .purgem DMA_LOAD
    .purgem DMA_ONE
    .purgem DMA_ANY
    .purgem PV_SLOT
    .purgem PV_PHASE
    .purgem BODY
    )ASM"
                 :
                 : [bf16] "n"(BF16 ? 1 : 0), [split] "n"(SPLIT ? 1 : 0), [nz] "n"(NZ ? 1 : 0), [mask_on] "n"(MASK ? 1 : 0),
                   [mask_lo] "s"(maskLo), [mask_hi] "s"(maskHi), [mask_bytes] "s"(maskBytes), [mask_token_bytes] "s"(maskTokenBytes),
                   [real_heads] "s"(realHeads), [qrope] "s"(qRope), [rope_lo] "s"(ropeLo),
                   [rope_hi] "s"(ropeHi), [roperowbytes] "s"(ropeRowBytes), [scale] "s"(scale2), [bshift] "s"(blockShift), [table] "s"(table),
                   [rowbytes] "s"(rowBytes), [cache_lo] "s"(cacheLo), [cache_hi] "s"(cacheHi), [q] "s"(q), [out] "s"(out),
                   [lse] "s"(lse), [tokbegin] "s"(tokBegin), [tokend] "s"(tokEnd), [lds] "s"(ldsBase), [wave] "s"(wave),
                   [complete] "s"(complete), [nh] "s"(heads), [qlast] "s"(lastHead)
                 : "memory", "vcc", "scc", "m0", ATBMI_REGS_0_99("v"), ATBMI_REGS_100_111("v"), ATBMI_REGS_112_255("v"),
                   ATBMI_REGS_0_99("a"), ATBMI_REGS_100_111("a"), ATBMI_REGS_112_255("a"), ATBMI_SREGS_36_69("s"), "s70", "s71");
}

// One wave range per workgroup; the grid is a multiple of 8 x head groups.
template <bool BF16, bool SPLIT, bool NZ, bool MASK>
__global__ __launch_bounds__(NW *WAVE) void PaMlaAsmKernel(const PaArgs a, const PaStreamPlan p)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    // Workgroups go to the 8 XCDs round-robin and every XCD has an L2 of its own. XCD x takes the x-th eighth
    // of the ranges: consecutive ranges walk the same sequences, so the (three to five) ranges of a sequence
    // fetch its 147 KB of query rows from HBM once and from their common L2 after that; the head groups of a
    // range, which read the same cache rows, sit on one XCD as well.
    const int perXcd = gridDim.x / (8 * p.headGroups);
    const int xcd = blockIdx.x % 8;
    const int slot = blockIdx.x / 8;
    const int hgIdx = slot % p.headGroups;
    const int wr = xcd * perXcd + slot / p.headGroups;
    if (wr >= p.numWgRanges) {
        return;
    }
    const int s0 = PaRangeBegin(wr, p.totalSteps, p.numWaveRanges);
    const int s1 = PaRangeBegin(wr + 1, p.totalSteps, p.numWaveRanges);
    if (s0 >= s1) {
        return;
    }
    const uint32_t ldsBase = static_cast<uint32_t>(
        reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) unsigned char *)smem));
    // (a head count that is not a multiple of 128 leaves the last workgroup waves with fewer than 32 heads, or with
    // none: those still stage their rows of every tile, compute on a repeated query row and store nothing)
    const int h0 = hgIdx * PA_MLA_HEADS_PER_WG + static_cast<int>(wave) * HPW;
    // (a pass may hold several query tokens of its sequence: their rows follow each other in q and out as more heads
    // would, so the pass has tokens x heads rows)
    constexpr float LOG2E = 1.4426950408889634f;
    const float scale2 = a.qkScale * LOG2E;
    const uint32_t blockShift = static_cast<uint32_t>(__builtin_ctz(static_cast<unsigned>(a.blockSize)));

    auto uniform = [](int v) { return __builtin_amdgcn_readfirstlane(v); };
    int seqIdx = uniform(p.firstSeq ? p.firstSeq[wr] : p.inlineFirst[wr]);
    while (uniform(mfma::PlanSeq(p, seqIdx + 1).stepBegin) <= s0) {
        ++seqIdx;
    }
    for (; seqIdx < p.numSeqs; ++seqIdx) {
        const PaSeq sq = mfma::PlanSeq(p, seqIdx);
        const int tableRow = uniform(sq.tableRow);
        const int ctxLen = uniform(sq.ctxLen);
        const int stepBegin = uniform(sq.stepBegin);
        const int qRow = uniform(sq.qRow);
        if (stepBegin >= s1) {
            break;
        }
        const int seqEnd = uniform(mfma::PlanSeq(p, seqIdx + 1).stepBegin);
        const int segBegin = max(s0, stepBegin);
        const int segEnd = min(s1, seqEnd);
        Segment sg;
        sg.cache = a.kc;
        sg.table = a.tables + static_cast<int64_t>(tableRow) * a.maxBlocksPerSeq;
        sg.rowBytes = static_cast<uint32_t>(a.kRowStride * 2);
        sg.blockShift = blockShift;
        sg.tokBegin = static_cast<uint32_t>((segBegin - stepBegin) * STEP);
        sg.tokEnd = static_cast<uint32_t>(min(ctxLen, (segEnd - stepBegin) * STEP));
        sg.complete = (segBegin == stepBegin && segEnd == seqEnd) ? 1u : 0u;
        const int passHeads = uniform(sq.nTok) * a.H;
        const int liveHeads = min(max(passHeads - h0, 0), HPW);
        const int hq = liveHeads > 0 ? h0 : 0; // where this wave's query rows are read from
        const int64_t rowHead = static_cast<int64_t>(qRow) * a.H + h0;
        const int64_t rowQuery = static_cast<int64_t>(qRow) * a.H + hq;
        sg.heads = static_cast<uint32_t>(liveHeads);
        sg.q = reinterpret_cast<const uint16_t *>(a.q) + rowQuery * (SPLIT ? DV : D);
        sg.qRope = SPLIT ? reinterpret_cast<const uint16_t *>(a.qRope) + rowQuery * (D - DV) : nullptr;
        sg.ropeCache = SPLIT ? a.kRope : nullptr;
        sg.ropeRowBytes = SPLIT ? static_cast<uint32_t>(a.ropeRowStride * 2) : 0u;
        if (sg.complete) {
            sg.out = reinterpret_cast<uint16_t *>(a.out) + rowHead * DV;
            sg.lse = a.lse ? reinterpret_cast<uint16_t *>(a.lse) + rowHead : nullptr;
        } else {
            const int slot = 2 * wr + (segBegin == s0 ? 0 : 1);
            const int64_t ph = static_cast<int64_t>(slot) * p.foldTokens * a.H + h0;
            sg.out = reinterpret_cast<uint16_t *>(a.partO) + ph * DV;
            sg.lse = a.partLse + ph;
        }
        if (MASK) {
            // one mask row per query row (no stride between heads): the row of this pass
            sg.mask = reinterpret_cast<const uint16_t *>(a.mask) + static_cast<int64_t>(uniform(sq.maskRow)) * a.maskBatchStride;
            sg.maskTokenBytes = static_cast<uint32_t>(a.maskRowStep * a.maskBatchStride * 2);
            sg.maskBytes = (static_cast<uint32_t>(uniform(sq.nTok) - 1) * sg.maskTokenBytes + static_cast<uint32_t>(a.maskLen) * 2u + 3u) & ~3u;
        } else {
            sg.mask = nullptr;
            sg.maskBytes = 0;
            sg.maskTokenBytes = 0;
        }
        sg.realHeads = static_cast<uint32_t>(a.H);
        RunSegment<BF16, SPLIT, NZ, MASK>(sg, ldsBase, wave, scale2);
    }
}

template <bool BF16, bool SPLIT, bool NZ, bool MASK> int LaunchAsmBuild(const PaArgs &args, const PaStreamPlan &plan, hipStream_t stream)
{
    static_assert(SPLIT || !NZ, "fractal-NZ caches come with the split layout");
    auto kernel = PaMlaAsmKernel<BF16, SPLIT, NZ, MASK>;
    const int configured = ConfigureKernelLds(reinterpret_cast<const void *>(kernel), LDS_BYTES);
    if (configured != OK) {
        return configured;
    }
    if (plan.tokenSlices != 1 || plan.numWaveRanges != plan.numWgRanges || plan.foldTokens < 1 || plan.foldTokens > 8 ||
        plan.headGroups != (plan.foldTokens * args.H + PA_MLA_HEADS_PER_WG - 1) / PA_MLA_HEADS_PER_WG || args.G != 1 || args.D != D || args.Dv != DV ||
        args.ropeDim != (SPLIT ? D - DV : 0) || (args.nzShift > 0) != NZ || args.blockSize < 16 || (args.blockSize & (args.blockSize - 1)) != 0 ||
        args.kRowStride * 2 > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: plan or shape does not fit the 128-head MLA kernel");
    }
    const int64_t grid = (static_cast<int64_t>(plan.numWgRanges) + 7) / 8 * 8 * plan.headGroups;
    if (grid <= 0 || grid > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: grid of %lld workgroups is out of range", (long long)grid);
    }
    if (MASK && (args.maskHeadStride != 0 || args.maskBatchStride % 2 != 0 || reinterpret_cast<uintptr_t>(args.mask) % 4 != 0)) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: the 128-head MLA kernel takes one mask row per query row, rows 4-byte aligned");
    }
    kernel<<<static_cast<unsigned>(grid), NW * WAVE, LDS_BYTES, stream>>>(args, plan);
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}

template <bool BF16, bool SPLIT, bool NZ = false> int LaunchAsm(const PaArgs &args, const PaStreamPlan &plan, hipStream_t stream)
{
    return args.mask != nullptr ? LaunchAsmBuild<BF16, SPLIT, NZ, true>(args, plan, stream)
                                : LaunchAsmBuild<BF16, SPLIT, NZ, false>(args, plan, stream);
}

} // namespace mla
} // namespace atbmi
#endif
