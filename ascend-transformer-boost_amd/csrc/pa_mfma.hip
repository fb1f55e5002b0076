// Shape coverage and dispatch of the MFMA decode-attention kernel.
#include <cstdlib>
#include "pa_internal.h"

namespace atbmi {

bool PaMfmaSupports(const AtbmiPaShape &s)
{
    if (s.blockSize % 16 != 0) {
        return false; // a 16-token sub-tile must not straddle cache blocks
    }
    const int d = s.headDimK;
    const int dv = s.headDimV;
    if (s.mlaCombined) {
        return s.kvDtype != ATBMI_INT8 && ((d == 576 && dv == 512) || (d == 192 && dv == 128));
    }
    if (d != dv) {
        return false;
    }
    // every multiple of 32 up to 256 (int8 rows: from 64)
    return d % 32 == 0 && d >= (s.kvDtype == ATBMI_INT8 ? 64 : 32) && d <= 256;
}

bool PaMlaWide(const AtbmiPaShape &s)
{
    static const bool enabled = [] {
        const char *v = getenv("ATBMI_PA_MLA_WIDE");
        return !(v && v[0] == '0');
    }();
    return enabled && s.mlaCombined && s.kvDtype != ATBMI_INT8 && s.headDimK == 576 && s.headDimV == 512 &&
           s.numKvHeads == 1 && s.numHeads >= 1 && s.blockSize >= 16 &&
           (s.blockSize & (s.blockSize - 1)) == 0 && // (the kernel finds a token's block by shifting)
           (s.qScale == 0.0f || s.qScale == 1.0f) && !s.hasLogN && // (those take the 16-head kernel)
           // a mask with one row per query row or sequence (no stride between heads), rows on even elements
           (!s.hasMask || (s.maskHeadStride == 0 && s.maskBatchStride % 2 == 0));
}

bool PaMfmaSharedTile(const AtbmiPaShape &s)
{
    if (PaMlaWide(s)) {
        return false;
    }
    if (!s.mlaCombined || s.headDimK != 576 || s.headDimV != 512 || s.numKvHeads <= 0) {
        return false;
    }
    const int group = s.numHeads / s.numKvHeads;
    const int headTiles = (group + PA_MFMA_HEAD_TILE - 1) / PA_MFMA_HEAD_TILE;
    return (s.numKvHeads * headTiles) % 4 == 0;
}

int PaMfmaWaves(const AtbmiPaShape &s)
{
    if (PaMlaWide(s)) {
        return PA_MLA_WAVES;
    }
    if (PaMfmaSharedTile(s)) {
        // 16 heads x (576 + 512) channels of Q and accumulators need a whole SIMD's registers
        return 4;
    }
    // eight waves' K/V tiles fit the 160 KB of LDS up to 128-channel rows
    // (and for the 192/128 combined cache); wider rows run four waves
    return (s.headDimK <= 128 || (s.mlaCombined && s.headDimK <= 192)) ? 8 : 4;
}

int LaunchPaMfma(const AtbmiPaShape &s, const PaArgs &args, const PaStreamPlan &plan, hipStream_t stream)
{
    int rc;
    if (PaMlaWide(s)) {
        return LaunchPaMlaWide(s, args, plan, stream);
    }
    if (s.kvDtype == ATBMI_INT8) {
        rc = LaunchPaMfmaInt8(s, args, plan, stream);
    } else if (s.qDtype == ATBMI_BF16) {
        rc = LaunchPaMfmaBf16(s, args, plan, stream);
    } else {
        rc = LaunchPaMfmaF16(s, args, plan, stream);
    }
    if (rc < 0) {
        return Fail(ERR_INVALID_PARAM, "pa_decode: no MFMA kernel for head sizes %d/%d", s.headDimK, s.headDimV);
    }
    return rc;
}

} // namespace atbmi
