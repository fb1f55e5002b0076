// Shared host/device helpers of the MI355X kernel layer.
#ifndef ATBMI_COMMON_H
#define ATBMI_COMMON_H
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include "atbmi_kernels.h"

namespace atbmi {

// Return codes are atb::ErrorType values.
constexpr int OK = 0;
constexpr int ERR_INVALID_PARAM = 1;
constexpr int ERR_RT_FAIL = 4;
constexpr int ERR_OUT_OF_DEVICE_MEMORY = 26;
constexpr int ERR_OUT_OF_HOST_MEMORY = 27;

constexpr int WAVE = 64;

// Records the message atbmi_last_error() hands back and returns `code`.
int Fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define ATBMI_HIP_CHECK(expr)                                                                       \
    do {                                                                                            \
        hipError_t e_ = (expr);                                                                     \
        if (e_ != hipSuccess) {                                                                     \
            return ::atbmi::Fail(::atbmi::ERR_RT_FAIL, "%s failed: %s", #expr, hipGetErrorString(e_)); \
        }                                                                                           \
    } while (0)

// One physical work item of the split-K plan: the token range
// [tokBegin, tokEnd) of one sequence, handled by one workgroup per KV head.
struct PaWorkItem {
    int32_t qRow;        // row of q / out this sequence uses
    int32_t seq;         // row of blockTables
    int32_t tokBegin;
    int32_t tokEnd;
    int32_t partialBase; // first partial slot this item writes
    int32_t direct;      // 1: the only chunk of its sequence, write `out` directly
    int32_t pad0;
    int32_t pad1;
};

// Per non-empty sequence: where its partials live, for the merge kernel.
struct PaSeqInfo {
    int32_t qRow;
    int32_t firstPartial;
    int32_t numPartials;
    int32_t ctxLen;
};

// Kernel arguments shared by the attention kernels and the merge kernel.
struct PaArgs {
    const void *q;
    const void *kc;
    const void *vc;
    const int32_t *tables;
    const float *kScale;
    const int32_t *kOff;
    const float *vScale;
    const int32_t *vOff;
    void *out;
    const PaWorkItem *items;
    const PaSeqInfo *seqs;
    float *partO;   // [numPartials][H][Dv] normalised partial outputs
    float *partLse; // [numPartials][H] log2-domain log-sum-exp
    int32_t H, G, D, Dv;
    int32_t blockSize, maxBlocksPerSeq;
    int32_t qIsBf16;
    int32_t groupSize; // H / G
    float qkScale;
    float qScale; // 0 when unused
    int64_t kRowStride; // elements between consecutive tokens in the key cache (G*D)
    int64_t vRowStride; // same for the value cache (G*Dv, or G*D when V aliases K)
    int32_t vHeadStride; // elements between KV heads inside a value row (Dv, or D when V aliases K)
    int32_t finishV;     // 1: partial outputs are still in int8 units; the final write applies vScale/vOff
};

__device__ __forceinline__ float Bf16ToFloat(uint16_t v)
{
    return __uint_as_float(static_cast<uint32_t>(v) << 16);
}

// Round-to-nearest-even fp32 -> bf16, NaN kept quiet.
__device__ __forceinline__ uint16_t FloatToBf16(float f)
{
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        return static_cast<uint16_t>((u >> 16) | 0x40u);
    }
    u += 0x7fffu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

__device__ __forceinline__ float HalfBitsToFloat(uint16_t v)
{
    return static_cast<float>(__builtin_bit_cast(_Float16, v));
}

__device__ __forceinline__ uint16_t FloatToHalfBits(float f)
{
    return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
}

__device__ __forceinline__ float Load16(const void *p, int64_t idx, bool bf16)
{
    uint16_t raw = reinterpret_cast<const uint16_t *>(p)[idx];
    return bf16 ? Bf16ToFloat(raw) : HalfBitsToFloat(raw);
}

__device__ __forceinline__ void Store16(void *p, int64_t idx, float v, bool bf16)
{
    reinterpret_cast<uint16_t *>(p)[idx] = bf16 ? FloatToBf16(v) : FloatToHalfBits(v);
}

} // namespace atbmi
#endif
