// KV-cache write kernels for gfx950: ReshapeAndCache (byte copy by slot),
// the per-channel int8 quantiser and the fused quantise+write.
//
// All three are tiny, launch-latency-bound kernels (a decode step writes one
// row per sequence); the only hardware concern is that every HBM access is a
// full-width vector access, so rows are moved as 16-byte pieces whenever the
// row size and base addresses allow it.
#include "atbmi_common.h"

namespace atbmi {
namespace {

constexpr int COPY_THREADS = 256;

// grid.x = token, grid.y = 0 (key) / 1 (value). One workgroup copies one row.
// VecT is the widest type all addresses are aligned to.
template <typename VecT>
__global__ __launch_bounds__(COPY_THREADS) void ReshapeAndCacheKernel(const uint8_t *__restrict__ key,
                                                                      const uint8_t *__restrict__ value,
                                                                      uint8_t *__restrict__ keyCache,
                                                                      uint8_t *__restrict__ valueCache,
                                                                      const int32_t *__restrict__ slots,
                                                                      int64_t kRowBytes, int64_t vRowBytes,
                                                                      int64_t numSlots)
{
    const int64_t token = blockIdx.x;
    const int64_t slot = slots[token];
    if (slot < 0 || slot >= numSlots) {
        return;
    }
    const bool isValue = blockIdx.y == 1;
    const int64_t rowBytes = isValue ? vRowBytes : kRowBytes;
    const VecT *src = reinterpret_cast<const VecT *>((isValue ? value : key) + token * rowBytes);
    VecT *dst = reinterpret_cast<VecT *>((isValue ? valueCache : keyCache) + slot * rowBytes);
    const int64_t n = rowBytes / static_cast<int64_t>(sizeof(VecT));
    for (int64_t i = threadIdx.x; i < n; i += COPY_THREADS) {
        dst[i] = src[i];
    }
}

// A key or value input that is a strided view: element (token, head, channel) sits
// `offset + token * tokenStride + head * headStride + channel * chanStride` bytes from the base.
struct StridedRows {
    const uint8_t *base;
    int64_t offset, tokenStride, headStride, chanStride;
    int64_t headBytes; // headDim * element size: what one head contributes to a cache row
};

// grid.x = token, grid.y = 0 (key) / 1 (value). One workgroup gathers one strided row into its slot.
// VecT is the widest type every head's start is aligned to when the channels are contiguous,
// otherwise the element type (one element per access).
template <typename VecT>
__global__ __launch_bounds__(COPY_THREADS) void ReshapeAndCacheStridedKernel(StridedRows k, StridedRows v,
                                                                             uint8_t *__restrict__ keyCache,
                                                                             uint8_t *__restrict__ valueCache,
                                                                             const int32_t *__restrict__ slots,
                                                                             int64_t heads, int64_t numSlots)
{
    const int64_t token = blockIdx.x;
    const int64_t slot = slots[token];
    if (slot < 0 || slot >= numSlots) {
        return;
    }
    const bool isValue = blockIdx.y == 1;
    const StridedRows &r = isValue ? v : k;
    const int64_t perHead = r.headBytes / static_cast<int64_t>(sizeof(VecT));
    const uint8_t *src = r.base + r.offset + token * r.tokenStride;
    uint8_t *dst = (isValue ? valueCache : keyCache) + slot * heads * r.headBytes;
    for (int64_t i = threadIdx.x; i < heads * perHead; i += COPY_THREADS) {
        const int64_t h = i / perHead;
        const int64_t c = i - h * perHead;
        reinterpret_cast<VecT *>(dst)[i] = *reinterpret_cast<const VecT *>(src + h * r.headStride + c * r.chanStride);
    }
}

// q = clamp(rint(x / s) + offset, -128, 127); IEEE divide, ties to even.
__device__ __forceinline__ int8_t QuantOne(float x, float s, int32_t offset)
{
    float r = rintf(__fdiv_rn(x, s));
    if (r != r) {
        return 0;
    }
    r += static_cast<float>(offset);
    r = fminf(fmaxf(r, -128.0f), 127.0f);
    return static_cast<int8_t>(static_cast<int32_t>(r));
}

__global__ __launch_bounds__(256) void QuantPerChannelKernel(const void *__restrict__ x, int32_t isBf16,
                                                             const float *__restrict__ scale,
                                                             const int32_t *__restrict__ offset,
                                                             int8_t *__restrict__ out, int64_t total,
                                                             int64_t channels)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int64_t c = i % channels;
        const float v = Load16(x, i, isBf16 != 0);
        out[i] = QuantOne(v, scale[c], offset ? offset[c] : 0);
    }
}

// grid.x = token, grid.y = 0 (key) / 1 (value): quantise one row straight
// into its cache slot.
__global__ __launch_bounds__(256) void ReshapeAndCacheQuantKernel(const void *__restrict__ key,
                                                                  const void *__restrict__ value, int32_t isBf16,
                                                                  const float *__restrict__ kScale,
                                                                  const float *__restrict__ vScale,
                                                                  int8_t *__restrict__ keyCache,
                                                                  int8_t *__restrict__ valueCache,
                                                                  const int32_t *__restrict__ slots, int64_t kRow,
                                                                  int64_t vRow, int64_t numSlots)
{
    const int64_t token = blockIdx.x;
    const int64_t slot = slots[token];
    if (slot < 0 || slot >= numSlots) {
        return;
    }
    const bool isValue = blockIdx.y == 1;
    const int64_t row = isValue ? vRow : kRow;
    const void *src = isValue ? value : key;
    const float *scale = isValue ? vScale : kScale;
    int8_t *dst = (isValue ? valueCache : keyCache) + slot * row;
    for (int64_t c = threadIdx.x; c < row; c += blockDim.x) {
        dst[c] = QuantOne(Load16(src, token * row + c, isBf16 != 0), scale[c], 0);
    }
}

bool Aligned(const void *p, uintptr_t a)
{
    return (reinterpret_cast<uintptr_t>(p) % a) == 0;
}

} // namespace
} // namespace atbmi

using namespace atbmi;

extern "C" int atbmi_reshape_and_cache(const void *key, const void *value, void *keyCache, void *valueCache,
                                       const int32_t *slotMapping, int64_t numTokens, int64_t numKvHeads,
                                       int64_t headDimK, int64_t headDimV, int64_t numSlots, int32_t elemBytes,
                                       void *stream)
{
    if (!key || !keyCache || !slotMapping) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache: key, keyCache and slotMapping must be non-null");
    }
    if ((value == nullptr) != (valueCache == nullptr)) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache: value and valueCache must both be given or both be null");
    }
    if (numTokens < 0 || numKvHeads <= 0 || headDimK <= 0 || numSlots <= 0 || (value && headDimV <= 0)) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache: bad extents");
    }
    if (elemBytes != 1 && elemBytes != 2) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache: elemBytes must be 1 or 2, got %d", elemBytes);
    }
    if (numTokens == 0) {
        return OK;
    }
    if (numTokens > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache: too many tokens");
    }
    const int64_t kRowBytes = numKvHeads * headDimK * elemBytes;
    const int64_t vRowBytes = value ? numKvHeads * headDimV * elemBytes : kRowBytes;
    // Widest vector every row start is aligned to.
    uintptr_t align = 16;
    while (align > 1 && !(kRowBytes % align == 0 && vRowBytes % align == 0 && Aligned(key, align) &&
                          Aligned(keyCache, align) && (!value || (Aligned(value, align) && Aligned(valueCache, align))))) {
        align >>= 1;
    }
    dim3 grid(static_cast<unsigned>(numTokens), value ? 2 : 1);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint8_t *k8 = static_cast<const uint8_t *>(key);
    const uint8_t *v8 = static_cast<const uint8_t *>(value);
    uint8_t *kc8 = static_cast<uint8_t *>(keyCache);
    uint8_t *vc8 = static_cast<uint8_t *>(valueCache);
    switch (align) {
        case 16:
            ReshapeAndCacheKernel<uint4><<<grid, COPY_THREADS, 0, s>>>(k8, v8, kc8, vc8, slotMapping, kRowBytes,
                                                                        vRowBytes, numSlots);
            break;
        case 8:
            ReshapeAndCacheKernel<uint2><<<grid, COPY_THREADS, 0, s>>>(k8, v8, kc8, vc8, slotMapping, kRowBytes,
                                                                        vRowBytes, numSlots);
            break;
        case 4:
            ReshapeAndCacheKernel<uint32_t><<<grid, COPY_THREADS, 0, s>>>(k8, v8, kc8, vc8, slotMapping, kRowBytes,
                                                                           vRowBytes, numSlots);
            break;
        case 2:
            ReshapeAndCacheKernel<uint16_t><<<grid, COPY_THREADS, 0, s>>>(k8, v8, kc8, vc8, slotMapping, kRowBytes,
                                                                           vRowBytes, numSlots);
            break;
        default:
            ReshapeAndCacheKernel<uint8_t><<<grid, COPY_THREADS, 0, s>>>(k8, v8, kc8, vc8, slotMapping, kRowBytes,
                                                                          vRowBytes, numSlots);
            break;
    }
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}

extern "C" int atbmi_reshape_and_cache_strided(const void *key, const void *value, void *keyCache, void *valueCache,
                                               const int32_t *slotMapping, int64_t numTokens, int64_t numKvHeads,
                                               int64_t headDimK, int64_t headDimV, int64_t numSlots,
                                               int32_t elemBytes, const int64_t *keyStrides, int64_t keyOffset,
                                               const int64_t *valueStrides, int64_t valueOffset, void *stream)
{
    if (!key || !keyCache || !slotMapping || !keyStrides) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache_strided: key, keyCache, slotMapping, keyStrides must be non-null");
    }
    if ((value == nullptr) != (valueCache == nullptr) || (value && !valueStrides)) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache_strided: value, valueCache and valueStrides go together");
    }
    if (numTokens < 0 || numTokens > 0x7fffffffLL || numKvHeads <= 0 || headDimK <= 0 || numSlots <= 0 ||
        (value && headDimV <= 0)) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache_strided: bad extents");
    }
    if (elemBytes != 1 && elemBytes != 2) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache_strided: elemBytes must be 1 or 2, got %d", elemBytes);
    }
    if (numTokens == 0) {
        return OK;
    }
    auto rows = [&](const void *base, const int64_t *strides, int64_t offset, int64_t headDim) {
        StridedRows r;
        r.base = static_cast<const uint8_t *>(base);
        r.offset = offset * elemBytes;
        r.tokenStride = strides[0] * elemBytes;
        r.headStride = strides[1] * elemBytes;
        r.chanStride = strides[2] * elemBytes;
        r.headBytes = headDim * elemBytes;
        return r;
    };
    const StridedRows k = rows(key, keyStrides, keyOffset, headDimK);
    const StridedRows v = value ? rows(value, valueStrides, valueOffset, headDimV) : k;
    // Widest access: whole vectors when the channels of a head are contiguous and every head of every
    // token starts on the vector's alignment, single elements otherwise.
    uintptr_t align = static_cast<uintptr_t>(elemBytes);
    if (k.chanStride == elemBytes && v.chanStride == elemBytes) {
        align = 16;
        auto fits = [&](const StridedRows &r, const void *cache) {
            return Aligned(r.base, align) && Aligned(cache, align) && r.offset % static_cast<int64_t>(align) == 0 &&
                   r.tokenStride % static_cast<int64_t>(align) == 0 && r.headStride % static_cast<int64_t>(align) == 0 &&
                   r.headBytes % static_cast<int64_t>(align) == 0;
        };
        while (align > static_cast<uintptr_t>(elemBytes) && !(fits(k, keyCache) && (!value || fits(v, valueCache)))) {
            align >>= 1;
        }
    }
    dim3 grid(static_cast<unsigned>(numTokens), value ? 2 : 1);
    hipStream_t s = static_cast<hipStream_t>(stream);
    uint8_t *kc8 = static_cast<uint8_t *>(keyCache);
    uint8_t *vc8 = static_cast<uint8_t *>(valueCache);
    StridedRows kk = k, vv = v;
    if (align > static_cast<uintptr_t>(elemBytes)) { // contiguous channels: the step between accesses is the vector
        kk.chanStride = vv.chanStride = static_cast<int64_t>(align);
    }
    switch (align) {
        case 16:
            ReshapeAndCacheStridedKernel<uint4><<<grid, COPY_THREADS, 0, s>>>(kk, vv, kc8, vc8, slotMapping, numKvHeads, numSlots);
            break;
        case 8:
            ReshapeAndCacheStridedKernel<uint2><<<grid, COPY_THREADS, 0, s>>>(kk, vv, kc8, vc8, slotMapping, numKvHeads, numSlots);
            break;
        case 4:
            ReshapeAndCacheStridedKernel<uint32_t><<<grid, COPY_THREADS, 0, s>>>(kk, vv, kc8, vc8, slotMapping, numKvHeads, numSlots);
            break;
        case 2:
            ReshapeAndCacheStridedKernel<uint16_t><<<grid, COPY_THREADS, 0, s>>>(kk, vv, kc8, vc8, slotMapping, numKvHeads, numSlots);
            break;
        default:
            ReshapeAndCacheStridedKernel<uint8_t><<<grid, COPY_THREADS, 0, s>>>(kk, vv, kc8, vc8, slotMapping, numKvHeads, numSlots);
            break;
    }
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}

extern "C" int atbmi_quant_per_channel(const void *x, int32_t xDtype, const float *scale, const int32_t *offset,
                                       int8_t *out, int64_t rows, int64_t channels, void *stream)
{
    if (!x || !scale || !out) {
        return Fail(ERR_INVALID_PARAM, "quant_per_channel: x, scale and out must be non-null");
    }
    if (xDtype != ATBMI_F16 && xDtype != ATBMI_BF16) {
        return Fail(ERR_INVALID_PARAM, "quant_per_channel: x must be fp16 or bf16");
    }
    if (rows < 0 || channels <= 0) {
        return Fail(ERR_INVALID_PARAM, "quant_per_channel: bad extents");
    }
    const int64_t total = rows * channels;
    if (total == 0) {
        return OK;
    }
    int64_t blocks = (total + 255) / 256;
    if (blocks > 65536) {
        blocks = 65536;
    }
    QuantPerChannelKernel<<<static_cast<unsigned>(blocks), 256, 0, static_cast<hipStream_t>(stream)>>>(
        x, xDtype == ATBMI_BF16, scale, offset, out, total, channels);
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}

extern "C" int atbmi_reshape_and_cache_quant(const void *key, const void *value, int32_t kvDtype,
                                             const float *kScale, const float *vScale, int8_t *keyCache,
                                             int8_t *valueCache, const int32_t *slotMapping, int64_t numTokens,
                                             int64_t numKvHeads, int64_t headDimK, int64_t headDimV,
                                             int64_t numSlots, void *stream)
{
    if (!key || !keyCache || !kScale || !slotMapping) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache_quant: key, kScale, keyCache, slotMapping must be non-null");
    }
    if ((value == nullptr) != (valueCache == nullptr) || (value && !vScale)) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache_quant: value, vScale and valueCache go together");
    }
    if (kvDtype != ATBMI_F16 && kvDtype != ATBMI_BF16) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache_quant: key/value must be fp16 or bf16");
    }
    if (numTokens < 0 || numTokens > 0x7fffffffLL || numKvHeads <= 0 || headDimK <= 0 || numSlots <= 0 ||
        (value && headDimV <= 0)) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache_quant: bad extents");
    }
    if (numTokens == 0) {
        return OK;
    }
    dim3 grid(static_cast<unsigned>(numTokens), value ? 2 : 1);
    ReshapeAndCacheQuantKernel<<<grid, 256, 0, static_cast<hipStream_t>(stream)>>>(
        key, value, kvDtype == ATBMI_BF16, kScale, vScale, keyCache, valueCache, slotMapping,
        numKvHeads * headDimK, value ? numKvHeads * headDimV : 0, numSlots);
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}
