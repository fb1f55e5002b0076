// KV-cache write kernels for gfx950: ReshapeAndCache (byte copy by slot),
// the per-channel int8 quantiser and the fused quantise+write.
//
// All three are tiny, launch-latency-bound kernels (a decode step writes one
// row per sequence); the only hardware concern is that every HBM access is a
// full-width vector access, so rows are moved as 16-byte pieces whenever the
// row size and base addresses allow it.
#include <algorithm>
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

// Fractal-NZ caches: a cache row of C elements is cut into pieces of `lastDim` elements and a block of blockSize
// slots is stored piece-major, [numBlocks, C / lastDim, blockSize, lastDim]. grid.x = group of NZ_TOKENS tokens,
// grid.y = 0 (key) / 1 (value). Neighbouring lanes take the same piece of neighbouring tokens: tokens of a
// prompt sit in consecutive slots, so a piece of the group lands in one contiguous run of the cache
// (NZ_TOKENS * pieceBytes), and the lanes that share a token read consecutive pieces of its row.
constexpr int NZ_TOKENS = 8;
typedef uint32_t NzVec16 __attribute__((ext_vector_type(4))); // (plain vector types: the non-temporal store takes no structs)
typedef uint32_t NzVec8 __attribute__((ext_vector_type(2)));

struct NzRows {
    const uint8_t *src;
    uint8_t *cache;
    int64_t rowBytes;   // bytes of one token's row
    int64_t pieceBytes; // lastDim * element size: 16 or 32
};

template <typename VecT>
__global__ __launch_bounds__(COPY_THREADS) void ReshapeAndCacheNzKernel(NzRows k, NzRows v,
                                                                        const int32_t *__restrict__ slots,
                                                                        int64_t numTokens, int64_t blockSize,
                                                                        int64_t numSlots)
{
    const NzRows &r = blockIdx.y == 1 ? v : k;
    const int perPiece = static_cast<int>(r.pieceBytes / static_cast<int64_t>(sizeof(VecT)));
    const int lanesPerPiece = perPiece * NZ_TOKENS; // divides COPY_THREADS for every VecT and piece size
    const int sub = threadIdx.x % lanesPerPiece;
    const int tok = sub / perPiece;
    const int within = sub - tok * perPiece;
    const int64_t token = static_cast<int64_t>(blockIdx.x) * NZ_TOKENS + tok;
    if (token >= numTokens) {
        return;
    }
    const int64_t slot = slots[token];
    if (slot < 0 || slot >= numSlots) {
        return;
    }
    const int64_t block = slot / blockSize;
    const int64_t offset = slot - block * blockSize;
    const VecT *src = reinterpret_cast<const VecT *>(r.src + token * r.rowBytes) + within;
    uint8_t *dst = r.cache + block * blockSize * r.rowBytes + offset * r.pieceBytes +
                   within * static_cast<int64_t>(sizeof(VecT));
    const int pieces = static_cast<int>(r.rowBytes / r.pieceBytes);
    const int step = COPY_THREADS / lanesPerPiece;
    const int64_t pieceStride = blockSize * r.pieceBytes;
    // all loads of a batch before its stores (the compiler cannot reorder them itself: the caches may alias the rows)
    constexpr int BATCH = 4;
    for (int p0 = threadIdx.x / lanesPerPiece; p0 < pieces; p0 += step * BATCH) {
        VecT held[BATCH];
#pragma unroll
        for (int i = 0; i < BATCH; ++i) {
            const int p = p0 + i * step;
            if (p < pieces) {
                held[i] = src[p * perPiece];
            }
        }
#pragma unroll
        for (int i = 0; i < BATCH; ++i) {
            const int p = p0 + i * step;
            if (p < pieces) {
                __builtin_nontemporal_store(held[i], reinterpret_cast<VecT *>(dst + p * pieceStride));
            }
        }
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

// RMSNorm of the latent row + rotary embedding of the rotary row, written side by side into the
// token's slot of a single cache (the producer of the combined MLA cache). One wave per token, four
// tokens per workgroup; fp32 arithmetic, one rounding to the 16-bit type at the end:
//   cache[slot][0 : normDim]       = (x * (1 / sqrt(mean(x^2) + epsilon))) * gamma
//   cache[slot][normDim + i]       = r[i] * cos[i] - r[i + half] * sin[i]            (i < half)
//   cache[slot][normDim + half + i] = r[half + i] * cos[half + i] + r[i] * sin[half + i]
constexpr int NORM_ROPE_WAVES = 4;
typedef uint32_t RowVec __attribute__((ext_vector_type(4)));
// A cache row is written once and read much later by another kernel: non-temporal, so that the write
// stream does not claim cache lines on its way out.
__device__ __forceinline__ void StoreRowPiece(uint16_t *p, uint4 v)
{
    __builtin_nontemporal_store(RowVec{v.x, v.y, v.z, v.w}, reinterpret_cast<RowVec *>(p));
}

__device__ __forceinline__ float Half16(uint32_t word, int hi, bool bf16)
{
    const uint16_t h = static_cast<uint16_t>(word >> (16 * hi));
    return bf16 ? Bf16ToFloat(h) : HalfBitsToFloat(h);
}
__device__ __forceinline__ uint32_t PackPair(float lo, float hi, bool bf16)
{
    const uint32_t l = bf16 ? FloatToBf16(lo) : FloatToHalfBits(lo);
    const uint32_t h = bf16 ? FloatToBf16(hi) : FloatToHalfBits(hi);
    return l | (h << 16);
}
// (x * inv) * gamma for 8 channels, inv = 1 / rms: the order of the reference's golden
__device__ __forceinline__ uint4 NormPiece(uint4 v, uint4 g, float inv, bool bf16)
{
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w};
    uint32_t o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        o[e] = PackPair(__fmul_rn(__fmul_rn(inv, Half16(w[e], 0, bf16)), Half16(gw[e], 0, bf16)),
                        __fmul_rn(__fmul_rn(inv, Half16(w[e], 1, bf16)), Half16(gw[e], 1, bf16)), bf16);
    }
    return uint4{o[0], o[1], o[2], o[3]};
}
__device__ __forceinline__ float SumSquares(uint4 v, bool bf16)
{
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    float sq = 0.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float f = Half16(w[e >> 1], e & 1, bf16);
        sq += f * f;
    }
    return sq;
}

// FAST: rows of at most 512 latent channels and at most 128 rotary channels: everything a lane needs is
// requested up front (one 16-byte piece of the latent row and of gamma, one rotary pair) and the latent
// row stays in registers between the two passes. Otherwise the row is read twice (the second time
// from the caches). The kernel is bound by its vector instructions as much as by memory (a row is
// only 2.5 KB): the element type is a template parameter and every lane has work in every phase.
template <bool FAST, bool BF16>
__global__ __launch_bounds__(NORM_ROPE_WAVES *WAVE) void NormRopeCacheKernel(
    const uint16_t *__restrict__ x, const uint16_t *__restrict__ gamma, const uint16_t *__restrict__ rope,
    const uint16_t *__restrict__ cosTab, const uint16_t *__restrict__ sinTab, const int32_t *__restrict__ slots,
    uint16_t *__restrict__ cache, int64_t numTokens, int32_t normDim, int32_t ropeDim, int64_t numSlots,
    float epsilon)
{
    const int lane = threadIdx.x % WAVE;
    constexpr bool bf16 = BF16;
    const int half = ropeDim / 2;
    // a wave walks the tokens with the stride of the whole launch
    const int64_t stride = static_cast<int64_t>(gridDim.x) * NORM_ROPE_WAVES;
    for (int64_t token = static_cast<int64_t>(blockIdx.x) * NORM_ROPE_WAVES + threadIdx.x / WAVE; token < numTokens;
         token += stride) {
        // The slot is asked for first and looked at last (FAST): a row's loads do not wait for it, and
        // the few rows that turn out to be skipped cost their loads.
        const int64_t slot = slots[token];
        if (!FAST && (slot < 0 || slot >= numSlots)) {
            continue;
        }
        const uint16_t *xr = x + token * normDim;
        const uint16_t *rr = rope + token * ropeDim;
        const uint16_t *cr = cosTab + token * ropeDim;
        const uint16_t *sr = sinTab + token * ropeDim;
        // Rotary pair (i, half + i): two products and a sum, each rounded, as the reference kernel's
        // vector unit does them.
        auto turn = [&](int i, uint16_t *out) {
            const float a = Load16(rr, i, bf16), b = Load16(rr, i + half, bf16);
            const float lo = __fadd_rn(__fmul_rn(a, Load16(cr, i, bf16)), __fmul_rn(-b, Load16(sr, i, bf16)));
            const float hi = __fadd_rn(__fmul_rn(b, Load16(cr, i + half, bf16)), __fmul_rn(a, Load16(sr, i + half, bf16)));
            Store16(out, normDim + i, lo, bf16);
            Store16(out, normDim + half + i, hi, bf16);
        };
        // normDim is a multiple of 8 (checked by the host): a lane takes 8 consecutive channels at a time
        if constexpr (FAST) {
            const int c = lane * 8;
            const bool mine = c < normDim;
            const bool turns = lane < half;
            uint4 xv = {0u, 0u, 0u, 0u}, gv = xv;
            uint16_t ra = 0, rb = 0, ca = 0, cb = 0, sa = 0, sb = 0;
            if (mine) {
                xv = *reinterpret_cast<const uint4 *>(xr + c);
                gv = *reinterpret_cast<const uint4 *>(gamma + c);
            }
            if (turns) {
                ra = rr[lane]; rb = rr[half + lane];
                ca = cr[lane]; cb = cr[half + lane];
                sa = sr[lane]; sb = sr[half + lane];
            }
            float sq = SumSquares(xv, bf16);
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                sq += __shfl_xor(sq, off, WAVE);
            }
            const float inv = __fdiv_rn(1.0f, __fsqrt_rn(__fdiv_rn(sq, static_cast<float>(normDim)) + epsilon));
            if (slot < 0 || slot >= numSlots) {
                continue;
            }
            uint16_t *out = cache + slot * (static_cast<int64_t>(normDim) + ropeDim);
            if (mine) {
                StoreRowPiece(out + c, NormPiece(xv, gv, inv, bf16));
            }
            if (turns) {
                const float a = Half16(ra, 0, bf16), b = Half16(rb, 0, bf16);
                const float lo = __fadd_rn(__fmul_rn(a, Half16(ca, 0, bf16)), __fmul_rn(-b, Half16(sa, 0, bf16)));
                const float hi = __fadd_rn(__fmul_rn(b, Half16(cb, 0, bf16)), __fmul_rn(a, Half16(sb, 0, bf16)));
                Store16(out, normDim + lane, lo, bf16);
                Store16(out, normDim + half + lane, hi, bf16);
            }
        } else {
            uint16_t *out = cache + slot * (static_cast<int64_t>(normDim) + ropeDim);
            float sq = 0.0f;
            for (int c = lane * 8; c < normDim; c += WAVE * 8) {
                sq += SumSquares(*reinterpret_cast<const uint4 *>(xr + c), bf16);
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                sq += __shfl_xor(sq, off, WAVE);
            }
            const float inv = __fdiv_rn(1.0f, __fsqrt_rn(__fdiv_rn(sq, static_cast<float>(normDim)) + epsilon));
            for (int c = lane * 8; c < normDim; c += WAVE * 8) { // second pass: the row is still in the caches
                StoreRowPiece(out + c, NormPiece(*reinterpret_cast<const uint4 *>(xr + c),
                                                 *reinterpret_cast<const uint4 *>(gamma + c), inv, bf16));
            }
            for (int i = lane; i < half; i += WAVE) {
                turn(i, out);
            }
        }
    }
}

// ElewiseOperation's per-channel quantiser and dequantiser: the scale has the type of x (16-bit) and
// the offset is int8; "channel" is the element's index modulo the number of scale entries (the scale
// covers the trailing dimensions of x, or is a single value).
//   quant:        clamp(rint(fp16(x / scale)) + offset, -128, 127): the quotient is rounded to fp16
//                 before it is rounded to an integer, as the reference golden's fp16 division does
//                 (for bf16 inputs too: the golden converts them to fp16 first)
//   dequant:      fp16((x - offset) * scale), saturated at +-65504
// VEC = 8: eight consecutive elements per thread with 16-byte accesses on the 16-bit side.
__device__ __forceinline__ int8_t QuantOne16(float x, float s, int32_t offset, bool bf16)
{
    (void)bf16; // (bf16 inputs take the same route: the reference golden converts them to fp16 and divides there)
    const float q = HalfBitsToFloat(FloatToHalfBits(__fdiv_rn(x, s)));
    float r = rintf(q);
    if (r != r) {
        return 0;
    }
    r += static_cast<float>(offset);
    r = fminf(fmaxf(r, -128.0f), 127.0f);
    return static_cast<int8_t>(static_cast<int32_t>(r));
}

// The same result with the division replaced by a multiplication with y = RN(1 / s) and one correction step
// (q = x y; r = x - s q exactly, by fused multiply-add; q' = q + r y): q' is the correctly rounded x / s
// for finite non-zero s and 1 / s, because x and s carry at most 11 significant bits: q is within two
// units of the quotient, the correction leaves an error below 2^-47 of it, and a quotient of two such
// numbers that is not itself representable stays at least 2^-36 away from every rounding boundary.
// Scales that are 0, infinite or NaN (special = true) take the division.
__device__ __forceinline__ int8_t QuantOne16Fast(float x, float s, float y, float offset, bool special)
{
    float q;
    if (__builtin_expect(special, 0)) {
        q = __fdiv_rn(x, s);
    } else {
        const float q0 = __fmul_rn(x, y);
        const float r = __fmaf_rn(-s, q0, x);
        q = __fmaf_rn(r, y, q0);
        q = fabsf(q0) < INFINITY ? q : q0; // x infinite or NaN: the product already is the answer
    }
    float v = rintf(HalfBitsToFloat(FloatToHalfBits(q)));
    if (v != v) {
        return 0;
    }
    v = fminf(fmaxf(v + offset, -128.0f), 127.0f);
    return static_cast<int8_t>(static_cast<int32_t>(v));
}

__device__ __forceinline__ uint16_t DequantOne(int8_t x, float s, int32_t offset)
{
    // The product is exact in fp32 (9 bits times 11). Its zero must keep the product's sign (0 * -s = -0
    // in the golden): the compiler would otherwise merge the multiply and the conversion into one
    // fused multiply-add with +0, which turns -0 into +0, so the product is made opaque first.
    float p = static_cast<float>(static_cast<int32_t>(x) - offset) * s;
    asm volatile("" : "+v"(p));
    uint16_t h = FloatToHalfBits(p);
    if ((h & 0x7fffu) == 0x7c00u) { // overflowed to infinity: the golden clips to the largest finite value
        h = static_cast<uint16_t>((h & 0x8000u) | 0x7bffu);
    }
    return h;
}

template <int VEC, bool DEQUANT>
__global__ __launch_bounds__(256) void ElewisePerChannelKernel(const void *__restrict__ x,
                                                               const uint16_t *__restrict__ scale,
                                                               const int8_t *__restrict__ offset,
                                                               void *__restrict__ out, int64_t total,
                                                               int64_t channels, int32_t isBf16)
{
    const bool bf16 = isBf16 != 0;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x * VEC;
    // per-channel values of the thread's current 8 channels (VEC == 8): they are looked up again only when
    // the channels change, which with the launcher's grid they do not
    int64_t cached = -1;
    float sf[8], inv[8], offF[8];
    int8_t off[8];
    bool special = false;
    for (int64_t i = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * VEC; i < total; i += stride) {
        const int64_t c = i % channels;
        if constexpr (VEC == 8) {
          if (c != cached) {
            cached = c;
            uint32_t sw[4] = {0u, 0u, 0u, 0u};
            if (channels > 1) {
                const uint4 sv = *reinterpret_cast<const uint4 *>(scale + c);
                sw[0] = sv.x; sw[1] = sv.y; sw[2] = sv.z; sw[3] = sv.w;
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                off[e] = 0;
            }
            if (offset) {
                if (channels > 1) {
                    const uint2 ov = *reinterpret_cast<const uint2 *>(offset + c);
                    const uint32_t ow[2] = {ov.x, ov.y};
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        off[e] = static_cast<int8_t>(ow[e >> 2] >> (8 * (e & 3)));
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        off[e] = offset[0];
                    }
                }
            }
            special = false;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint16_t h = channels > 1 ? static_cast<uint16_t>(sw[e >> 1] >> (16 * (e & 1))) : scale[0];
                sf[e] = bf16 ? Bf16ToFloat(h) : HalfBitsToFloat(h);
                if constexpr (!DEQUANT) {
                    inv[e] = __fdiv_rn(1.0f, sf[e]);
                    offF[e] = static_cast<float>(off[e]);
                    special = special || !(fabsf(inv[e]) < INFINITY) || inv[e] == 0.0f;
                }
            }
          }
            if constexpr (DEQUANT) {
                const uint2 xv = *reinterpret_cast<const uint2 *>(static_cast<const int8_t *>(x) + i);
                const uint32_t xw[2] = {xv.x, xv.y};
                uint32_t o[4];
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    const uint32_t lo = DequantOne(static_cast<int8_t>(xw[e >> 2] >> (8 * (e & 3))), sf[e], off[e]);
                    const uint32_t hi = DequantOne(static_cast<int8_t>(xw[(e + 1) >> 2] >> (8 * ((e + 1) & 3))), sf[e + 1], off[e + 1]);
                    o[e >> 1] = lo | (hi << 16);
                }
                *reinterpret_cast<uint4 *>(static_cast<uint16_t *>(out) + i) = uint4{o[0], o[1], o[2], o[3]};
            } else {
                const uint4 xv = *reinterpret_cast<const uint4 *>(static_cast<const uint16_t *>(x) + i);
                const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
                uint32_t o[2] = {0u, 0u};
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const uint16_t h = static_cast<uint16_t>(xw[e >> 1] >> (16 * (e & 1)));
                    const float xf = bf16 ? Bf16ToFloat(h) : HalfBitsToFloat(h);
                    const uint32_t q = static_cast<uint8_t>(QuantOne16Fast(xf, sf[e], inv[e], offF[e], special));
                    o[e >> 2] |= q << (8 * (e & 3));
                }
                *reinterpret_cast<uint2 *>(static_cast<int8_t *>(out) + i) = uint2{o[0], o[1]};
            }
        } else {
            const float sf = Load16(scale, c, bf16);
            const int32_t off = offset ? offset[c] : 0;
            if constexpr (DEQUANT) {
                static_cast<uint16_t *>(out)[i] = DequantOne(static_cast<const int8_t *>(x)[i], sf, off);
            } else {
                static_cast<int8_t *>(out)[i] = QuantOne16(Load16(x, i, bf16), sf, off, bf16);
            }
        }
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

template <typename VecT>
static void LaunchNz(const NzRows &k, const NzRows &v, const int32_t *slots, int64_t numTokens, int64_t blockSize,
                     int64_t numSlots, hipStream_t s)
{
    dim3 grid(static_cast<unsigned>((numTokens + NZ_TOKENS - 1) / NZ_TOKENS), 2);
    ReshapeAndCacheNzKernel<VecT><<<grid, COPY_THREADS, 0, s>>>(k, v, slots, numTokens, blockSize, numSlots);
}

extern "C" int atbmi_reshape_and_cache_nz(const void *key, const void *value, void *keyCache, void *valueCache,
                                          const int32_t *slotMapping, int64_t numTokens, int64_t keyRowElems,
                                          int64_t valueRowElems, int64_t blockSize, int64_t numBlocks,
                                          int32_t keyElemBytes, int32_t valueElemBytes, void *stream)
{
    if (!key || !value || !keyCache || !valueCache || !slotMapping) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache_nz: key, value, the caches and slotMapping must be non-null");
    }
    if ((keyElemBytes != 1 && keyElemBytes != 2) || (valueElemBytes != 1 && valueElemBytes != 2)) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache_nz: element sizes must be 1 or 2, got %d and %d", keyElemBytes,
                    valueElemBytes);
    }
    // a piece is 32 int8 or 16 two-byte elements of a key row, 16 elements of a value row
    const int64_t keyLast = keyElemBytes == 1 ? 32 : 16;
    const int64_t valueLast = 16;
    if (numTokens < 0 || keyRowElems <= 0 || valueRowElems <= 0 || blockSize <= 0 || numBlocks <= 0 ||
        keyRowElems % keyLast != 0 || valueRowElems % valueLast != 0) {
        return Fail(ERR_INVALID_PARAM,
                    "reshape_and_cache_nz: bad extents (key row %lld must be a multiple of %lld, value row %lld of 16)",
                    static_cast<long long>(keyRowElems), static_cast<long long>(keyLast),
                    static_cast<long long>(valueRowElems));
    }
    if (numTokens == 0) {
        return OK;
    }
    if (numTokens > 0x7fffffffLL) {
        return Fail(ERR_INVALID_PARAM, "reshape_and_cache_nz: too many tokens");
    }
    const NzRows k{static_cast<const uint8_t *>(key), static_cast<uint8_t *>(keyCache), keyRowElems * keyElemBytes,
                   keyLast * keyElemBytes};
    const NzRows v{static_cast<const uint8_t *>(value), static_cast<uint8_t *>(valueCache),
                   valueRowElems * valueElemBytes, valueLast * valueElemBytes};
    // pieces are 32 or 16 bytes, so the widest access is set by the base addresses
    uintptr_t align = 16;
    while (align > 1 && !(k.pieceBytes % align == 0 && v.pieceBytes % align == 0 && Aligned(key, align) &&
                          Aligned(value, align) && Aligned(keyCache, align) && Aligned(valueCache, align))) {
        align >>= 1;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t numSlots = numBlocks * blockSize;
    switch (align) {
        case 16: LaunchNz<NzVec16>(k, v, slotMapping, numTokens, blockSize, numSlots, s); break;
        case 8: LaunchNz<NzVec8>(k, v, slotMapping, numTokens, blockSize, numSlots, s); break;
        case 4: LaunchNz<uint32_t>(k, v, slotMapping, numTokens, blockSize, numSlots, s); break;
        case 2: LaunchNz<uint16_t>(k, v, slotMapping, numTokens, blockSize, numSlots, s); break;
        default: LaunchNz<uint8_t>(k, v, slotMapping, numTokens, blockSize, numSlots, s); break;
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

extern "C" int atbmi_norm_rope_reshape_and_cache(const void *x, const void *gamma, const void *keyRope,
                                                 const void *cosTable, const void *sinTable,
                                                 const int32_t *slotMapping, void *keyCache, int64_t numTokens,
                                                 int64_t normDim, int64_t ropeDim, int64_t numSlots, int32_t dtype,
                                                 float epsilon, void *stream)
{
    if (!x || !gamma || !keyRope || !cosTable || !sinTable || !slotMapping || !keyCache) {
        return Fail(ERR_INVALID_PARAM, "norm_rope_reshape_and_cache: every tensor must be non-null");
    }
    if (dtype != ATBMI_F16 && dtype != ATBMI_BF16) {
        return Fail(ERR_INVALID_PARAM, "norm_rope_reshape_and_cache: tensors must be fp16 or bf16");
    }
    if (numTokens < 0 || numTokens > 0x7fffffffLL || normDim <= 0 || ropeDim <= 0 || numSlots <= 0 ||
        normDim > (1 << 20) || ropeDim > (1 << 20)) {
        return Fail(ERR_INVALID_PARAM, "norm_rope_reshape_and_cache: bad extents");
    }
    if (normDim % 8 != 0 || ropeDim % 2 != 0) {
        return Fail(ERR_INVALID_PARAM, "norm_rope_reshape_and_cache: normDim must be a multiple of 8 and ropeDim even, "
                                       "got %lld and %lld", (long long)normDim, (long long)ropeDim);
    }
    if (!Aligned(x, 16) || !Aligned(gamma, 16) || !Aligned(keyCache, 16) || (ropeDim * 2) % 16 != 0) {
        return Fail(ERR_INVALID_PARAM, "norm_rope_reshape_and_cache: x, gamma and keyCache must be 16-byte aligned and "
                                       "a rotary row a multiple of 16 bytes");
    }
    if (numTokens == 0) {
        return OK;
    }
    // one wave per token up to 262 144 tokens (more waves in flight hide more of each row's load latency
    // than longer-lived waves do); beyond that the waves loop over the tokens
    const unsigned grid = static_cast<unsigned>(std::min<int64_t>((numTokens + NORM_ROPE_WAVES - 1) / NORM_ROPE_WAVES, 65536));
    // the register-resident form: one 16-byte piece of the latent row and one rotary pair per lane
    const bool fast = normDim <= WAVE * 8 && ropeDim <= WAVE * 2;
    const bool bf16 = dtype == ATBMI_BF16;
    auto kernel = fast ? (bf16 ? NormRopeCacheKernel<true, true> : NormRopeCacheKernel<true, false>)
                       : (bf16 ? NormRopeCacheKernel<false, true> : NormRopeCacheKernel<false, false>);
    kernel<<<grid, NORM_ROPE_WAVES * WAVE, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const uint16_t *>(x), static_cast<const uint16_t *>(gamma), static_cast<const uint16_t *>(keyRope),
        static_cast<const uint16_t *>(cosTable), static_cast<const uint16_t *>(sinTable), slotMapping,
        static_cast<uint16_t *>(keyCache), numTokens, static_cast<int32_t>(normDim), static_cast<int32_t>(ropeDim),
        numSlots, epsilon);
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}

namespace {
template <bool DEQUANT>
int LaunchElewisePerChannel(const char *what, const void *x, const void *scale, const int8_t *offset, void *out,
                            int64_t total, int64_t channels, int32_t dtype, void *stream)
{
    if (!x || !scale || !out) {
        return Fail(ERR_INVALID_PARAM, "%s: x, scale and out must be non-null", what);
    }
    if (dtype != ATBMI_F16 && !(dtype == ATBMI_BF16 && !DEQUANT)) {
        return Fail(ERR_INVALID_PARAM, "%s: unsupported element type %d", what, dtype);
    }
    if (total < 0 || channels <= 0 || (total % channels) != 0) {
        return Fail(ERR_INVALID_PARAM, "%s: %lld elements do not divide into rows of %lld scale entries", what,
                    (long long)total, (long long)channels);
    }
    if (total == 0) {
        return OK;
    }
    const bool wide = total % 8 == 0 && (channels == 1 || channels % 8 == 0) && Aligned(x, 16) && Aligned(out, 16) &&
                      Aligned(scale, 16) && (!offset || Aligned(offset, 8));
    const int64_t items = wide ? total / 8 : total;
    int64_t blocks = std::min<int64_t>((items + 255) / 256, 1 << 20);
    if (wide && channels > 1) {
        // A thread keeps its 8 channels while it walks the rows if the launch's stride (blocks * 2048 elements)
        // is a multiple of the channel count: round the grid to the next multiple that makes it one, unless
        // that would leave most of it idle.
        int64_t a = channels, b = 2048;
        while (b != 0) {
            const int64_t t = a % b;
            a = b;
            b = t;
        }
        const int64_t unit = channels / a; // blocks must be a multiple of this
        if (unit <= blocks) {
            blocks = blocks / unit * unit;
            blocks = std::min<int64_t>(blocks, std::max<int64_t>(unit, 2048 / unit * unit));
        }
    }
    const unsigned grid = static_cast<unsigned>(blocks);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (wide) {
        ElewisePerChannelKernel<8, DEQUANT><<<grid, 256, 0, s>>>(x, static_cast<const uint16_t *>(scale), offset, out, total,
                                                                 channels, dtype == ATBMI_BF16);
    } else {
        ElewisePerChannelKernel<1, DEQUANT><<<grid, 256, 0, s>>>(x, static_cast<const uint16_t *>(scale), offset, out, total,
                                                                 channels, dtype == ATBMI_BF16);
    }
    ATBMI_HIP_CHECK(hipGetLastError());
    return OK;
}
} // namespace

extern "C" int atbmi_elewise_quant_per_channel(const void *x, const void *scale, const int8_t *offset, int8_t *out,
                                               int64_t total, int64_t channels, int32_t dtype, void *stream)
{
    return LaunchElewisePerChannel<false>("elewise_quant_per_channel", x, scale, offset, out, total, channels, dtype, stream);
}

extern "C" int atbmi_elewise_dequant_per_channel(const int8_t *x, const void *scale, const int8_t *offset, void *out,
                                                 int64_t total, int64_t channels, void *stream)
{
    return LaunchElewisePerChannel<true>("elewise_dequant_per_channel", x, scale, offset, out, total, channels, ATBMI_F16,
                                         stream);
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
