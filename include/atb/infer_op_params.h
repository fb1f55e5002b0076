// Parameter structs of the two inference operators this library implements:
// ReshapeAndCache (KV-cache write) and PagedAttention (decode attention over
// a block-table-addressed KV cache). Field order, enumerator values and sizes
// follow the reference so that a param filled by existing code is read the
// same way (reference include/atb/infer_op_params.h:39-42, :488-526,
// :1859-1963; sizes pinned by tests/unittest/ops/test_op_param_size.cpp:47,51).
#ifndef ATB_INFER_OP_PARAMS_H
#define ATB_INFER_OP_PARAMS_H
#include <cstdint>
#include <acl/acl.h>
#include "atb/svector.h"

namespace atb {
namespace infer {

enum InputLayout : int {
    TYPE_BSND = 0, // [tokens, heads, head_dim] queries, [blocks, block, heads, dim] caches
    TYPE_BNSD      // head-major caches [numBlocks, kvHeads, blockSize, headSize]
};

// Writes one K row and one V row per token into the paged caches at the
// slot the slot mapping names; negative slots are skipped.
struct ReshapeAndCacheParam {
    enum CompressType : int {
        COMPRESS_TYPE_UNDEFINED = 0,
        COMPRESS_TYPE_KVHEAD,     // head compression (alibi): inputs + wins, seqLens
        COMPRESS_TYPE_KVHEAD_ROPE // head compression (rope): inputs + wins, seqLens, offsetIndex
    };
    enum KvCacheCfg : int {
        K_CACHE_V_CACHE = 0, // inputs: key, value, keyCache, valueCache, slotMapping
        K_CACHE_V_BYPASS,    // inputs: key, keyCache, slotMapping (single cache, e.g. MLA latent)
        K_CACHE_V_CACHE_NZ   // fractal-NZ caches [blocks, heads*headSize/L, blockSize, L], L = 32 (int8 key) or 16
    };

    CompressType compressType = COMPRESS_TYPE_UNDEFINED;
    KvCacheCfg kvCacheCfg = K_CACHE_V_CACHE;
    uint8_t rsv[16] = {0}; // must stay zero
};

// ReshapeAndCache whose key / value inputs are strided views: two (or one) more pairs of host
// int64 inputs give the element strides [3] and the element offset [1] of each
// (reference include/atb/infer_op_params.h:531-568).
struct ReshapeAndCacheWithStrideParam {
    enum CompressType : int {
        COMPRESS_TYPE_UNDEFINED = 0,
        COMPRESS_TYPE_KVHEAD,     // rejected at creation with strided inputs
        COMPRESS_TYPE_KVHEAD_ROPE // rejected at creation with strided inputs
    };
    enum KvCacheCfg : int {
        K_CACHE_V_CACHE = 0, // inputs: key, value, keyCache, valueCache, slotMapping, kStrides, vStrides, kOffset, vOffset
        K_CACHE_V_BYPASS,    // inputs: key, keyCache, slotMapping, kStrides, kOffset
    };

    CompressType compressType = COMPRESS_TYPE_UNDEFINED;
    KvCacheCfg kvCacheCfg = K_CACHE_V_CACHE;
    uint8_t rsv[16] = {0}; // must stay zero
};

// ReshapeAndCache for caches compressed by dropping a window of tokens per (sequence, head) pair:
// inputs key, value [tokens, heads, headSize], keyCache, valueCache [blocks, blockSize, 1, headSize],
// slotMapping, wins [batch * heads], seqLen [batch], offsetIndex [batch * heads]; outputs the caches
// (reference include/atb/infer_op_params.h:2883-2894).
struct ReshapeAndCacheOmniParam {
    uint8_t rsv[8] = {0}; // must stay zero
};

// Decode attention: one query token per sequence against that sequence's
// cached keys/values, found through blockTables and bounded by contextLens.
struct PagedAttentionParam {
    int32_t headNum = 0;   // query heads, > 0
    float qkScale = 1.0;   // multiplies Q.K^T before the softmax
    int32_t kvHeadNum = 0; // KV heads; 0 means "same as headNum"

    enum MaskType : int {
        UNDEFINED = 0, // no mask input
        MASK_TYPE_NORM,
        MASK_TYPE_ALIBI,
        MASK_TYPE_SPEC,
        MASK_TYPE_MASK_FREE,    // Atlas 300I Duo only: InferShape / Setup return ERROR_INVALID_TENSOR_DIM elsewhere
        MASK_TYPE_NORM_COMPRESS // Atlas 300I Duo only: refused at creation elsewhere
    };
    MaskType maskType = UNDEFINED;

    bool batchRunStatusEnable = false;

    enum QuantType : int {
        TYPE_QUANT_UNDEFINED = 0,
        TYPE_QUANT_UNQUANT = 0,     // fp16/bf16 query and caches
        TYPE_DEQUANT_FUSION = 1,    // fp16/bf16 query, int8 caches + per-channel descale (and offset)
        TYPE_QUANT_QKV_OFFLINE = 2, // int8 query and caches
        TYPE_QUANT_QKV_ONLINE = 3
    };
    QuantType quantType = TYPE_QUANT_UNQUANT;

    aclDataType outDataType = ACL_DT_UNDEFINED; // only read by the QKV-quant modes

    bool hasQuantOffset = false; // dequant fusion: kOffset / vOffset inputs present

    enum CompressType : int {
        COMPRESS_TYPE_UNDEFINED = 0,
        COMPRESS_TYPE_KVHEAD,
        COMPRESS_TYPE_KVHEAD_ROPE,
        COMPRESS_TYPE_MAX
    };
    CompressType compressType = COMPRESS_TYPE_UNDEFINED;

    enum CalcType : int {
        CALC_TYPE_UNDEFINED = 0,
        CALC_TYPE_SPEC // several query tokens per sequence (speculative decode)
    };
    CalcType calcType = CALC_TYPE_UNDEFINED;

    enum ScaleType : int {
        SCALE_TYPE_TOR = 0,
        SCALE_TYPE_LOGN,
        SCALE_TYPE_MAX
    };
    ScaleType scaleType = SCALE_TYPE_TOR;

    InputLayout inputLayout = TYPE_BSND;

    // > 0: the key cache is a combined MLA latent cache and V is its first
    // mlaVHeadSize channels; no valueCache input. Range [0, 576].
    uint32_t mlaVHeadSize = 0;

    float qScale = 0; // pre-multiplies Q; ignored when 0 or 1

    uint8_t rsv[64] = {0}; // must stay zero
};

// Decode attention over the compressed latent cache of multi-head latent
// attention, with the query and the cache rows given as 512 latent channels
// plus 64 rotary channels in two tensors each; V is the 512 latent channels.
// (reference include/atb/infer_op_params.h:2899-2984)
struct MultiLatentAttentionParam {
    int32_t headNum = 0;   // query heads: 8, 16, 32, 64 or 128
    float qkScale = 1.0;   // multiplies Q.K^T before the softmax, in (0, 1]
    int32_t kvHeadNum = 0; // 1

    enum MaskType : int {
        UNDEFINED = 0,         // no mask input
        MASK_TYPE_SPEC,        // one mask row per query token, with CALC_TYPE_SPEC
        MASK_TYPE_MASK_FREE,   // compressed causal mask: a [125 + 2 q, 128] template (decode), [512, 512] (prefill)
        MASK_TYPE_CAUSAL_MASK, // causal, no mask tensor
        MASK_TYPE_SWA_NORM     // sliding window of windowSize tokens (prefill only)
    };
    MaskType maskType = UNDEFINED;

    enum CalcType : int {
        CALC_TYPE_UNDEFINED = 0, // one query token per sequence
        CALC_TYPE_SPEC,          // qSeqlen input: several query tokens per sequence
        CALC_TYPE_RING,          // second output: the log-sum-exp of every row
        CALC_TYPE_SPEC_AND_RING, // both
        CALC_TYPE_PREFILL        // prompt attention over key / value tensors instead of the caches
    };
    CalcType calcType = CALC_TYPE_UNDEFINED;

    enum CacheMode : uint8_t {
        KVCACHE = 0,  // one 576-channel cache; rejected by the reference itself
        KROPE_CTKV,   // latent cache [blocks, 128, 1, 512] + rotary cache [blocks, 128, 1, 64]
        INT8_NZCACHE, // int8 latent cache [blocks, 16, 128, 32] + 16-bit rotary cache, fractal-NZ; int8 query
        NZCACHE       // the 16-bit caches in fractal-NZ: [blocks, 32, 128, 16] + [blocks, 4, 128, 16]
    };
    CacheMode cacheMode = KVCACHE;

    uint32_t windowSize = 0;

    enum MaskUseStatusType : int {
        MASK_USE_STATUS_TYPE_UNDEFINED = 0,
        MASK_USE_STATUS_TYPE_BATCH_MASK, // input maskUseStatus [batch]: 0 lets a sequence's query tokens see its whole context
        MASK_USE_STATUS_TYPE_MAX
    };
    MaskUseStatusType maskUseStatusType = MASK_USE_STATUS_TYPE_UNDEFINED;

    uint8_t rsv[32] = {0}; // must stay zero
};

// Elementwise operations (reference include/atb/infer_op_params.h:354-421). Built here: the two
// per-channel forms that sit beside the int8 KV cache, ELEWISE_QUANT_PER_CHANNEL (x, scale, offset ->
// int8) and ELEWISE_DEQUANT_PER_CHANNEL (int8 x, scale, offset -> fp16); the other types are
// rejected when the operation is created.
struct ElewiseParam {
    enum ElewiseType : int {
        ELEWISE_UNDEFINED = 0,
        ELEWISE_CAST,
        ELEWISE_MULS,
        ELEWISE_COS,
        ELEWISE_SIN,
        ELEWISE_NEG,
        ELEWISE_QUANT,
        ELEWISE_LOGICAL_NOT,
        ELEWISE_ADD,
        ELEWISE_MUL,
        ELEWISE_REALDIV,
        ELEWISE_LOGICAL_AND,
        ELEWISE_LOGICAL_OR,
        ELEWISE_LESS,
        ELEWISE_GREATER,
        ELEWISE_SUB,
        ELEWISE_EQUAL,
        ELEWISE_QUANT_PER_CHANNEL,
        ELEWISE_DEQUANT_PER_CHANNEL,
        ELEWISE_DYNAMIC_QUANT,
        ELEWISE_TANH,
        ELEWISE_TYPE_MAX
    };
    struct QuantParam {
        float inputScale = 1.0f;
        bool asymmetric = false;
        int inputOffset = 0;
        uint8_t rsv[20] = {0}; // must stay zero
    };
    struct MulsParam {
        float varAttr = 0.0f;
        uint8_t rsv[12] = {0}; // must stay zero
    };
    ElewiseType elewiseType = ELEWISE_UNDEFINED;
    QuantParam quantParam;
    MulsParam mulsParam;
    aclDataType outTensorType = ACL_DT_UNDEFINED;
    uint8_t rsv[8] = {0}; // must stay zero
};

// Rotary position embedding of query and key rows (reference include/atb/infer_op_params.h:1605-1617).
struct RopeParam {
    int32_t rotaryCoeff = 4; // 2: rotate halves; 4: the two halves of a head separately; headDim: interleaved pairs
    int32_t cosFormat = 0;   // 0: cos / sin hold a row per token; 1: a row per position of a sequence
    uint8_t rsv[8] = {0};    // must stay zero
};

// RMSNorm of the latent row, rotary embedding of the rotary row and the write of both, side by side,
// into a single cache: the step that fills the combined MLA cache
// (reference include/atb/infer_op_params.h:2697-2716).
struct NormRopeReshapeParam {
    uint32_t precisionMode = 0; // passed through to the kernel by the reference; the arithmetic here is fp32 always
    uint32_t rotaryCoeff = 2;   // 2: rotate halves (the only form the reference's goldens define)
    float epsilon = 1e-5;       // added to the mean square; |epsilon| must not be below FLT_MIN
    uint8_t rsv[16] = {0};      // must stay zero
};

// Copies whole blocks of the key and value caches onto other blocks of the same caches
// (reference include/atb/infer_op_params.h:1208-1217).
struct BlockCopyParam {
    uint8_t rsv[16] = {0}; // must stay zero
};

// Gathers the cached rows of every sequence into contiguous key / value tensors, the
// reverse of ReshapeAndCache (reference include/atb/infer_op_params.h:3070-3101).
struct PagedCacheLoadParam {
    enum KvCacheCfg : int8_t {
        K_CACHE_V_CACHE_NZ = 0, // fractal-NZ caches [blocks, heads*headSize/L, blockSize, L], L = 32 (int8) or 16
        K_CACHE_V_CACHE_ND      // caches [blocks, blockSize, heads, headSize]
    };
    KvCacheCfg kvCacheCfg = K_CACHE_V_CACHE_NZ;
    bool isSeqLensCumsumMode = false; // seqLens holds running sums [batch + 1] instead of lengths [batch]
    bool hasSeqStarts = false;        // seqStarts gives the first cached position of every sequence
    uint8_t rsv[61] = {0};            // must stay zero
};

static_assert(sizeof(ReshapeAndCacheParam) == 24, "ReshapeAndCacheParam ABI size");
static_assert(sizeof(ReshapeAndCacheWithStrideParam) == 24, "ReshapeAndCacheWithStrideParam ABI size");
static_assert(sizeof(ReshapeAndCacheOmniParam) == 8, "ReshapeAndCacheOmniParam ABI size");
static_assert(sizeof(ElewiseParam) == 64 && sizeof(ElewiseParam::QuantParam) == 32 && sizeof(ElewiseParam::MulsParam) == 16,
              "ElewiseParam ABI size");
static_assert(sizeof(RopeParam) == 16, "RopeParam ABI size");
static_assert(sizeof(NormRopeReshapeParam) == 28, "NormRopeReshapeParam ABI size");
static_assert(sizeof(BlockCopyParam) == 16, "BlockCopyParam ABI size");
static_assert(sizeof(PagedCacheLoadParam) == 64, "PagedCacheLoadParam ABI size");
static_assert(sizeof(MultiLatentAttentionParam) == 64, "MultiLatentAttentionParam ABI size");
static_assert(sizeof(PagedAttentionParam) == 120, "PagedAttentionParam ABI size");

} // namespace infer
} // namespace atb
#endif
