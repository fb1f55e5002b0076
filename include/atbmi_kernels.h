/*
 * atbmi_kernels.h - C ABI of the MI355X (gfx950) kernel layer under the ATB
 * PagedAttention / ReshapeAndCache operators.
 *
 * This is the boundary the C++ operator layer (atb::Operation) calls, and the
 * one a foreign-language binding would bind: plain pointers, sizes and POD
 * structs, no C++ types, no exceptions. Every pointer named "device" is an HBM
 * address; "host" pointers are ordinary CPU memory. `stream` is a hipStream_t
 * passed as void* (NULL = the default stream). All launches are asynchronous.
 *
 * Return value: 0 on success, otherwise an atb::ErrorType value
 * (1 = invalid parameter, 4 = HIP runtime failure, 26 = out of device memory,
 * 27 = out of host memory). atbmi_last_error() gives a readable reason.
 *
 * In the reference these entry points correspond to the device side of the
 * MKI kernels that the ATB runners launch:
 *   reshape_and_cache  -> src/kernels/mixkernels/reshape_and_cache/op_kernel/reshape_and_cache_nd.cpp:146-192
 *   quant_per_channel  -> ElewiseOperation ELEWISE_QUANT_PER_CHANNEL (include/atb/infer_op_params.h:378)
 *   pa_plan_*          -> PagedAttentionTiling (src/kernels/mixkernels/pagedattention/tiling/paged_attention_tiling.cpp:419-470)
 *   pa_decode          -> paged_attention_mask (src/kernels/mixkernels/pagedattention/op_kernel/paged_attention_mask_mix.cce:24-163)
 *                         and the MLA combined-cache kernel (op_kernel/paged_MLAttention_combine_cache_mask_mix.cce)
 */
#ifndef ATBMI_KERNELS_H
#define ATBMI_KERNELS_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types of tensors crossing this boundary. */
typedef enum AtbmiDtype {
    ATBMI_F16 = 0,
    ATBMI_BF16 = 1,
    ATBMI_INT8 = 2
} AtbmiDtype;

/* Which attention kernel a plan uses. AUTO picks the MFMA kernel when the
 * shape is one it is built for and the scalar kernel otherwise. */
typedef enum AtbmiPaKernel {
    ATBMI_PA_KERNEL_AUTO = 0,
    ATBMI_PA_KERNEL_SCALAR = 1,
    ATBMI_PA_KERNEL_MFMA = 2
} AtbmiPaKernel;

/* Readable reason for the last non-zero return on the calling thread. */
const char *atbmi_last_error(void);

/* Number of HIP devices visible, or a negative value when the HIP runtime
 * cannot be initialised. Makes no allocation. */
int atbmi_device_count(void);

/*
 * KV-cache write. For each token i in [0, numTokens): s = slotMapping[i];
 * s < 0 (or s >= numSlots) skips the token, otherwise the numKvHeads*headDimK
 * elements of key[i] are copied to keyCache viewed as [numSlots, numKvHeads*headDimK]
 * at row s, and the same for value/valueCache with headDimV. A byte copy:
 * elemBytes (1 or 2) is all that matters about the dtype. value and valueCache
 * may both be NULL (single-cache form).
 * Replaces: reshape_and_cache_nd.cpp:90-124 (ProcessKVUnequal et al.).
 */
int atbmi_reshape_and_cache(const void *keyDevice, const void *valueDevice, void *keyCacheDevice,
                            void *valueCacheDevice, const int32_t *slotMappingDevice, int64_t numTokens,
                            int64_t numKvHeads, int64_t headDimK, int64_t headDimV, int64_t numSlots,
                            int32_t elemBytes, void *stream);

/*
 * KV-cache write under head compression (ReshapeAndCacheParam::compressType): the caches hold one head per
 * slot, [numSlots, headSize], and pair i = b * numHeads + h (sequence b of `batch`, head h) owns the slots from
 * slotMapping[i] on (slotMapping[i] < 0 skips the pair). Sequence b is the seqLens[b] rows of key / value
 * [numTokens, numHeads, headSize] after those of the sequences before it. All index tensors are device memory.
 *   offsetIndex == NULL (COMPRESS_TYPE_KVHEAD): the last wins[i] tokens of the sequence, head h, in order.
 *   offsetIndex != NULL (COMPRESS_TYPE_KVHEAD_ROPE), o = offsetIndex[i]: o == -1 copies the whole sequence;
 *     otherwise the tokens before o, then ONE slot with the mean of the wins[i] tokens from o on (fp32 sum in
 *     token order, divided by wins[i], rounded to nearest even), then the tokens after the window; wins[i] == 0
 *     copies everything. fp16 / bf16 only.
 * Rows that would be read outside key / value or written outside the caches are left out.
 * Replaces: reshape_and_cache_compress.cpp / reshape_and_cache_compress_rope.cpp of the reference
 * (src/kernels/mixkernels/reshape_and_cache/op_kernel/; goldens tests/apitest/kernelstest/mix/
 * test_reshape_and_cache_wins.py:61-88 and test_reshape_and_cache_wins_rope.py:78-131).
 */
int atbmi_reshape_and_cache_compress(const void *keyDevice, const void *valueDevice, void *keyCacheDevice,
                                     void *valueCacheDevice, const int32_t *slotMappingDevice,
                                     const int32_t *winsDevice, const int32_t *seqLensDevice,
                                     const int32_t *offsetIndexDevice, int64_t batch, int64_t numHeads,
                                     int64_t headSize, int64_t numTokens, int64_t numSlots, int32_t dtype,
                                     void *stream);

/*
 * KV-cache write of ReshapeAndCacheOmniOperation: the arguments and the layout of atbmi_reshape_and_cache_compress,
 * offsetIndex required, and a window that leaves nothing behind. With o = offsetIndex[i] and w = wins[i], pair i
 * writes the tokens [0, o) of its sequence and then at once the tokens [o + w, seqLens[b]) to consecutive slots from
 * slotMapping[i] on; o == -1, w <= 0 or o >= seqLens[b] copies the whole sequence; a window that runs past the end
 * of the sequence leaves only the tokens before it. A byte copy (fp16 / bf16 rows in the reference, one-byte rows
 * work too).
 * Replaces: reshape_and_cache_omni_compress.cpp:87-110 of the reference (src/kernels/mixkernels/reshape_and_cache/
 * op_kernel/, parameters read as reshape_and_cache_base.h:276-289 does; goldens
 * tests/framework/python/CsvOpsTestTool/data_generation.py:9797-9846 and
 * tests/apitest/kernelstest/mix/test_reshape_and_cache_omni_compress.py:80-116).
 */
int atbmi_reshape_and_cache_omni(const void *keyDevice, const void *valueDevice, void *keyCacheDevice,
                                 void *valueCacheDevice, const int32_t *slotMappingDevice,
                                 const int32_t *winsDevice, const int32_t *seqLensDevice,
                                 const int32_t *offsetIndexDevice, int64_t batch, int64_t numHeads, int64_t headSize,
                                 int64_t numTokens, int64_t numSlots, int32_t dtype, void *stream);

/*
 * KV-cache write into fractal-NZ caches (ReshapeAndCacheParam::K_CACHE_V_CACHE_NZ), the writer of the caches
 * MultiLatentAttention reads with cacheMode NZCACHE / INT8_NZCACHE. keyCache is
 * [numBlocks, keyRowElems / L, blockSize, L] with L = 32 for one-byte and 16 for two-byte keys, valueCache
 * [numBlocks, valueRowElems / 16, blockSize, 16]: element c of token i's key row (numKvHeads * headDimK elements)
 * goes to block s / blockSize, piece c / L, row s % blockSize, place c % L, s = slotMapping[i]; s < 0 (or
 * s >= numBlocks * blockSize) skips the token. Key and value may differ in element size (int8 latent rows with
 * 16-bit rotary rows). A byte copy.
 * Replaces: reshape_and_cache_nz.cpp:85-178 of the reference (src/kernels/mixkernels/reshape_and_cache/op_kernel/;
 * golden tests/apitest/kernelstest/mix/test_reshape_and_cache_nz.py:45-66).
 */
int atbmi_reshape_and_cache_nz(const void *keyDevice, const void *valueDevice, void *keyCacheDevice,
                               void *valueCacheDevice, const int32_t *slotMappingDevice, int64_t numTokens,
                               int64_t keyRowElems, int64_t valueRowElems, int64_t blockSize, int64_t numBlocks,
                               int32_t keyElemBytes, int32_t valueElemBytes, void *stream);

/*
 * KV-cache write from strided views of key / value: element (token, head, channel) of key is read
 * keyOffset + token * keyStrides[0] + head * keyStrides[1] + channel * keyStrides[2] ELEMENTS from
 * keyDevice (the same for value); everything else as atbmi_reshape_and_cache. The stride arrays are
 * host memory and are read before the call returns.
 * Replaces: ReshapeAndCacheWithStrideOperation's kernel launch, which sets strides and offset on the
 * key / value tensors of the ReshapeAndCache kernel (reference src/ops/ops_infer/
 * reshape_and_cache_with_stride/reshape_and_cache_with_stride_ops_runner.cpp:78-104; golden
 * tests/unittest/ops/reshape_and_cache_with_stride/test_reshape_and_cache_with_stride.cpp:219-245).
 */
int atbmi_reshape_and_cache_strided(const void *keyDevice, const void *valueDevice, void *keyCacheDevice,
                                    void *valueCacheDevice, const int32_t *slotMappingDevice, int64_t numTokens,
                                    int64_t numKvHeads, int64_t headDimK, int64_t headDimV, int64_t numSlots,
                                    int32_t elemBytes, const int64_t *keyStridesHost, int64_t keyOffset,
                                    const int64_t *valueStridesHost, int64_t valueOffset, void *stream);

/*
 * RMSNorm + rotary embedding + cache write in one kernel, the producer of the combined (MLA) cache:
 * for token i with slot s = slotMapping[i] in [0, numSlots),
 *   keyCache[s][0 : normDim]            = gamma * x[i] / sqrt(mean(x[i]^2) + epsilon)
 *   keyCache[s][normDim : normDim+ropeDim] = r * cos[i] + rotate_half(r) * sin[i],  r = keyRope[i],
 *   rotate_half(r) = concat(-r[ropeDim/2:], r[:ropeDim/2]),
 * computed in fp32 and rounded once to dtype (fp16 or bf16, the type of every tensor). keyCache is
 * viewed as [numSlots, normDim + ropeDim]; other slots keep their content.
 * Replaces: the RmsNormAndRopeAndReshapeAndCache kernel behind NormRopeReshapeOperation (reference
 * src/kernels/mixkernels/rms_norm_and_rope_and_reshape_and_cache/op_kernel/
 * rms_norm_and_rope_and_reshape_and_cache.cpp:160-305; golden tests/apitest/opstest/python/operations/
 * norm_rope_reshape/test_norm_rope_reshape.py:21-71).
 */
int atbmi_norm_rope_reshape_and_cache(const void *xDevice, const void *gammaDevice, const void *keyRopeDevice,
                                      const void *cosDevice, const void *sinDevice, const int32_t *slotMappingDevice,
                                      void *keyCacheDevice, int64_t numTokens, int64_t normDim, int64_t ropeDim,
                                      int64_t numSlots, int32_t dtype, float epsilon, void *stream);

/*
 * Rotary position embedding of query and key rows (q [numTokens, hiddenQ], k [numTokens, hiddenK],
 * fp16 or bf16). The cos / sin tables have rows of headDim entries (the type of q, or fp32 with
 * fp16 rows when tableIsFloat); a row of q or k is cut into units of headDim channels, a unit into
 * rotaryCoeff / 2 chunks of 2 * stride channels (stride = headDim / rotaryCoeff), and in a chunk
 *   out[i]          = x[i] * cos[i'] - x[i + stride] * sin[i']
 *   out[i + stride] = x[i + stride] * cos[i' + stride] + x[i] * sin[i' + stride]     (i' = i's offset in its unit)
 * in fp32, rounded once. cosFormat 0: table row r belongs to token r. cosFormat 1: to position r of
 * every sequence; seqLens (int32 [batch], device) then gives the tokens their positions; tokens past
 * the last sequence, or with a row outside the table, are left alone. qOut / kOut may be q / k.
 * Replaces: the Rope kernel behind RopeOperation (reference src/ops/ops_infer/rope/rope_ops_runner.cpp:43-72;
 * golden tests/apitest/opstest/python/operations/rope/test_rope_operation2.py:120-218, cosFormat 1
 * test_rope_operation3.py:29-55).
 */
int atbmi_rope(const void *qDevice, const void *kDevice, const void *cosDevice, const void *sinDevice,
               const int32_t *seqLensDevice, void *qOutDevice, void *kOutDevice, int64_t numTokens, int64_t hiddenQ,
               int64_t hiddenK, int64_t headDim, int64_t tableRows, int64_t batch, int32_t rotaryCoeff,
               int32_t cosFormat, int32_t dtype, int32_t tableIsFloat, void *stream);

/*
 * ElewiseOperation's per-channel quantiser and dequantiser. x holds `total` elements, scale (the
 * type of x for the quantiser, fp16 for the dequantiser) and offset (int8, may be NULL) hold
 * `channels` entries each; element i uses entry i % channels (the scale covers the trailing
 * dimensions of x, or is a single value).
 *   quantiser:   out = clamp(rint(fp16(x / scale)) + offset, -128, 127) as int8: the quotient is
 *                rounded to fp16 first (the reference golden divides in fp16, bf16 inputs included);
 *                ties to even, NaN -> 0
 *   dequantiser: out = fp16((x - offset) * scale), saturated at +-65504
 * Replaces: the ELEWISE_QUANT_PER_CHANNEL / ELEWISE_DEQUANT_PER_CHANNEL kernels behind ElewiseOperation
 * (reference src/ops/ops_infer/elewise/elewise_operation.cpp:451-472; goldens tests/apitest/opstest/
 * python/operations/elewise/test_elewise_quant.py:24-32, test_elewise_dequant.py:23-31).
 */
int atbmi_elewise_quant_per_channel(const void *xDevice, const void *scaleDevice, const int8_t *offsetDevice,
                                    int8_t *outDevice, int64_t total, int64_t channels, int32_t dtype, void *stream);
int atbmi_elewise_dequant_per_channel(const int8_t *xDevice, const void *scaleDevice, const int8_t *offsetDevice,
                                      void *outDevice, int64_t total, int64_t channels, void *stream);

/*
 * Per-channel int8 quantiser: out[r][c] = clamp(rint(float(x[r][c]) / scale[c]) + offset[c], -128, 127),
 * IEEE fp32 divide, round-half-even, NaN -> 0. offset may be NULL.
 * Replaces: the ELEWISE_QUANT_PER_CHANNEL kernel (golden
 * tests/apitest/opstest/python/operations/elewise/test_elewise_quant.py:24-32).
 */
int atbmi_quant_per_channel(const void *xDevice, int32_t xDtype, const float *scaleDevice,
                            const int32_t *offsetDevice, int8_t *outDevice, int64_t rows, int64_t channels,
                            void *stream);

/*
 * BlockCopy: copies whole cache blocks inside the key cache and the value cache. Source i
 * (srcBlocks[i]) goes to the destinations dstBlocks[cumSum[i-1] .. cumSum[i]) (cumSum[-1] = 0).
 * All index vectors are int32 device memory; keyBlockBytes / valueBlockBytes are the bytes of
 * one block (blockSize * heads * headSize * sizeof element). valueCache may be NULL. Sources
 * and destinations must be disjoint sets (the copies run in parallel); an index outside
 * [0, numBlocks) skips that copy.
 * Replaces: BlockCopyOperation's kernel (reference src/ops/ops_infer/block_copy/
 * block_copy_operation.cpp:69-99 inputs, golden tests/apitest/opstest/python/operations/
 * block_copy/test_block_copy.py golden_calc).
 */
int atbmi_block_copy(void *keyCacheDevice, void *valueCacheDevice, const int32_t *srcBlocksDevice,
                     const int32_t *dstBlocksDevice, const int32_t *cumSumDevice, int64_t srcCount, int64_t dstCount,
                     int64_t numBlocks, int64_t keyBlockBytes, int64_t valueBlockBytes, void *stream);

/*
 * PagedCacheLoad, ND caches: gathers the rows of every sequence from the paged caches into
 * contiguous key / value tensors, the reverse of ReshapeAndCache. Token t of sequence b is
 * the row at offset t % blockSize of block blockTables[b][seqStarts[b] / blockSize + t / blockSize]
 * and lands in output row (tokens of the sequences before b) + t. seqLens (int32, device) holds
 * the lengths [batch], or with cumsumMode their running sum [batch + 1] starting at 0; seqStarts
 * may be NULL (all 0). A negative or out-of-range block id leaves its output rows untouched, as do
 * rows at or past outRows. maxSeqLen bounds every length (the launch is sized by it; the lengths
 * themselves are only known on the device).
 * Replaces: PagedCacheLoadOperation's ND kernel (reference src/ops/ops_infer/paged_cache_load/
 * paged_cache_load_operation.cpp:20-50 inputs, golden tests/apitest/opstest/python/operations/
 * paged_cache_load/test_paged_cache_load_operation_nd.py:57-170).
 */
int atbmi_paged_cache_load(const void *keyCacheDevice, const void *valueCacheDevice, const int32_t *blockTablesDevice,
                           const int32_t *seqLensDevice, const int32_t *seqStartsDevice, void *keyDevice,
                           void *valueDevice, int64_t batch, int64_t maxBlocksPerSeq, int64_t blockSize,
                           int64_t numBlocks, int64_t keyRowBytes, int64_t valueRowBytes, int64_t outRows,
                           int64_t maxSeqLen, int32_t cumsumMode, void *stream);

/*
 * PagedCacheLoad, fractal-NZ caches (PagedCacheLoadParam::K_CACHE_V_CACHE_NZ): the same gather from caches
 * [numBlocks, rowBytes / pieceBytes, blockSize, piece], where a row is cut into pieces of keyPieceBytes /
 * valuePieceBytes (32 int8 or 16 two-byte elements) and a block holds piece 0 of all its rows, then piece 1, ...
 * The outputs are plain rows [outRows, rowBytes]. seqLens holds the lengths [batch]; there are no sequence starts
 * and no running-sum form in this layout (reference paged_cache_load_operation.cpp:63-67).
 * Replaces: PagedCacheLoadOperation's NZ kernel (golden tests/apitest/kernelstest/mix/
 * test_paged_cache_load_nz.py:72-131).
 */
int atbmi_paged_cache_load_nz(const void *keyCacheDevice, const void *valueCacheDevice,
                              const int32_t *blockTablesDevice, const int32_t *seqLensDevice, void *keyDevice,
                              void *valueDevice, int64_t batch, int64_t maxBlocksPerSeq, int64_t blockSize,
                              int64_t numBlocks, int64_t keyRowBytes, int64_t valueRowBytes, int64_t keyPieceBytes,
                              int64_t valuePieceBytes, int64_t outRows, int64_t maxSeqLen, void *stream);

/*
 * Fused quantise + KV-cache write (extension; the reference runs the
 * quantiser and ReshapeAndCache as two operators): key/value are fp16/bf16
 * [numTokens, numKvHeads, headDim*], kScale/vScale are fp32 [numKvHeads*headDim*],
 * caches are int8. Same slot rules as atbmi_reshape_and_cache, same
 * arithmetic as atbmi_quant_per_channel with no offset.
 */
int atbmi_reshape_and_cache_quant(const void *keyDevice, const void *valueDevice, int32_t kvDtype,
                                  const float *kScaleDevice, const float *vScaleDevice, int8_t *keyCacheDevice,
                                  int8_t *valueCacheDevice, const int32_t *slotMappingDevice, int64_t numTokens,
                                  int64_t numKvHeads, int64_t headDimK, int64_t headDimV, int64_t numSlots,
                                  void *stream);

/* Static description of a paged decode-attention problem. */
/* Row of the mask a query row uses, in units of maskBatchStride
 * (reference tiling/paged_attention_tiling_dependency.cpp:557-569, GetLookaheadMaskOffset):
 *   SEQUENCE  the index of its sequence in hostContextLens (one-token decode: NORM / ALIBI masks)
 *   QUERY     its own index among the query rows (MASK_TYPE_SPEC: mask [numQueryRows, maxLen])
 *   POSITION  its position in the sequence, contextLen - queryLen + i for the i-th query token
 *             (a square causal NORM mask [maxLen, maxLen] under CALC_TYPE_SPEC) */
typedef enum AtbmiPaMaskRow {
    ATBMI_PA_MASK_ROW_SEQUENCE = 0,
    ATBMI_PA_MASK_ROW_QUERY = 1,
    ATBMI_PA_MASK_ROW_POSITION = 2
} AtbmiPaMaskRow;

/* Order of the dimensions inside one cache block (reference include/atb/infer_op_params.h, InputLayout):
 *   TOKEN_MAJOR  [numBlocks, blockSize, G, D]  TYPE_BSND
 *   HEAD_MAJOR   [numBlocks, G, blockSize, D]  TYPE_BNSD (PagedAttentionParam::inputLayout; 16-bit
 *                caches with separate key and value caches only)
 *   FRACTAL_NZ   [numBlocks, D / 16, blockSize, 16]: channel c of the token at offset t of a block sits at
 *                (c / 16) * blockSize * 16 + t * 16 + c % 16 of the block (MultiLatentAttentionParam::NZCACHE,
 *                reference include/atb/infer_op_params.h:2949-2955; only the split latent layout, ropeDim 64,
 *                16-bit, with a power-of-two block size: keyCache [numBlocks, 32, blockSize, 16] and
 *                keyRopeCache [numBlocks, 4, blockSize, 16]) */
typedef enum AtbmiPaKvLayout {
    ATBMI_PA_KV_TOKEN_MAJOR = 0,
    ATBMI_PA_KV_HEAD_MAJOR = 1,
    ATBMI_PA_KV_FRACTAL_NZ = 2
} AtbmiPaKvLayout;

typedef struct AtbmiPaShape {
    int32_t qDtype;          /* ATBMI_F16 or ATBMI_BF16; the output has the same type */
    int32_t kvDtype;         /* ATBMI_F16 / ATBMI_BF16 (== qDtype) or ATBMI_INT8 */
    int32_t numHeads;        /* query heads H */
    int32_t numKvHeads;      /* KV heads G, H % G == 0 */
    int32_t headDimK;        /* D: channels of q and of a key row */
    int32_t headDimV;        /* Dv: channels of a value row and of the output */
    int32_t blockSize;       /* tokens per cache block */
    int32_t numBlocks;       /* blocks in the cache pool */
    int32_t maxBlocksPerSeq; /* row length of blockTables */
    int32_t numQueryRows;    /* rows of q / out */
    int32_t mlaCombined;     /* 1: no value cache; V = first Dv channels of the key cache row */
    int32_t hasOffset;       /* int8 KV: kOffset / vOffset are given */
    int32_t kernel;          /* AtbmiPaKernel */
    int32_t hasMask;         /* 1: an additive score bias (AtbmiPaTensors.mask) is given */
    float qkScale;           /* multiplies q.k before the softmax */
    float qScale;            /* pre-multiplies q (rounded to qDtype) unless 0 or 1 */
    int64_t maskBatchStride; /* elements between the mask rows of consecutive sequences (0: shared) */
    int64_t maskHeadStride;  /* elements between the mask rows of consecutive query heads (0: shared) */
    int32_t maskLen;         /* tokens per mask row, >= every context length */
    int32_t hasLogN;         /* 1: a per-sequence factor on qkScale (AtbmiPaTensors.logN) is given */
    int32_t descalePacked;   /* 1: kScale / vScale are uint64 arrays whose low 32 bits hold the fp32 value,
                                as atb::Utils::QuantParamConvert packs them (reference src/atb/utils/utils.cpp:153-164) */
    int32_t maskRowBy;       /* AtbmiPaMaskRow: which mask row (in units of maskBatchStride) a query row uses */
    int32_t ropeDim;         /* 0, or 64 with mlaCombined, headDimK 576 and headDimV 512: the split latent layout of
                                MultiLatentAttentionParam::KROPE_CTKV (reference include/atb/infer_op_params.h:2949-2958):
                                query and keyCache hold rows of headDimK - ropeDim channels, queryRope and
                                keyRopeCache the remaining ropeDim channels of the same rows */
    int32_t kvLayout;        /* AtbmiPaKvLayout of keyCache and valueCache */
    /* Head compression (PagedAttentionParam::compressType, reference
     * src/kernels/mixkernels/pagedattention/tiling/paged_attention_tiling.cpp:36-80,217-226): every (sequence,
     * KV head) pair of the model becomes a sequence of its own here, with its own context length and block-table
     * row, numKvHeads = 1 and numHeads = the model's heads per KV head; query / out rows are the same memory read
     * as [tokens * kvHeads, numHeads, D]. Three things then still follow the model's indices: */
    int32_t maskSeqDiv;      /* > 1 with maskRowBy SEQUENCE: sequence b uses mask row b / maskSeqDiv (a mask with one
                                row per model sequence) */
    int32_t maskSeqMod;      /* > 0 with maskRowBy SEQUENCE: ... row b % maskSeqMod (a mask with one row group per
                                model KV head and none per sequence); applied after maskSeqDiv */
    int32_t descaleHeads;    /* > 0, int8 KV: kScale / vScale (and the offsets) hold descaleHeads slices of D / Dv
                                entries and sequence b uses slice b % descaleHeads; numKvHeads must be 1 */
    int32_t hasRazorOffset;  /* 1: AtbmiPaTensors.razorOffset is given (COMPRESS_TYPE_KVHEAD_ROPE) */
} AtbmiPaShape;

/* Device tensors of one decode call.
 *   query       [numQueryRows, H, D]                qDtype
 *   keyCache    [numBlocks, blockSize, G, D]        kvDtype ([numBlocks, G, blockSize, D] when head-major)
 *   valueCache  [numBlocks, blockSize, G, Dv]       kvDtype (NULL when mlaCombined; head-major like keyCache)
 *   blockTables [batch, maxBlocksPerSeq]            int32
 *   kScale/vScale [G*D] / [G*Dv] fp32 (or uint64-packed fp32, see descalePacked), kOffset/vOffset same
 *               length int32 (int8 KV only)
 *   out         [numQueryRows, H, Dv]               qDtype
 *   mask        qDtype, hasMask only: the score of sequence b (its index in hostContextLens), head h and
 *               token t gets mask[b * maskBatchStride + h * maskHeadStride + t] added after the qkScale
 *               multiplication. Covers the reference's MASK_TYPE_NORM ([batch, 1, maxLen]: batch stride
 *               maxLen, head stride 0; [1, maxLen]: both 0) and MASK_TYPE_ALIBI ([heads, 1, maxLen]: batch
 *               stride 0; [batch, heads | 1, 1, maxLen]) layouts of a decode step
 *               (tiling/paged_attention_tiling.cpp:36-80).
 *   logN        fp32 [batch], hasLogN only: sequence b uses qkScale * logN[b] (SCALE_TYPE_LOGN).
 */
typedef struct AtbmiPaTensors {
    const void *query;
    const void *keyCache;
    const void *valueCache;
    const int32_t *blockTables;
    const float *kScale;
    const int32_t *kOffset;
    const float *vScale;
    const int32_t *vOffset;
    void *out;
    const void *mask;
    const float *logN;
    const void *queryRope;    /* [numQueryRows, H, ropeDim] qDtype, ropeDim > 0 only */
    const void *keyRopeCache; /* [numBlocks, blockSize, G, ropeDim] qDtype, ropeDim > 0 only */
    const float *razorOffset; /* hasRazorOffset only: fp32 [numBlocks, blockSize], added to q.k of the token in that
                                 cache slot before the qkScale multiplication (numKvHeads 1, token-major caches) */
    void *lse;                /* NULL, or [numQueryRows, H] qDtype: receives the natural-log log-sum-exp of the
                                 scaled (and masked) scores of every planned query row and head — the second
                                 output of MultiLatentAttentionParam::CALC_TYPE_RING */
} AtbmiPaTensors;

typedef struct AtbmiPaPlan AtbmiPaPlan; /* opaque; owned by the caller, not thread-safe */

/* Validates the shape and creates an empty plan. Host only. */
int atbmi_pa_plan_create(const AtbmiPaShape *shape, AtbmiPaPlan **plan);

/* Splits the batch into KV chunks for the given host context lengths
 * (sequence b attends to tokens [0, hostContextLens[b])). A sequence of length
 * 0 is skipped and takes no query row: query/out row index = number of
 * non-empty sequences before it. Host only, O(batch + chunks). */
int atbmi_pa_plan_update(AtbmiPaPlan *plan, const int32_t *hostContextLens, int32_t batch);

/* The same with several query tokens per sequence (CALC_TYPE_SPEC: speculative / multi-token decoding;
 * replaces the qSeqLen handling of the reference, src/ops/ops_infer/paged_attention/param.cpp:39-62 and
 * tiling/paged_attention_tiling_dependency.cpp:580-620). Sequence b brings hostQueryLens[b] consecutive
 * query rows (0 <= hostQueryLens[b] <= hostContextLens[b]; none when its context length is 0), each of
 * which attends to all hostContextLens[b] tokens: which of them a row may see is the mask's business
 * (AtbmiPaShape.maskRowBy). hostQueryLens == NULL means one row per sequence. Up to 16 / (numHeads /
 * numKvHeads) query tokens of a sequence share one pass over its K and V rows. */
int atbmi_pa_plan_update_multi(AtbmiPaPlan *plan, const int32_t *hostContextLens, const int32_t *hostQueryLens,
                               int32_t batch);

/* Causal query rows for the updates that follow: the t-th of a sequence's n query rows then attends to its
 * first hostContextLens[b] - n + t + 1 tokens only, with no mask involved. This is how the reference's MLA
 * tiling makes several query tokens causal when it runs one job per query token (128 heads, or an int8 cache:
 * src/kernels/mixkernels/multi_latent_attention/tiling/mla_tiling.cpp:139-144,
 * mla_tiling_dependency.cpp:292-316). perSequence, NULL or a host array of `count` flags that is copied,
 * exempts the sequences whose flag is 0 (the reference's maskUseStatus); an update with another batch than
 * `count` is refused. enable == 0 returns to whole contexts. Query tokens of a sequence then take a pass each. */
int atbmi_pa_plan_set_causal_rows(AtbmiPaPlan *plan, int32_t enable, const int32_t *perSequence, int32_t count);

/* Empty sequences for the updates that follow: with enable != 0 a sequence whose context length is 0 still owns its
 * hostQueryLens[b] (or one) query rows, which are neither read nor written, and the rows of the sequences behind it
 * stay where they are. This is what the reference's MultiLatentAttention tiling does (it moves on by qSeqLen whatever
 * kvSeqLen is, src/kernels/mixkernels/multi_latent_attention/tiling/mla_tiling.cpp:146-149), whereas its PagedAttention
 * tiling gives such a sequence no row (tiling/paged_attention_tiling_dependency.cpp:593,654,706), the default here. */
int atbmi_pa_plan_set_empty_keep_rows(AtbmiPaPlan *plan, int32_t enable);

/* Device workspace bytes atbmi_pa_decode needs for the current plan. */
uint64_t atbmi_pa_plan_workspace_size(const AtbmiPaPlan *plan);

/* Number of KV chunks (workgroup launches per KV head) in the current plan. */
int64_t atbmi_pa_plan_num_chunks(const AtbmiPaPlan *plan);

/* Algorithmic HBM bytes of one decode call with the current plan: valid K/V
 * rows + q + out + block-table entries + context lengths + scale vectors +
 * every distinct mask row over the tokens it biases + logN. */
uint64_t atbmi_pa_plan_algorithmic_bytes(const AtbmiPaPlan *plan);

/* Uploads the plan into the workspace and launches the attention kernel (and
 * the split merge kernel when any sequence has more than one chunk). */
int atbmi_pa_decode(AtbmiPaPlan *plan, const AtbmiPaTensors *tensors, void *workspaceDevice,
                    uint64_t workspaceBytes, void *stream);

/*
 * atbmi_pa_decode without a workspace and without any allocation. No counterpart in the reference: it is
 * for callers that cannot allocate device or pinned memory around the call (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc). The partial rows of the split go into a static
 * device array of atbmi_pa_static_scratch_bytes() bytes (32 MiB) that every GPU the library runs on holds
 * until the process ends. Refused with 1 (invalid parameter) when the current plan needs more than that
 * (atbmi_pa_plan_workspace_size), or when its tables do not travel in the kernel arguments (scalar-kernel
 * plans; more than 160 passes or 512 workgroup ranges): use atbmi_pa_decode then. Kernel timing
 * (atbmi_timing_enable) does not cover it. All calls on one GPU share the array: calls that may overlap on
 * one GPU (different streams, different threads) race; calls on one stream are safe. Results are those of
 * atbmi_pa_decode, bit for bit. The FIRST call on a device, and the first with each kernel variant (head size, cache
 * type, with or without a mask), looks up the array's address and raises the kernel's LDS limit, two runtime calls
 * that do not belong inside a stream capture: make one call of each variant before capturing.
 */
int atbmi_pa_decode_static(AtbmiPaPlan *plan, const AtbmiPaTensors *tensors, void *stream);
uint64_t atbmi_pa_static_scratch_bytes(void);

void atbmi_pa_plan_destroy(AtbmiPaPlan *plan);

/*
 * Prefill attention of MultiLatentAttention (MultiLatentAttentionParam::CALC_TYPE_PREFILL; reference
 * src/ops/ops_infer/multi_latent_attention/multi_latent_attention_ops_runner_prefill.cpp:33-131, kernel library
 * src/kernels/mixkernels/multi_latent_attention/mla_operation.cpp:184-235 and tiling/mla_tiling.cpp:286-327):
 * flash attention over variable-length sequences with 128 + 64 key channels and 128 value channels per head.
 * Sequence b owns hostQLens[b] consecutive rows of query / queryRope / out and hostKvLens[b] rows of key /
 * keyRope / value: consecutive as well (kvPaddedRows 0, tensors [tokens, kvHeads, channels]), or rows
 * [b * kvPaddedRows, b * kvPaddedRows + hostKvLens[b]) (tensors [batch, kvPaddedRows, kvHeads * channels]).
 * Query head h attends over KV head h / (numHeads / numKvHeads).
 *   mask NONE    every query sees every key of its sequence (MaskType UNDEFINED)
 *        CAUSAL  query i sees keys j <= i (MASK_TYPE_CAUSAL_MASK, and MASK_TYPE_MASK_FREE, whose 512 x 512 mask
 *                input is the strictly upper triangular matrix that says the same; its values are not read)
 *        WINDOW  j <= i and j > i - windowSize (MASK_TYPE_SWA_NORM; the mask input is not read either)
 * With a mask the two lengths of a sequence must agree. The lengths are host arrays, read during the call.
 */
typedef enum AtbmiMlaPrefillMask {
    ATBMI_MLA_PREFILL_MASK_NONE = 0,
    ATBMI_MLA_PREFILL_MASK_CAUSAL = 1,
    ATBMI_MLA_PREFILL_MASK_WINDOW = 2
} AtbmiMlaPrefillMask;

typedef struct AtbmiMlaPrefillCall {
    int32_t dtype;             /* AtbmiDtype of every tensor: ATBMI_F16 or ATBMI_BF16 */
    int32_t numHeads;
    int32_t numKvHeads;        /* divides numHeads */
    int32_t mask;              /* AtbmiMlaPrefillMask */
    int32_t windowSize;        /* WINDOW only, > 0 */
    float qkScale;
    int32_t batch;
    int32_t reserved;
    int64_t kvPaddedRows;      /* 0: key rows of the sequences follow each other */
    const int32_t *hostQLens;  /* [batch], host memory */
    const int32_t *hostKvLens; /* [batch], host memory */
    const void *query;         /* [sum qLens, numHeads, 128] */
    const void *queryRope;     /* [sum qLens, numHeads, 64] */
    const void *key;           /* [key rows, numKvHeads, 128] */
    const void *keyRope;       /* [key rows, numKvHeads, 64] */
    const void *value;         /* [key rows, numKvHeads, 128] */
    void *out;                 /* [sum qLens, numHeads, 128] */
} AtbmiMlaPrefillCall;

/* Validates the call (pointers aside) and reports the device workspace it needs: 32 bytes per block of
 * 128 queries. Host only. */
int atbmi_mla_prefill_workspace_size(const AtbmiMlaPrefillCall *call, uint64_t *bytes);
/* Uploads the block list into the workspace and launches the kernel on `stream`; does not wait. */
int atbmi_mla_prefill(const AtbmiMlaPrefillCall *call, void *workspaceDevice, uint64_t workspaceBytes, void *stream);

/*
 * Decode attention of MultiLatentAttention over the int8 fractal-NZ cache (MultiLatentAttentionParam::INT8_NZCACHE;
 * reference src/ops/ops_infer/multi_latent_attention/multi_latent_attention_operation.cpp:427-476 for the shapes,
 * kernel library src/kernels/mixkernels/multi_latent_attention/op_kernel/mla_int8.cce, golden
 * tests/apitest/opstest/python/operations/multi_latent_attention/test_multi_latent_attention_int8nz.py:115-121,179-262):
 * the 512 latent channels of queries and cache rows are int8 with one fp32 descale per head for the scores
 * (qkDescale) and one for the values (pvDescale), the 64 rotary channels stay 16-bit, and the softmax weights
 * of every cache block (128 tokens) are quantised to int8 against the block's largest weight before they
 * multiply the int8 value rows; all integer products are exact.
 *   query       int8 [numQueryRows, numHeads, 512]       queryRope  16-bit [numQueryRows, numHeads, 64]
 *   kvCache     int8 [numBlocks, 512 / 32, 128, 32]      kRopeCache 16-bit [numBlocks, 64 / 16, 128, 16]
 *   blockTables int32 [batch, maxBlocksPerSeq] (device)  qkDescale, pvDescale fp32 [numHeads]
 *   mask        NULL, or 16-bit [numQueryRows, maskLen] added to the scaled scores of its query row
 *   out         16-bit [numQueryRows, numHeads, 512]     lse        NULL, or fp32 [numQueryRows, numHeads]
 * Sequence b attends to hostContextLens[b] tokens with hostQueryLens[b] consecutive query rows (NULL: one
 * each; a sequence of length 0 keeps its rows, which are neither read nor written, as the reference's tiling
 * moves on by qSeqLen whatever kvSeqLen is: tiling/mla_tiling.cpp:146-149). With causalRows != 0 the t-th of a sequence's n query rows
 * attends to its first hostContextLens[b] - n + t + 1 tokens only, unless hostCausalUse (NULL, or [batch])
 * holds 0 for the sequence: the reference golden's handling of several query tokens in this mode
 * (test_multi_latent_attention_int8nz.py:356-364). The lengths and flags are host arrays, read during the call.
 */
typedef struct AtbmiMlaInt8Call {
    int32_t outDtype;          /* ATBMI_F16 or ATBMI_BF16: type of queryRope, kRopeCache, mask and out */
    int32_t numHeads;
    int32_t blockSize;         /* 128 */
    int32_t numBlocks;
    int32_t maxBlocksPerSeq;
    int32_t batch;
    int32_t numQueryRows;
    int32_t hasMask;
    int32_t maskLen;
    float qkScale;
    const int32_t *hostContextLens; /* [batch], host memory */
    const int32_t *hostQueryLens;   /* NULL or [batch], host memory */
    int32_t causalRows;
    const int32_t *hostCausalUse;   /* NULL or [batch], host memory */
    const void *query;
    const void *queryRope;
    const void *kvCache;
    const void *kRopeCache;
    const int32_t *blockTables;
    const float *qkDescale;
    const float *pvDescale;
    const void *mask;
    void *out;
    float *lse;
} AtbmiMlaInt8Call;

/* Validates the call (pointers aside) and reports the device workspace it needs: 16 bytes per query row, and, when
 * the call has too few heads to fill the chip and its rows are cut into pieces (up to four), the pieces' output rows
 * and log-sum-exps. */
int atbmi_mla_int8_workspace_size(const AtbmiMlaInt8Call *call, uint64_t *bytes);
/* Launches the kernel (and, for rows cut into pieces, the merge kernel) on `stream`; does not wait. The list of
 * query rows travels in the kernel arguments when it has at most 128 entries and is uploaded into the workspace
 * otherwise (the workspace is asked for either way). */
int atbmi_mla_int8_decode(const AtbmiMlaInt8Call *call, void *workspaceDevice, uint64_t workspaceBytes, void *stream);

/*
 * PagedAttention decode with int8 queries over int8 caches (PagedAttentionParam::quantType TYPE_QUANT_QKV_ONLINE /
 * TYPE_QUANT_QKV_OFFLINE; reference src/ops/ops_infer/paged_attention/paged_attention_operation.cpp:250-275,429-436
 * for the parameters and inputs, kernel library src/kernels/mixkernels/pagedattention/paged_attention_operation.cpp:
 * 357-403 for the descale shapes, golden tests/apitest/kernelstest/mix/test_paged_attention_common.py:104-110,147-229):
 * query, keys and values are int8 with one fp32 descale per QUERY head for the scores (kDescale) and one for the
 * values (vDescale); the softmax weights of every tile of 64 tokens are quantised to int8 before they multiply the
 * int8 value rows, against the tile's largest weight (online) or with the factor pScale[head] (offline); all integer
 * products are exact.
 *   query       int8 [numQueryRows, numHeads, headDim]            kDescale, vDescale, pScale  fp32 [numHeads]
 *   keyCache, valueCache  int8 [numBlocks, blockSize, numKvHeads, headDim]   blockTables int32 [batch, maxBlocksPerSeq]
 *   mask        NULL, or 16-bit (the output's type): the bias of sequence b, head h, token t is
 *               mask[b * maskSeqStride + h * maskHeadStride + t] (elements; a stride of 0 shares the row), added to
 *               the scaled scores
 *   out         16-bit [numQueryRows, numHeads, headDim]
 * One query token per sequence; a sequence of length 0 takes no query row. headDim is 64, 128 or 256; pScale is
 * expected to keep w x pScale within 127, as the reference's own generator does. Long contexts are cut into pieces
 * that are worked on side by side and merged, as the reference's kernel and golden do (:171-229); offline the weights
 * are taken against the running maximum, which starts anew in every piece, so the result depends on the cut in its
 * last digits (pieceTiles fixes it). The lengths are a host array, read
 * during the call.
 */
typedef struct AtbmiPaInt8QCall {
    int32_t outDtype;          /* ATBMI_F16 or ATBMI_BF16: type of mask and out */
    int32_t numHeads;
    int32_t numKvHeads;
    int32_t headDim;
    int32_t blockSize;
    int32_t numBlocks;
    int32_t maxBlocksPerSeq;
    int32_t batch;
    int32_t numQueryRows;
    int32_t offline;           /* 0: weights quantised against the tile's maximum; 1: with pScale */
    int32_t hasMask;
    int32_t maskLen;           /* positions a mask row covers, >= every context length */
    int32_t pieceTiles;        /* c > 0: a context of n units of 128 tokens is cut into ceil(n / c) pieces of
                                  ceil(n / pieces) units, merged by their log-sum-exps. 0: the library cuts: the
                                  64-token tiles of all sequences, in order, are one list cut into equal shares,
                                  share w beginning at tile floor(tiles x w / shares), with shares = min(tiles / 4,
                                  workgroups the chip holds at once); a sequence is cut where a share begins
                                  inside it */
    float qkScale;
    int64_t maskSeqStride;
    int64_t maskHeadStride;
    const int32_t *hostContextLens; /* [batch], host memory */
    const void *query;
    const void *keyCache;
    const void *valueCache;
    const int32_t *blockTables;
    const float *kDescale;
    const float *vDescale;
    const float *pScale;       /* offline only */
    const void *mask;
    void *out;
    int32_t maskRowByQuery;    /* 0: the mask row of a sequence is its index in hostContextLens; 1: the index of its query
                                * row (MASK_TYPE_SPEC: mask [numQueryRows, maskLen], maskSeqStride = maskLen), which differs
                                * when sequences without context come before it */
} AtbmiPaInt8QCall;

/* Validates the call (pointers aside) and reports the device workspace it needs: the table of context pieces
 * (32 bytes each) and, for sequences cut into several pieces, their partial rows (in the output's 16-bit type) and
 * fp32 log-sum-exps. The library's own cut
 * (pieceTiles = 0) follows the number of CUs of the current device, so size and launch belong on the same device;
 * a launch that finds the workspace too small fails with an error and runs nothing. */
int atbmi_pa_int8q_workspace_size(const AtbmiPaInt8QCall *call, uint64_t *bytes);
/* Uploads the tables into the workspace and launches the kernel (and the merge of cut sequences) on `stream`;
 * does not wait. */
int atbmi_pa_int8q_decode(const AtbmiPaInt8QCall *call, void *workspaceDevice, uint64_t workspaceBytes, void *stream);

/*
 * MultiLatentAttention with maskType MASK_TYPE_MASK_FREE and several query tokens (decode calcTypes; replaces the
 * mask handling of the reference's device kernel, src/kernels/mixkernels/multi_latent_attention/op_kernel/
 * mla.cce:3719-3750 with 2581-2592, and the shape rule of tiling/mla_tiling.cpp:156-166): expands the compressed
 * mask, a template [templateRows, 128] (templateBatch == 0) or [templateBatch = batch, templateRows, 128] of 16-bit
 * values, into one mask row per query token, outMask 16-bit [numQueryRows, maskLen], to be handed to the decode
 * plan as a mask with one row per query row (AtbmiPaShape.maskRowBy = ATBMI_PA_MASK_ROW_QUERY). Sequence b has
 * hostContextLens[b] tokens and hostQueryLens[b] query rows (also when its context is empty: rows of zeros), as a
 * plan with atbmi_pa_plan_set_empty_keep_rows has them; both are host arrays read during the call.
 */
typedef struct AtbmiMlaMaskFreeCall {
    int32_t batch;
    int32_t numQueryRows;
    int32_t templateBatch; /* 0, or batch */
    int32_t templateRows;  /* 125 + 2 q in the reference's tests */
    int32_t maskLen;       /* elements per row of outMask, >= every context length */
    const int32_t *hostContextLens;
    const int32_t *hostQueryLens;
    const void *maskTemplate;
    void *outMask;
} AtbmiMlaMaskFreeCall;

/* Validates the call (pointers aside) and reports the device workspace it needs (16 bytes per query row). */
int atbmi_mla_mask_free_workspace_size(const AtbmiMlaMaskFreeCall *call, uint64_t *bytes);
/* Uploads the row list into the workspace and launches the expansion on `stream`; does not wait. */
int atbmi_mla_mask_free_expand(const AtbmiMlaMaskFreeCall *call, void *workspaceDevice, uint64_t workspaceBytes,
                               void *stream);

/*
 * Kernel timing for benchmarks. atbmi_timing_enable(n) with n > 0 makes every
 * n-th atbmi_pa_decode bracket its attention kernel with HIP events on the
 * launch stream (the events themselves cost a few microseconds of stream
 * time, hence the sampling); 0 turns it off.
 * atbmi_timing_read waits for the recorded events, adds them up, returns the
 * sum in milliseconds and the number of timed launches, and clears the record.
 */
int atbmi_timing_enable(int32_t enable);
int atbmi_timing_read(double *totalMs, int64_t *launches);
/* The same, and also the sum from the start of the attention kernel to the end of the merge kernel that
 * follows it (equal to the first sum for calls that need no merge). Any pointer may be NULL. */
int atbmi_timing_read_split(double *kernelMs, double *withMergeMs, int64_t *launches);
/* The same record launch by launch (milliseconds), at most `capacity` launches; clears the record. */
int atbmi_timing_read_samples(float *kernelMs, float *withMergeMs, int64_t capacity, int64_t *launches);
/* whole != 0: a timed call is bracketed as ONE interval, from in front of the attention kernel to behind its merge
 * kernel, with no event between the two (an event there costs the merge kernel about a microsecond of stream time);
 * both figures of a read are then that interval. 0 (the default): three events, as described above. */
int atbmi_timing_whole_calls(int32_t whole);

#ifdef __cplusplus
}
#endif
#endif
