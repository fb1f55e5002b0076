/*
 * atb_capi.h - flat C view of the atb::Operation API, for callers that cannot
 * include C++ headers (ctypes / cffi / JNI test drivers and benchmarks).
 *
 * Each function forwards to the C++ call named in its comment and returns its
 * atb::Status unchanged. It plays the part of the reference's own test
 * driver, which builds an operation from a param, binds host tensors, then
 * runs InferShape -> Setup -> Execute
 * (reference tests/framework/c++/atb_torch/operation/operation_torch.cpp:313-415).
 * The reference ships C wrappers only for other operators
 * (include/atb/atb_acl.h:99-116); PagedAttention and ReshapeAndCache have none.
 */
#ifndef ATB_CAPI_H
#define ATB_CAPI_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* atb::Tensor flattened: desc {dtype, format, shape}, deviceData, hostData, dataSize. */
typedef struct AtbCTensor {
    int32_t dtype;  /* aclDataType */
    int32_t format; /* aclFormat */
    int64_t dims[8];
    uint64_t dimNum;
    void *deviceData;
    void *hostData;
    uint64_t dataSize;
} AtbCTensor;

/* atb::CreateContext + Context::SetExecuteStream(stream). */
int32_t atb_c_create_context(void *stream, void **context);
/* Context::SetExecuteStream. */
int32_t atb_c_context_set_stream(void *context, void *stream);
/* Context::SetExecuteStreams: `count` streams, the first of which is the one atb_c_context_set_stream sets. */
int32_t atb_c_context_set_streams(void *context, void *const *streams, uint32_t count);
/* Context::SetExecuteType (0 normal, 1 pre-launch, 2 launch). */
int32_t atb_c_context_set_execute_type(void *context, int32_t type);
/* atb::DestroyContext. */
int32_t atb_c_destroy_context(void *context);

/* atb::CreateOperation for infer::PagedAttentionParam, ReshapeAndCacheParam,
 * ReshapeAndCacheWithStrideParam, ReshapeAndCacheOmniParam, RopeParam, ElewiseParam, NormRopeReshapeParam,
 * MultiLatentAttentionParam, BlockCopyParam and PagedCacheLoadParam. opName is the operation's name
 * ("PagedAttentionOperation", "ReshapeAndCacheOperation", "ReshapeAndCacheWithStrideOperation",
 * "ReshapeAndCacheOmniOperation", "RopeOperation", "ElewiseOperation", "NormRopeReshapeOperation",
 * "MultiLatentAttentionOperation", "BlockCopyOperation", "PagedCacheLoadOperation"); param points at the bytes of
 * the matching C++ param struct (120 / 24 / 24 / 8 / 16 / 64 / 28 / 64 / 16 / 64 bytes). */
int32_t atb_c_create_operation(const char *opName, const void *param, uint64_t paramSize, void **operation);
/* atb::DestroyOperation. */
int32_t atb_c_destroy_operation(void *operation);

/* Operation::GetInputNum / GetOutputNum / GetName (name copied into buf). */
uint32_t atb_c_op_input_num(void *operation);
uint32_t atb_c_op_output_num(void *operation);
int32_t atb_c_op_name(void *operation, char *buf, uint64_t bufSize);

/* Operation::InferShape; only desc fields of the tensors are read/written. */
int32_t atb_c_op_infer_shape(void *operation, const AtbCTensor *inDescs, uint32_t numIn, AtbCTensor *outDescs,
                             uint32_t outCapacity, uint32_t *numOut);
/* Operation::Setup. context may be NULL to exercise the error path. */
int32_t atb_c_op_setup(void *operation, const AtbCTensor *inTensors, uint32_t numIn, const AtbCTensor *outTensors,
                       uint32_t numOut, uint64_t *workspaceSize, void *context);
/* Operation::Execute. */
int32_t atb_c_op_execute(void *operation, const AtbCTensor *inTensors, uint32_t numIn,
                         const AtbCTensor *outTensors, uint32_t numOut, void *workspace, uint64_t workspaceSize,
                         void *context);

/* atb::SetExecuteStreamId / atb::GetExecuteStreamId: which of the context's streams the operation launches on. */
int32_t atb_c_op_set_stream_id(void *operation, uint32_t streamId);
uint32_t atb_c_op_get_stream_id(void *operation);

/* atb::Utils::GetTensorSize on the desc fields. */
uint64_t atb_c_tensor_size(const AtbCTensor *tensor);

/* atb::Utils::QuantParamConvert (reference include/atb/utils.h:82): fp32 bits into the low half of uint64. */
void atb_c_quant_param_convert(const float *src, uint64_t *dest, uint64_t itemCount);

/* sizeof(infer::PagedAttentionParam), sizeof(infer::ReshapeAndCacheParam),
 * sizeof(infer::MultiLatentAttentionParam). */
uint64_t atb_c_sizeof_paged_attention_param(void);
uint64_t atb_c_sizeof_reshape_and_cache_param(void);
uint64_t atb_c_sizeof_multi_latent_attention_param(void);

#ifdef __cplusplus
}
#endif
#endif
