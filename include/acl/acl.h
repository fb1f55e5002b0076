// Minimal stand-in for the CANN runtime header that atb/types.h pulls in.
// Only what the PagedAttention / ReshapeAndCache path touches is declared: tensor
// element types, tensor formats, the stream handle and the tensor handle of the
// aclnn-style wrappers.
// Enumerator values are the CANN ones, so packs built by existing callers
// keep their meaning (value table: reference
// tests/framework/python/CsvOpsTestTool/atb_csv_ops_test.py:33-40).
// On MI355X an aclrtStream carries a hipStream_t.
#ifndef ATB_MI_ACL_SHIM_H
#define ATB_MI_ACL_SHIM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    ACL_DT_UNDEFINED = -1,
    ACL_FLOAT = 0,
    ACL_FLOAT16 = 1,
    ACL_INT8 = 2,
    ACL_INT32 = 3,
    ACL_UINT8 = 4,
    ACL_INT16 = 6,
    ACL_UINT16 = 7,
    ACL_UINT32 = 8,
    ACL_INT64 = 9,
    ACL_UINT64 = 10,
    ACL_DOUBLE = 11,
    ACL_BOOL = 12,
    ACL_STRING = 13,
    ACL_COMPLEX64 = 16,
    ACL_COMPLEX128 = 17,
    ACL_BF16 = 27,
} aclDataType;

typedef enum {
    ACL_FORMAT_UNDEFINED = -1,
    ACL_FORMAT_NCHW = 0,
    ACL_FORMAT_NHWC = 1,
    ACL_FORMAT_ND = 2,
    ACL_FORMAT_NC1HWC0 = 3,
    ACL_FORMAT_FRACTAL_Z = 4,
    ACL_FORMAT_FRACTAL_NZ = 29,
    ACL_FORMAT_NCDHW = 30,
} aclFormat;

typedef void *aclrtStream;

/* The tensor handle of CANN's aclnn-style interfaces (there: aclnn/acl_meta.h), as far as the
 * two-call C wrappers of atb/atb_acl.h need it: a view shape, an element type, a format and the
 * address of the data (device memory, or host memory for the operands the wrappers read on the
 * host). stride, offset and the storage shape are accepted and kept, and must describe a
 * contiguous tensor that starts at tensorData. */
typedef struct aclTensor aclTensor;
typedef int aclnnStatus;
#define ACL_SUCCESS 0
#define ACL_ERROR_INVALID_PARAM 100000

aclTensor *aclCreateTensor(const int64_t *viewDims, uint64_t viewDimsNum, aclDataType dataType, const int64_t *stride,
                           int64_t offset, aclFormat format, const int64_t *storageDims, uint64_t storageDimsNum,
                           void *tensorData);
aclnnStatus aclDestroyTensor(const aclTensor *tensor);
/* *viewDims is allocated with new[]; the caller releases it with delete[] (as CANN's does). */
aclnnStatus aclGetViewShape(const aclTensor *tensor, int64_t **viewDims, uint64_t *viewDimsNum);
aclnnStatus aclGetDataType(const aclTensor *tensor, aclDataType *dataType);
aclnnStatus aclGetFormat(const aclTensor *tensor, aclFormat *format);
aclnnStatus aclGetRawTensorAddr(const aclTensor *tensor, void **addr);
/* Bytes per element; 0 for a type without a fixed size. */
size_t aclDataTypeSize(aclDataType dataType);

#ifdef __cplusplus
}
#endif
#endif
