// Minimal stand-in for the CANN runtime header that atb/types.h pulls in.
// Only the three things the PagedAttention / ReshapeAndCache path touches are
// declared: tensor element types, tensor formats and the stream handle.
// Enumerator values are the CANN ones, so packs built by existing callers
// keep their meaning (value table: reference
// tests/framework/python/CsvOpsTestTool/atb_csv_ops_test.py:33-40).
// On MI355X an aclrtStream carries a hipStream_t.
#ifndef ATB_MI_ACL_SHIM_H
#define ATB_MI_ACL_SHIM_H

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

#ifdef __cplusplus
}
#endif
#endif
