"""ctypes binding of the two in-tree libraries.

`kernels()` loads lib/libatbmi_kernels.so (the C ABI of the HIP kernels) and
`atb()` loads lib/libatb.so (the atb::Operation layer through its flat C view).
Both raise if the library has not been built: there is no fallback path.

The classes below are a thin driver in the order the reference's own test
harness uses (reference tests/framework/c++/atb_torch/operation/operation_torch.cpp:313-415):
create the operation from its param, InferShape, allocate outputs, build the
VariantPack, bind host tensors (contextLens), Setup, allocate the workspace,
Execute. PyTorch is used only to hold device memory and the HIP stream.
"""
import ctypes
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
# ATB_MI_LIB_DIR names another build of the two libraries (the sanitizer build, lib_sanitize)
_LIB = os.environ.get("ATB_MI_LIB_DIR") or os.path.join(_PKG, "lib")

# aclDataType / aclFormat values (include/acl/acl.h)
ACL_FLOAT, ACL_FLOAT16, ACL_INT8, ACL_INT32, ACL_INT64, ACL_BF16 = 0, 1, 2, 3, 9, 27
ACL_FORMAT_ND, ACL_FORMAT_FRACTAL_NZ = 2, 29
ACL_DTYPE_BY_NAME = {
    "float": 0, "float16": 1, "int8": 2, "int32": 3, "uint8": 4, "int16": 6, "uint16": 7, "uint32": 8,
    "int64": 9, "uint64": 10, "double": 11, "bool": 12, "bf16": 27,
}
ACL_FORMAT_BY_NAME = {"nchw": 0, "nhwc": 1, "nd": 2, "fractal_nz": 29, "ncdhw": 30}

# atb::ErrorType (include/atb/types.h)
ERROR_NAMES = [
    "NO_ERROR", "ERROR_INVALID_PARAM", "ERROR_INVALID_GRAPH", "ERROR_INTERNAL_ERROR", "ERROR_RT_FAIL",
    "ERROR_INVALID_IN_TENSOR_NUM", "ERROR_INVALID_TENSOR_DTYPE", "ERROR_INVALID_TENSOR_FORMAT",
    "ERROR_INVALID_TENSOR_DIM", "ERROR_INVALID_TENSOR_SIZE", "ERROR_OPERATION_NULL_RUNNER",
    "ERROR_GRAPH_INFERSHAPE_FUNC_FAIL", "ERROR_CANN_ERROR", "ERROR_INVALID_TENSOR_INI_MATCH",
    "ERROR_INVALID_TENSOR_ADDR", "ERROR_INVALID_TENSOR_NUM", "ERROR_INVALID_TENSOR_DIM_NUM",
    "ERROR_INVALID_SINGLE_OPERATION_PARAM", "ERROR_GRAPH_NODE_RESHAPE_FUNC_FAIL", "ERROR_INVALID_GRAPH_NODE_CHUNK",
    "ERROR_INVALID_CONTEXT_ADDR", "ERROR_INVALID_STREAM", "ERROR_INVALID_WORKSPACE_SIZE",
    "ERROR_INVALID_WORKSPACE_ADDR", "ERROR_INVALID_OPERATION_ADDR", "ERROR_HCCL_FAIL",
    "ERROR_OUT_OF_DEVICE_MEMORY", "ERROR_OUT_OF_HOST_MEMORY", "ERROR_COMM_EMPTY", "ERROR_COPY_HOST_MEMORY_FAIL",
]
ERROR_CODE = {n: i for i, n in enumerate(ERROR_NAMES)}

ATBMI_F16, ATBMI_BF16, ATBMI_INT8 = 0, 1, 2
ATBMI_PA_KERNEL_AUTO, ATBMI_PA_KERNEL_SCALAR, ATBMI_PA_KERNEL_MFMA = 0, 1, 2
ATBMI_PA_MASK_ROW_SEQUENCE, ATBMI_PA_MASK_ROW_QUERY, ATBMI_PA_MASK_ROW_POSITION = 0, 1, 2


class AtbCTensor(ctypes.Structure):
    _fields_ = [
        ("dtype", ctypes.c_int32), ("format", ctypes.c_int32), ("dims", ctypes.c_int64 * 8),
        ("dimNum", ctypes.c_uint64), ("deviceData", ctypes.c_void_p), ("hostData", ctypes.c_void_p),
        ("dataSize", ctypes.c_uint64),
    ]


class PagedAttentionParam(ctypes.Structure):
    """Byte image of atb::infer::PagedAttentionParam (120 bytes)."""
    _fields_ = [
        ("headNum", ctypes.c_int32), ("qkScale", ctypes.c_float), ("kvHeadNum", ctypes.c_int32),
        ("maskType", ctypes.c_int32), ("batchRunStatusEnable", ctypes.c_bool), ("quantType", ctypes.c_int32),
        ("outDataType", ctypes.c_int32), ("hasQuantOffset", ctypes.c_bool), ("compressType", ctypes.c_int32),
        ("calcType", ctypes.c_int32), ("scaleType", ctypes.c_int32), ("inputLayout", ctypes.c_int32),
        ("mlaVHeadSize", ctypes.c_uint32), ("qScale", ctypes.c_float), ("rsv", ctypes.c_uint8 * 64),
    ]

    def __init__(self, **kw):
        super().__init__()
        self.qkScale = 1.0
        self.outDataType = -1
        for k, v in kw.items():
            if not hasattr(self, k):
                raise AttributeError("PagedAttentionParam has no field " + k)
            setattr(self, k, v)


class ReshapeAndCacheParam(ctypes.Structure):
    """Byte image of atb::infer::ReshapeAndCacheParam (24 bytes)."""
    _fields_ = [("compressType", ctypes.c_int32), ("kvCacheCfg", ctypes.c_int32), ("rsv", ctypes.c_uint8 * 16)]

    def __init__(self, **kw):
        super().__init__()
        for k, v in kw.items():
            if not hasattr(self, k):
                raise AttributeError("ReshapeAndCacheParam has no field " + k)
            setattr(self, k, v)


class ReshapeAndCacheWithStrideParam(ReshapeAndCacheParam):
    """Byte image of atb::infer::ReshapeAndCacheWithStrideParam (24 bytes, the same fields)."""


class ReshapeAndCacheOmniParam(ctypes.Structure):
    """Byte image of atb::infer::ReshapeAndCacheOmniParam (8 reserved bytes)."""
    _fields_ = [("rsv", ctypes.c_uint8 * 8)]


class ElewiseParam(ctypes.Structure):
    """Byte image of atb::infer::ElewiseParam (64 bytes: type, QuantParam 32, MulsParam 16, out type, rsv)."""
    _fields_ = [("elewiseType", ctypes.c_int32), ("inputScale", ctypes.c_float), ("asymmetric", ctypes.c_bool),
                ("inputOffset", ctypes.c_int32), ("quantRsv", ctypes.c_uint8 * 20), ("varAttr", ctypes.c_float),
                ("mulsRsv", ctypes.c_uint8 * 12), ("outTensorType", ctypes.c_int32), ("rsv", ctypes.c_uint8 * 8)]
    ELEWISE_QUANT_PER_CHANNEL, ELEWISE_DEQUANT_PER_CHANNEL = 17, 18

    def __init__(self, **kw):
        super().__init__()
        self.inputScale = 1.0
        self.outTensorType = -1
        for k, v in kw.items():
            if not hasattr(self, k):
                raise AttributeError("ElewiseParam has no field " + k)
            setattr(self, k, v)


class RopeParam(ctypes.Structure):
    """Byte image of atb::infer::RopeParam (16 bytes)."""
    _fields_ = [("rotaryCoeff", ctypes.c_int32), ("cosFormat", ctypes.c_int32), ("rsv", ctypes.c_uint8 * 8)]

    def __init__(self, **kw):
        super().__init__()
        self.rotaryCoeff = 4
        for k, v in kw.items():
            if not hasattr(self, k):
                raise AttributeError("RopeParam has no field " + k)
            setattr(self, k, v)


class NormRopeReshapeParam(ctypes.Structure):
    """Byte image of atb::infer::NormRopeReshapeParam (28 bytes)."""
    _fields_ = [("precisionMode", ctypes.c_uint32), ("rotaryCoeff", ctypes.c_uint32), ("epsilon", ctypes.c_float),
                ("rsv", ctypes.c_uint8 * 16)]

    def __init__(self, **kw):
        super().__init__()
        self.rotaryCoeff = 2
        self.epsilon = 1e-5
        for k, v in kw.items():
            if not hasattr(self, k):
                raise AttributeError("NormRopeReshapeParam has no field " + k)
            setattr(self, k, v)


class BlockCopyParam(ctypes.Structure):
    """Byte image of atb::infer::BlockCopyParam (16 bytes)."""
    _fields_ = [("rsv", ctypes.c_uint8 * 16)]


class PagedCacheLoadParam(ctypes.Structure):
    """Byte image of atb::infer::PagedCacheLoadParam (64 bytes)."""
    _fields_ = [("kvCacheCfg", ctypes.c_int8), ("isSeqLensCumsumMode", ctypes.c_bool), ("hasSeqStarts", ctypes.c_bool),
                ("rsv", ctypes.c_uint8 * 61)]

    def __init__(self, **kw):
        super().__init__()
        for k, v in kw.items():
            if not hasattr(self, k):
                raise AttributeError("PagedCacheLoadParam has no field " + k)
            setattr(self, k, v)


class MultiLatentAttentionParam(ctypes.Structure):
    """Byte image of atb::infer::MultiLatentAttentionParam (64 bytes)."""
    _fields_ = [("headNum", ctypes.c_int32), ("qkScale", ctypes.c_float), ("kvHeadNum", ctypes.c_int32),
                ("maskType", ctypes.c_int32), ("calcType", ctypes.c_int32), ("cacheMode", ctypes.c_uint8),
                ("windowSize", ctypes.c_uint32), ("maskUseStatusType", ctypes.c_int32), ("rsv", ctypes.c_uint8 * 32)]

    def __init__(self, **kw):
        super().__init__()
        self.qkScale = 1.0
        for k, v in kw.items():
            if not hasattr(self, k):
                raise AttributeError("MultiLatentAttentionParam has no field " + k)
            setattr(self, k, v)


class AtbmiPaShape(ctypes.Structure):
    _fields_ = [
        ("qDtype", ctypes.c_int32), ("kvDtype", ctypes.c_int32), ("numHeads", ctypes.c_int32),
        ("numKvHeads", ctypes.c_int32), ("headDimK", ctypes.c_int32), ("headDimV", ctypes.c_int32),
        ("blockSize", ctypes.c_int32), ("numBlocks", ctypes.c_int32), ("maxBlocksPerSeq", ctypes.c_int32),
        ("numQueryRows", ctypes.c_int32), ("mlaCombined", ctypes.c_int32), ("hasOffset", ctypes.c_int32),
        ("kernel", ctypes.c_int32), ("hasMask", ctypes.c_int32), ("qkScale", ctypes.c_float),
        ("qScale", ctypes.c_float), ("maskBatchStride", ctypes.c_int64), ("maskHeadStride", ctypes.c_int64),
        ("maskLen", ctypes.c_int32), ("hasLogN", ctypes.c_int32),
        ("descalePacked", ctypes.c_int32), ("maskRowBy", ctypes.c_int32), ("ropeDim", ctypes.c_int32),
        ("kvLayout", ctypes.c_int32), ("maskSeqDiv", ctypes.c_int32), ("maskSeqMod", ctypes.c_int32),
        ("descaleHeads", ctypes.c_int32), ("hasRazorOffset", ctypes.c_int32),
    ]


class AtbmiPaTensors(ctypes.Structure):
    _fields_ = [(n, ctypes.c_void_p) for n in
                ("query", "keyCache", "valueCache", "blockTables", "kScale", "kOffset", "vScale", "vOffset", "out",
                 "mask", "logN", "queryRope", "keyRopeCache", "razorOffset", "lse")]


class AtbmiMlaPrefillCall(ctypes.Structure):
    """One atbmi_mla_prefill call (include/atbmi_kernels.h)."""
    _fields_ = [("dtype", ctypes.c_int32), ("numHeads", ctypes.c_int32), ("numKvHeads", ctypes.c_int32),
                ("mask", ctypes.c_int32), ("windowSize", ctypes.c_int32), ("qkScale", ctypes.c_float),
                ("batch", ctypes.c_int32), ("reserved", ctypes.c_int32), ("kvPaddedRows", ctypes.c_int64),
                ("hostQLens", ctypes.c_void_p), ("hostKvLens", ctypes.c_void_p), ("query", ctypes.c_void_p),
                ("queryRope", ctypes.c_void_p), ("key", ctypes.c_void_p), ("keyRope", ctypes.c_void_p),
                ("value", ctypes.c_void_p), ("out", ctypes.c_void_p)]


ATBMI_MLA_PREFILL_MASK_NONE, ATBMI_MLA_PREFILL_MASK_CAUSAL, ATBMI_MLA_PREFILL_MASK_WINDOW = 0, 1, 2


class AtbmiMlaInt8Call(ctypes.Structure):
    """One atbmi_mla_int8_decode call (include/atbmi_kernels.h)."""
    _fields_ = [("outDtype", ctypes.c_int32), ("numHeads", ctypes.c_int32), ("blockSize", ctypes.c_int32),
                ("numBlocks", ctypes.c_int32), ("maxBlocksPerSeq", ctypes.c_int32), ("batch", ctypes.c_int32),
                ("numQueryRows", ctypes.c_int32), ("hasMask", ctypes.c_int32), ("maskLen", ctypes.c_int32),
                ("qkScale", ctypes.c_float), ("hostContextLens", ctypes.c_void_p), ("hostQueryLens", ctypes.c_void_p),
                ("causalRows", ctypes.c_int32), ("hostCausalUse", ctypes.c_void_p)] + [(n, ctypes.c_void_p) for n in (
                    "query", "queryRope", "kvCache", "kRopeCache", "blockTables", "qkDescale", "pvDescale", "mask", "out",
                    "lse")]

class AtbmiPaInt8QCall(ctypes.Structure):
    """One atbmi_pa_int8q_decode call (include/atbmi_kernels.h)."""
    _fields_ = [(n, ctypes.c_int32) for n in ("outDtype", "numHeads", "numKvHeads", "headDim", "blockSize", "numBlocks",
                                              "maxBlocksPerSeq", "batch", "numQueryRows", "offline", "hasMask",
                                              "maskLen", "pieceTiles")] + [
        ("qkScale", ctypes.c_float), ("maskSeqStride", ctypes.c_int64), ("maskHeadStride", ctypes.c_int64)] + [
        (n, ctypes.c_void_p) for n in ("hostContextLens", "query", "keyCache", "valueCache", "blockTables", "kDescale",
                                       "vDescale", "pScale", "mask", "out")] + [("maskRowByQuery", ctypes.c_int32)]


class AtbmiMlaMaskFreeCall(ctypes.Structure):
    """One atbmi_mla_mask_free_expand call (include/atbmi_kernels.h)."""
    _fields_ = [("batch", ctypes.c_int32), ("numQueryRows", ctypes.c_int32), ("templateBatch", ctypes.c_int32),
                ("templateRows", ctypes.c_int32), ("maskLen", ctypes.c_int32), ("hostContextLens", ctypes.c_void_p),
                ("hostQueryLens", ctypes.c_void_p), ("maskTemplate", ctypes.c_void_p), ("outMask", ctypes.c_void_p)]


_kernels = None
_atb = None


def _load(name):
    path = os.path.join(_LIB, name)
    if not os.path.exists(path):
        raise RuntimeError("%s is not built; run `python3 %s`" % (path, os.path.join(_PKG, "build.py")))
    return ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)


def kernels():
    """libatbmi_kernels.so with argument types set."""
    global _kernels
    if _kernels is None:
        lib = _load("libatbmi_kernels.so")
        vp, i32, i64, u64 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_uint64
        lib.atbmi_last_error.restype = ctypes.c_char_p
        lib.atbmi_last_error.argtypes = []
        lib.atbmi_device_count.restype = ctypes.c_int
        lib.atbmi_reshape_and_cache.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i32, vp]
        lib.atbmi_reshape_and_cache_nz.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i32, i32, vp]
        lib.atbmi_reshape_and_cache_strided.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i32, vp, i64, vp,
                                                        i64, vp]
        lib.atbmi_reshape_and_cache_compress.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i32, vp]
        lib.atbmi_reshape_and_cache_omni.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i32, vp]
        lib.atbmi_norm_rope_reshape_and_cache.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i32,
                                                          ctypes.c_float, vp]
        lib.atbmi_rope.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i32, i32, i32, i32, vp]
        lib.atbmi_elewise_quant_per_channel.argtypes = [vp, vp, vp, vp, i64, i64, i32, vp]
        lib.atbmi_elewise_dequant_per_channel.argtypes = [vp, vp, vp, vp, i64, i64, vp]
        lib.atbmi_quant_per_channel.argtypes = [vp, i32, vp, vp, vp, i64, i64, vp]
        lib.atbmi_reshape_and_cache_quant.argtypes = [vp, vp, i32, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, vp]
        lib.atbmi_block_copy.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, vp]
        lib.atbmi_paged_cache_load.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, i64,
                                               i32, vp]
        lib.atbmi_paged_cache_load_nz.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, i64, i64, i64,
                                                  vp]
        lib.atbmi_pa_plan_create.argtypes = [ctypes.POINTER(AtbmiPaShape), ctypes.POINTER(vp)]
        lib.atbmi_pa_plan_update.argtypes = [vp, vp, i32]
        lib.atbmi_pa_plan_update_multi.argtypes = [vp, vp, vp, i32]
        lib.atbmi_pa_plan_update_multi.restype = i32
        lib.atbmi_mla_mask_free_workspace_size.argtypes = [vp, vp]
        lib.atbmi_mla_mask_free_expand.argtypes = [vp, vp, u64, vp]
        lib.atbmi_pa_plan_set_causal_rows.argtypes = [vp, i32, vp, i32]
        lib.atbmi_pa_plan_set_causal_rows.restype = i32
        lib.atbmi_pa_plan_workspace_size.argtypes = [vp]
        lib.atbmi_pa_plan_workspace_size.restype = u64
        lib.atbmi_pa_plan_num_chunks.argtypes = [vp]
        lib.atbmi_pa_plan_num_chunks.restype = i64
        lib.atbmi_pa_plan_algorithmic_bytes.argtypes = [vp]
        lib.atbmi_pa_plan_algorithmic_bytes.restype = u64
        lib.atbmi_pa_decode.argtypes = [vp, ctypes.POINTER(AtbmiPaTensors), vp, u64, vp]
        lib.atbmi_pa_decode_static.argtypes = [vp, ctypes.POINTER(AtbmiPaTensors), vp]
        lib.atbmi_pa_static_scratch_bytes.argtypes = []
        lib.atbmi_pa_static_scratch_bytes.restype = u64
        lib.atbmi_mla_prefill_workspace_size.argtypes = [ctypes.POINTER(AtbmiMlaPrefillCall), ctypes.POINTER(u64)]
        lib.atbmi_mla_prefill.argtypes = [ctypes.POINTER(AtbmiMlaPrefillCall), vp, u64, vp]
        lib.atbmi_mla_int8_workspace_size.argtypes = [ctypes.POINTER(AtbmiMlaInt8Call), ctypes.POINTER(u64)]
        lib.atbmi_mla_int8_decode.argtypes = [ctypes.POINTER(AtbmiMlaInt8Call), vp, u64, vp]
        lib.atbmi_pa_int8q_workspace_size.argtypes = [ctypes.POINTER(AtbmiPaInt8QCall), ctypes.POINTER(u64)]
        lib.atbmi_pa_int8q_decode.argtypes = [ctypes.POINTER(AtbmiPaInt8QCall), vp, u64, vp]
        lib.atbmi_pa_plan_destroy.argtypes = [vp]
        lib.atbmi_pa_plan_destroy.restype = None
        lib.atbmi_timing_enable.argtypes = [i32]
        lib.atbmi_timing_read.argtypes = [ctypes.POINTER(ctypes.c_double), ctypes.POINTER(i64)]
        lib.atbmi_timing_read_split.argtypes = [ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double),
                                                ctypes.POINTER(i64)]
        lib.atbmi_timing_read_samples.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_float), i64,
                                                  ctypes.POINTER(i64)]
        lib.atbmi_timing_whole_calls.argtypes = [i32]
        _kernels = lib
    return _kernels


def atb():
    """libatb.so (flat C view of atb::Operation) with argument types set."""
    global _atb
    if _atb is None:
        kernels()  # libatb.so depends on it
        lib = _load("libatb.so")
        vp, i32, u32, u64 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_uint32, ctypes.c_uint64
        tp = ctypes.POINTER(AtbCTensor)
        lib.atb_c_create_context.argtypes = [vp, ctypes.POINTER(vp)]
        lib.atb_c_context_set_stream.argtypes = [vp, vp]
        lib.atb_c_context_set_streams.argtypes = [vp, ctypes.POINTER(vp), u32]
        lib.atb_c_op_set_stream_id.argtypes = [vp, u32]
        lib.atb_c_op_get_stream_id.argtypes = [vp]
        lib.atb_c_op_get_stream_id.restype = u32
        lib.atb_c_context_set_execute_type.argtypes = [vp, i32]
        lib.atb_c_destroy_context.argtypes = [vp]
        lib.atb_c_create_operation.argtypes = [ctypes.c_char_p, vp, u64, ctypes.POINTER(vp)]
        lib.atb_c_destroy_operation.argtypes = [vp]
        lib.atb_c_op_input_num.argtypes = [vp]
        lib.atb_c_op_input_num.restype = u32
        lib.atb_c_op_output_num.argtypes = [vp]
        lib.atb_c_op_output_num.restype = u32
        lib.atb_c_op_name.argtypes = [vp, ctypes.c_char_p, u64]
        lib.atb_c_op_infer_shape.argtypes = [vp, tp, u32, tp, u32, ctypes.POINTER(u32)]
        lib.atb_c_op_setup.argtypes = [vp, tp, u32, tp, u32, ctypes.POINTER(u64), vp]
        lib.atb_c_op_execute.argtypes = [vp, tp, u32, tp, u32, vp, u64, vp]
        lib.atb_c_tensor_size.argtypes = [tp]
        lib.atb_c_tensor_size.restype = u64
        lib.atb_c_quant_param_convert.argtypes = [ctypes.c_void_p, ctypes.c_void_p, u64]
        lib.atb_c_quant_param_convert.restype = None
        lib.atb_c_sizeof_paged_attention_param.restype = u64
        lib.atb_c_sizeof_reshape_and_cache_param.restype = u64
        lib.atb_c_sizeof_multi_latent_attention_param.restype = u64
        # the aclnn-style tensor handle and the two-call wrappers of atb/atb_acl.h
        i64p = ctypes.POINTER(ctypes.c_int64)
        lib.aclCreateTensor.argtypes = [i64p, u64, i32, i64p, ctypes.c_int64, i32, i64p, u64, vp]
        lib.aclCreateTensor.restype = vp
        lib.aclDestroyTensor.argtypes = [vp]
        lib.aclGetDataType.argtypes = [vp, ctypes.POINTER(i32)]
        lib.aclGetFormat.argtypes = [vp, ctypes.POINTER(i32)]
        lib.aclGetRawTensorAddr.argtypes = [vp, ctypes.POINTER(vp)]
        lib.aclDataTypeSize.argtypes = [i32]
        lib.aclDataTypeSize.restype = ctypes.c_size_t
        lib.AtbMLAGetWorkspaceSize.argtypes = [vp] * 10 + [i32, ctypes.c_float, i32, ctypes.c_int, ctypes.c_int,
                                                           ctypes.c_uint8, vp, vp, ctypes.POINTER(u64),
                                                           ctypes.POINTER(vp), vp]
        lib.AtbMLA.argtypes = [vp, u64, vp, vp]
        lib.AtbMLAPreFillGetWorkspaceSize.argtypes = [vp] * 8 + [i32, ctypes.c_float, i32, ctypes.c_int, ctypes.c_uint8,
                                                                 vp, ctypes.POINTER(u64), ctypes.POINTER(vp), vp]
        lib.AtbMLAPreFill.argtypes = [vp, u64, vp, vp]
        lib.AtbPagedCacheLoadGetWorkspaceSize.argtypes = [vp] * 7 + [ctypes.c_int8, ctypes.c_bool, ctypes.c_bool,
                                                                     ctypes.POINTER(u64), ctypes.POINTER(vp), vp]
        lib.AtbPagedCacheLoad.argtypes = [vp, u64, vp, vp]
        _atb = lib
    return _atb


def acl_tensor(dtype, shape, data_ptr, fmt=ACL_FORMAT_ND):
    """aclCreateTensor for a contiguous tensor at data_ptr (device or host memory); release it with
    atb().aclDestroyTensor."""
    dims = (ctypes.c_int64 * len(shape))(*[int(d) for d in shape])
    strides = [1] * len(shape)
    for i in range(len(shape) - 2, -1, -1):
        strides[i] = strides[i + 1] * int(shape[i + 1])
    st = (ctypes.c_int64 * len(shape))(*strides)
    code = ACL_DTYPE_BY_NAME[dtype] if isinstance(dtype, str) else int(dtype)
    return atb().aclCreateTensor(dims, len(shape), code, st, 0, int(fmt), dims, len(shape), ctypes.c_void_p(data_ptr))


def acl_tensor_of(t):
    """aclTensor handle of a contiguous torch tensor (a CPU tensor gives a host address)."""
    return acl_tensor(_torch_acl_dtype(t), list(t.shape), t.data_ptr())


def last_kernel_error():
    return kernels().atbmi_last_error().decode()


def make_tensor(dtype, shape, device_ptr=None, host_ptr=None, fmt=ACL_FORMAT_ND, data_size=None):
    """AtbCTensor from raw pieces; dataSize defaults to Utils::GetTensorSize."""
    t = AtbCTensor()
    t.dtype = ACL_DTYPE_BY_NAME[dtype] if isinstance(dtype, str) else int(dtype)
    t.format = ACL_FORMAT_BY_NAME[fmt] if isinstance(fmt, str) else int(fmt)
    t.dimNum = len(shape)
    for i, d in enumerate(shape[:8]):
        t.dims[i] = int(d)
    t.deviceData = device_ptr
    t.hostData = host_ptr
    t.dataSize = atb().atb_c_tensor_size(ctypes.byref(t)) if data_size is None else int(data_size)
    return t


def _torch_acl_dtype(t):
    import torch
    return {torch.float16: ACL_FLOAT16, torch.bfloat16: ACL_BF16, torch.int8: ACL_INT8, torch.int32: ACL_INT32,
            torch.float32: ACL_FLOAT, torch.int64: ACL_INT64}[t.dtype]


def tensor_of(t, host=None):
    """AtbCTensor describing a contiguous torch tensor on the GPU; `host` is an
    optional contiguous CPU tensor bound as hostData (contextLens)."""
    if not t.is_contiguous():
        raise ValueError("tensor must be contiguous")
    c = make_tensor(_torch_acl_dtype(t), list(t.shape), device_ptr=t.data_ptr() if t.is_cuda else None,
                    host_ptr=(host.data_ptr() if host is not None else (None if t.is_cuda else t.data_ptr())))
    return c


class Context:
    """atb::Context bound to a HIP stream (a torch.cuda.Stream or a raw handle)."""

    def __init__(self, stream):
        self.stream = stream
        handle = stream.cuda_stream if hasattr(stream, "cuda_stream") else stream
        self.ptr = ctypes.c_void_p()
        st = atb().atb_c_create_context(ctypes.c_void_p(handle), ctypes.byref(self.ptr))
        if st != 0:
            raise RuntimeError("CreateContext failed: %s" % ERROR_NAMES[st])

    def set_execute_type(self, t):
        return atb().atb_c_context_set_execute_type(self.ptr, int(t))

    def set_streams(self, streams):
        """Context::SetExecuteStreams: torch streams or raw handles; an operation picks one by its stream id."""
        handles = [s.cuda_stream if hasattr(s, "cuda_stream") else s for s in streams]
        arr = (ctypes.c_void_p * max(1, len(handles)))(*handles)
        self.streams = list(streams)  # (kept alive)
        return atb().atb_c_context_set_streams(self.ptr, arr, len(handles))

    def close(self):
        if self.ptr:
            atb().atb_c_destroy_context(self.ptr)
            self.ptr = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Operation:
    """An atb::Operation created from a param struct. create() returns the status
    instead of raising, so error-path tests can read it."""

    def __init__(self, name, param):
        self.name = name
        self.param = param
        self.ptr = ctypes.c_void_p()
        self.status = atb().atb_c_create_operation(name.encode(), ctypes.byref(param), ctypes.sizeof(param),
                                                   ctypes.byref(self.ptr))
        self._keep = None

    @property
    def ok(self):
        return self.status == 0 and bool(self.ptr)

    def set_stream_id(self, stream_id):
        return atb().atb_c_op_set_stream_id(self.ptr, int(stream_id))

    def get_stream_id(self):
        return atb().atb_c_op_get_stream_id(self.ptr)

    def input_num(self):
        return atb().atb_c_op_input_num(self.ptr)

    def output_num(self):
        return atb().atb_c_op_output_num(self.ptr)

    def get_name(self):
        buf = ctypes.create_string_buffer(128)
        atb().atb_c_op_name(self.ptr, buf, 128)
        return buf.value.decode()

    def infer_shape(self, in_descs):
        arr = (AtbCTensor * max(1, len(in_descs)))(*in_descs)
        out = (AtbCTensor * 8)()
        n = ctypes.c_uint32(0)
        st = atb().atb_c_op_infer_shape(self.ptr, arr, len(in_descs), out, 8, ctypes.byref(n))
        return st, [out[i] for i in range(n.value)] if st == 0 else []

    def setup(self, in_tensors, out_tensors, context):
        ia = (AtbCTensor * max(1, len(in_tensors)))(*in_tensors)
        oa = (AtbCTensor * max(1, len(out_tensors)))(*out_tensors)
        ws = ctypes.c_uint64(0)
        ctx = context.ptr if isinstance(context, Context) else context
        st = atb().atb_c_op_setup(self.ptr, ia, len(in_tensors), oa, len(out_tensors), ctypes.byref(ws), ctx)
        return st, ws.value

    def execute(self, in_tensors, out_tensors, workspace_ptr, workspace_size, context):
        ia = (AtbCTensor * max(1, len(in_tensors)))(*in_tensors)
        oa = (AtbCTensor * max(1, len(out_tensors)))(*out_tensors)
        ctx = context.ptr if isinstance(context, Context) else context
        return atb().atb_c_op_execute(self.ptr, ia, len(in_tensors), oa, len(out_tensors),
                                      ctypes.c_void_p(workspace_ptr), workspace_size, ctx)

    def close(self):
        if self.ptr:
            atb().atb_c_destroy_operation(self.ptr)
            self.ptr = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class OperationRunner:
    """Runs one operation on torch GPU tensors the way the reference harness does:
    InferShape -> allocate outputs (or take caller-owned ones) -> Setup ->
    workspace -> Execute. The workspace tensor is kept and grown on demand."""

    def __init__(self, name, param, context):
        self.op = Operation(name, param)
        if not self.op.ok:
            raise RuntimeError("CreateOperation(%s) failed: %s" % (name, ERROR_NAMES[self.op.status]))
        self.context = context
        self.workspace = None

    def run(self, inputs, outputs=None, host_inputs=None):
        """inputs: torch GPU tensors (or ready-made AtbCTensor descriptions, for a view whose shape
        is not the tensor's own); host_inputs: {index: CPU tensor} bound as
        hostData; outputs: caller-owned output tensors (in-place cache update; torch tensors or
        ready-made AtbCTensor descriptions) or None to allocate from InferShape. Returns the output tensors."""
        import torch
        host_inputs = host_inputs or {}
        ins = [t if isinstance(t, AtbCTensor) else tensor_of(t, host_inputs.get(i)) for i, t in enumerate(inputs)]
        if outputs is None:
            st, descs = self.op.infer_shape(ins)
            if st != 0:
                raise RuntimeError("InferShape failed: %s" % ERROR_NAMES[st])
            rev = {ACL_FLOAT16: torch.float16, ACL_BF16: torch.bfloat16, ACL_INT8: torch.int8, ACL_FLOAT: torch.float32}
            outputs = [torch.empty([d.dims[i] for i in range(d.dimNum)], dtype=rev[d.dtype], device=inputs[0].device)
                       for d in descs]
        outs = [t if isinstance(t, AtbCTensor) else tensor_of(t) for t in outputs]
        st, ws = self.op.setup(ins, outs, self.context)
        if st != 0:
            raise RuntimeError("Setup failed: %s" % ERROR_NAMES[st])
        if ws > 0 and (self.workspace is None or self.workspace.numel() < ws):
            self.workspace = torch.empty(int(ws), dtype=torch.uint8, device=inputs[0].device)
        wptr = self.workspace.data_ptr() if ws > 0 else None
        st = self.op.execute(ins, outs, wptr, ws, self.context)
        if st != 0:
            raise RuntimeError("Execute failed: %s (%s)" % (ERROR_NAMES[st], last_kernel_error()))
        return outputs

    def close(self):
        self.op.close()
