"""The `torch_atb` Python surface of the reference for the operators this library has:
`Operation(param).forward([tensors]) -> [tensors]` with `name`, `input_num`, `output_num`, and
parameter classes with snake_case fields and nested enums
(reference src/torch_atb/bindings.cpp:49-93 Operation, :520-590 PagedAttentionParam,
:926-944 ReshapeAndCacheParam; src/torch_atb/operation_wrapper.cpp:230-311 forward = Setup + Execute +
stream synchronisation; src/torch_atb/resource/utils.cpp:53-90: a CPU tensor is bound as hostData,
any other tensor as deviceData).

    import importlib
    torch_atb = importlib.import_module("ascend-transformer-boost_amd").torch_atb
    op = torch_atb.Operation(torch_atb.PagedAttentionParam(head_num=32, kv_head_num=8, qk_scale=0.088))
    out, = op.forward([q, key_cache, value_cache, block_tables, context_lens_cpu])

Differences from the reference module, all forced by the operators themselves: tensors live on a ROCm
device ("cuda" in torch); the work runs on torch's current stream of the first device tensor (on a side
stream ordered after it when that is the null stream, which a Context does not take); operators
whose outputs are their inputs updated in place (ReshapeAndCache, NormRopeReshape, PagedCacheLoad) return those input
tensors instead of fresh ones. ReshapeAndCacheWithStrideParam, ReshapeAndCacheOmniParam, NormRopeReshapeParam,
MultiLatentAttentionParam, BlockCopyParam and PagedCacheLoadParam are not bound by the reference's module; they are offered here in the same style
(for ReshapeAndCacheWithStride, key / value are [tokens, heads, head_size] tensors that start at the base
of the storage which the strides and the offset index into).
"""
import enum
import re

from . import binding as _b


def _snake(name):
    return re.sub(r"(?<!^)(?=[A-Z])", "_", name).lower()


class _Param:
    """Base of the parameter classes: snake_case attributes over the byte image of the C++ struct."""
    _struct = None
    _op_name = None

    def __init__(self, **kwargs):
        object.__setattr__(self, "_c", self._struct())
        object.__setattr__(self, "_names", {_snake(f[0]): f[0] for f in self._struct._fields_ if f[0] != "rsv"})
        for k, v in kwargs.items():
            setattr(self, k, v)

    def __getattr__(self, key):
        names = object.__getattribute__(self, "_names")
        if key in names:
            return getattr(object.__getattribute__(self, "_c"), names[key])
        raise AttributeError(key)

    def __setattr__(self, key, value):
        if key not in self._names:
            raise AttributeError("%s has no field %s" % (type(self).__name__, key))
        setattr(self._c, self._names[key], int(value) if isinstance(value, enum.Enum) else value)

    def __repr__(self):
        return "%s: {%s}" % (type(self).__name__, ", ".join("%s: %r" % (k, getattr(self, k)) for k in self._names))


class InputLayout(enum.IntEnum):
    TYPE_BSND = 0
    TYPE_BNSD = 1


class PagedAttentionParam(_Param):
    _struct = _b.PagedAttentionParam
    _op_name = "PagedAttentionOperation"

    class MaskType(enum.IntEnum):
        UNDEFINED = 0
        MASK_TYPE_NORM = 1
        MASK_TYPE_ALIBI = 2
        MASK_TYPE_SPEC = 3

    class QuantType(enum.IntEnum):
        TYPE_QUANT_UNQUANT = 0
        TYPE_DEQUANT_FUSION = 1
        TYPE_QUANT_QKV_OFFLINE = 2
        TYPE_QUANT_QKV_ONLINE = 3

    class CompressType(enum.IntEnum):
        COMPRESS_TYPE_UNDEFINED = 0
        COMPRESS_TYPE_KVHEAD = 1
        COMPRESS_TYPE_KVHEAD_ROPE = 2
        COMPRESS_TYPE_MAX = 3

    class CalcType(enum.IntEnum):
        CALC_TYPE_UNDEFINED = 0
        CALC_TYPE_SPEC = 1

    class ScaleType(enum.IntEnum):
        SCALE_TYPE_TOR = 0
        SCALE_TYPE_LOGN = 1
        SCALE_TYPE_MAX = 2


class ReshapeAndCacheParam(_Param):
    _struct = _b.ReshapeAndCacheParam
    _op_name = "ReshapeAndCacheOperation"

    class CompressType(enum.IntEnum):
        COMPRESS_TYPE_UNDEFINED = 0
        COMPRESS_TYPE_KVHEAD = 1
        COMPRESS_TYPE_KVHEAD_ROPE = 2

    class KvCacheCfg(enum.IntEnum):
        K_CACHE_V_CACHE = 0
        K_CACHE_V_BYPASS = 1
        K_CACHE_V_CACHE_NZ = 2


class ReshapeAndCacheWithStrideParam(_Param):
    _struct = _b.ReshapeAndCacheWithStrideParam
    _op_name = "ReshapeAndCacheWithStrideOperation"

    class CompressType(enum.IntEnum):
        COMPRESS_TYPE_UNDEFINED = 0
        COMPRESS_TYPE_KVHEAD = 1
        COMPRESS_TYPE_KVHEAD_ROPE = 2

    class KvCacheCfg(enum.IntEnum):
        K_CACHE_V_CACHE = 0
        K_CACHE_V_BYPASS = 1


class ReshapeAndCacheOmniParam(_Param):
    _struct = _b.ReshapeAndCacheOmniParam
    _op_name = "ReshapeAndCacheOmniOperation"


class ElewiseParam(_Param):
    _struct = _b.ElewiseParam
    _op_name = "ElewiseOperation"

    class ElewiseType(enum.IntEnum):
        ELEWISE_QUANT_PER_CHANNEL = 17
        ELEWISE_DEQUANT_PER_CHANNEL = 18


class RopeParam(_Param):
    _struct = _b.RopeParam
    _op_name = "RopeOperation"


class NormRopeReshapeParam(_Param):
    _struct = _b.NormRopeReshapeParam
    _op_name = "NormRopeReshapeOperation"


class MultiLatentAttentionParam(_Param):
    _struct = _b.MultiLatentAttentionParam
    _op_name = "MultiLatentAttentionOperation"

    class MaskType(enum.IntEnum):
        UNDEFINED = 0
        MASK_TYPE_SPEC = 1
        MASK_TYPE_MASK_FREE = 2
        MASK_TYPE_CAUSAL_MASK = 3
        MASK_TYPE_SWA_NORM = 4

    class CalcType(enum.IntEnum):
        CALC_TYPE_UNDEFINED = 0
        CALC_TYPE_SPEC = 1
        CALC_TYPE_RING = 2
        CALC_TYPE_SPEC_AND_RING = 3
        CALC_TYPE_PREFILL = 4

    class CacheMode(enum.IntEnum):
        KVCACHE = 0
        KROPE_CTKV = 1
        INT8_NZCACHE = 2
        NZCACHE = 3


class BlockCopyParam(_Param):
    _struct = _b.BlockCopyParam
    _op_name = "BlockCopyOperation"


class PagedCacheLoadParam(_Param):
    _struct = _b.PagedCacheLoadParam
    _op_name = "PagedCacheLoadOperation"

    class KvCacheCfg(enum.IntEnum):
        K_CACHE_V_CACHE_NZ = 0
        K_CACHE_V_CACHE_ND = 1


# operation name -> indices of the inputs that its outputs are (updated in place), by input count
_IN_PLACE = {
    "ReshapeAndCacheOperation": {5: [2, 3], 3: [1], 7: [2, 3], 8: [2, 3]},  # 7 / 8: head compression
    "ReshapeAndCacheWithStrideOperation": {9: [2, 3], 5: [1]},
    "ReshapeAndCacheOmniOperation": {8: [2, 3]},
    "NormRopeReshapeOperation": {7: [6]},
    "PagedCacheLoadOperation": {7: [4, 5]},
}


class Operation:
    """An operator created from its parameter object; forward() runs it once."""

    def __init__(self, param):
        if not isinstance(param, _Param):
            raise TypeError("Operation() takes one of this module's parameter objects")
        self._op = _b.Operation(param._op_name, param._c)
        if not self._op.ok:
            raise RuntimeError("create operation fail: %s" % _b.ERROR_NAMES[self._op.status])
        self._contexts = {}
        self._side_streams = {}
        self._workspace = None

    @property
    def name(self):
        return self._op.get_name()

    @property
    def input_num(self):
        return self._op.input_num()

    @property
    def output_num(self):
        return self._op.output_num()

    def __repr__(self):
        return "op name: %s, input_num: %d, output_num: %d" % (self.name, self.input_num, self.output_num)

    def forward(self, in_tensors):
        import torch
        in_tensors = [t if t.is_contiguous() else t.contiguous() for t in in_tensors]
        device = next((t.device for t in in_tensors if t.is_cuda), None)
        if device is None:
            raise RuntimeError("call Forward fail, no input lives on the device")
        current = torch.cuda.current_stream(device)
        stream = current
        if current.cuda_stream == 0:
            # a Context wants a stream handle that is not null, and torch's default stream is the null
            # stream: run on a stream of this operation's own, ordered after the current one
            if device.index not in self._side_streams:
                self._side_streams[device.index] = torch.cuda.Stream(device=device)
            stream = self._side_streams[device.index]
            stream.wait_stream(current)
        key = (device.index, stream.cuda_stream)
        if key not in self._contexts:
            self._contexts[key] = _b.Context(stream)
        context = self._contexts[key]
        ins = [_b.tensor_of(t) for t in in_tensors]
        aliased = _IN_PLACE.get(self.name, {}).get(len(in_tensors))
        if aliased is not None:
            outputs = [in_tensors[i] for i in aliased]
        else:
            st, descs = self._op.infer_shape(ins)
            if st != 0:
                raise RuntimeError("call operation_->InferShape fail: %s" % _b.ERROR_NAMES[st])
            rev = {_b.ACL_FLOAT16: torch.float16, _b.ACL_BF16: torch.bfloat16, _b.ACL_INT8: torch.int8}
            outputs = [torch.empty([d.dims[i] for i in range(d.dimNum)], dtype=rev[d.dtype], device=device)
                       for d in descs]
        outs = [_b.tensor_of(t) for t in outputs]
        st, ws = self._op.setup(ins, outs, context)
        if st != 0:
            raise RuntimeError("call operation_->Setup fail: %s" % _b.ERROR_NAMES[st])
        if ws > 0 and (self._workspace is None or self._workspace.numel() < ws or self._workspace.device != device):
            with torch.cuda.stream(stream):
                self._workspace = torch.empty(int(ws), dtype=torch.uint8, device=device)
        st = self._op.execute(ins, outs, self._workspace.data_ptr() if ws > 0 else None, ws, context)
        if st != 0:
            raise RuntimeError("call operation_->Execute fail: %s (%s)" % (_b.ERROR_NAMES[st], _b.last_kernel_error()))
        stream.synchronize()
        return outputs

    def close(self):
        self._op.close()
        for c in self._contexts.values():
            c.close()
        self._contexts = {}
