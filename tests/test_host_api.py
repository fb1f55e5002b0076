"""Host-side behaviour of the atb::Operation layer, without a GPU.

The expected statuses come from the reference's own operator-API test tables
(tests/golden/*_cases.json, extracted from the reference CSVs by
tests/golden/make_csv_fixtures.py): one row = param + input/output
descriptions + the status the reference returns, tagged with the stage
(C: CreateOperation, I: InferShape, S: Setup). Setup never touches device
memory, so fake device addresses are enough here.
"""
import ctypes
import json
import os
import subprocess

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
FAKE_DEVICE = 0x10000


def _load(name):
    with open(os.path.join(HERE, "golden", name + "_cases.json")) as f:
        return json.load(f)["cases"]


PA_CASES = _load("paged_attention")
RAC_CASES = _load("reshape_and_cache")
MLA_CASES = _load("multi_latent_attention")
BLOCK_COPY_CASES = _load("block_copy")
CACHE_LOAD_CASES = _load("paged_cache_load")
NORM_ROPE_CASES = _load("norm_rope_reshape")
ROPE_CASES = _load("rope")
ELEWISE_CASES = _load("elewise")
OMNI_CASES = _load("reshape_and_cache_omni")


def _pa_unimplemented(p):
    """Features of PagedAttentionParam the reference accepts but this library rejects at creation: int8 queries
    (quantType QKV online / offline) together with the MLA cache."""
    return p.get("quantType", 0) >= 2 and p.get("mlaVHeadSize", 0) > 0


def _pa_mask_shape_refused(case):
    """Mask shapes the reference operation lets through Setup although its kernel would read past the
    tensor with them: a 3-dim ALIBI mask whose first dim is not the head count (the tiling makes the row length the
    head stride, tiling/paged_attention_tiling.cpp:43-47; the kernel library's own shape list has no such entry,
    paged_attention_operation.cpp:749-761), and with several query tokens per sequence (calcType 1) a NORM mask that
    is not the square causal one (the second query token of a sequence would read the next sequence's row, the last
    sequence's past the end). Refused here during Setup. (The 4-dim NORM mask, for which the tiling derives no
    strides, is taken as the reference's kernel reads it: the first row for everyone.)"""
    p = case["param"]
    if p.get("maskType", 0) not in (1, 2, 3) or _pa_unimplemented(p) or case["expected"] != "NO_ERROR":
        return False
    mask = case["in_shapes"][4 if p.get("mlaVHeadSize", 0) > 0 else 5]
    if p.get("calcType", 0) == 1:
        if p["maskType"] == 3:
            return not (len(mask) == 2 and mask[0] == case["in_shapes"][0][0])
        return not (len(mask) == 2 and mask[0] == mask[1])
    if p["maskType"] == 1:
        return False
    return len(mask) == 3 and mask[0] != p["headNum"]


def _rac_unimplemented(p):
    """Features of ReshapeAndCacheParam the reference accepts but this library rejects at creation: none."""
    return False


def _mla_unimplemented(p):
    """Features of MultiLatentAttentionParam the reference accepts but this library rejects at creation: none
    (MASK_TYPE_MASK_FREE with fewer than 128 heads is refused at Setup, which no table row reaches)."""
    return False


def _make_param(binding, op, p):
    cls = {"PagedAttentionOperation": binding.PagedAttentionParam,
           "MultiLatentAttentionOperation": binding.MultiLatentAttentionParam,
           "BlockCopyOperation": binding.BlockCopyParam,
           "PagedCacheLoadOperation": binding.PagedCacheLoadParam,
           "ReshapeAndCacheWithStrideOperation": binding.ReshapeAndCacheWithStrideParam,
           "ReshapeAndCacheOmniOperation": binding.ReshapeAndCacheOmniParam,
           "NormRopeReshapeOperation": binding.NormRopeReshapeParam,
           "RopeOperation": binding.RopeParam,
           "ElewiseOperation": binding.ElewiseParam,
           "ReshapeAndCacheOperation": binding.ReshapeAndCacheParam}[op]
    fields = {k: v for k, v in p.items() if k != "rsv"}
    param = cls(**fields) if fields else cls()
    for i, v in enumerate(p.get("rsv", [])):  # a row may set reserved bytes to see them refused
        param.rsv[i] = v
    return param


def _tensors(binding, dtypes, formats, shapes, host_arrays=None):
    """host_arrays: {input index: numpy array bound as hostData}."""
    out = []
    for i, (dt, fmt, shape) in enumerate(zip(dtypes, formats, shapes)):
        host = host_arrays[i].ctypes.data if host_arrays and i in host_arrays else None
        dt = {"float32": "float"}.get(dt, dt)  # the reference table spells ACL_FLOAT both ways
        out.append(binding.make_tensor(dt, shape, device_ptr=FAKE_DEVICE, host_ptr=host, fmt=fmt))
    return out


def _run_case(binding, case, ctx):
    """Returns (stage, status) of the first failing stage, or ("", 0)."""
    op = binding.Operation(case["op"], _make_param(binding, case["op"], case["param"]))
    if op.status != 0:
        return "C", op.status, None
    try:
        ins = _tensors(binding, case["in_dtypes"], case["in_formats"], case["in_shapes"])
        st, out_descs = op.infer_shape(ins)
        if st != 0:
            return "I", st, None
        host = {}
        if case["op"] == "PagedAttentionOperation":
            p = case["param"]
            lens_index = 3 if p.get("mlaVHeadSize", 0) > 0 else 4
            kc = case["in_shapes"][1]
            tables = case["in_shapes"][lens_index - 1]
            host[lens_index] = np.full((case["in_shapes"][lens_index][0],), min(kc[1] * tables[1], 7), dtype=np.int32)
            if p.get("batchRunStatusEnable", False):
                status_index = lens_index + (2 if p.get("maskType", 0) != 0 else 1)
                if status_index < len(case["in_shapes"]):
                    host[status_index] = np.ones((case["in_shapes"][status_index][0],), dtype=np.int32)
            if p.get("calcType", 0) == 1:
                qlens_index = lens_index + (2 if p.get("maskType", 0) != 0 else 1)
                if qlens_index < len(case["in_shapes"]):
                    host[qlens_index] = np.ones((case["in_shapes"][qlens_index][0],), dtype=np.int32)
        if case["op"] == "MultiLatentAttentionOperation" and case["param"].get("calcType", 0) == 4:
            # prefill: qSeqLen and kvSeqLen are host tensors; one sequence that fills the query
            for i in (5, 6):
                if i < len(case["in_shapes"]) and len(case["in_shapes"][i]) == 1:
                    host[i] = np.full((case["in_shapes"][i][0],), 1, dtype=np.int32)
        elif case["op"] == "MultiLatentAttentionOperation" and len(case["in_shapes"]) > 5:
            host[5] = np.full((case["in_shapes"][5][0],), 7, dtype=np.int32)
            if case["param"].get("calcType", 0) in (1, 3):
                host[len(case["in_shapes"]) - 1] = np.ones((case["in_shapes"][-1][0],), dtype=np.int32)
        ins = _tensors(binding, case["in_dtypes"], case["in_formats"], case["in_shapes"], host)
        outs = _tensors(binding, case["out_dtypes"], case["out_formats"], case["out_shapes"])
        st, _ = op.setup(ins, outs, ctx)
        if st != 0:
            return "S", st, out_descs
        return "", 0, out_descs
    finally:
        op.close()


@pytest.fixture(scope="module")
def ctx(binding):
    c = binding.Context(0x1)  # any non-null handle: Setup never uses the stream
    yield c
    c.close()


def _check(binding, case, ctx, unimplemented, refused_at_setup=False):
    stage, status, out_descs = _run_case(binding, case, ctx)
    expected = case["expected"]
    if unimplemented:
        # documented deviation: rejected when the operation is created
        assert (stage, status) == ("C", binding.ERROR_CODE["ERROR_INVALID_PARAM"])
        return
    if refused_at_setup:
        assert (stage, status) == ("S", binding.ERROR_CODE["ERROR_INVALID_PARAM"])
        return
    if expected == "NO_ERROR":
        assert (stage, status) == ("", 0), "%s: %s:%s" % (case["name"], stage, binding.ERROR_NAMES[status])
        got = [[d.dims[i] for i in range(d.dimNum)] for d in out_descs]
        assert got == case["out_shapes"]
        return
    if expected == "I:NO_ERROR":
        # the row only asks InferShape to succeed (its output shapes are not the operation's)
        assert stage not in ("C", "I"), "%s: %s:%s" % (case["name"], stage, binding.ERROR_NAMES[status])
        return
    want_stage, want_name = expected.split(":")
    assert stage == want_stage and binding.ERROR_NAMES[status] == want_name, \
        "%s: got %s:%s want %s" % (case["name"], stage, binding.ERROR_NAMES[status], expected)


@pytest.mark.parametrize("case", PA_CASES, ids=lambda c: "%d-%s" % (c["case"], c["name"]))
def test_paged_attention_table(binding, ctx, case):
    _check(binding, case, ctx, _pa_unimplemented(case["param"]) and not case["expected"].startswith("C:"),
           _pa_mask_shape_refused(case))


@pytest.mark.parametrize("case", MLA_CASES, ids=lambda c: "%d-%s" % (c["case"], c["name"]))
def test_multi_latent_attention_table(binding, ctx, case):
    _check(binding, case, ctx, _mla_unimplemented(case["param"]) and not case["expected"].startswith("C:"))


@pytest.mark.parametrize("case", BLOCK_COPY_CASES, ids=lambda c: "%d-%s" % (c["case"], c["name"]))
def test_block_copy_table(binding, ctx, case):
    _check(binding, case, ctx, False)


@pytest.mark.parametrize("case", CACHE_LOAD_CASES, ids=lambda c: "%d-%s" % (c["case"], c["name"]))
def test_paged_cache_load_table(binding, ctx, case):
    _check(binding, case, ctx, False)


@pytest.mark.parametrize("case", ELEWISE_CASES, ids=lambda c: "%d-%s" % (c["case"], c["name"]))
def test_elewise_per_channel_table(binding, ctx, case):
    _check(binding, case, ctx, False)


def test_elewise_checks(binding, ctx):
    """Creation (reference elewise_operation.cpp:40-99), the optional offset (:474-486) and what the kernel
    needs of the shapes."""
    E = binding.ERROR_CODE
    P = binding.ElewiseParam
    assert ctypes.sizeof(P) == 64   # reference tests/unittest/ops/test_op_param_size.cpp:25
    for t in (0, 21, 22, -1):       # out of range
        assert binding.Operation("ElewiseOperation", P(elewiseType=t)).status == E["ERROR_INVALID_PARAM"]
    for t in (1, 2, 6, 8, 19, 20):  # in range, not built here
        assert binding.Operation("ElewiseOperation", P(elewiseType=t)).status == E["ERROR_INVALID_PARAM"]
    for field in ("rsv", "quantRsv", "mulsRsv"):
        p = P(elewiseType=17)
        getattr(p, field)[1] = 1
        assert binding.Operation("ElewiseOperation", p).status == E["ERROR_INVALID_PARAM"]
    mk = binding.make_tensor
    op = binding.Operation("ElewiseOperation", P(elewiseType=17))
    assert op.get_name() == "ElewiseOperation" and (op.input_num(), op.output_num()) == (3, 1)
    ins = lambda x=(10, 8192), s=(8192,), o=(8192,): [mk("float16", x, FAKE_DEVICE), mk("float16", s, FAKE_DEVICE),
                                                     mk("int8", o, FAKE_DEVICE)]
    out = lambda shape=(10, 8192): [mk("int8", shape, FAKE_DEVICE)]
    st, descs = op.infer_shape(ins())
    assert st == 0 and descs[0].dtype == binding.ACL_INT8 and [descs[0].dims[i] for i in range(2)] == [10, 8192]
    assert op.setup(ins(), out(), ctx) == (0, 0)
    # the offset may be an empty tensor; nothing else may
    assert op.infer_shape(ins(o=(0,)))[0] == 0 and op.setup(ins(o=(0,)), out(), ctx) == (0, 0)
    assert op.infer_shape(ins(s=(0,)))[0] == E["ERROR_INVALID_TENSOR_SIZE"]
    # scale / offset must tile x, the output must have x's size
    assert op.setup(ins(s=(100,), o=(100,)), out(), ctx)[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.setup(ins(o=(4096,)), out(), ctx)[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.setup(ins(), out((10, 4096)), ctx)[0] == E["ERROR_INVALID_TENSOR_DIM"]
    op.close()
    op = binding.Operation("ElewiseOperation", P(elewiseType=18))
    d_ins = [mk("int8", (10, 64), FAKE_DEVICE), mk("float16", (64,), FAKE_DEVICE), mk("int8", (64,), FAKE_DEVICE)]
    st, descs = op.infer_shape(d_ins)
    assert st == 0 and descs[0].dtype == binding.ACL_FLOAT16
    bf = [mk("int8", (10, 64), FAKE_DEVICE), mk("bf16", (64,), FAKE_DEVICE), mk("int8", (64,), FAKE_DEVICE)]
    assert op.infer_shape(bf)[0] == E["ERROR_INVALID_TENSOR_INI_MATCH"]
    op.close()


@pytest.mark.parametrize("case", ROPE_CASES, ids=lambda c: "%d-%s" % (c["case"], c["name"]))
def test_rope_table(binding, ctx, case):
    _check(binding, case, ctx, False)


@pytest.mark.parametrize("case", NORM_ROPE_CASES, ids=lambda c: "%d-%s" % (c["case"], c["name"]))
def test_norm_rope_reshape_table(binding, ctx, case):
    _check(binding, case, ctx, False)


@pytest.mark.parametrize("case", RAC_CASES, ids=lambda c: "%d-%s" % (c["case"], c["name"]))
def test_reshape_and_cache_table(binding, ctx, case):
    _check(binding, case, ctx, _rac_unimplemented(case["param"]) and not case["expected"].startswith("C:"))


@pytest.mark.parametrize("case", OMNI_CASES, ids=lambda c: "%d-%s" % (c["csv_line"], c["name"]))
def test_reshape_and_cache_omni_table(binding, ctx, case):
    _check(binding, case, ctx, False)


def test_reshape_and_cache_omni_checks(binding, ctx):
    """What the reference's table (all refusals) leaves open: the name and tensor counts
    (reshape_and_cache_omni_operation.cpp:45,53-64), a pack that passes (shapes of the golden,
    tests/apitest/opstest/python/operations/reshape_and_cache_omni/test_reshape_and_cache_omni.py:134-150),
    the outputs taking the caches' descs (:77-83), each dim rule of :101-152 and the Setup rule of :164-169."""
    E = binding.ERROR_CODE
    P = binding.ReshapeAndCacheOmniParam
    assert ctypes.sizeof(P) == 8   # reference include/atb/infer_op_params.h:2889-2894
    op = binding.Operation("ReshapeAndCacheOmniOperation", P())
    assert op.status == 0 and op.get_name() == "ReshapeAndCacheOmniOperation"
    assert (op.input_num(), op.output_num()) == (8, 2)
    mk = binding.make_tensor

    def ins(dtype="float16", tokens=600, heads=4, d=128, batch=2, blocks=64, block=128, **over):
        shapes = {"key": [tokens, heads, d], "value": [tokens, heads, d], "kc": [blocks, block, 1, d],
                  "vc": [blocks, block, 1, d], "slots": [batch * heads], "wins": [batch * heads], "seq": [batch],
                  "offs": [batch * heads]}
        shapes.update(over)
        types = [dtype] * 4 + ["int32"] * 4
        return [mk(t, shapes[n], FAKE_DEVICE) for t, n in zip(types, ("key", "value", "kc", "vc", "slots", "wins",
                                                                     "seq", "offs"))]

    def outs(dtype="float16", kc=(64, 128, 1, 128), vc=(64, 128, 1, 128)):
        return [mk(dtype, list(kc), FAKE_DEVICE), mk(dtype, list(vc), FAKE_DEVICE)]

    for dtype in ("float16", "bf16"):
        st, descs = op.infer_shape(ins(dtype))
        assert st == 0 and [[d.dims[i] for i in range(d.dimNum)] for d in descs] == [[64, 128, 1, 128]] * 2
        assert op.setup(ins(dtype), outs(dtype), ctx) == (0, 0)
    assert op.infer_shape(ins("int8"))[0] == E["ERROR_INVALID_TENSOR_INI_MATCH"]
    assert op.infer_shape(ins(key=[600, 512]))[0] == E["ERROR_INVALID_TENSOR_DIM_NUM"]
    assert op.infer_shape(ins(seq=[2, 1]))[0] == E["ERROR_INVALID_TENSOR_DIM_NUM"]
    bad = [dict(d=48, kc=[64, 128, 1, 48], vc=[64, 128, 1, 48], key=[600, 4, 48], value=[600, 4, 48]),  # 32 | headSize
           dict(value=[599, 4, 128]), dict(value=[600, 2, 128]), dict(slots=[7]), dict(wins=[9]), dict(offs=[4]),
           dict(value=[600, 4, 64]), dict(kc=[64, 128, 1, 64]), dict(vc=[64, 128, 1, 256]), dict(vc=[32, 128, 1, 128]),
           dict(vc=[64, 64, 1, 128]), dict(kc=[64, 128, 2, 128]), dict(vc=[64, 128, 4, 128]),
           dict(batch=125)]  # 125 * 4 = 500 pairs
    for over in bad:
        assert op.infer_shape(ins(**over))[0] == E["ERROR_INVALID_TENSOR_DIM"], over
    assert op.infer_shape(ins(batch=124, tokens=1000))[0] == 0   # 496 pairs
    assert op.setup(ins(value=[599, 4, 128]), outs(), ctx)[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.setup(ins(), outs(kc=(64, 128, 1, 64)), ctx)[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.setup(ins(), outs("bf16"), ctx)[0] != 0
    op.close()
    p = P()
    p.rsv[7] = 1
    assert binding.Operation("ReshapeAndCacheOmniOperation", p).status == E["ERROR_INVALID_PARAM"]


def test_table_coverage():
    """Most rows of the reference tables must be checked at face value, not as deviations."""
    pa_dev = [c for c in PA_CASES if (_pa_unimplemented(c["param"]) and not c["expected"].startswith("C:")) or
              _pa_mask_shape_refused(c)]
    rac_dev = [c for c in RAC_CASES if _rac_unimplemented(c["param"]) and not c["expected"].startswith("C:")]
    assert len(PA_CASES) == 81 and len(PA_CASES) - len(pa_dev) == 78   # (3 mask shapes refused at Setup)
    assert len(RAC_CASES) == 38 and len(rac_dev) == 0
    # every MultiLatentAttention row is replayed at face value
    mla_dev = [c for c in MLA_CASES if _mla_unimplemented(c["param"]) and not c["expected"].startswith("C:")]
    assert len(MLA_CASES) == 147 and len(mla_dev) == 0
    assert len(OMNI_CASES) == 15   # all at face value


def test_param_sizes(binding):
    # reference tests/unittest/ops/test_op_param_size.cpp:47,51
    assert binding.atb().atb_c_sizeof_paged_attention_param() == 120
    assert binding.atb().atb_c_sizeof_reshape_and_cache_param() == 24
    assert ctypes.sizeof(binding.PagedAttentionParam) == 120
    assert ctypes.sizeof(binding.ReshapeAndCacheParam) == 24
    # :68
    assert binding.atb().atb_c_sizeof_multi_latent_attention_param() == 64
    assert ctypes.sizeof(binding.MultiLatentAttentionParam) == 64


def test_reserved_bytes_must_be_zero(binding):
    p = binding.PagedAttentionParam(headNum=8, kvHeadNum=8)
    p.rsv[63] = 1
    assert binding.Operation("PagedAttentionOperation", p).status == binding.ERROR_CODE["ERROR_INVALID_PARAM"]
    r = binding.ReshapeAndCacheParam()
    r.rsv[0] = 1
    assert binding.Operation("ReshapeAndCacheOperation", r).status == binding.ERROR_CODE["ERROR_INVALID_PARAM"]


def test_names_and_tensor_counts(binding):
    cases = [
        (binding.PagedAttentionParam(headNum=8, kvHeadNum=8), 5),
        (binding.PagedAttentionParam(headNum=8, kvHeadNum=8, quantType=1), 7),
        (binding.PagedAttentionParam(headNum=8, kvHeadNum=8, quantType=1, hasQuantOffset=True), 9),
        (binding.PagedAttentionParam(headNum=8, kvHeadNum=1, mlaVHeadSize=512), 4),
        (binding.PagedAttentionParam(headNum=8, kvHeadNum=8, maskType=1), 6),
        (binding.PagedAttentionParam(headNum=8, kvHeadNum=8, maskType=2, batchRunStatusEnable=True, scaleType=1), 8),
        (binding.PagedAttentionParam(headNum=8, kvHeadNum=8, maskType=1, quantType=1, hasQuantOffset=True), 10),
        (binding.PagedAttentionParam(headNum=8, kvHeadNum=1, mlaVHeadSize=512, maskType=1), 5),
    ]
    for p, n in cases:
        op = binding.Operation("PagedAttentionOperation", p)
        assert op.ok and op.get_name() == "PagedAttentionOperation"
        assert (op.input_num(), op.output_num()) == (n, 1)
        op.close()
    op = binding.Operation("ReshapeAndCacheOperation", binding.ReshapeAndCacheParam())
    assert op.get_name() == "ReshapeAndCacheOperation" and (op.input_num(), op.output_num()) == (5, 2)
    op.close()
    op = binding.Operation("ReshapeAndCacheOperation", binding.ReshapeAndCacheParam(kvCacheCfg=1))
    assert (op.input_num(), op.output_num()) == (3, 1)
    op.close()
    # reference reshape_and_cache_with_stride_operation.cpp:116-138
    op = binding.Operation("ReshapeAndCacheWithStrideOperation", binding.ReshapeAndCacheWithStrideParam())
    assert op.get_name() == "ReshapeAndCacheWithStrideOperation" and (op.input_num(), op.output_num()) == (9, 2)
    op.close()
    op = binding.Operation("ReshapeAndCacheWithStrideOperation", binding.ReshapeAndCacheWithStrideParam(kvCacheCfg=1))
    assert (op.input_num(), op.output_num()) == (5, 1)
    op.close()


def _c1_pack(binding, lens_host, q_rows=4, tables_rows=4):
    ins = [
        binding.make_tensor("float16", [q_rows, 8, 128], FAKE_DEVICE),
        binding.make_tensor("float16", [64, 128, 8, 128], FAKE_DEVICE),
        binding.make_tensor("float16", [64, 128, 8, 128], FAKE_DEVICE),
        binding.make_tensor("int32", [tables_rows, 4], FAKE_DEVICE),
        binding.make_tensor("int32", [len(lens_host)], FAKE_DEVICE,
                            host_ptr=lens_host.ctypes.data if lens_host is not None else None),
    ]
    outs = [binding.make_tensor("float16", [q_rows, 8, 128], FAKE_DEVICE)]
    return ins, outs


def test_setup_reads_host_context_lens(binding, ctx):
    op = binding.Operation("PagedAttentionOperation",
                           binding.PagedAttentionParam(headNum=8, kvHeadNum=8, qkScale=0.088))
    lens = np.array([469, 339, 432, 71], dtype=np.int32)
    ins, outs = _c1_pack(binding, lens)
    st, ws = op.setup(ins, outs, ctx)
    assert st == 0
    # missing hostData: the lengths cannot be read (reference param.cpp:16-62)
    ins[4].hostData = None
    st, _ = op.setup(ins, outs, ctx)
    assert binding.ERROR_NAMES[st] == "ERROR_INVALID_PARAM"
    # a length beyond what the block table can address
    bad = np.array([469, 339, 4 * 128 + 1, 71], dtype=np.int32)
    ins, outs = _c1_pack(binding, bad)
    st, _ = op.setup(ins, outs, ctx)
    assert binding.ERROR_NAMES[st] == "ERROR_INVALID_PARAM"
    op.close()


def test_setup_workspace_grows_with_split_count(binding, ctx):
    op = binding.Operation("PagedAttentionOperation",
                           binding.PagedAttentionParam(headNum=32, kvHeadNum=8, qkScale=0.088))

    def setup(lens):
        lens = np.asarray(lens, dtype=np.int32)
        ins = [
            binding.make_tensor("bf16", [len(lens), 32, 128], FAKE_DEVICE),
            binding.make_tensor("bf16", [4096, 128, 8, 128], FAKE_DEVICE),
            binding.make_tensor("bf16", [4096, 128, 8, 128], FAKE_DEVICE),
            binding.make_tensor("int32", [len(lens), 256], FAKE_DEVICE),
            binding.make_tensor("int32", [len(lens)], FAKE_DEVICE, host_ptr=lens.ctypes.data),
        ]
        outs = [binding.make_tensor("bf16", [len(lens), 32, 128], FAKE_DEVICE)]
        st, ws = op.setup(ins, outs, ctx)
        assert st == 0
        return ws

    short = setup([100] * 4)
    long = setup([32768] * 4)
    assert long > short >= 0
    op.close()


def test_operation_stream_id(binding):
    """SetExecuteStreamId / GetExecuteStreamId (reference include/atb/operation.h:150,159,
    src/atb/operation/operation.cpp:24-55, operation_base.cpp:1356-1379): the default is stream 0, the id is
    kept, and Execute refuses an id the context has no stream for."""
    e = binding.ERROR_CODE
    op = binding.Operation("PagedAttentionOperation",
                           binding.PagedAttentionParam(headNum=8, kvHeadNum=8, qkScale=0.088))
    assert op.get_stream_id() == 0
    assert op.set_stream_id(1) == 0 and op.get_stream_id() == 1
    assert binding.atb().atb_c_op_set_stream_id(None, 1) == e["ERROR_INVALID_PARAM"]
    assert binding.atb().atb_c_op_get_stream_id(None) == 0
    lens = np.array([469, 339, 432, 71], dtype=np.int32)
    ins, outs = _c1_pack(binding, lens)
    one = binding.Context(0x1)
    st, ws = op.setup(ins, outs, one)
    assert st == 0
    # the context holds one stream only: nothing is launched
    assert op.execute(ins, outs, FAKE_DEVICE, max(ws, 1), one) == e["ERROR_INVALID_PARAM"]
    assert one.set_streams([]) == e["ERROR_INVALID_PARAM"]
    one.close()
    op.close()


def test_setup_and_execute_error_paths(binding, ctx):
    e = binding.ERROR_CODE
    op = binding.Operation("PagedAttentionOperation",
                           binding.PagedAttentionParam(headNum=8, kvHeadNum=8, qkScale=0.088))
    lens = np.array([469, 339, 432, 71], dtype=np.int32)
    ins, outs = _c1_pack(binding, lens)
    # Execute before any Setup
    assert op.execute(ins, outs, FAKE_DEVICE, 1 << 20, ctx) == e["ERROR_INVALID_PARAM"]
    # Setup without a context
    st, _ = op.setup(ins, outs, None)
    assert st == e["ERROR_INVALID_PARAM"]
    # wrong tensor count
    st, _ = op.setup(ins[:4], outs, ctx)
    assert st == e["ERROR_INVALID_IN_TENSOR_NUM"]
    st, _ = op.setup(ins, [], ctx)
    assert st == e["ERROR_INVALID_IN_TENSOR_NUM"]
    # a zero-sized dim is an invalid tensor size, 9 dims an invalid dim count
    bad = list(ins)
    bad[0] = binding.make_tensor("float16", [4, 0, 128], FAKE_DEVICE)
    st, _ = op.setup(bad, outs, ctx)
    assert st == e["ERROR_INVALID_TENSOR_SIZE"]
    bad[0] = binding.make_tensor("float16", [4, 8, 128], FAKE_DEVICE)
    bad[0].dimNum = 9
    st, _ = op.setup(bad, outs, ctx)
    assert st == e["ERROR_INVALID_TENSOR_DIM"]
    # query head count differs from headNum: caught by the kernel-level checks
    bad = list(ins)
    bad[0] = binding.make_tensor("float16", [4, 16, 128], FAKE_DEVICE)
    st, _ = op.setup(bad, [binding.make_tensor("float16", [4, 16, 128], FAKE_DEVICE)], ctx)
    assert st == e["ERROR_INVALID_PARAM"]

    st, ws = op.setup(ins, outs, ctx)
    assert st == 0
    # a failed Setup invalidates the previous one
    st, _ = op.setup(ins[:4], outs, ctx)
    assert st != 0
    assert op.execute(ins, outs, FAKE_DEVICE, 1 << 20, ctx) == e["ERROR_INVALID_PARAM"]

    st, ws = op.setup(ins, outs, ctx)
    assert st == 0
    # different context
    other = binding.Context(0x2)
    assert op.execute(ins, outs, FAKE_DEVICE, max(ws, 1), other) == e["ERROR_INVALID_PARAM"]
    other.close()
    # workspace too small / null
    if ws > 0:
        assert op.execute(ins, outs, FAKE_DEVICE, ws - 1, ctx) == e["ERROR_INVALID_PARAM"]
        assert op.execute(ins, outs, None, ws, ctx) == e["ERROR_INVALID_PARAM"]
    # dataSize changed since Setup
    changed = list(ins)
    changed[0] = binding.make_tensor("float16", [4, 8, 128], FAKE_DEVICE, data_size=17)
    assert op.execute(changed, outs, FAKE_DEVICE, max(ws, 1), ctx) == e["ERROR_INVALID_PARAM"]
    # tensor with no data pointer at all
    nodata = list(ins)
    nodata[1] = binding.make_tensor("float16", [64, 128, 8, 128], None)
    assert op.execute(nodata, outs, FAKE_DEVICE, max(ws, 1), ctx) == e["ERROR_INVALID_PARAM"]
    # null stream
    nostream = binding.Context(None)
    st, ws2 = op.setup(ins, outs, nostream)
    assert st == 0
    assert op.execute(ins, outs, FAKE_DEVICE, max(ws2, 1), nostream) == e["ERROR_INVALID_PARAM"]
    nostream.close()
    # split execute: LAUNCH without a PRELAUNCH
    st, ws = op.setup(ins, outs, ctx)
    ctx.set_execute_type(2)
    try:
        assert op.execute(ins, outs, FAKE_DEVICE, max(ws, 1), ctx) == e["ERROR_INVALID_PARAM"]
    finally:
        ctx.set_execute_type(0)
    op.close()


def test_mask_status_and_logn_inputs(binding, ctx):
    """Setup-time rules for the optional inputs: mask layouts (reference
    tiling/paged_attention_tiling.cpp:36-74), the host-side status vector
    (param.cpp:39-49), logN sizes (paged_attention_operation.cpp:900-924), and
    the smaller query of a dynamic batch (:679-688, :935-941)."""
    e = binding.ERROR_CODE
    lens = np.array([5, 0, 7, 200], dtype=np.int32)
    status = np.array([1, 0, 1, 1], dtype=np.int32)

    def pack(mask_shape=None, q_rows=4, out_rows=None, status_host=True, logn=None, mask_dtype="float16"):
        ins = [
            binding.make_tensor("float16", [q_rows, 32, 128], FAKE_DEVICE),
            binding.make_tensor("float16", [8, 64, 16, 128], FAKE_DEVICE),
            binding.make_tensor("float16", [8, 64, 16, 128], FAKE_DEVICE),
            binding.make_tensor("int32", [4, 4], FAKE_DEVICE),
            binding.make_tensor("int32", [4], FAKE_DEVICE, host_ptr=lens.ctypes.data),
        ]
        if mask_shape is not None:
            ins.append(binding.make_tensor(mask_dtype, mask_shape, FAKE_DEVICE))
        if status_host is not None:
            ins.append(binding.make_tensor("int32", [4], FAKE_DEVICE,
                                           host_ptr=status.ctypes.data if status_host else None))
        if logn is not None:
            ins.append(binding.make_tensor("float", logn, FAKE_DEVICE))
        outs = [binding.make_tensor("float16", [q_rows if out_rows is None else out_rows, 32, 128], FAKE_DEVICE)]
        return ins, outs

    def setup(op, *a, **k):
        return op.setup(*pack(*a, **k), ctx)[0]

    norm = binding.Operation("PagedAttentionOperation", binding.PagedAttentionParam(
        headNum=32, kvHeadNum=16, qkScale=0.088, maskType=1))
    for shape, want in (([4, 1, 256], 0), ([1, 256], 0), ([4, 1, 200], 0), ([4, 1, 199], e["ERROR_INVALID_PARAM"]),
                        ([3, 1, 256], e["ERROR_INVALID_PARAM"]), ([4, 2, 256], e["ERROR_INVALID_PARAM"]),
                        ([4, 32, 1, 256], 0), ([4, 1, 1, 256], 0),   # (read as the reference's kernel reads them: row 0)
                        ([4, 16, 1, 256], e["ERROR_INVALID_PARAM"]), ([3, 32, 1, 256], e["ERROR_INVALID_PARAM"]),
                        ([2, 256], e["ERROR_INVALID_PARAM"])):
        assert setup(norm, shape, status_host=None) == want, shape
    # the mask has q's dtype
    assert setup(norm, [4, 1, 256], status_host=None, mask_dtype="bf16") == e["ERROR_INVALID_TENSOR_INI_MATCH"]
    norm.close()

    alibi = binding.Operation("PagedAttentionOperation", binding.PagedAttentionParam(
        headNum=32, kvHeadNum=16, qkScale=0.088, maskType=2))
    for shape, want in (([32, 1, 256], 0), ([4, 32, 1, 256], 0), ([4, 1, 1, 256], 0),
                        ([4, 1, 256], e["ERROR_INVALID_PARAM"]), ([4, 16, 1, 256], e["ERROR_INVALID_PARAM"]),
                        ([4, 32, 2, 256], e["ERROR_INVALID_PARAM"]), ([1, 256], e["ERROR_INVALID_PARAM"])):
        assert setup(alibi, shape, status_host=None) == want, shape
    alibi.close()

    dyn = binding.Operation("PagedAttentionOperation", binding.PagedAttentionParam(
        headNum=32, kvHeadNum=16, qkScale=0.088, batchRunStatusEnable=True, scaleType=1))
    assert setup(dyn, logn=[4]) == 0
    assert setup(dyn, q_rows=3, logn=[4]) == 0                      # three running sequences, three query rows
    assert setup(dyn, q_rows=2, logn=[4]) == e["ERROR_INVALID_PARAM"]  # fewer rows than non-empty sequences
    assert setup(dyn, q_rows=5, logn=[4]) == e["ERROR_INVALID_TENSOR_DIM"]
    assert setup(dyn, q_rows=3, out_rows=4, logn=[4]) == e["ERROR_INVALID_TENSOR_DIM"]
    assert setup(dyn, status_host=False, logn=[4]) == e["ERROR_INVALID_PARAM"]
    assert setup(dyn, logn=[5]) == e["ERROR_INVALID_TENSOR_DIM"]
    assert setup(dyn, logn=[4, 1]) == e["ERROR_INVALID_TENSOR_DIM"]
    dyn.close()
    # without the dynamic batch the query must cover every sequence of contextLens
    plain = binding.Operation("PagedAttentionOperation", binding.PagedAttentionParam(
        headNum=32, kvHeadNum=16, qkScale=0.088))
    assert setup(plain, status_host=None) == 0
    plain.close()


def test_several_query_tokens_inputs(binding, ctx):
    """CALC_TYPE_SPEC: qSeqLens follows the mask, is read on the host (reference param.cpp:96-110)
    and has one entry per sequence; masks are (query rows, maxS) for MASK_TYPE_SPEC and the
    square (maxS, maxS) for MASK_TYPE_NORM; the query rows must cover the sum of the lengths."""
    e = binding.ERROR_CODE
    lens = np.array([10, 64, 0, 64], dtype=np.int32)
    qlens = np.array([1, 15, 7, 6], dtype=np.int32)   # the empty sequence brings no rows: 22 in all

    def setup(op, mask_shape, q_rows=22, qlens_host=qlens, qlens_shape=(4,)):
        ins = [
            binding.make_tensor("float16", [q_rows, 32, 128], FAKE_DEVICE),
            binding.make_tensor("float16", [8, 64, 16, 128], FAKE_DEVICE),
            binding.make_tensor("float16", [8, 64, 16, 128], FAKE_DEVICE),
            binding.make_tensor("int32", [4, 2], FAKE_DEVICE),
            binding.make_tensor("int32", [4], FAKE_DEVICE, host_ptr=lens.ctypes.data),
            binding.make_tensor("float16", mask_shape, FAKE_DEVICE),
            binding.make_tensor("int32", list(qlens_shape), FAKE_DEVICE,
                                host_ptr=qlens_host.ctypes.data if qlens_host is not None else None),
        ]
        outs = [binding.make_tensor("float16", [q_rows, 32, 128], FAKE_DEVICE)]
        return op.setup(ins, outs, ctx)[0]

    spec = binding.Operation("PagedAttentionOperation", binding.PagedAttentionParam(
        headNum=32, kvHeadNum=16, qkScale=0.088, maskType=3, calcType=1))
    assert spec.ok and spec.input_num() == 7
    assert setup(spec, [22, 64]) == 0
    assert setup(spec, [24, 64], q_rows=24) == 0                      # spare query rows are left alone
    assert setup(spec, [21, 64], q_rows=21) == e["ERROR_INVALID_PARAM"]  # 22 rows planned
    assert setup(spec, [20, 64]) == e["ERROR_INVALID_PARAM"]          # one mask row per query row
    assert setup(spec, [22, 63]) == e["ERROR_INVALID_PARAM"]          # shorter than a context
    assert setup(spec, [4, 1, 64]) == e["ERROR_INVALID_PARAM"]
    assert setup(spec, [22, 64], qlens_host=None) == e["ERROR_INVALID_PARAM"]
    assert setup(spec, [22, 64], qlens_shape=(3,)) == e["ERROR_INVALID_PARAM"]
    too_long = np.array([11, 1, 0, 1], dtype=np.int32)              # more query tokens than context
    assert setup(spec, [22, 64], qlens_host=too_long) == e["ERROR_INVALID_PARAM"]
    spec.close()
    norm = binding.Operation("PagedAttentionOperation", binding.PagedAttentionParam(
        headNum=32, kvHeadNum=16, qkScale=0.088, maskType=1, calcType=1))
    assert setup(norm, [64, 64]) == 0
    assert setup(norm, [128, 128]) == 0
    assert setup(norm, [22, 64]) == e["ERROR_INVALID_PARAM"]
    assert setup(norm, [4, 1, 64]) == e["ERROR_INVALID_PARAM"]
    norm.close()
    # the reference's creation rules: SPEC needs the NORM or SPEC mask, and neither dequant nor logN
    for bad in (dict(maskType=0), dict(maskType=2), dict(maskType=1, quantType=1), dict(maskType=1, scaleType=1),
                dict(maskType=1, batchRunStatusEnable=True)):
        op = binding.Operation("PagedAttentionOperation", binding.PagedAttentionParam(
            headNum=32, kvHeadNum=16, qkScale=0.088, calcType=1, **bad))
        assert op.status == e["ERROR_INVALID_PARAM"], bad
    # MASK_TYPE_SPEC without CALC_TYPE_SPEC: one query token per sequence, one mask row per query row
    op = binding.Operation("PagedAttentionOperation", binding.PagedAttentionParam(headNum=32, kvHeadNum=16, maskType=3))
    assert op.status == 0 and op.input_num() == 6
    op.close()


def test_multi_latent_attention_counts_shapes_and_setup(binding, ctx):
    """Tensor counts and InferShape per calcType (reference multi_latent_attention_operation.cpp:245-283),
    host-side lengths, and the output shapes Setup insists on."""
    e = binding.ERROR_CODE
    mk = binding.MultiLatentAttentionParam
    for kw, n_in, n_out in ((dict(), 6, 1), (dict(calcType=1), 7, 1), (dict(calcType=1, maskType=1), 8, 1),
                            (dict(calcType=2), 6, 2), (dict(calcType=3, maskType=1), 8, 2),
                            (dict(calcType=1, maskType=2), 8, 1),       # MASK_FREE brings its template
                            (dict(calcType=1, maskType=3), 7, 1),       # CAUSAL_MASK has no mask tensor
                            (dict(calcType=3, maskUseStatusType=1), 8, 2),
                            (dict(calcType=3, maskType=2, maskUseStatusType=1), 9, 2),
                            (dict(calcType=3, cacheMode=2, maskUseStatusType=1), 10, 2)):
        op = binding.Operation("MultiLatentAttentionOperation", mk(**dict(dict(headNum=32, kvHeadNum=1, qkScale=0.07,
                                                                             cacheMode=1), **kw)))
        assert op.ok and (op.input_num(), op.output_num()) == (n_in, n_out), kw
        op.close()
    for bad in (dict(headNum=12), dict(kvHeadNum=2), dict(cacheMode=0), dict(maskType=1), dict(qkScale=1.5),
                dict(qkScale=0.0), dict(calcType=5), dict(cacheMode=4), dict(calcType=4, headNum=32),
                dict(cacheMode=2, calcType=2, maskType=1),
                dict(calcType=1, maskType=4), dict(calcType=1, maskUseStatusType=1), dict(maskUseStatusType=1),
                dict(calcType=3, maskUseStatusType=2), dict(calcType=3, maskUseStatusType=-1)):
        kw = dict(headNum=32, kvHeadNum=1, qkScale=0.07, cacheMode=1)
        kw.update(bad)
        assert binding.Operation("MultiLatentAttentionOperation", mk(**kw)).status == e["ERROR_INVALID_PARAM"], bad
    p = mk(headNum=32, kvHeadNum=1, qkScale=0.07, cacheMode=1)
    p.rsv[31] = 1
    assert binding.Operation("MultiLatentAttentionOperation", p).status == e["ERROR_INVALID_PARAM"]

    lens = np.array([10, 300, 0, 64], dtype=np.int32)
    qlens = np.array([1, 3, 2, 2], dtype=np.int32)   # 8 query rows: the sequence without context keeps its two

    def pack(rows=4, mask=None, with_qlens=False, lens_host=True, qlens_host=True, dtype="float16", block=128):
        ins = [
            binding.make_tensor(dtype, [rows, 32, 512], FAKE_DEVICE),
            binding.make_tensor(dtype, [rows, 32, 64], FAKE_DEVICE),
            binding.make_tensor(dtype, [16, block, 1, 512], FAKE_DEVICE),
            binding.make_tensor(dtype, [16, block, 1, 64], FAKE_DEVICE),
            binding.make_tensor("int32", [4, 3], FAKE_DEVICE),
            binding.make_tensor("int32", [4], FAKE_DEVICE, host_ptr=lens.ctypes.data if lens_host else None),
        ]
        if mask is not None:
            ins.append(binding.make_tensor(dtype, mask, FAKE_DEVICE))
        if with_qlens:
            ins.append(binding.make_tensor("int32", [4], FAKE_DEVICE, host_ptr=qlens.ctypes.data if qlens_host else None))
        return ins

    def outs(rows=4, lse=False, dtype="float16", width=512):
        o = [binding.make_tensor(dtype, [rows, 32, width], FAKE_DEVICE)]
        if lse:
            o.append(binding.make_tensor(dtype, [rows, 32, 1], FAKE_DEVICE))
        return o

    ring = binding.Operation("MultiLatentAttentionOperation", mk(headNum=32, kvHeadNum=1, qkScale=0.07, cacheMode=1,
                                                                 calcType=2))
    st, descs = ring.infer_shape(pack(dtype="bf16"))
    assert st == 0 and [[d.dims[i] for i in range(d.dimNum)] for d in descs] == [[4, 32, 512], [4, 32, 1]]
    assert all(d.dtype == binding.ACL_DTYPE_BY_NAME["bf16"] for d in descs)
    assert ring.setup(pack(), outs(lse=True), ctx)[0] == 0
    assert ring.setup(pack(lens_host=False), outs(lse=True), ctx)[0] == e["ERROR_INVALID_PARAM"]
    assert ring.setup(pack(), outs(lse=True, width=576), ctx)[0] == e["ERROR_INVALID_PARAM"]
    assert ring.setup(pack(block=64), outs(lse=True), ctx)[0] == e["ERROR_INVALID_TENSOR_DIM"]
    # only the plain decode calcType ties the token count to the batch (reference :577-580)
    assert ring.setup(pack(rows=5), outs(rows=5, lse=True), ctx)[0] == 0
    plain = binding.Operation("MultiLatentAttentionOperation", mk(headNum=32, kvHeadNum=1, qkScale=0.07, cacheMode=1))
    assert plain.setup(pack(), outs(), ctx)[0] == 0
    assert plain.setup(pack(rows=5), outs(rows=5), ctx)[0] == e["ERROR_INVALID_TENSOR_DIM"]
    plain.close()
    assert ring.setup(pack(dtype="bf16"), outs(lse=True), ctx)[0] == e["ERROR_INVALID_TENSOR_INI_MATCH"]
    ring.close()

    spec = binding.Operation("MultiLatentAttentionOperation", mk(headNum=32, kvHeadNum=1, qkScale=0.07, cacheMode=1,
                                                                 calcType=1, maskType=1))
    assert spec.setup(pack(rows=8, mask=[8, 300], with_qlens=True), outs(rows=8), ctx)[0] == 0
    assert spec.setup(pack(rows=8, mask=[8, 299], with_qlens=True), outs(rows=8), ctx)[0] == e["ERROR_INVALID_PARAM"]
    assert spec.setup(pack(rows=8, mask=[7, 300], with_qlens=True), outs(rows=8), ctx)[0] == e["ERROR_INVALID_PARAM"]
    assert spec.setup(pack(rows=7, mask=[7, 300], with_qlens=True), outs(rows=7), ctx)[0] == e["ERROR_INVALID_PARAM"]
    assert spec.setup(pack(rows=8, mask=[8, 300], with_qlens=True, qlens_host=False), outs(rows=8), ctx)[0] == \
        e["ERROR_INVALID_PARAM"]
    spec.close()


def test_multi_latent_attention_causal_rows_and_mask_use_status(binding, ctx):
    """Several query tokens on the reference's job-per-token path (128 heads, or the int8 cache): the mask tensor is
    not read, maskUseStatus is an optional host tensor [batch] (reference multi_latent_attention_operation.cpp:
    536-575, ops_runner :117-131, tiling mla_tiling.cpp:139-144); MASK_TYPE_MASK_FREE with fewer heads is refused
    at Setup."""
    e = binding.ERROR_CODE
    mk = binding.MultiLatentAttentionParam
    lens = np.array([10, 300, 0, 64], dtype=np.int32)
    qlens = np.array([1, 3, 2, 2], dtype=np.int32)   # 8 query rows: the sequence without context keeps its two
    use = np.array([1, 0, 1, 1], dtype=np.int32)

    def pack(heads, mask=None, use_shape=None, use_host=True, qlens_host=qlens):
        ins = [binding.make_tensor("float16", [8, heads, 512], FAKE_DEVICE),
               binding.make_tensor("float16", [8, heads, 64], FAKE_DEVICE),
               binding.make_tensor("float16", [16, 128, 1, 512], FAKE_DEVICE),
               binding.make_tensor("float16", [16, 128, 1, 64], FAKE_DEVICE),
               binding.make_tensor("int32", [4, 3], FAKE_DEVICE),
               binding.make_tensor("int32", [4], FAKE_DEVICE, host_ptr=lens.ctypes.data)]
        if mask is not None:
            ins.append(binding.make_tensor("float16", mask, FAKE_DEVICE))
        ins.append(binding.make_tensor("int32", [4], FAKE_DEVICE, host_ptr=qlens_host.ctypes.data))
        if use_shape is not None:
            ins.append(binding.make_tensor("int32", use_shape, FAKE_DEVICE, host_ptr=use.ctypes.data if use_host else None))
        return ins

    def outs(heads, lse=True):
        o = [binding.make_tensor("float16", [8, heads, 512], FAKE_DEVICE)]
        return o + ([binding.make_tensor("float16", [8, heads, 1], FAKE_DEVICE)] if lse else [])

    # 128 heads: any mask shape passes, because the tensor is not read; the flags come from the host
    op = binding.Operation("MultiLatentAttentionOperation", mk(headNum=128, kvHeadNum=1, qkScale=0.07, cacheMode=1,
                                                               calcType=3, maskType=2, maskUseStatusType=1))
    assert op.ok and op.input_num() == 9
    assert op.setup(pack(128, mask=[129, 128], use_shape=[4]), outs(128), ctx)[0] == 0
    assert op.setup(pack(128, mask=[4, 129, 128], use_shape=[4]), outs(128), ctx)[0] == 0
    assert op.setup(pack(128, mask=[129, 128], use_shape=[0]), outs(128), ctx)[0] == 0        # optional: left out
    assert op.setup(pack(128, mask=[129, 128], use_shape=[4], use_host=False), outs(128), ctx)[0] == e["ERROR_INVALID_PARAM"]
    assert op.setup(pack(128, mask=[129, 128], use_shape=[3]), outs(128), ctx)[0] == e["ERROR_INVALID_TENSOR_DIM"]
    assert op.setup(pack(128, mask=[129, 128], use_shape=[4, 1]), outs(128), ctx)[0] == e["ERROR_INVALID_TENSOR_DIM_NUM"]
    # more query tokens than context cannot be made causal
    assert op.setup(pack(128, mask=[129, 128], use_shape=[4], qlens_host=np.array([11, 3, 0, 2], np.int32)),
                    outs(128), ctx)[0] == e["ERROR_INVALID_PARAM"]
    op.close()
    # fewer heads: the template is expanded into the workspace, one row of 384 (300 rounded up to whole cache blocks)
    # 16-bit values per query token, after the plan's own bytes and the 16-byte row records
    op = binding.Operation("MultiLatentAttentionOperation", mk(headNum=32, kvHeadNum=1, qkScale=0.07, cacheMode=1,
                                                               calcType=1, maskType=2))
    # (the same call with the mask rows handed over ready-made plans the same kernel and needs only the plan's bytes)
    plain = binding.Operation("MultiLatentAttentionOperation", mk(headNum=32, kvHeadNum=1, qkScale=0.07, cacheMode=1,
                                                                  calcType=1, maskType=1))
    st, ws = op.setup(pack(32, mask=[131, 128]), outs(32, lse=False), ctx)
    st0, ws0 = plain.setup(pack(32, mask=[8, 384]), outs(32, lse=False), ctx)
    assert (st, st0) == (0, 0) and ws >= ws0 + 8 * 16 + 8 * 384 * 2 and ws <= ws0 + 8 * 16 + 8 * 384 * 2 + 1024
    assert op.setup(pack(32, mask=[4, 131, 128]), outs(32, lse=False), ctx)[0] == 0           # a template per sequence
    assert op.setup(pack(32, mask=[3, 131, 128]), outs(32, lse=False), ctx)[0] == e["ERROR_INVALID_PARAM"]
    assert op.setup(pack(32, mask=[131, 64]), outs(32, lse=False), ctx)[0] == e["ERROR_INVALID_PARAM"]
    assert op.setup(pack(32, mask=[131]), outs(32, lse=False), ctx)[0] == e["ERROR_INVALID_PARAM"]
    # the 300-token sequence with 3 query tokens reads template rows up to 44 - 1 + 2; 64 tokens, 2 query tokens: 64
    assert op.setup(pack(32, mask=[65, 128]), outs(32, lse=False), ctx)[0] == 0
    assert op.setup(pack(32, mask=[64, 128]), outs(32, lse=False), ctx)[0] == e["ERROR_INVALID_PARAM"]
    op.close()
    plain.close()
    # CAUSAL_MASK: no mask tensor, any head count
    op = binding.Operation("MultiLatentAttentionOperation", mk(headNum=32, kvHeadNum=1, qkScale=0.07, cacheMode=1,
                                                               calcType=1, maskType=3))
    assert op.ok and op.setup(pack(32), outs(32, lse=False), ctx)[0] == 0
    op.close()


def test_multi_latent_attention_int8_nz_cache_checks(binding, ctx):
    """cacheMode INT8_NZCACHE: int8 query [T, H, 512] and latent cache [blocks, 16, 128, 32], 16-bit rotary parts,
    qkDescale / pvDescale fp32 [H] after the mask and qSeqlen, fp32 log-sum-exp (reference
    multi_latent_attention_operation.cpp:245-283 counts and InferShape, :427-476 shapes, :493-541 descales and
    outputs; ops_configs/atb_ops_info.ini:6741-6771, 6825-6858, 6918-6945)."""
    e = binding.ERROR_CODE
    mk = binding.MultiLatentAttentionParam
    lens = np.array([10, 300, 0, 64], dtype=np.int32)
    qlens = np.array([1, 3, 2, 2], dtype=np.int32)   # 8 query rows: the sequence without context keeps its two

    def pack(rows=4, kv=(16, 16, 128, 32), kr=(16, 4, 128, 16), dtype="float16", with_qlens=False, q_dtype="int8",
             descale=(32,), fmt="fractal_nz", mask=None):
        ins = [binding.make_tensor(q_dtype, [rows, 32, 512], FAKE_DEVICE),
               binding.make_tensor(dtype, [rows, 32, 64], FAKE_DEVICE),
               binding.make_tensor("int8", list(kv), FAKE_DEVICE, fmt=fmt),
               binding.make_tensor(dtype, list(kr), FAKE_DEVICE, fmt=fmt),
               binding.make_tensor("int32", [4, 3], FAKE_DEVICE),
               binding.make_tensor("int32", [4], FAKE_DEVICE, host_ptr=lens.ctypes.data)]
        if mask is not None:
            ins.append(binding.make_tensor(dtype, list(mask), FAKE_DEVICE))
        if with_qlens:
            ins.append(binding.make_tensor("int32", [4], FAKE_DEVICE, host_ptr=qlens.ctypes.data))
        ins += [binding.make_tensor("float", list(descale), FAKE_DEVICE) for _ in range(2)]
        return ins

    def outs(rows=4, lse=None, dtype="float16"):
        o = [binding.make_tensor(dtype, [rows, 32, 512], FAKE_DEVICE)]
        if lse:
            o.append(binding.make_tensor(lse, [rows, 32, 1], FAKE_DEVICE))
        return o

    plain = binding.Operation("MultiLatentAttentionOperation", mk(headNum=32, kvHeadNum=1, qkScale=0.07, cacheMode=2))
    assert plain.ok and (plain.input_num(), plain.output_num()) == (8, 1)
    st, descs = plain.infer_shape(pack(dtype="bf16"))
    assert st == 0 and descs[0].dtype == binding.ACL_DTYPE_BY_NAME["bf16"]      # the rotary query's type, not int8
    st, ws = plain.setup(pack(), outs(), ctx)
    assert st == 0 and ws == 256                                                # 16 bytes per query row, to a multiple of 256
    assert plain.setup(pack(q_dtype="float16"), outs(), ctx)[0] == e["ERROR_INVALID_TENSOR_INI_MATCH"]
    assert plain.setup(pack(fmt="nd"), outs(), ctx)[0] == e["ERROR_INVALID_TENSOR_INI_MATCH"]
    for bad in (dict(kv=(16, 32, 128, 16)), dict(kv=(16, 16, 64, 32), kr=(16, 4, 64, 16)), dict(kr=(16, 2, 128, 32)),
                dict(kv=(16, 8, 128, 32))):
        assert plain.setup(pack(**bad), outs(), ctx)[0] == e["ERROR_INVALID_TENSOR_DIM"], bad
    assert plain.setup(pack(descale=(31,)), outs(), ctx)[0] == e["ERROR_INVALID_PARAM"]
    plain.close()
    ring = binding.Operation("MultiLatentAttentionOperation", mk(headNum=32, kvHeadNum=1, qkScale=0.07, cacheMode=2,
                                                                 calcType=2))
    assert ring.ok and (ring.input_num(), ring.output_num()) == (8, 2)
    st, descs = ring.infer_shape(pack())
    assert st == 0 and descs[1].dtype == binding.ACL_DTYPE_BY_NAME["float"]
    assert [d.dims[i] for d in descs for i in range(d.dimNum)] == [4, 32, 512, 4, 32, 1]
    assert ring.setup(pack(), outs(lse="float"), ctx)[0] == 0
    assert ring.setup(pack(), outs(lse="float16"), ctx)[0] == e["ERROR_INVALID_TENSOR_INI_MATCH"]
    assert ring.setup(pack(descale=(31,)), outs(lse="float"), ctx)[0] == e["ERROR_INVALID_TENSOR_DIM"]
    assert ring.setup(pack(descale=(4, 8)), outs(lse="float"), ctx)[0] == e["ERROR_INVALID_TENSOR_DIM_NUM"]
    ring.close()
    both = binding.Operation("MultiLatentAttentionOperation", mk(headNum=32, kvHeadNum=1, qkScale=0.07, cacheMode=2,
                                                                 calcType=3))
    assert both.ok and (both.input_num(), both.output_num()) == (9, 2)
    assert both.setup(pack(rows=8, with_qlens=True), outs(rows=8, lse="float"), ctx)[0] == 0
    both.close()
    spec = binding.Operation("MultiLatentAttentionOperation", mk(headNum=32, kvHeadNum=1, qkScale=0.07, cacheMode=2,
                                                                 calcType=1, maskType=1))
    assert spec.ok and spec.input_num() == 10
    assert spec.setup(pack(rows=8, with_qlens=True, mask=(8, 300)), outs(rows=8), ctx)[0] == 0
    # the int8 kernels of the reference never read the mask (tiling/mla_tiling.cpp:142-144): its shape is not looked at
    assert spec.setup(pack(rows=8, with_qlens=True, mask=(8, 299)), outs(rows=8), ctx)[0] == 0
    spec.close()


def test_multi_latent_attention_prefill_checks(binding, ctx):
    """calcType PREFILL: creation rules (reference multi_latent_attention_operation.cpp:175-206), tensor counts
    (:245-266), output shaped like the query (:268-283, :306-320), both key layouts (:718-737), lengths read from
    hostData and equal per sequence (multi_latent_attention_ops_runner_prefill.cpp:98-110)."""
    e = binding.ERROR_CODE
    mk = binding.MultiLatentAttentionParam
    base = dict(headNum=4, kvHeadNum=4, qkScale=0.07, cacheMode=1, calcType=4)
    for kw, n_in in ((dict(), 7), (dict(maskType=2), 8), (dict(maskType=3), 7), (dict(maskType=4, windowSize=100), 8),
                     (dict(maskType=3, kvHeadNum=2), 7), (dict(headNum=1, kvHeadNum=1), 7),
                     (dict(headNum=128, kvHeadNum=128), 7)):
        op = binding.Operation("MultiLatentAttentionOperation", mk(**dict(base, **kw)))
        assert op.ok and (op.input_num(), op.output_num()) == (n_in, 1), kw
        assert op.get_name() == "MultiLatentAttentionOperation"
        op.close()
    for bad in (dict(headNum=0, kvHeadNum=0), dict(headNum=129, kvHeadNum=129), dict(kvHeadNum=2), dict(maskType=1),
                dict(cacheMode=3), dict(cacheMode=0), dict(maskType=4), dict(qkScale=2.0)):
        assert binding.Operation("MultiLatentAttentionOperation", mk(**dict(base, **bad))).status == \
            e["ERROR_INVALID_PARAM"], bad

    q_lens = np.array([100, 0, 28], dtype=np.int32)
    kv_lens = q_lens.copy()

    def pack(q=(128, 4, 128), qr=(128, 4, 64), k=(128, 4, 128), kr=(128, 4, 64), v=(128, 4, 128), mask=None,
             ql=q_lens, kl=kv_lens, dtype="float16", host=True):
        ins = [binding.make_tensor(dtype, list(s), FAKE_DEVICE) for s in (q, qr, k, kr, v)]
        ins.append(binding.make_tensor("int32", [len(ql)], FAKE_DEVICE, host_ptr=ql.ctypes.data if host else None))
        ins.append(binding.make_tensor("int32", [len(kl)], FAKE_DEVICE, host_ptr=kl.ctypes.data if host else None))
        if mask is not None:
            ins.append(binding.make_tensor(dtype, list(mask), FAKE_DEVICE))
        return ins

    def out(shape=(128, 4, 128), dtype="float16"):
        return [binding.make_tensor(dtype, list(shape), FAKE_DEVICE)]

    op = binding.Operation("MultiLatentAttentionOperation", mk(**base))
    st, descs = op.infer_shape(pack(dtype="bf16"))
    assert st == 0 and [[d.dims[i] for i in range(d.dimNum)] for d in descs] == [[128, 4, 128]]
    assert descs[0].dtype == binding.ACL_DTYPE_BY_NAME["bf16"]
    st, ws = op.setup(pack(), out(), ctx)
    assert st == 0 and ws == 2 * 32   # one block of 128 queries per non-empty sequence, 32 bytes each
    # 2-dim query and output, keys padded per sequence as [batch, maxSeqLen, kvHeads * channels]
    flat = dict(q=(128, 512), qr=(128, 256), k=(3, 100, 512), kr=(3, 100, 256), v=(3, 100, 512))
    st, descs = op.infer_shape(pack(**flat))
    assert st == 0 and [[d.dims[i] for i in range(d.dimNum)] for d in descs] == [[128, 512]]
    assert op.setup(pack(**flat), out((128, 512)), ctx)[0] == 0
    short = dict(flat, k=(3, 99, 512), kr=(3, 99, 256), v=(3, 99, 512))
    assert op.setup(pack(**short), out((128, 512)), ctx)[0] == e["ERROR_INVALID_PARAM"]      # 100 keys in 99 rows
    assert op.setup(pack(host=False), out(), ctx)[0] == e["ERROR_INVALID_PARAM"]
    assert op.setup(pack(kl=np.array([100, 0, 27], dtype=np.int32)), out(), ctx)[0] == e["ERROR_INVALID_PARAM"]
    assert op.setup(pack(ql=np.array([100, 1, 28], dtype=np.int32), kl=np.array([100, 1, 28], dtype=np.int32)), out(),
                    ctx)[0] == e["ERROR_INVALID_PARAM"]                                          # 129 rows of 128
    assert op.setup(pack(), out((128, 4, 64)), ctx)[0] == e["ERROR_INVALID_TENSOR_DIM"]
    assert op.setup(pack(), out((128, 512)), ctx)[0] == e["ERROR_INVALID_TENSOR_DIM_NUM"]
    assert op.setup(pack(mask=(512, 512)), out(), ctx)[0] == e["ERROR_INVALID_IN_TENSOR_NUM"]
    assert op.setup(pack(dtype="bf16"), out(), ctx)[0] == e["ERROR_INVALID_TENSOR_INI_MATCH"]
    for bad in (dict(q=(128, 4, 127)), dict(qr=(128, 4, 32)), dict(qr=(127, 4, 64)), dict(k=(128, 3, 128)),
                dict(kr=(128, 4, 32)), dict(v=(128, 4, 64)), dict(v=(127, 4, 128))):
        assert op.setup(pack(**bad), out(), ctx)[0] == e["ERROR_INVALID_TENSOR_DIM"], bad
    op.close()

    free = binding.Operation("MultiLatentAttentionOperation", mk(**dict(base, maskType=2)))
    assert free.setup(pack(mask=(512, 512)), out(), ctx)[0] == 0
    assert free.setup(pack(mask=(512, 511)), out(), ctx)[0] == e["ERROR_INVALID_TENSOR_DIM"]
    assert free.setup(pack(mask=(1, 512, 512)), out(), ctx)[0] == 0
    assert free.setup(pack(), out(), ctx)[0] == e["ERROR_INVALID_IN_TENSOR_NUM"]
    free.close()
    # CAUSAL_MASK takes no mask tensor, keys only in the padded layout, and may group query heads over KV heads
    causal = binding.Operation("MultiLatentAttentionOperation", mk(**dict(base, maskType=3, kvHeadNum=2)))
    padded = dict(k=(3, 100, 256), kr=(3, 100, 128), v=(3, 100, 256))
    assert causal.setup(pack(**padded), out(), ctx)[0] == 0
    assert causal.setup(pack(k=(128, 2, 128), kr=(128, 2, 64), v=(128, 2, 128)), out(), ctx)[0] == \
        e["ERROR_INVALID_TENSOR_DIM"]
    causal.close()
    swa = binding.Operation("MultiLatentAttentionOperation", mk(**dict(base, maskType=4, windowSize=50)))
    assert swa.setup(pack(mask=(100, 100)), out(), ctx)[0] == 0
    assert swa.setup(pack(mask=(99, 100)), out(), ctx)[0] == e["ERROR_INVALID_PARAM"]
    swa.close()


def test_multi_latent_attention_nz_cache_checks(binding, ctx):
    """cacheMode NZCACHE: caches [blocks, channels / 16, 128, 16] in the fractal-NZ format (reference
    multi_latent_attention_operation.cpp:394-425). Only the plain decode has a dtype / format table in the
    reference (ops_configs/atb_ops_info.ini:6946-6967); with qSeqlen, a mask or the log-sum-exp output the
    section name it builds does not exist and the table check is skipped (operation_base.cpp:229-233)."""
    e = binding.ERROR_CODE
    mk = binding.MultiLatentAttentionParam
    lens = np.array([10, 300, 0, 64], dtype=np.int32)
    qlens = np.array([1, 3, 2, 2], dtype=np.int32)

    def pack(kv=(16, 32, 128, 16), kr=(16, 4, 128, 16), fmt="fractal_nz", dtype="float16", rows=4, with_qlens=False):
        ins = [binding.make_tensor(dtype, [rows, 32, 512], FAKE_DEVICE),
               binding.make_tensor(dtype, [rows, 32, 64], FAKE_DEVICE),
               binding.make_tensor(dtype, list(kv), FAKE_DEVICE, fmt=fmt),
               binding.make_tensor(dtype, list(kr), FAKE_DEVICE, fmt=fmt),
               binding.make_tensor("int32", [4, 3], FAKE_DEVICE),
               binding.make_tensor("int32", [4], FAKE_DEVICE, host_ptr=lens.ctypes.data)]
        if with_qlens:
            ins.append(binding.make_tensor("int32", [4], FAKE_DEVICE, host_ptr=qlens.ctypes.data))
        return ins

    def outs(rows=4, lse=False, dtype="float16"):
        o = [binding.make_tensor(dtype, [rows, 32, 512], FAKE_DEVICE)]
        if lse:
            o.append(binding.make_tensor(dtype, [rows, 32, 1], FAKE_DEVICE))
        return o

    op = binding.Operation("MultiLatentAttentionOperation", mk(headNum=32, kvHeadNum=1, qkScale=0.07, cacheMode=3))
    assert op.ok and (op.input_num(), op.output_num()) == (6, 1)
    st, descs = op.infer_shape(pack())
    assert st == 0 and [[d.dims[i] for i in range(d.dimNum)] for d in descs] == [[4, 32, 512]]
    assert op.setup(pack(), outs(), ctx)[0] == 0
    assert op.setup(pack(dtype="bf16"), outs(dtype="bf16"), ctx)[0] == 0
    assert op.setup(pack(fmt="nd"), outs(), ctx)[0] == e["ERROR_INVALID_TENSOR_INI_MATCH"]
    for bad in (dict(kv=(16, 32, 64, 16), kr=(16, 4, 64, 16)),      # block size is 128
                dict(kr=(16, 4, 256, 16)), dict(kr=(15, 4, 128, 16)),
                dict(kv=(16, 16, 128, 32)), dict(kr=(16, 2, 128, 32)),  # 16 channels per slab row
                dict(kv=(16, 31, 128, 16)), dict(kr=(16, 8, 128, 16)),  # 512 and 64 channels
                dict(kv=(16, 128, 1, 512), kr=(16, 128, 1, 64))):       # the token-major shapes
        assert op.setup(pack(**bad), outs(), ctx)[0] == e["ERROR_INVALID_TENSOR_DIM"], bad
    assert op.setup(pack(rows=5), outs(rows=5), ctx)[0] == e["ERROR_INVALID_TENSOR_DIM"]
    op.close()
    # with the log-sum-exp output or qSeqlen no table is checked; the dim checks are the same
    ring = binding.Operation("MultiLatentAttentionOperation", mk(headNum=32, kvHeadNum=1, qkScale=0.07, cacheMode=3,
                                                                 calcType=2))
    assert ring.ok and ring.output_num() == 2
    assert ring.setup(pack(), outs(lse=True), ctx)[0] == 0
    assert ring.setup(pack(fmt="nd"), outs(lse=True), ctx)[0] == 0
    assert ring.setup(pack(kv=(16, 31, 128, 16)), outs(lse=True), ctx)[0] == e["ERROR_INVALID_TENSOR_DIM"]
    ring.close()
    spec = binding.Operation("MultiLatentAttentionOperation", mk(headNum=32, kvHeadNum=1, qkScale=0.07, cacheMode=3,
                                                                 calcType=1))
    assert spec.ok and spec.input_num() == 7
    assert spec.setup(pack(rows=8, with_qlens=True), outs(rows=8), ctx)[0] == 0
    spec.close()


def test_paged_attention_bnsd_checks(binding, ctx):
    """inputLayout = TYPE_BNSD: caches [numBlocks, kvHeads, blockSize, headSize]. Parameter combinations
    (reference paged_attention_operation.cpp:302-323), dim checks (:697-726, :965-994) and the head
    counts, which the reference leaves to its kernel library."""
    E = binding.ERROR_CODE
    P = binding.PagedAttentionParam
    base = dict(headNum=32, kvHeadNum=16, qkScale=0.088, inputLayout=1)
    for extra in (dict(calcType=1), dict(compressType=1), dict(quantType=1), dict(scaleType=1),
                  dict(mlaVHeadSize=512, kvHeadNum=1)):
        assert binding.Operation("PagedAttentionOperation", P(**dict(base, **extra))).status == E["ERROR_INVALID_PARAM"]
    lens = np.full((4,), 100, dtype=np.int32)
    mk = binding.make_tensor

    def pack(q=(4, 32, 128), kc=(9, 16, 64, 128), vc=(9, 16, 64, 128), tables=(4, 8), dtype="float16", mask=None):
        t = [mk(dtype, q, FAKE_DEVICE), mk(dtype, kc, FAKE_DEVICE), mk(dtype, vc, FAKE_DEVICE),
             mk("int32", tables, FAKE_DEVICE), mk("int32", (4,), FAKE_DEVICE, host_ptr=lens.ctypes.data)]
        if mask:
            t.append(mk(dtype, mask, FAKE_DEVICE))
        return t

    out = lambda shape=(4, 32, 128), dtype="float16": [mk(dtype, shape, FAKE_DEVICE)]
    for mask_type, mask in ((0, None), (1, (4, 1, 512)), (2, (32, 1, 512))):
        op = binding.Operation("PagedAttentionOperation", P(**dict(base, maskType=mask_type)))
        assert op.status == 0
        st, descs = op.infer_shape(pack(mask=mask))
        assert st == 0 and [descs[0].dims[i] for i in range(3)] == [4, 32, 128]
        assert op.setup(pack(mask=mask), out(), ctx)[0] == 0
        assert op.setup(pack(mask=mask, dtype="bf16"), out(dtype="bf16"), ctx)[0] == 0
        op.close()
    op = binding.Operation("PagedAttentionOperation", P(**base))
    assert op.infer_shape(pack(kc=(9, 16, 64)))[0] == E["ERROR_INVALID_TENSOR_DIM_NUM"]
    assert op.infer_shape(pack(q=(4, 32 * 128)))[0] == E["ERROR_INVALID_TENSOR_DIM_NUM"]
    assert op.infer_shape(pack(vc=(9, 16, 64, 64)))[0] == E["ERROR_INVALID_TENSOR_DIM"]    # head sizes
    assert op.infer_shape(pack(q=(4, 32, 64)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.infer_shape(pack(vc=(8, 16, 64, 128)))[0] == E["ERROR_INVALID_TENSOR_DIM"]   # numBlocks
    assert op.infer_shape(pack(vc=(9, 16, 32, 128)))[0] == E["ERROR_INVALID_TENSOR_DIM"]   # blockSize
    assert op.setup(pack(), out((4, 32, 64)), ctx)[0] == E["ERROR_INVALID_TENSOR_DIM"]
    # what the reference's kernel library refuses: head counts of the caches and of the output
    assert op.infer_shape(pack(kc=(9, 64, 16, 128), vc=(9, 64, 16, 128)))[0] == 0  # token-major caches fit the dim rules
    assert op.setup(pack(kc=(9, 64, 16, 128), vc=(9, 64, 16, 128)), out(), ctx)[0] == E["ERROR_INVALID_PARAM"]
    assert op.setup(pack(vc=(9, 8, 64, 128)), out(), ctx)[0] == E["ERROR_INVALID_PARAM"]
    assert op.setup(pack(), out((4, 16, 128)), ctx)[0] == E["ERROR_INVALID_PARAM"]
    assert op.setup(pack(kc=(9, 16, 24, 128), vc=(9, 16, 24, 128)), out(), ctx)[0] == E["ERROR_INVALID_PARAM"]  # 16-aligned
    op.close()


def test_paged_attention_head_compression_checks(binding, ctx):
    """compressType KVHEAD / KVHEAD_ROPE: parameter combinations (reference paged_attention_operation.cpp:197-215,
    225,266,294,309,339), the razorOffset input and its dims (:426-427,877-898), and what the reference's kernel
    library asks of the shapes (mixkernels/pagedattention/paged_attention_operation.cpp:316-325,342-354,754-758)."""
    E = binding.ERROR_CODE
    P = binding.PagedAttentionParam
    base = dict(headNum=32, kvHeadNum=8, qkScale=0.088)
    for bad in (dict(compressType=3), dict(compressType=-1), dict(compressType=2, maskType=1),
                dict(compressType=2, batchRunStatusEnable=True), dict(compressType=1, calcType=1, maskType=1),
                dict(compressType=1, scaleType=1), dict(compressType=1, inputLayout=1),
                dict(compressType=1, mlaVHeadSize=64, kvHeadNum=1), dict(compressType=1, quantType=2, outDataType=1)):
        assert binding.Operation("PagedAttentionOperation", P(**dict(base, **bad))).status == E["ERROR_INVALID_PARAM"], bad
    lens = np.full((32,), 100, dtype=np.int32)
    mk = binding.make_tensor

    def pack(q=(4, 32, 128), kc=(64, 128, 1, 128), vc=(64, 128, 1, 128), tables=(32, 8), n_lens=32, dtype="float16",
             extra=()):
        return [mk(dtype, q, FAKE_DEVICE), mk(dtype, kc, FAKE_DEVICE), mk(dtype, vc, FAKE_DEVICE),
                mk("int32", tables, FAKE_DEVICE), mk("int32", (n_lens,), FAKE_DEVICE, host_ptr=lens.ctypes.data)] + [
                    mk(dt, shape, FAKE_DEVICE) for dt, shape in extra]

    out = lambda dtype="float16": [mk(dtype, (4, 32, 128), FAKE_DEVICE)]
    op = binding.Operation("PagedAttentionOperation", P(**dict(base, compressType=1)))
    assert op.status == 0 and op.infer_shape(pack())[0] == 0
    assert op.setup(pack(), out(), ctx)[0] == 0
    assert op.infer_shape(pack(vc=(64, 128, 1, 96)))[0] == E["ERROR_INVALID_TENSOR_DIM"]       # K and V head sizes
    assert op.setup(pack(kc=(64, 128, 8, 128), vc=(64, 128, 8, 128)), out(), ctx)[0] == E["ERROR_INVALID_PARAM"]
    assert op.setup(pack(tables=(4, 8), n_lens=4), out(), ctx)[0] == E["ERROR_INVALID_PARAM"]  # one length per pair
    op.close()
    # masks: one row per model sequence, per head of the model, or both
    for mask_type, shape, ok in ((1, (1, 512), True), (1, (4, 1, 512), True), (1, (32, 1, 512), False),
                                 (2, (32, 1, 512), True), (2, (4, 32, 1, 512), True), (2, (4, 1, 1, 512), True),
                                 (2, (32, 32, 1, 512), False), (2, (4, 4, 1, 512), False)):
        op = binding.Operation("PagedAttentionOperation", P(**dict(base, compressType=1, maskType=mask_type)))
        st = op.setup(pack(extra=[("float16", shape)]), out(), ctx)[0]
        assert st == (0 if ok else E["ERROR_INVALID_PARAM"]), (mask_type, shape)
        op.close()
    # int8 cache: descales of the model's KV heads; fp16 queries only
    op = binding.Operation("PagedAttentionOperation", P(**dict(base, compressType=1, quantType=1)))
    i8 = lambda dtype="float16", n=8 * 128: [
        mk(dtype, (4, 32, 128), FAKE_DEVICE), mk("int8", (64, 128, 1, 128), FAKE_DEVICE),
        mk("int8", (64, 128, 1, 128), FAKE_DEVICE), mk("int32", (32, 8), FAKE_DEVICE),
        mk("int32", (32,), FAKE_DEVICE, host_ptr=lens.ctypes.data), mk("float", (n,), FAKE_DEVICE),
        mk("float", (n,), FAKE_DEVICE)]
    assert op.setup(i8(), out(), ctx)[0] == 0
    assert op.setup(i8(n=128), out(), ctx)[0] == E["ERROR_INVALID_PARAM"]
    assert op.setup(i8(dtype="bf16"), out("bf16"), ctx)[0] == E["ERROR_INVALID_PARAM"]
    op.close()
    # KVHEAD_ROPE: one more input, fp32 [numBlocks, blockSize]
    op = binding.Operation("PagedAttentionOperation", P(**dict(base, compressType=2)))
    assert op.status == 0 and op.input_num() == 6
    assert op.setup(pack(extra=[("float", (64, 128))]), out(), ctx)[0] == 0
    assert op.setup(pack(dtype="bf16", extra=[("float", (64, 128))]), out("bf16"), ctx)[0] == 0
    assert op.setup(pack(extra=[("float", (64, 64))]), out(), ctx)[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.setup(pack(extra=[("float", (32, 128))]), out(), ctx)[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.setup(pack(extra=[("float", (64 * 128,))]), out(), ctx)[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.infer_shape(pack(extra=[("float16", (64, 128))]))[0] == E["ERROR_INVALID_TENSOR_INI_MATCH"]
    assert op.infer_shape(pack())[0] == E["ERROR_INVALID_IN_TENSOR_NUM"]
    op.close()


def test_reshape_and_cache_head_compression_checks(binding, ctx):
    """ReshapeAndCacheParam::compressType (reference reshape_and_cache_operation.cpp:61-80 create, :124-136 input
    counts, :286-305 dim rules; kernel library reshape_and_cache_operation.cpp:198-229,246-275 for the index tensors)."""
    E = binding.ERROR_CODE
    P = binding.ReshapeAndCacheParam
    for bad in (P(compressType=3), P(compressType=-1), P(compressType=1, kvCacheCfg=1), P(compressType=2, kvCacheCfg=2)):
        assert binding.Operation("ReshapeAndCacheOperation", bad).status == E["ERROR_INVALID_PARAM"]
    mk = binding.make_tensor

    def pack(n_extra, dtype="float16", key=(100, 4, 128), value=(100, 4, 128), kc=(32, 128, 1, 128), vc=(32, 128, 1, 128),
             pairs=8, batch=2, extra_dtype="int32"):
        t = [mk(dtype, key, FAKE_DEVICE), mk(dtype, value, FAKE_DEVICE), mk(dtype, kc, FAKE_DEVICE),
             mk(dtype, vc, FAKE_DEVICE), mk("int32", (pairs,), FAKE_DEVICE), mk(extra_dtype, (pairs,), FAKE_DEVICE),
             mk("int32", (batch,), FAKE_DEVICE)]
        if n_extra == 3:
            t.append(mk("int32", (pairs,), FAKE_DEVICE))
        return t

    outs = lambda dtype="float16": [mk(dtype, (32, 128, 1, 128), FAKE_DEVICE) for _ in range(2)]
    for compress, n_extra in ((1, 2), (2, 3)):
        op = binding.Operation("ReshapeAndCacheOperation", P(compressType=compress))
        assert op.status == 0 and op.input_num() == 5 + n_extra and op.output_num() == 2
        st, descs = op.infer_shape(pack(n_extra))
        assert st == 0 and [descs[1].dims[i] for i in range(4)] == [32, 128, 1, 128]
        assert op.setup(pack(n_extra), outs(), ctx) == (0, 0)
        assert op.setup(pack(n_extra, dtype="bf16"), outs("bf16"), ctx) == (0, 0)
        int8 = op.infer_shape(pack(n_extra, dtype="int8"))[0]
        assert int8 == (0 if compress == 1 else E["ERROR_INVALID_TENSOR_INI_MATCH"])  # the window mean is 16-bit only
        assert op.infer_shape(pack(n_extra, extra_dtype="int64"))[0] == E["ERROR_INVALID_TENSOR_INI_MATCH"]
        assert op.infer_shape(pack(5 - n_extra))[0] == E["ERROR_INVALID_IN_TENSOR_NUM"]
        assert op.infer_shape(pack(n_extra, kc=(32, 128, 4, 128), vc=(32, 128, 4, 128)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
        assert op.infer_shape(pack(n_extra, value=(100, 4, 64), vc=(32, 128, 1, 64)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
        assert op.infer_shape(pack(n_extra, key=(100, 4, 48), value=(100, 4, 48), kc=(32, 128, 1, 48),
                                   vc=(32, 128, 1, 48)))[0] == E["ERROR_INVALID_TENSOR_DIM"]      # multiple of 32
        assert op.infer_shape(pack(n_extra, value=(99, 4, 128)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
        assert op.setup(pack(n_extra, pairs=7), outs(), ctx)[0] == E["ERROR_INVALID_PARAM"]       # batch * heads entries
        assert op.setup(pack(n_extra, batch=3), outs(), ctx)[0] == E["ERROR_INVALID_PARAM"]
        op.close()


def test_reshape_and_cache_with_stride_checks(binding, ctx):
    """Creation, tensor-count, dim and host-data checks of ReshapeAndCacheWithStrideOperation
    (reference reshape_and_cache_with_stride_operation.cpp:51-88,163-299; the strides and offsets
    are host tensors read at Setup, reshape_and_cache_with_stride_ops_runner.cpp:78-104)."""
    E = binding.ERROR_CODE
    P = binding.ReshapeAndCacheWithStrideParam
    for bad in (P(compressType=1), P(compressType=2), P(compressType=3), P(kvCacheCfg=2), P(compressType=-1)):
        assert binding.Operation("ReshapeAndCacheWithStrideOperation", bad).status == E["ERROR_INVALID_PARAM"]
    r = P()
    r.rsv[3] = 1
    assert binding.Operation("ReshapeAndCacheWithStrideOperation", r).status == E["ERROR_INVALID_PARAM"]

    k_strides = np.array([2 * 8 * 128, 128, 1], dtype=np.int64)
    v_strides = np.array([2 * 8 * 128, 128, 1], dtype=np.int64)
    k_off = np.array([0], dtype=np.int64)
    v_off = np.array([8 * 128], dtype=np.int64)

    def pack(dtype="float16", key=(4, 8, 128), value=(4, 8, 128), kc=(16, 32, 8, 128), vc=(16, 32, 8, 128), slots=(4,),
             stride_shape=(3,), hosts=True, stride_dtype="int64"):
        mk = binding.make_tensor
        hp = lambda a: a.ctypes.data if hosts else None
        return [mk(dtype, key, FAKE_DEVICE), mk(dtype, value, FAKE_DEVICE), mk(dtype, kc, FAKE_DEVICE),
                mk(dtype, vc, FAKE_DEVICE), mk("int32", slots, FAKE_DEVICE),
                mk(stride_dtype, stride_shape, None, host_ptr=hp(k_strides)),
                mk(stride_dtype, stride_shape, None, host_ptr=hp(v_strides)),
                mk("int64", (1,), None, host_ptr=hp(k_off)), mk("int64", (1,), None, host_ptr=hp(v_off))]

    op = binding.Operation("ReshapeAndCacheWithStrideOperation", P())
    st, descs = op.infer_shape(pack())
    assert st == 0 and [descs[i].dims[j] for i in range(2) for j in range(4)] == [16, 32, 8, 128] * 2
    outs = lambda: [binding.make_tensor("float16", (16, 32, 8, 128), FAKE_DEVICE) for _ in range(2)]
    assert op.setup(pack(), outs(), ctx) == (0, 0)
    assert op.infer_shape(pack(key=(4, 8)))[0] == E["ERROR_INVALID_TENSOR_DIM_NUM"]
    assert op.infer_shape(pack(stride_shape=(3, 1)))[0] == E["ERROR_INVALID_TENSOR_DIM_NUM"]
    assert op.infer_shape(pack(value=(5, 8, 128)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.infer_shape(pack(value=(4, 4, 128)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.infer_shape(pack(vc=(16, 64, 8, 128)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.infer_shape(pack(vc=(8, 32, 8, 128)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.infer_shape(pack(kc=(16, 32, 4, 128)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.infer_shape(pack(kc=(16, 32, 8, 64)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
    # different head sizes of key and value are fine as long as each matches its cache
    assert op.infer_shape(pack(value=(4, 8, 64), vc=(16, 32, 8, 64)))[0] == 0
    assert op.infer_shape(pack(dtype="int8"))[0] == E["ERROR_INVALID_TENSOR_INI_MATCH"]
    assert op.infer_shape(pack(stride_dtype="int32"))[0] == E["ERROR_INVALID_TENSOR_INI_MATCH"]
    # outputs must describe the caches
    wrong = [binding.make_tensor("float16", (16, 32, 8, 64), FAKE_DEVICE) for _ in range(2)]
    assert op.setup(pack(), wrong, ctx)[0] == E["ERROR_INVALID_TENSOR_DIM"]
    # strides / offsets without host data, or not three strides
    assert op.setup(pack(hosts=False), outs(), ctx)[0] == E["ERROR_INVALID_PARAM"]
    assert op.setup(pack(stride_shape=(2,)), outs(), ctx)[0] == E["ERROR_INVALID_TENSOR_DIM"]
    op.close()

    op = binding.Operation("ReshapeAndCacheWithStrideOperation", P(kvCacheCfg=1))
    mk = binding.make_tensor
    siso = lambda key=(4, 1, 576), kc=(16, 32, 1, 576), slots=(4,): [
        mk("bf16", key, FAKE_DEVICE), mk("bf16", kc, FAKE_DEVICE), mk("int32", slots, FAKE_DEVICE),
        mk("int64", (3,), None, host_ptr=k_strides.ctypes.data), mk("int64", (1,), None, host_ptr=k_off.ctypes.data)]
    assert op.infer_shape(siso())[0] == 0
    assert op.setup(siso(), [mk("bf16", (16, 32, 1, 576), FAKE_DEVICE)], ctx) == (0, 0)
    assert op.infer_shape(siso(slots=(5,)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.infer_shape(siso(kc=(16, 32, 2, 576)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.infer_shape(siso(kc=(16, 32, 1, 512)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.infer_shape(siso(key=(4, 576)))[0] == E["ERROR_INVALID_TENSOR_DIM_NUM"]
    op.close()


def test_norm_rope_reshape_checks(binding, ctx):
    """Creation, dim and output checks of NormRopeReshapeOperation (reference
    norm_rope_reshape_operation.cpp:35-55,77-106,113-201; kernel-library checks
    rms_norm_and_rope_and_reshape_and_cache_operation.cpp:63-117)."""
    E = binding.ERROR_CODE
    P = binding.NormRopeReshapeParam
    assert binding.Operation("NormRopeReshapeOperation", P(epsilon=0.0)).status == E["ERROR_INVALID_PARAM"]
    assert binding.Operation("NormRopeReshapeOperation", P(epsilon=1e-39)).status == E["ERROR_INVALID_PARAM"]
    assert binding.Operation("NormRopeReshapeOperation", P(epsilon=-1e-5)).status == 0   # |epsilon| is what counts
    assert binding.Operation("NormRopeReshapeOperation", P(rotaryCoeff=4)).status == E["ERROR_INVALID_PARAM"]
    assert ctypes.sizeof(P) == 28
    mk = binding.make_tensor

    def pack(x=(64, 1, 512), gamma=(512,), rope=(64, 64), cos=(64, 64), sin=(64, 64), slots=(64,),
             cache=(192, 128, 1, 576), gamma_dtype="float16"):
        return [mk("float16", x, FAKE_DEVICE), mk(gamma_dtype, gamma, FAKE_DEVICE), mk("float16", rope, FAKE_DEVICE),
                mk("float16", cos, FAKE_DEVICE), mk("float16", sin, FAKE_DEVICE), mk("int32", slots, FAKE_DEVICE),
                mk("float16", cache, FAKE_DEVICE)]

    op = binding.Operation("NormRopeReshapeOperation", P())
    assert op.get_name() == "NormRopeReshapeOperation" and (op.input_num(), op.output_num()) == (7, 1)
    st, descs = op.infer_shape(pack())
    assert st == 0 and [descs[0].dims[i] for i in range(4)] == [192, 128, 1, 576]
    out = lambda shape=(192, 128, 1, 576), dtype="float16", fmt="nd": [mk(dtype, shape, FAKE_DEVICE, fmt=fmt)]
    assert op.setup(pack(), out(), ctx) == (0, 0)
    assert op.infer_shape(pack(x=(64, 512)))[0] == E["ERROR_INVALID_TENSOR_DIM_NUM"]
    assert op.infer_shape(pack(cache=(192, 128, 576)))[0] == E["ERROR_INVALID_TENSOR_DIM_NUM"]
    assert op.infer_shape(pack(gamma=(496,)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.infer_shape(pack(rope=(63, 64)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.infer_shape(pack(cos=(63, 64)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.infer_shape(pack(cos=(64, 32)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.infer_shape(pack(sin=(64, 32)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.infer_shape(pack(cache=(192, 128, 1, 512)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.infer_shape(pack(x=(64, 1, 520), gamma=(520,), cache=(192, 128, 1, 584)))[0] == E["ERROR_INVALID_TENSOR_DIM"]
    # rows far beyond the reference's Ascend buffer bound are fine here
    assert op.infer_shape(pack(x=(64, 1, 16384), gamma=(16384,), cache=(192, 128, 1, 16448)))[0] == 0
    # the output against the cache: a dtype or format outside the operation's table is caught by the table
    # check that runs first; then rank and dims
    assert op.setup(pack(), out(dtype="bf16"), ctx)[0] == E["ERROR_INVALID_TENSOR_INI_MATCH"]
    assert op.setup(pack(), out(fmt="fractal_nz"), ctx)[0] == E["ERROR_INVALID_TENSOR_INI_MATCH"]
    assert op.setup(pack(), out(shape=(192, 128, 576)), ctx)[0] == E["ERROR_INVALID_TENSOR_SIZE"]
    assert op.setup(pack(), out(shape=(192, 64, 1, 576)), ctx)[0] == E["ERROR_INVALID_TENSOR_DIM"]
    # the kernel library's own checks, met at Setup: one head, equal row counts, rows in units of 16
    assert op.setup(pack(x=(64, 2, 512)), out(), ctx)[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.setup(pack(slots=(63,)), out(), ctx)[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.setup(pack(sin=(63, 64)), out(), ctx)[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.setup(pack(rope=(64, 8), cos=(64, 8), sin=(64, 8), cache=(192, 128, 1, 520)),
                    out(shape=(192, 128, 1, 520)), ctx)[0] == E["ERROR_INVALID_TENSOR_DIM"]
    op.close()


def test_torch_atb_surface(pkg):
    """The reference's torch binding surface: snake_case parameter fields, nested enums, name and
    tensor counts (reference src/torch_atb/bindings.cpp:84-93, :520-590, :926-944)."""
    ta = pkg.torch_atb
    p = ta.PagedAttentionParam(head_num=32, qk_scale=0.088, kv_head_num=8,
                               mask_type=ta.PagedAttentionParam.MaskType.MASK_TYPE_ALIBI, batch_run_status_enable=True,
                               scale_type=ta.PagedAttentionParam.ScaleType.SCALE_TYPE_LOGN)
    assert (p.head_num, p.kv_head_num, p.mask_type, p.batch_run_status_enable, p.scale_type) == (32, 8, 2, True, 1)
    assert abs(p.qk_scale - 0.088) < 1e-7 and "head_num: 32" in repr(p)
    op = ta.Operation(p)
    assert (op.name, op.input_num, op.output_num) == ("PagedAttentionOperation", 8, 1)
    assert repr(op) == "op name: PagedAttentionOperation, input_num: 8, output_num: 1"
    op.close()
    with pytest.raises(AttributeError):
        ta.PagedAttentionParam(headNum=1)
    with pytest.raises(RuntimeError):
        ta.Operation(ta.PagedAttentionParam(head_num=0))
    rac = ta.Operation(ta.ReshapeAndCacheParam(kv_cache_cfg=ta.ReshapeAndCacheParam.KvCacheCfg.K_CACHE_V_BYPASS))
    assert (rac.name, rac.input_num, rac.output_num) == ("ReshapeAndCacheOperation", 3, 1)
    rac.close()
    mla = ta.Operation(ta.MultiLatentAttentionParam(head_num=128, kv_head_num=1, qk_scale=0.07,
                                                    cache_mode=ta.MultiLatentAttentionParam.CacheMode.KROPE_CTKV,
                                                    calc_type=ta.MultiLatentAttentionParam.CalcType.CALC_TYPE_RING))
    assert (mla.input_num, mla.output_num) == (6, 2)
    mla.close()
    omni = ta.Operation(ta.ReshapeAndCacheOmniParam())
    assert (omni.name, omni.input_num, omni.output_num) == ("ReshapeAndCacheOmniOperation", 8, 2)
    omni.close()


def test_dequant_vector_lengths(binding, ctx):
    e = binding.ERROR_CODE
    op = binding.Operation("PagedAttentionOperation",
                           binding.PagedAttentionParam(headNum=32, kvHeadNum=16, quantType=1, qkScale=0.088))
    lens = np.array([5, 6, 7, 8], dtype=np.int32)

    def pack(n):
        return [
            binding.make_tensor("float16", [4, 32, 128], FAKE_DEVICE),
            binding.make_tensor("int8", [4, 64, 16, 128], FAKE_DEVICE),
            binding.make_tensor("int8", [4, 64, 16, 128], FAKE_DEVICE),
            binding.make_tensor("int32", [4, 32], FAKE_DEVICE),
            binding.make_tensor("int32", [4], FAKE_DEVICE, host_ptr=lens.ctypes.data),
            binding.make_tensor("float", [n], FAKE_DEVICE),
            binding.make_tensor("float", [2048], FAKE_DEVICE),
        ]
    outs = [binding.make_tensor("float16", [4, 32, 128], FAKE_DEVICE)]
    assert op.setup(pack(2048), outs, ctx)[0] == 0
    assert op.setup(pack(128), outs, ctx)[0] == e["ERROR_INVALID_PARAM"]
    # uint64-packed descales (Utils::QuantParamConvert): both vectors or neither
    ins = pack(2048)
    ins[5] = binding.make_tensor("int64", [2048], FAKE_DEVICE)
    assert op.setup(ins, outs, ctx)[0] == e["ERROR_INVALID_TENSOR_INI_MATCH"]
    ins[6] = binding.make_tensor("int64", [2048], FAKE_DEVICE)
    assert op.setup(ins, outs, ctx)[0] == 0
    ins[5] = binding.make_tensor("int64", [128], FAKE_DEVICE)
    assert op.setup(ins, outs, ctx)[0] == e["ERROR_INVALID_PARAM"]
    op.close()


def test_int8_query_quantisation_param_and_tensor_rules(binding, ctx):
    """quantType TYPE_QUANT_QKV_OFFLINE / ONLINE (reference paged_attention_operation.cpp:250-275 parameter rules,
    :429-436 inputs kDescale, vDescale (+ pScale offline), :455-459 the output takes outDataType; kernel library
    paged_attention_operation.cpp:357-403: one fp32 descale per query head)."""
    e = binding.ERROR_CODE
    P = binding.PagedAttentionParam
    for bad in (dict(outDataType=0), dict(outDataType=binding.ACL_FLOAT16, hasQuantOffset=True),
                dict(outDataType=binding.ACL_FLOAT16, calcType=1, maskType=1),
                dict(outDataType=binding.ACL_FLOAT16, compressType=1),
                dict(outDataType=binding.ACL_FLOAT16, scaleType=1),
                dict(outDataType=binding.ACL_FLOAT16, mlaVHeadSize=512, kvHeadNum=1)):
        kw = dict(headNum=32, kvHeadNum=2, quantType=3, qkScale=0.088)
        kw.update(bad)
        op = binding.Operation("PagedAttentionOperation", P(**kw))
        assert op.status == e["ERROR_INVALID_PARAM"], bad
    lens = np.array([5, 0, 700, 8], dtype=np.int32)

    def pack(offline, heads=32, mask="bf16", q="int8"):
        ins = [binding.make_tensor(q, [4, 32, 128], FAKE_DEVICE), binding.make_tensor("int8", [9, 128, 2, 128], FAKE_DEVICE),
               binding.make_tensor("int8", [9, 128, 2, 128], FAKE_DEVICE), binding.make_tensor("int32", [4, 6], FAKE_DEVICE),
               binding.make_tensor("int32", [4], FAKE_DEVICE, host_ptr=lens.ctypes.data),
               binding.make_tensor(mask, [4, 1, 768], FAKE_DEVICE),
               binding.make_tensor("float", [heads], FAKE_DEVICE), binding.make_tensor("float", [32], FAKE_DEVICE)]
        return ins + ([binding.make_tensor("float", [32], FAKE_DEVICE)] if offline else [])
    for quant, offline in ((3, False), (2, True)):
        op = binding.Operation("PagedAttentionOperation", P(headNum=32, kvHeadNum=2, quantType=quant, qkScale=0.088,
                                                            maskType=1, outDataType=binding.ACL_BF16))
        assert op.ok and op.input_num() == (9 if offline else 8) and op.output_num() == 1
        st, descs = op.infer_shape(pack(offline))
        assert st == 0 and descs[0].dtype == binding.ACL_BF16 and [descs[0].dims[i] for i in range(3)] == [4, 32, 128]
        outs = [binding.make_tensor("bf16", [4, 32, 128], FAKE_DEVICE)]
        st, ws = op.setup(pack(offline), outs, ctx)
        # 13 tiles of 64 tokens in three shares: the sequence of 700 tokens is cut twice; piece table, merge table,
        # three partial rows of 2 x 16 heads in the output's 16-bit type, their log-sum-exps in fp32
        assert st == 0 and ws == 256 + 256 + 3 * 2 * 16 * 128 * 2 + 3 * 2 * 16 * 4
        assert op.setup(pack(offline, heads=2), outs, ctx)[0] == e["ERROR_INVALID_PARAM"]        # descales per query head
        assert op.setup(pack(offline, mask="float16"), outs, ctx)[0] == e["ERROR_INVALID_TENSOR_INI_MATCH"]
        assert op.setup(pack(offline, q="float16"), outs, ctx)[0] == e["ERROR_INVALID_TENSOR_INI_MATCH"]
        assert op.setup(pack(not offline), outs, ctx)[0] == e["ERROR_INVALID_IN_TENSOR_NUM"]
        lens[2] = 6 * 128 + 1                                   # longer than its block-table row
        assert op.setup(pack(offline), outs, ctx)[0] == e["ERROR_INVALID_PARAM"]
        lens[2] = 700
        op.close()


def test_quant_param_convert(binding):
    """reference tests/unittest/core/test_utils.cpp:37-50: the low 32 bits carry the float, the rest is 0;
    null arguments are ignored."""
    lib = binding.atb()
    lib.atb_c_quant_param_convert(None, None, 0)
    src = np.array([1.0, 2.3, 3.0, 4.0, 5.0, -0.0, np.inf], dtype=np.float32)
    dest = np.full(len(src), 0xFFFFFFFFFFFFFFFF, dtype=np.uint64)
    lib.atb_c_quant_param_convert(src.ctypes.data, dest.ctypes.data, len(src))
    assert np.array_equal(dest, src.view(np.uint32).astype(np.uint64))
    assert np.array_equal((dest & 0xFFFFFFFF).astype(np.uint32).view(np.float32), src)


def test_tensor_size_helper(binding):
    t = binding.make_tensor("bf16", [3, 5, 7], FAKE_DEVICE)
    assert t.dataSize == 3 * 5 * 7 * 2
    assert binding.make_tensor("int64", [4], FAKE_DEVICE).dataSize == 32
    assert binding.make_tensor("float", [2, 0], FAKE_DEVICE).dataSize == 0
    t = binding.make_tensor("float", [2, 2], FAKE_DEVICE)
    t.dimNum = 0
    assert binding.atb().atb_c_tensor_size(ctypes.byref(t)) == 0


def _declared_symbols(header):
    import re
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(atbmi_[a-z0-9_]+|atb_c_[a-z0-9_]+)\s*\(", text)))


@pytest.mark.parametrize("header,lib", [("atbmi_kernels.h", "libatbmi_kernels.so"), ("atb_capi.h", "libatb.so")])
def test_every_declared_symbol_is_exported(pkg, header, lib):
    names = _declared_symbols(header)
    assert len(names) >= 10
    path = os.path.join(ROOT, "ascend-transformer-boost_amd", "lib", lib)
    handle = ctypes.CDLL(path)
    for n in names:
        assert hasattr(handle, n), "%s does not export %s" % (lib, n)


def test_acl_tensor_handle_and_two_call_wrappers(binding, ctx):
    """The aclnn-style tensor handle and AtbMLAGetWorkspaceSize / AtbPagedCacheLoadGetWorkspaceSize up to
    Setup (reference include/atb/atb_acl.h:99-116,251-267; atb_acl_mla.cpp:25-116)."""
    lib = binding.atb()
    E = binding.ERROR_CODE
    t = binding.acl_tensor("bf16", [4, 128, 512], FAKE_DEVICE)
    assert t
    dt, fmt, addr = ctypes.c_int32(), ctypes.c_int32(), ctypes.c_void_p()
    assert lib.aclGetDataType(t, ctypes.byref(dt)) == 0 and dt.value == binding.ACL_BF16
    assert lib.aclGetFormat(t, ctypes.byref(fmt)) == 0 and fmt.value == binding.ACL_FORMAT_ND
    assert lib.aclGetRawTensorAddr(t, ctypes.byref(addr)) == 0 and addr.value == FAKE_DEVICE
    assert lib.aclGetDataType(None, ctypes.byref(dt)) != 0
    lib.aclDestroyTensor(t)
    assert [lib.aclDataTypeSize(c) for c in (binding.ACL_INT8, binding.ACL_FLOAT16, binding.ACL_BF16, binding.ACL_FLOAT,
                                             binding.ACL_INT64, -1)] == [1, 2, 2, 4, 8, 0]

    lens = np.array([100, 7, 300, 1], dtype=np.int32)
    mk = binding.acl_tensor
    handles = dict(q=mk("float16", [4, 32, 512], FAKE_DEVICE), qr=mk("float16", [4, 32, 64], FAKE_DEVICE),
                   kv=mk("float16", [16, 128, 1, 512], FAKE_DEVICE), kr=mk("float16", [16, 128, 1, 64], FAKE_DEVICE),
                   tables=mk("int32", [4, 3], FAKE_DEVICE), lens=mk("int32", [4], lens.ctypes.data),
                   out=mk("float16", [4, 32, 512], FAKE_DEVICE), lse=mk("float16", [4, 32, 1], FAKE_DEVICE))
    ws, op = ctypes.c_uint64(0), ctypes.c_void_p()

    def mla(calc_type, cache_mode=1, out="out", lse=None, op_ref=op):
        h = handles
        return lib.AtbMLAGetWorkspaceSize(h["q"], h["qr"], h["kv"], h["kr"], h["tables"], h["lens"], None, None, None, None,
                                          32, 0.1, 1, 0, calc_type, cache_mode, h[out], h[lse] if lse else None,
                                          ctypes.byref(ws), ctypes.byref(op_ref), ctx.ptr)
    assert mla(0) == 0 and op.value and ws.value > 0
    first = op.value
    assert mla(0) == 0 and op.value == first          # an existing operation is reused
    ring = ctypes.c_void_p()
    assert mla(2, lse="lse", op_ref=ring) == 0 and ring.value and ring.value != first
    nz = ctypes.c_void_p()
    assert mla(0, cache_mode=4, op_ref=nz) == E["ERROR_INVALID_PARAM"] and not nz.value   # no such cache mode
    lens[2] = 3 * 128 + 1                              # longer than its block table: Setup refuses
    assert mla(0) == E["ERROR_INVALID_PARAM"]
    assert lib.AtbMLA(None, 0, None, ctx.ptr) == E["ERROR_INVALID_OPERATION_ADDR"]
    # a handle with more than 8 dims does not convert: the wrapper returns that status, not Setup's
    # (reference atb_acl_mla.cpp:69-96 checks every conversion)
    lens[2] = 300
    wide = mk("float16", [1] * 9, FAKE_DEVICE)
    good = handles["out"]
    handles["out"] = wide
    assert mla(0) == E["ERROR_INVALID_TENSOR_DIM"]
    handles["out"] = good
    lib.aclDestroyTensor(wide)
    for o in (op, ring):
        lib.atb_c_destroy_operation(o)

    load = ctypes.c_void_p()
    hc = dict(kc=mk("float16", [16, 128, 8, 128], FAKE_DEVICE), vc=mk("float16", [16, 128, 8, 128], FAKE_DEVICE),
              tables=mk("int32", [4, 3], FAKE_DEVICE), lens=mk("int32", [4], FAKE_DEVICE),
              key=mk("float16", [400, 8, 128], FAKE_DEVICE), value=mk("float16", [400, 8, 128], FAKE_DEVICE),
              starts=mk("int32", [4], FAKE_DEVICE))
    assert lib.AtbPagedCacheLoadGetWorkspaceSize(hc["kc"], hc["vc"], hc["tables"], hc["lens"], hc["key"], hc["value"],
                                                 hc["starts"], 1, False, True, ctypes.byref(ws), ctypes.byref(load),
                                                 ctx.ptr) == 0 and load.value
    lib.atb_c_destroy_operation(load)
    # without seqStarts the wrapper binds six tensors, and the ND operation takes seven: refused, as in the reference
    # (atb_acl_paged_cache_load.cpp:37-41 against paged_cache_load_operation.cpp:93-100)
    six = ctypes.c_void_p()
    assert lib.AtbPagedCacheLoadGetWorkspaceSize(hc["kc"], hc["vc"], hc["tables"], hc["lens"], hc["key"], hc["value"],
                                                 None, 1, False, False, ctypes.byref(ws), ctypes.byref(six),
                                                 ctx.ptr) == E["ERROR_INVALID_IN_TENSOR_NUM"]
    lib.atb_c_destroy_operation(six)
    # the fractal-NZ layout (kvCacheCfg 0): six tensors, caches [blocks, channels / 16, blockSize, 16], rows [tokens, channels]
    nzf = binding.ACL_FORMAT_BY_NAME["fractal_nz"]
    hn = dict(kc=mk("float16", [16, 64, 128, 16], FAKE_DEVICE, nzf), vc=mk("float16", [16, 64, 128, 16], FAKE_DEVICE, nzf),
              key=mk("float16", [400, 1024], FAKE_DEVICE), value=mk("float16", [400, 1024], FAKE_DEVICE))
    nzload = ctypes.c_void_p()
    assert lib.AtbPagedCacheLoadGetWorkspaceSize(hn["kc"], hn["vc"], hc["tables"], hc["lens"], hn["key"], hn["value"],
                                                 None, 0, False, False, ctypes.byref(ws), ctypes.byref(nzload),
                                                 ctx.ptr) == 0 and nzload.value
    # token-major handles do not match that operation's dtype / format table
    assert lib.AtbPagedCacheLoadGetWorkspaceSize(hc["kc"], hc["vc"], hc["tables"], hc["lens"], hc["key"], hc["value"],
                                                 None, 0, False, False, ctypes.byref(ws), ctypes.byref(nzload),
                                                 ctx.ptr) == E["ERROR_INVALID_TENSOR_INI_MATCH"]
    lib.atb_c_destroy_operation(nzload)
    hc.update({"nz_" + k: v for k, v in hn.items()})
    for h in list(handles.values()) + list(hc.values()):
        lib.aclDestroyTensor(h)


def test_cpp_caller_builds_and_runs_against_the_public_headers(pkg, tmp_path):
    """tests/cpp/atb_caller.cpp uses nothing but atb/atb_infer.h, the way a caller of the reference does
    (context, CreateOperation, InferShape, Setup, the error paths); it is compiled with the host compiler
    against include/ and the built libraries and run on the CPU."""
    lib_dir = os.path.join(ROOT, "ascend-transformer-boost_amd", "lib")
    exe = str(tmp_path / "atb_caller")
    build = subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-I" + os.path.join(ROOT, "include"),
                            os.path.join(HERE, "cpp", "atb_caller.cpp"), "-o", exe, "-L" + lib_dir, "-latb",
                            "-latbmi_kernels", "-Wl,-rpath," + lib_dir], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                           text=True)
    assert build.returncode == 0, build.stdout
    run = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=60)
    assert run.returncode == 0 and run.stdout.strip().endswith("ok"), run.stdout + run.stderr


def test_cpp_api_symbols_are_exported(pkg):
    """The C++ entry points an ATB caller links against."""
    path = os.path.join(ROOT, "ascend-transformer-boost_amd", "lib", "libatb.so")
    out = subprocess.run(["nm", "-DC", "--defined-only", path], stdout=subprocess.PIPE, text=True).stdout
    for needle in [
        "atb::CreateOperation<atb::infer::PagedAttentionParam>",
        "atb::CreateOperation<atb::infer::ReshapeAndCacheParam>",
        "atb::CreateOperation<atb::infer::ReshapeAndCacheWithStrideParam>",
        "atb::CreateOperation<atb::infer::ReshapeAndCacheOmniParam>",
        "atb::CloneOperationParam<atb::infer::ReshapeAndCacheOmniParam>",
        "atb::UpdateOperationParam<atb::infer::ReshapeAndCacheOmniParam>",
        "atb::CreateOperation<atb::infer::NormRopeReshapeParam>",
        "atb::CreateOperation<atb::infer::RopeParam>",
        "atb::CreateOperation<atb::infer::ElewiseParam>",
        "atb::DestroyOperation(atb::Operation*)",
        "atb::CreateContext(atb::Context**)",
        "atb::DestroyContext(atb::Context*)",
        "atb::Utils::GetTensorSize(atb::TensorDesc const&)",
        "atb::Utils::GetTensorNumel(atb::Tensor const&)",
        "atb::Utils::GetAtbVersion",
        "AtbMLAGetWorkspaceSize", "AtbMLA", "AtbPagedCacheLoadGetWorkspaceSize", "AtbPagedCacheLoad",
        "aclCreateTensor", "aclDestroyTensor", "aclGetViewShape", "aclGetDataType", "aclGetFormat", "aclDataTypeSize",
    ]:
        assert needle in out, needle


def test_kernel_layer_validates_without_a_gpu(binding):
    """Argument validation of the C ABI happens before any HIP call."""
    k = binding.kernels()
    assert k.atbmi_reshape_and_cache(None, None, None, None, None, 1, 1, 1, 1, 1, 2, None) == 1
    assert b"non-null" in k.atbmi_last_error()
    assert k.atbmi_reshape_and_cache(1, None, 1, None, 1, 1, 1, 1, 1, 1, 3, None) == 1
    assert k.atbmi_quant_per_channel(1, 5, 1, None, 1, 1, 1, None) == 1
    assert k.atbmi_norm_rope_reshape_and_cache(16, 16, 16, 16, 16, 16, None, 1, 512, 64, 128, 0, 1e-5, None) == 1
    assert k.atbmi_norm_rope_reshape_and_cache(16, 16, 16, 16, 16, 16, 16, 1, 500, 64, 128, 0, 1e-5, None) == 1
    assert k.atbmi_norm_rope_reshape_and_cache(16, 16, 16, 16, 16, 16, 16, 1, 512, 64, 128, 2, 1e-5, None) == 1
    assert k.atbmi_norm_rope_reshape_and_cache(16, 8, 16, 16, 16, 16, 16, 1, 512, 64, 128, 0, 1e-5, None) == 1
    assert k.atbmi_norm_rope_reshape_and_cache(16, 16, 16, 16, 16, 16, 16, 0, 512, 64, 128, 0, 1e-5, None) == 0
    strides = np.array([256, 128, 1], dtype=np.int64)
    assert k.atbmi_reshape_and_cache_strided(1, None, 1, None, 1, 1, 1, 1, 1, 1, 2, None, 0, None, 0, None) == 1
    assert k.atbmi_reshape_and_cache_strided(1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 2, strides.ctypes.data, 0, None, 0, None) == 1
    assert k.atbmi_reshape_and_cache_strided(1, None, 1, None, 1, 0, 1, 1, 1, 1, 2, strides.ctypes.data, 0, None, 0,
                                             None) == 0
    shape = binding.AtbmiPaShape(qDtype=0, kvDtype=0, numHeads=8, numKvHeads=3, headDimK=128, headDimV=128,
                                 blockSize=128, numBlocks=4, maxBlocksPerSeq=4, numQueryRows=4, qkScale=1.0)
    plan = ctypes.c_void_p()
    assert k.atbmi_pa_plan_create(ctypes.byref(shape), ctypes.byref(plan)) == 1
    shape.numKvHeads = 8
    assert k.atbmi_pa_plan_create(ctypes.byref(shape), ctypes.byref(plan)) == 0
    lens = np.array([100, 0, 512, 7], dtype=np.int32)
    assert k.atbmi_pa_plan_update(plan, lens.ctypes.data, 4) == 0
    assert k.atbmi_pa_plan_num_chunks(plan) >= 3
    # bytes: valid rows * G*(D+Dv)*2 + 3 rows of q/out + table entries + lens
    want = (100 + 512 + 7) * 8 * 256 * 2 + 3 * 8 * 256 * 2 + (1 + 4 + 1) * 4 + 4 * 4
    assert k.atbmi_pa_plan_algorithmic_bytes(plan) == want
    lens[2] = 513
    assert k.atbmi_pa_plan_update(plan, lens.ctypes.data, 4) == 1
    k.atbmi_pa_plan_destroy(plan)
    # a mask needs a row length and non-negative strides; its bytes count per distinct row
    lens[2] = 512
    shape.hasMask = 1
    assert k.atbmi_pa_plan_create(ctypes.byref(shape), ctypes.byref(plan)) == 1
    for batch_stride, head_stride, extra in ((0, 0, 512), (512, 0, 619), (0, 512, 8 * 512), (8 * 512, 512, 8 * 619)):
        shape.maskLen, shape.maskBatchStride, shape.maskHeadStride, shape.hasLogN = 512, batch_stride, head_stride, 1
        assert k.atbmi_pa_plan_create(ctypes.byref(shape), ctypes.byref(plan)) == 0
        assert k.atbmi_pa_plan_update(plan, lens.ctypes.data, 4) == 0
        assert k.atbmi_pa_plan_algorithmic_bytes(plan) == want + extra * 2 + 4 * 4
        k.atbmi_pa_plan_destroy(plan)
    shape.maskBatchStride = -1
    assert k.atbmi_pa_plan_create(ctypes.byref(shape), ctypes.byref(plan)) == 1
    # several query rows per sequence: K/V count once, q/out and the mask once per row
    shape.maskBatchStride, shape.maskHeadStride, shape.maskRowBy, shape.hasLogN = 512, 0, 1, 0
    shape.numQueryRows = 9
    assert k.atbmi_pa_plan_create(ctypes.byref(shape), ctypes.byref(plan)) == 0
    qlens = np.array([3, 5, 4, 2], dtype=np.int32)    # sequence 1 is empty: 3 + 4 + 2 rows
    assert k.atbmi_pa_plan_update_multi(plan, lens.ctypes.data, qlens.ctypes.data, 4) == 0
    rows_ctx = 3 * 100 + 4 * 512 + 2 * 7
    want_multi = (100 + 512 + 7) * 8 * 256 * 2 + 9 * 8 * 256 * 2 + (1 + 4 + 1) * 4 + 4 * 4 + rows_ctx * 2 + 4 * 4
    assert k.atbmi_pa_plan_algorithmic_bytes(plan) == want_multi
    qlens[3] = 8                                       # more query tokens than the 7 of context
    assert k.atbmi_pa_plan_update_multi(plan, lens.ctypes.data, qlens.ctypes.data, 4) == 1
    qlens[3] = 3                                       # 10 rows, the query holds 9
    assert k.atbmi_pa_plan_update_multi(plan, lens.ctypes.data, qlens.ctypes.data, 4) == 1
    k.atbmi_pa_plan_destroy(plan)
    shape.maskRowBy = 3
    assert k.atbmi_pa_plan_create(ctypes.byref(shape), ctypes.byref(plan)) == 1


def test_pa_plan_refuses_inconsistent_layout_and_compression_fields(binding):
    """AtbmiPaShape.kvLayout, maskSeqDiv / maskSeqMod, descaleHeads and hasRazorOffset are validated on the host
    before any kernel sees them; the razor offsets add 4 bytes per attended slot to the algorithmic bytes."""
    k = binding.kernels()
    plan = ctypes.c_void_p()

    def create(**kw):
        base = dict(qDtype=0, kvDtype=0, numHeads=8, numKvHeads=1, headDimK=128, headDimV=128, blockSize=128,
                    numBlocks=8, maxBlocksPerSeq=4, numQueryRows=4, qkScale=1.0)
        base.update(kw)
        rc = k.atbmi_pa_plan_create(ctypes.byref(binding.AtbmiPaShape(**base)), ctypes.byref(plan))
        if rc == 0:
            k.atbmi_pa_plan_destroy(plan)
        return rc

    assert create() == 0
    assert create(kvLayout=1, numKvHeads=4) == 0
    assert create(kvLayout=2) == 1
    assert create(kvLayout=1, mlaCombined=1, headDimK=576, headDimV=512) == 1
    assert create(maskSeqDiv=-1) == 1 and create(maskSeqMod=-2) == 1 and create(descaleHeads=-1) == 1
    assert create(kvDtype=2, descaleHeads=4) == 0
    assert create(kvDtype=0, descaleHeads=4) == 1                       # descale slices need an int8 cache
    assert create(kvDtype=2, descaleHeads=4, numKvHeads=2) == 1         # ... and one KV head
    assert create(hasRazorOffset=1) == 0
    assert create(hasRazorOffset=1, numKvHeads=2) == 1
    assert create(hasRazorOffset=1, kvLayout=1) == 1
    shape = binding.AtbmiPaShape(qDtype=0, kvDtype=0, numHeads=8, numKvHeads=1, headDimK=128, headDimV=128,
                                 blockSize=128, numBlocks=8, maxBlocksPerSeq=4, numQueryRows=4, qkScale=1.0)
    lens = np.array([100, 0, 512, 7], dtype=np.int32)
    sizes = []
    for razor in (0, 1):
        shape.hasRazorOffset = razor
        assert k.atbmi_pa_plan_create(ctypes.byref(shape), ctypes.byref(plan)) == 0
        assert k.atbmi_pa_plan_update(plan, lens.ctypes.data, 4) == 0
        sizes.append(k.atbmi_pa_plan_algorithmic_bytes(plan))
        k.atbmi_pa_plan_destroy(plan)
    assert sizes[1] - sizes[0] == (100 + 512 + 7) * 4
    # the compressed cache write refuses what its kernels do not cover
    assert k.atbmi_reshape_and_cache_compress(16, 16, 16, 16, 16, 16, 16, None, 2, 4, 48, 100, 256, 0, None) == 1   # 32-aligned
    assert k.atbmi_reshape_and_cache_compress(16, 16, 16, 16, 16, 16, 16, 16, 2, 4, 128, 100, 256, 2, None) == 1   # int8 mean
    assert k.atbmi_reshape_and_cache_compress(16, 16, 16, 16, 16, 16, 16, 16, 2, 4, 2048, 100, 256, 0, None) == 1  # > 1024
    assert k.atbmi_reshape_and_cache_compress(16, 16, 16, 16, 16, None, 16, None, 2, 4, 128, 100, 256, 0, None) == 1
    assert k.atbmi_reshape_and_cache_compress(16, 8, 16, 16, 16, 16, 16, None, 2, 4, 128, 100, 256, 0, None) == 1   # alignment
    assert k.atbmi_reshape_and_cache_compress(16, 16, 16, 16, 16, 16, 16, None, 0, 4, 128, 0, 256, 0, None) == 0    # nothing to do
    assert k.atbmi_reshape_and_cache_omni(16, 16, 16, 16, 16, 16, 16, None, 2, 4, 128, 100, 256, 0, None) == 1      # offsetIndex
    assert b"offsetIndex" in k.atbmi_last_error()
    assert k.atbmi_reshape_and_cache_omni(16, 16, 16, 16, 16, 16, 16, 16, 2, 4, 48, 100, 256, 0, None) == 1
    assert k.atbmi_reshape_and_cache_omni(16, 16, 16, 8, 16, 16, 16, 16, 2, 4, 128, 100, 256, 0, None) == 1
    assert k.atbmi_reshape_and_cache_omni(16, 16, 16, 16, 16, 16, 16, 16, 0, 4, 128, 0, 256, 0, None) == 0


def test_mla_int8_rows_are_cut_when_heads_are_few(binding):
    """The int8 MLA kernel runs one workgroup a CU: a call with few heads cuts every row's blocks into equal pieces
    (and asks for room for the pieces' rows and log-sum-exps), a call that fills the chip does not."""
    k = binding.kernels()
    lens = np.full(64, 4096, dtype=np.int32)

    def size(heads, batch=64):
        call = binding.AtbmiMlaInt8Call(outDtype=binding.ATBMI_BF16, numHeads=heads, blockSize=128, numBlocks=4096,
                                        maxBlocksPerSeq=32, batch=batch, numQueryRows=batch, hasMask=0, maskLen=0,
                                        qkScale=0.1, hostContextLens=lens.ctypes.data)
        ws = ctypes.c_uint64(0)
        assert k.atbmi_mla_int8_workspace_size(ctypes.byref(call), ctypes.byref(ws)) == 0, binding.last_kernel_error()
        return int(ws.value)

    def pieces(heads, batch=64):
        table_only = lambda p: (batch * p * 16 + 255) // 256 * 256
        for p in (1, 2, 3, 4):
            rows = batch * p
            want = table_only(p) + (0 if p == 1 else rows * heads * 512 * 2 + (rows * heads * 4 + 255) // 256 * 256)
            if size(heads, batch) == want:
                return p
        raise AssertionError("unexpected workspace size %d" % size(heads, batch))

    assert pieces(128) == 1      # 256 workgroups of two head tiles
    assert pieces(64) == 2       # 128 workgroups of two head tiles, twice
    assert pieces(32) == 2       # 128 workgroups of one head tile, twice
    assert pieces(16) == 4       # 64 workgroups, four times
    assert pieces(128, batch=8) == 4
    lens[:] = 1000               # eight blocks a row: pieces of at least four blocks in the longest row
    assert pieces(16) == 2


def test_int8_query_mask_fetches_stay_inside_the_rows(binding):
    """The int8-query kernel fetches 16-bit mask values as aligned 32-bit words, from the word that holds a
    row's first element to the word that holds its last. Host arithmetic over every parity of base, strides and
    row length: the words stay inside the row exactly when base % 4 == 0 and strides and length are even, and
    that is the rule the call checks (by name) before anything touches the device."""
    k = binding.kernels()
    lens = np.array([6, 5], dtype=np.int32)

    def call(mask, seq_stride, head_stride, mask_len):
        c = binding.AtbmiPaInt8QCall(outDtype=binding.ATBMI_F16, numHeads=4, numKvHeads=2, headDim=128, blockSize=128,
                                     numBlocks=4, maxBlocksPerSeq=2, batch=2, numQueryRows=2, hasMask=1,
                                     maskLen=mask_len, qkScale=1.0, maskSeqStride=seq_stride,
                                     maskHeadStride=head_stride, hostContextLens=lens.ctypes.data, mask=mask)
        size = ctypes.c_uint64(0)
        return k.atbmi_pa_int8q_workspace_size(ctypes.byref(c), ctypes.byref(size))

    for base in (0x10000, 0x10002):
        for seq_stride in (0, 6, 7, 8):
            for head_stride in (0, 6, 7):
                for mask_len in (6, 7, 8):
                    inside = True
                    for b in range(2):
                        for h in range(4):
                            row = base + 2 * (b * seq_stride + h * head_stride)   # byte address of the row
                            first = row // 4 * 4
                            last = (row + 2 * (mask_len - 1)) // 4 * 4
                            inside &= first >= row and last + 4 <= row + 2 * mask_len
                    rule = base % 4 == 0 and seq_stride % 2 == 0 and head_stride % 2 == 0 and mask_len % 2 == 0
                    assert inside == rule, (base, seq_stride, head_stride, mask_len)
                    rc = call(base, seq_stride, head_stride, mask_len)
                    assert (rc == 0) == rule, (base, seq_stride, head_stride, mask_len)
                    if rc != 0:
                        assert b"4-byte" in k.atbmi_last_error()


def test_mask_free_is_created_and_refused_at_infer_shape(binding, ctx):
    """MASK_TYPE_MASK_FREE off Atlas 300I Duo (reference paged_attention_operation.cpp:769-791,805-840): the
    operation is created, InferShape and Setup return ERROR_INVALID_TENSOR_DIM; NORM_COMPRESS is refused at creation."""
    E = binding.ERROR_CODE
    P = binding.PagedAttentionParam
    assert binding.Operation("PagedAttentionOperation", P(headNum=8, kvHeadNum=8, qkScale=1.0, maskType=5)).status == \
        E["ERROR_INVALID_PARAM"]
    op = binding.Operation("PagedAttentionOperation", P(headNum=8, kvHeadNum=8, qkScale=1.0, maskType=4))
    assert op.status == 0 and op.input_num() == 6
    mk = binding.make_tensor
    lens = np.full((2,), 5, dtype=np.int32)
    ins = [mk("float16", (2, 8, 128), FAKE_DEVICE), mk("float16", (4, 128, 8, 128), FAKE_DEVICE),
           mk("float16", (4, 128, 8, 128), FAKE_DEVICE), mk("int32", (2, 2), FAKE_DEVICE),
           mk("int32", (2,), FAKE_DEVICE, host_ptr=lens.ctypes.data), mk("float16", (1, 8, 128, 16), FAKE_DEVICE)]
    assert op.infer_shape(ins)[0] == E["ERROR_INVALID_TENSOR_DIM"]
    assert op.setup(ins, [mk("float16", (2, 8, 128), FAKE_DEVICE)], ctx)[0] == E["ERROR_INVALID_TENSOR_DIM"]
    # dim-number mistakes are still reported first
    ins[1] = mk("float16", (4, 128, 8 * 128), FAKE_DEVICE)
    assert op.infer_shape(ins)[0] == E["ERROR_INVALID_TENSOR_DIM_NUM"]
    op.close()


def test_no_wave_range_of_a_plan_is_empty(binding):
    """A range without steps writes no partial row, yet the merge kernel reads the slot of every range
    between a row's first and last: the planner must never make more ranges than 32-token steps."""
    k = binding.kernels()
    cases = []
    for heads, kv, dk, dv, mla in ((8, 1, 128, 128, 0), (8, 2, 128, 128, 0), (4, 4, 64, 64, 0), (32, 8, 128, 128, 0),
                                   (16, 1, 576, 512, 1), (128, 1, 576, 512, 1), (32, 1, 192, 128, 1), (12, 1, 256, 256, 0)):
        for lens in ([96], [64], [33], [1], [224], [32, 32], [40, 1, 70], [129, 0, 31], [225, 17], [4096], [7] * 5):
            cases.append((heads, kv, dk, dv, mla, lens))
    for heads, kv, dk, dv, mla, lens in cases:
        shape = binding.AtbmiPaShape(qDtype=0, kvDtype=0, numHeads=heads, numKvHeads=kv, headDimK=dk, headDimV=dv,
                                     blockSize=128, numBlocks=64, maxBlocksPerSeq=32, numQueryRows=len(lens),
                                     mlaCombined=mla, qkScale=1.0, kernel=binding.ATBMI_PA_KERNEL_MFMA)
        plan = ctypes.c_void_p()
        assert k.atbmi_pa_plan_create(ctypes.byref(shape), ctypes.byref(plan)) == 0, (heads, kv, dk)
        arr = np.array(lens, dtype=np.int32)
        assert k.atbmi_pa_plan_update(plan, arr.ctypes.data, len(lens)) == 0
        steps = int(sum((n + 31) // 32 for n in lens))
        ranges = k.atbmi_pa_plan_num_chunks(plan)
        assert 1 <= ranges <= steps, (heads, kv, dk, lens, ranges, steps)
        if steps == 1:
            assert k.atbmi_pa_plan_workspace_size(plan) == 0
        k.atbmi_pa_plan_destroy(plan)


def test_query_tokens_of_a_sequence_share_a_pass_of_the_128_head_mla_kernel(binding):
    """With fewer than 128 heads the 128-head MLA kernel takes the query tokens of a sequence as more heads of one pass
    over its context (128 / heads of them, at most 8): the plan then has the steps, and so the ranges, of one token per
    sequence. With 128 heads, or a mask whose rows the kernel cannot address (odd stride: the 16-head tiles take it, one
    pass per token), every token is a pass of its own."""
    k = binding.kernels()

    def ranges(heads, q_len, mask_stride=0):
        shape = binding.AtbmiPaShape(qDtype=1, kvDtype=1, numHeads=heads, numKvHeads=1, headDimK=576, headDimV=512,
                                     blockSize=128, numBlocks=64, maxBlocksPerSeq=32, numQueryRows=2 * q_len,
                                     mlaCombined=1, qkScale=1.0, kernel=binding.ATBMI_PA_KERNEL_MFMA,
                                     hasMask=1 if mask_stride else 0, maskLen=mask_stride, maskBatchStride=mask_stride,
                                     maskRowBy=1 if mask_stride else 0)
        plan = ctypes.c_void_p()
        assert k.atbmi_pa_plan_create(ctypes.byref(shape), ctypes.byref(plan)) == 0, k.atbmi_last_error()
        lens, qn = np.array([4096, 4096], dtype=np.int32), np.array([q_len, q_len], dtype=np.int32)
        assert k.atbmi_pa_plan_update_multi(plan, lens.ctypes.data, qn.ctypes.data, 2) == 0, k.atbmi_last_error()
        n, ws = k.atbmi_pa_plan_num_chunks(plan), k.atbmi_pa_plan_workspace_size(plan)
        k.atbmi_pa_plan_destroy(plan)
        return n, ws

    one, ws_one = ranges(16, 1)
    four, ws_four = ranges(16, 4)
    assert four == one and ws_four > ws_one          # the same ranges; a slot holds the partial rows of four tokens
    assert ranges(16, 8)[0] == one and ranges(16, 9)[0] > one   # eight tokens a pass at most
    assert ranges(32, 4)[0] == one and ranges(64, 2)[0] == one
    assert ranges(64, 3)[0] > one                    # 128 / 64 = 2 tokens a pass
    assert ranges(128, 2)[0] > ranges(128, 1)[0]     # the rows of 128 heads are full
    assert ranges(16, 4, mask_stride=4096)[0] == one
    assert ranges(16, 4, mask_stride=4097)[0] > one


def test_plan_refuses_a_context_longer_than_the_mask_row(binding):
    k = binding.kernels()
    shape = binding.AtbmiPaShape(qDtype=0, kvDtype=0, numHeads=8, numKvHeads=8, headDimK=128, headDimV=128,
                                 blockSize=128, numBlocks=8, maxBlocksPerSeq=8, numQueryRows=2, qkScale=1.0,
                                 hasMask=1, maskLen=300, maskBatchStride=300)
    plan = ctypes.c_void_p()
    assert k.atbmi_pa_plan_create(ctypes.byref(shape), ctypes.byref(plan)) == 0
    arr = np.array([300, 12], dtype=np.int32)
    assert k.atbmi_pa_plan_update(plan, arr.ctypes.data, 2) == 0
    arr[1] = 301
    assert k.atbmi_pa_plan_update(plan, arr.ctypes.data, 2) == 1
    assert b"mask" in k.atbmi_last_error()
    k.atbmi_pa_plan_destroy(plan)


def test_bench_refuses_more_than_one_gpu():
    """The benchmark is a one-GPU program: asked for more it says so and exits, before it touches a device."""
    import sys
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE,
                         stderr=subprocess.PIPE, text=True, timeout=120)
    assert run.returncode != 0 and "one GPU" in run.stderr and run.stdout.strip() == ""
