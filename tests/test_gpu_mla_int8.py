"""GPU parity of MultiLatentAttention's int8 cache mode (INT8_NZCACHE): the HIP kernel through the C ABI and
through atb::Operation against the CPU oracle, which restates the reference golden
(tests/apitest/opstest/python/operations/multi_latent_attention/test_multi_latent_attention_int8nz.py:115-121,
179-262) with the same tile of 128 tokens. All integer products are exact on both sides; what differs is the
order of fp32 sums and the last bit of exp, which now and then moves an int8 weight by one step of 127: tolerance
rtol = atol = 2e-3 (fp16) / 2e-2 (bf16) on outputs of magnitude <= 5 * 5 / 127. Beside it the reference's own
criterion for this operator (precision_calcu.py:111-140, compare_cv): against the golden that quantises the whole
context as one tile, the kernel's errors may not exceed the tiled golden's by the factors 10 / 2 / 2."""
import ctypes
import math

import numpy as np
import pytest
import torch

from pa_harness import assert_close, dtype_code, random_tables

pytestmark = pytest.mark.gpu

TOL = {torch.float16: 2e-3, torch.bfloat16: 2e-2}


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return torch.device("cuda:0")


@pytest.fixture(scope="module")
def stream(dev):
    return torch.cuda.Stream(device=dev)


def _case(seed, dev, ctx, heads, dtype, q_lens=None, with_mask=False, causal=None):
    """Inputs drawn the way the reference test draws them (:478-506: uniform in [-5, 5], descales in +-5/127)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    ctx = np.asarray(ctx, np.int32)
    block = 128
    pool = int(((ctx + block - 1) // block).sum()) + 3
    tables = random_tables(rng, ctx, block, pool)
    # (a sequence without context keeps its query rows: reference tiling/mla_tiling.cpp:146-149)
    rows = int(sum((1 if q_lens is None else q_lens[b]) for b in range(len(ctx))))
    written = np.concatenate([np.full(1 if q_lens is None else q_lens[b], ctx[b] > 0) for b in range(len(ctx))])
    q8 = torch.from_numpy(rng.integers(-5, 6, size=(rows, heads, 512)).astype(np.int8))
    qr = torch.from_numpy(rng.uniform(-5, 5, size=(rows, heads, 64)).astype(np.float32)).to(dtype)
    kv8 = torch.from_numpy(rng.integers(-5, 6, size=(pool, block, 1, 512)).astype(np.int8))
    kr = torch.from_numpy(rng.uniform(-5, 5, size=(pool, block, 1, 64)).astype(np.float32)).to(dtype)
    qd = torch.from_numpy(rng.uniform(-5 / 127, 5 / 127, size=heads).astype(np.float32))
    pd = torch.from_numpy(rng.uniform(-5 / 127, 5 / 127, size=heads).astype(np.float32))
    mask = None
    if with_mask:
        m = np.zeros((rows, int(ctx.max())), np.float32)
        r = 0
        for b in range(len(ctx)):   # the look-ahead mask of several query tokens: token i of n does not see the last n - 1 - i
            n = 1 if q_lens is None else q_lens[b]
            for i in range(n):
                if n - 1 - i > 0 and ctx[b] > 0:
                    m[r, ctx[b] - (n - 1 - i):ctx[b]] = -10000.0
                r += 1
        mask = torch.from_numpy(m).to(dtype)
    return dict(q8=q8, qr=qr, kv8=kv8, kr=kr, tables=torch.from_numpy(tables), ctx=ctx, qd=qd, pd=pd, mask=mask,
                q_lens=q_lens, rows=rows, heads=heads, dtype=dtype, causal=causal, written=written)


def _nz(oracle, t, n0):
    """[blocks, 128, 1, channels] -> fractal-NZ [blocks, channels / n0, 128, n0] (same element type)."""
    if t.dtype == torch.int8:
        return torch.from_numpy(oracle.nd_to_nz(t.numpy()[:, :, 0, :], n0))
    return torch.from_numpy(oracle.nd_to_nz(t.view(torch.int16).numpy()[:, :, 0, :], n0)).view(t.dtype)


def _oracle(oracle, c, scale, tile, lse=None):
    return oracle.mla_int8_decode(c["q8"].numpy(), c["qr"].float().numpy(), c["kv8"].numpy(), c["kr"].float().numpy(),
                                  c["tables"].numpy(), c["ctx"], c["qd"].numpy(), c["pd"].numpy(), scale, tile=tile,
                                  mask=None if c["mask"] is None else c["mask"].float().numpy(), q_lens=c["q_lens"],
                                  lse_out=lse, causal_rows=c["causal"])


def int8_cabi(binding, oracle, stream, dev, c, scale, want_lse=False):
    k = binding.kernels()
    t = {n: c[n].to(dev) for n in ("q8", "qr", "tables", "qd", "pd")}
    kv_nz = _nz(oracle, c["kv8"], 32).to(dev)
    kr_nz = _nz(oracle, c["kr"], 16).to(dev)
    mask = c["mask"].to(dev) if c["mask"] is not None else None
    lens = np.ascontiguousarray(c["ctx"], dtype=np.int32)
    ql = None if c["q_lens"] is None else np.ascontiguousarray(np.asarray(c["q_lens"], dtype=np.int32))
    use = None if c["causal"] in (None, True) else np.ascontiguousarray(np.asarray(c["causal"], dtype=np.int32))
    call = binding.AtbmiMlaInt8Call(
        outDtype=dtype_code(binding, c["qr"]), numHeads=c["heads"], blockSize=128, numBlocks=kv_nz.shape[0],
        maxBlocksPerSeq=c["tables"].shape[1], batch=len(lens), numQueryRows=c["rows"], hasMask=0 if mask is None else 1,
        maskLen=0 if mask is None else mask.shape[1], qkScale=scale, hostContextLens=lens.ctypes.data,
        hostQueryLens=None if ql is None else ql.ctypes.data, causalRows=0 if c["causal"] is None else 1,
        hostCausalUse=None if use is None else use.ctypes.data)
    ws_bytes = ctypes.c_uint64(0)
    if k.atbmi_mla_int8_workspace_size(ctypes.byref(call), ctypes.byref(ws_bytes)) != 0:
        raise RuntimeError("mla_int8_workspace_size: " + binding.last_kernel_error())
    with torch.cuda.stream(stream):
        ws = torch.empty(max(int(ws_bytes.value), 16), dtype=torch.uint8, device=dev)
        out = torch.full((c["rows"], c["heads"], 512), 7.0, dtype=c["dtype"], device=dev)
        lse = torch.zeros((c["rows"], c["heads"]), dtype=torch.float32, device=dev) if want_lse else None
        call.query, call.queryRope, call.kvCache = t["q8"].data_ptr(), t["qr"].data_ptr(), kv_nz.data_ptr()
        call.kRopeCache, call.blockTables = kr_nz.data_ptr(), t["tables"].data_ptr()
        call.qkDescale, call.pvDescale = t["qd"].data_ptr(), t["pd"].data_ptr()
        call.mask = mask.data_ptr() if mask is not None else None
        call.out = out.data_ptr()
        call.lse = lse.data_ptr() if lse is not None else None
        if k.atbmi_mla_int8_decode(ctypes.byref(call), ws.data_ptr(), ws_bytes.value, stream.cuda_stream) != 0:
            raise RuntimeError("mla_int8_decode: " + binding.last_kernel_error())
    stream.synchronize()
    return (out, lse) if want_lse else out


def _errors(golden, x):
    """Largest relative, mean relative and root-mean-square error (reference precision_calcu.py:78-109)."""
    golden = np.asarray(golden, np.float32)
    x = np.asarray(x, np.float32)
    rel = np.abs(x - golden) / (np.abs(golden) + 1e-7)
    return rel.max(), rel.mean(), math.sqrt(np.mean((x - golden) ** 2))


def _double_golden(true_out, golden, got, dtype):
    floor = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -8    # CV_FUSION thresholds (:56-62)
    e_got, e_gold = _errors(true_out, got), _errors(true_out, golden)
    rates = [g / max(r, floor) for g, r in zip(e_got, e_gold)]
    return rates[0] < 10 and rates[1] < 2 and rates[2] < 2, rates


# ctx, heads, dtype, q_lens, mask, causal rows    (reference :668-766: 32 sequences of 256 tokens, 32 / 128 heads;
# :1270-1367 several query tokens: row j of q sees context + j - q + 1 tokens (:356-364), per sequence with
# batch_list. The mask cases exercise the kernel layer's own mask input, which the operation does not use.)
INT8_MATRIX = [
    ([256] * 32, 32, torch.float16, None, False, None),
    ([256] * 8, 128, torch.float16, None, False, None),
    ([256] * 32, 32, torch.bfloat16, None, False, None),
    ([700, 0, 1, 128, 129, 1500], 8, torch.float16, None, False, None),
    ([515, 33, 2048], 64, torch.bfloat16, [2, 1, 3], True, None),
    ([300, 1000, 0, 77], 16, torch.float16, [2, 2, 1, 4], True, None),
    ([256, 256], 128, torch.float16, [2, 2], False, True),
    ([515, 129, 2048, 4], 64, torch.bfloat16, [2, 1, 3, 4], False, True),
    ([300, 1000, 0, 130], 16, torch.float16, [2, 2, 1, 4], False, [1, 0, 1, 1]),
    # more query rows than travel in the kernel arguments: the row list goes through the workspace
    ([130] * 70, 16, torch.float16, [2] * 70, False, True),
]


@pytest.mark.parametrize("case", INT8_MATRIX, ids=lambda c: "b%d_h%d_%s%s" % (
    len(c[0]), c[1], str(c[2]).split(".")[-1], ("_multi" if c[3] else "") + ("_causal" if c[5] is not None else "")))
def test_mla_int8_nz_kernel(binding, oracle, dev, stream, case):
    ctx, heads, dtype, q_lens, with_mask, causal = case
    c = _case(600 + heads + len(ctx), dev, ctx, heads, dtype, q_lens, with_mask, causal)
    scale = 1.0 / math.sqrt(576.0)
    want_lse = np.zeros((c["rows"], heads), np.float32)
    want = _oracle(oracle, c, scale, 128, want_lse)
    got, lse = int8_cabi(binding, oracle, stream, dev, c, scale, want_lse=True)
    # the rows of a sequence without context are nobody's: the call leaves them as they were (7 / 0 here)
    idle = torch.from_numpy(~c["written"])
    assert torch.all(got[idle] == 7.0) and torch.all(lse[idle] == 0.0)
    want[~c["written"]] = 7.0
    assert_close(got, want, TOL[dtype], "int8 NZ %s" % (case,))
    assert_close(lse, want_lse, 1e-3, "int8 NZ lse")
    # the reference's criterion: errors against the whole-context golden no worse than the tiled golden's
    true_out = _oracle(oracle, c, scale, 1 << 30)
    true_out[~c["written"]] = 7.0
    rounded = torch.from_numpy(want).to(dtype).float().numpy()
    ok, rates = _double_golden(true_out, rounded, got.float().cpu().numpy(), dtype)
    assert ok, "double-golden rates %s" % (rates,)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_mla_int8_nz_tiles_far_apart(binding, oracle, dev, stream, dtype):
    """Tiles whose scores lie far apart (a bias per cache block through the kernel layer's mask input): blocks that
    weigh 2^-29 and 2^-87 of the heaviest, a heaviest block that comes late, blocks hidden altogether, a row whose
    first blocks are all hidden. The online rescaling, the unit the accumulators are kept in and the tiles that are
    too light to count all have to agree with the golden's plain arithmetic."""
    ctx = [1100, 640, 384]
    c = _case(777, dev, ctx, 32, dtype, None, True, None)
    bias = np.zeros((3, max(ctx)), np.float32)
    for b, per_block in enumerate([[0, -20, -60, 15, -np.inf, -3, 30, -45, -20],
                                   [-np.inf, -np.inf, -60, 0, 12],
                                   [-60, -60, -60]]):
        for k, v in enumerate(per_block):
            bias[b, k * 128:(k + 1) * 128] = v
    bias[0, 700] = -np.inf      # single hidden tokens inside a visible block
    bias[1, 639] = 25.0         # the last token alone outweighs everything before it
    c["mask"] = torch.from_numpy(bias).to(dtype)
    scale = 1.0 / math.sqrt(576.0)
    want_lse = np.zeros((c["rows"], 32), np.float32)
    want = _oracle(oracle, c, scale, 128, want_lse)
    got, lse = int8_cabi(binding, oracle, stream, dev, c, scale, want_lse=True)
    assert_close(got, want, TOL[dtype], "int8 NZ, tiles far apart")
    assert_close(lse, want_lse, 1e-3, "int8 NZ lse, tiles far apart")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_mla_int8_nz_through_operation_api(binding, oracle, dev, stream, dtype):
    """MultiLatentAttentionOperation with cacheMode INT8_NZCACHE through InferShape / Setup / Execute: plain decode,
    log-sum-exp output (fp32), several query tokens (each sees the context up to itself, with or without a mask
    tensor, which the reference's int8 kernels do not read: tiling/mla_tiling.cpp:139-144; golden :356-364), and
    maskUseStatus, which exempts sequences from that (golden batch_list, :1348-1367). Inputs: query (int8),
    queryRope, kvCache (int8, fractal-NZ), kvCacheRope (fractal-NZ), blockTables, contextLens, [mask], [qSeqlen],
    qkDescale, pvDescale, [maskUseStatus] (reference multi_latent_attention_operation.cpp:245-266)."""
    heads = 32
    scale = 1.0 / math.sqrt(576.0)
    ctx = [700, 33, 1500, 128]
    q_lens = [2, 1, 3, 1]
    c = binding.Context(stream)
    for calc, mask_type, use in ((0, 0, None), (2, 0, None), (1, 1, None), (3, 0, None), (1, 0, None),
                                 (3, 0, [1, 1, 0, 1]), (3, 0, [])):
        multi, ring = calc in (1, 3), calc in (2, 3)
        causal = None if not multi else (use if use else True)
        case = _case(700 + calc, dev, ctx, heads, dtype, q_lens if multi else None, mask_type == 1, causal)
        mask_tensor, case["mask"] = case["mask"], None   # (handed to the operation, not used by it)
        kv_nz = _nz(oracle, case["kv8"], 32).to(dev)
        kr_nz = _nz(oracle, case["kr"], 16).to(dev)
        lens = torch.from_numpy(case["ctx"])
        nz_desc = lambda t: binding.make_tensor(binding._torch_acl_dtype(t), list(t.shape), device_ptr=t.data_ptr(),
                                                fmt="fractal_nz")
        ins = [case["q8"].to(dev), case["qr"].to(dev), nz_desc(kv_nz), nz_desc(kr_nz), case["tables"].to(dev), lens.to(dev)]
        host = {5: lens}
        if mask_type == 1:
            ins.append(mask_tensor.to(dev))
        if multi:
            qn = torch.tensor(q_lens, dtype=torch.int32)
            host[len(ins)] = qn
            ins.append(qn.to(dev))
        ins += [case["qd"].to(dev), case["pd"].to(dev)]
        if use is not None:
            flags = torch.tensor(use, dtype=torch.int32)
            if use:
                host[len(ins)] = flags
            ins.append(flags.to(dev) if use else binding.make_tensor("int32", [0], device_ptr=0))
        op = binding.OperationRunner("MultiLatentAttentionOperation", binding.MultiLatentAttentionParam(
            headNum=heads, kvHeadNum=1, qkScale=scale, cacheMode=2, calcType=calc, maskType=mask_type,
            maskUseStatusType=0 if use is None else 1), c)
        with torch.cuda.stream(stream):
            outs = op.run(ins, host_inputs=host)
        stream.synchronize()
        assert len(outs) == (2 if ring else 1) and tuple(outs[0].shape) == (case["rows"], heads, 512)
        assert outs[0].dtype == dtype
        want_lse = np.zeros((case["rows"], heads), np.float32)
        want = _oracle(oracle, case, scale, 128, want_lse)
        assert_close(outs[0], want, TOL[dtype], "calcType %d" % calc)
        if ring:
            assert tuple(outs[1].shape) == (case["rows"], heads, 1) and outs[1].dtype == torch.float32
            assert_close(outs[1][..., 0], want_lse, 1e-3, "lse calcType %d" % calc)
        op.close()
    c.close()
