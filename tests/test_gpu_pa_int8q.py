"""GPU parity of PagedAttention with int8 queries over int8 caches (quantType TYPE_QUANT_QKV_ONLINE / OFFLINE): the
HIP kernel through the C ABI and through atb::Operation against the CPU oracle, which restates the reference golden
(tests/apitest/kernelstest/mix/test_paged_attention_common.py:104-110,147-229,256-276) with the same tile of 128
tokens. All integer products are exact on both sides; what differs is the order of fp32 sums and the last bit of
exp, which now and then moves an int8 weight by one step of 127: tolerance rtol = atol = 2e-3 (fp16) / 2e-2 (bf16)
on outputs of magnitude <= 5 * 5 / 127. Beside it the reference's own criterion (compare_cv, :716-724 with
precision_calcu.py:111-140): against the golden that quantises the whole context as one tile, the kernel's errors
may not exceed the tiled golden's by the factors 10 / 2 / 2."""
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


def _case(seed, ctx, heads, kv_heads, d, block, dtype, mask=None, offline=False):
    """Inputs drawn the way the reference test draws them (:444-452 uniform in [-5, 5] cast to int8, :540-543
    descales in +-5/127, the offline factor in [0, 127]); mask: None, "norm" ([batch, 1, maxS], :500-504) or "alibi"
    ([batch, heads, 1, maxS], :487-498)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    ctx = np.asarray(ctx, np.int32)
    pool = int(((ctx + block - 1) // block).sum()) + 3
    tables = random_tables(rng, ctx, block, pool)
    rows = int((ctx > 0).sum())
    c = dict(
        q8=torch.from_numpy(rng.uniform(-5, 5, size=(rows, heads, d)).astype(np.int8)),
        k8=torch.from_numpy(rng.uniform(-5, 5, size=(pool, block, kv_heads, d)).astype(np.int8)),
        v8=torch.from_numpy(rng.uniform(-5, 5, size=(pool, block, kv_heads, d)).astype(np.int8)),
        kd=torch.from_numpy(rng.uniform(-5 / 127, 5 / 127, size=heads).astype(np.float32)),
        vd=torch.from_numpy(rng.uniform(-5 / 127, 5 / 127, size=heads).astype(np.float32)),
        ps=torch.from_numpy(rng.uniform(0, 127, size=heads).astype(np.float32)) if offline else None,
        tables=torch.from_numpy(tables), ctx=ctx, rows=rows, heads=heads, kv_heads=kv_heads, d=d, block=block,
        dtype=dtype, mask=None, mask_kind=mask)
    max_len = int(ctx.max())
    if mask == "norm":
        m = np.zeros((len(ctx), 1, max_len), np.float32)
        for i in range(len(ctx)):
            m[i, :, :i] = -10000.0
        c["mask"] = torch.from_numpy(m).to(dtype)
    elif mask == "alibi":
        slopes = np.array([2.0 ** (-8.0 * (i + 1) / heads) for i in range(heads)], np.float32)
        m = np.zeros((len(ctx), heads, 1, max_len), np.float32)
        for i, n in enumerate(ctx):
            if n > 0:
                m[i, :, 0, :n] = slopes[:, None] * (np.arange(n) - n + 1).astype(np.float32)[None, :]
        c["mask"] = torch.from_numpy(m).to(dtype)
    return c


PIECE_TILES = 6   # contexts of more than 6 tiles are cut, in the C-ABI tests and in their oracle alike


TILE = 64   # tokens whose weights the library quantises together


def library_cuts(c, compute_units):
    """Where the library cuts the sequences of a call with pieceTiles = 0: the tiles of 64 tokens of all sequences, in
    order, are one list cut into equal shares (share w starts at tile floor(tiles * w / shares)); shares =
    min(tiles // 4, workgroups the chip holds at once), a workgroup being up to 8 waves (4 for head size 256), one
    per (KV head, tile of 16 query heads) pair, with 2 * 64 * (D + 16) bytes of the CU's 160 KiB each. Returns
    {sequence: [tokens]}."""
    pairs = c["kv_heads"] * -(-(c["heads"] // c["kv_heads"]) // 16)
    most = 8 if c["d"] <= 128 else 4
    groups = -(-pairs // most)
    waves = -(-pairs // groups)
    per_cu = max(1, min(8 // waves, 160 * 1024 // (waves * 2 * 64 * (c["d"] + 16))))
    tiles = [-(-int(n) // 64) for n in c["ctx"]]
    total = sum(tiles)
    shares = max(1, min(total // 4, compute_units * per_cu // groups))
    starts = [total * w // shares for w in range(1, shares)]
    cuts, at = {}, 0
    for b, n in enumerate(tiles):
        here = [(s - at) * 64 for s in starts if at < s < at + n]
        assert all(y - x <= min(8192, 64 * c["block"]) for x, y in zip([0] + here, here + [int(c["ctx"][b])]))
        if here:
            cuts[b] = here
        at += n
    return cuts


def _oracle(oracle, c, scale, tile, piece_tiles=PIECE_TILES, piece_cuts=None):
    """tile: "own" for the library's tile, None for the whole context as one tile; piece_tiles counts tiles of 128
    tokens, as the C ABI does."""
    if tile == "own":
        tile = TILE
    return oracle.paged_attention_int8q(
        c["q8"].numpy(), c["k8"].numpy(), c["v8"].numpy(), c["tables"].numpy(), c["ctx"], c["kd"].numpy(), c["vd"].numpy(),
        scale, p_scale=None if c["ps"] is None else c["ps"].numpy(), tile=tile,
        mask=None if c["mask"] is None else c["mask"].float().numpy(), mask_per_head=False, out_init=7.0,
        piece_tiles=None if piece_cuts is not None else piece_tiles, piece_unit=None if tile is None else 128,
        piece_cuts=piece_cuts)


def int8q_cabi(binding, stream, dev, c, scale, piece_tiles=PIECE_TILES):
    k = binding.kernels()
    t = {n: c[n].to(dev) for n in ("q8", "k8", "v8", "tables", "kd", "vd")}
    ps = c["ps"].to(dev) if c["ps"] is not None else None
    mask = c["mask"].to(dev) if c["mask"] is not None else None
    lens = np.ascontiguousarray(c["ctx"], dtype=np.int32)
    max_len = 0 if mask is None else mask.shape[-1]
    call = binding.AtbmiPaInt8QCall(
        outDtype=dtype_code(binding, torch.empty(0, dtype=c["dtype"])), numHeads=c["heads"], numKvHeads=c["kv_heads"],
        headDim=c["d"], blockSize=c["block"], numBlocks=c["k8"].shape[0], maxBlocksPerSeq=c["tables"].shape[1],
        batch=len(lens), numQueryRows=c["rows"], offline=0 if ps is None else 1, hasMask=0 if mask is None else 1,
        maskLen=max_len, pieceTiles=piece_tiles, qkScale=scale,
        maskSeqStride=0 if mask is None else (max_len if c["mask_kind"] == "norm" else c["heads"] * max_len),
        maskHeadStride=max_len if c["mask_kind"] == "alibi" else 0, hostContextLens=lens.ctypes.data)
    ws_bytes = ctypes.c_uint64(0)
    if k.atbmi_pa_int8q_workspace_size(ctypes.byref(call), ctypes.byref(ws_bytes)) != 0:
        raise RuntimeError("pa_int8q_workspace_size: " + binding.last_kernel_error())
    with torch.cuda.stream(stream):
        ws = torch.empty(max(int(ws_bytes.value), 16), dtype=torch.uint8, device=dev)
        out = torch.full((c["rows"], c["heads"], c["d"]), 7.0, dtype=c["dtype"], device=dev)
        call.query, call.keyCache, call.valueCache = t["q8"].data_ptr(), t["k8"].data_ptr(), t["v8"].data_ptr()
        call.blockTables, call.kDescale, call.vDescale = t["tables"].data_ptr(), t["kd"].data_ptr(), t["vd"].data_ptr()
        call.pScale = ps.data_ptr() if ps is not None else None
        call.mask = mask.data_ptr() if mask is not None else None
        call.out = out.data_ptr()
        if k.atbmi_pa_int8q_decode(ctypes.byref(call), ws.data_ptr(), ws_bytes.value, stream.cuda_stream) != 0:
            raise RuntimeError("pa_int8q_decode: " + binding.last_kernel_error())
    stream.synchronize()
    return out


def _errors(golden, x):
    """Largest relative, mean relative and root-mean-square error (reference precision_calcu.py:78-109)."""
    golden = np.asarray(golden, np.float32)
    x = np.asarray(x, np.float32)
    rel = np.abs(x - golden) / (np.abs(golden) + 1e-7)
    return rel.max(), rel.mean(), math.sqrt(np.mean((x - golden) ** 2))


def _double_golden(true_out, golden, got, dtype):
    floor = 2.0 ** -11 if dtype == torch.float16 else 2.0 ** -8    # CV_FUSION thresholds (precision_calcu.py:56-62)
    e_got, e_gold = _errors(true_out, got), _errors(true_out, golden)
    rates = [g / max(r, floor) for g, r in zip(e_got, e_gold)]
    return rates[0] < 10 and rates[1] < 2 and rates[2] < 2, rates


# ctx, heads, kv heads, head size, block size, dtype, mask, offline
# (reference :3011-3227: 9 sequences [3000, 300, 14000, 33, 65, 1, 16, 14000, 300] with 32 heads over 2 KV heads,
# head size 128, block 128, NORM / ALIBI / no mask, bf16 and fp16 outputs, online and offline; contexts cut to keep
# the CPU oracle within seconds)
INT8Q_MATRIX = [
    ([3000, 300, 1400, 33, 65, 1, 16, 0, 300], 32, 2, 128, 128, torch.bfloat16, "norm", False),
    ([3000, 300, 1400, 33, 65, 1, 16, 1400, 300], 32, 2, 128, 128, torch.float16, "alibi", False),
    ([700, 129, 128, 4], 32, 2, 128, 128, torch.float16, None, True),
    ([700, 129, 128, 4], 32, 8, 128, 128, torch.bfloat16, "norm", True),
    ([515, 33, 2048], 64, 8, 128, 128, torch.float16, None, False),       # 8 heads a KV head: half a head tile
    ([300, 1000, 0, 77], 40, 1, 128, 64, torch.float16, None, False),     # 40 heads over one KV head: three head tiles
    ([300, 100, 77], 8, 8, 64, 16, torch.float16, "norm", False),         # head size 64, 16-token blocks, MHA
    ([260, 31], 12, 4, 256, 32, torch.bfloat16, None, False),             # head size 256
    ([700, 260, 31], 24, 12, 256, 64, torch.float16, "norm", True),       # head size 256: 12 KV heads in workgroups of 4 waves
    ([330, 64, 1100], 16, 4, 64, 64, torch.bfloat16, "alibi", False),     # head size 64, blocks of 64 tokens = a wave's tile
    # one KV head with at most 16 query heads: workgroups of one wave
    ([700, 129, 128, 4, 1500], 8, 1, 128, 128, torch.float16, "norm", False),
    ([700, 129, 128, 4, 1500], 16, 1, 128, 128, torch.bfloat16, "alibi", True),
    ([300, 100, 77], 4, 1, 64, 16, torch.float16, None, False),
    ([260, 31], 12, 1, 256, 32, torch.bfloat16, None, False),
]


@pytest.mark.parametrize("case", INT8Q_MATRIX, ids=lambda c: "ctx%d_h%d_g%d_d%d_b%d_%s_%s_%s" % (
    max(c[0]), c[1], c[2], c[3], c[4], str(c[5]).split(".")[-1], c[6], "offline" if c[7] else "online"))
def test_int8q_kernel_against_the_oracle(binding, oracle, dev, stream, case):
    ctx, heads, kv_heads, d, block, dtype, mask, offline = case
    c = _case(710 + heads + d, ctx, heads, kv_heads, d, block, dtype, mask, offline)
    scale = 1.0 / math.sqrt(d)
    got = int8q_cabi(binding, stream, dev, c, scale)
    want = _oracle(oracle, c, scale, "own")
    assert_close(got, want, TOL[dtype], "the library's tile")
    # the reference's criterion: compared with the whole context as one tile, no worse than the tiled golden
    ok, rates = _double_golden(_oracle(oracle, c, scale, None), want, got.float().cpu().numpy(), dtype)
    assert ok, rates
    assert float(got.float().abs().max()) > 0


@pytest.mark.parametrize("offline", [False, True])
def test_int8q_library_cut_on_many_short_and_one_long_sequence(binding, oracle, dev, stream, offline):
    """pieceTiles = 0 on shapes that stress the walk over pieces: 200 sequences of 0 .. 150 tokens (pieces of one to
    three tiles, so the requests run one or two pieces ahead of the arithmetic), workgroups of six waves (12 KV
    heads); then one sequence of 20 000 tokens, which every share boundary cuts."""
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    rng = np.random.Generator(np.random.PCG64(77))
    ctx = rng.integers(0, 151, size=200).astype(np.int32)
    ctx[:4] = [0, 1, 64, 65]
    for case_ctx, heads, kv_heads, d, block, mask in ((ctx, 12, 12, 128, 32, "norm"), ([20000], 8, 2, 128, 128, None)):
        c = _case(930 + len(case_ctx), case_ctx, heads, kv_heads, d, block, torch.float16, mask, offline)
        scale = 1.0 / math.sqrt(d)
        cuts = library_cuts(c, cus)
        assert cuts
        got = int8q_cabi(binding, stream, dev, c, scale, piece_tiles=0)
        assert_close(got, _oracle(oracle, c, scale, "own", piece_cuts=cuts), TOL[torch.float16], "the library's cut")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_int8q_masks_of_minus_infinity(binding, oracle, dev, stream, dtype):
    """A mask of -inf over the first 130 tokens of a sequence (its first two tiles see nothing, and with pieces of
    one unit its first piece reaches the merge with a log-sum-exp of -inf), over all of another (its output is
    zero), and over a tile in the middle of a third."""
    ctx, heads, kv_heads, d, block = [300, 70, 400], 8, 2, 128, 128
    c = _case(940, ctx, heads, kv_heads, d, block, dtype, "norm", False)
    m = np.zeros((3, 1, 400), np.float32)
    m[0, 0, :130] = -np.inf
    m[1, 0, :] = -np.inf
    m[2, 0, 128:192] = -np.inf
    c["mask"] = torch.from_numpy(m).to(dtype)
    scale = 1.0 / math.sqrt(d)
    for piece_tiles in (1, 100):
        got = int8q_cabi(binding, stream, dev, c, scale, piece_tiles=piece_tiles)
        want = _oracle(oracle, c, scale, "own", piece_tiles=piece_tiles)
        assert np.isfinite(want).all() and np.abs(want[1]).max() == 0
        assert_close(got, want, TOL[dtype], "pieces of %d units" % piece_tiles)
        assert float(got[1].float().abs().max()) == 0


def test_int8q_long_pieces_and_small_blocks(binding, oracle, dev, stream):
    """A context of 71 units of 128 tokens in one piece (pieceTiles = 100) and in two (pieceTiles = 64: 36 + 35 units),
    offline, where the cut shows in the int8 weights; then blocks of 64 tokens with two KV heads."""
    ctx, heads, kv_heads, d, block, dtype = [9000, 130], 4, 1, 64, 128, torch.float16
    c = _case(911, ctx, heads, kv_heads, d, block, dtype, None, True)
    scale = 1.0 / math.sqrt(d)
    whole = _oracle(oracle, c, scale, "own", piece_tiles=100)
    halves = _oracle(oracle, c, scale, "own", piece_tiles=64)
    assert np.abs(whole - halves).max() > 0
    assert_close(int8q_cabi(binding, stream, dev, c, scale, piece_tiles=100), whole, TOL[dtype], "one piece")
    assert_close(int8q_cabi(binding, stream, dev, c, scale, piece_tiles=64), halves, TOL[dtype], "two pieces")
    c = _case(912, ctx, 4, 2, d, 64, dtype, None, True)
    got = int8q_cabi(binding, stream, dev, c, scale, piece_tiles=32)
    assert_close(got, _oracle(oracle, c, scale, "own", piece_tiles=32), TOL[dtype], "blocks of 64 tokens")


def test_int8q_rejects_what_it_cannot_run(binding, dev, stream):
    k = binding.kernels()
    lens = np.array([5, 300], np.int32)
    call = binding.AtbmiPaInt8QCall(outDtype=binding.ATBMI_F16, numHeads=32, numKvHeads=8, headDim=128, blockSize=128,
                                    numBlocks=8, maxBlocksPerSeq=2, batch=2, numQueryRows=2, qkScale=0.1,
                                    hostContextLens=lens.ctypes.data)
    ws = ctypes.c_uint64(0)
    assert k.atbmi_pa_int8q_workspace_size(ctypes.byref(call), ctypes.byref(ws)) != 0        # 300 tokens in 2 blocks
    assert "exceeds" in binding.last_kernel_error()
    lens[1] = 200
    assert k.atbmi_pa_int8q_workspace_size(ctypes.byref(call), ctypes.byref(ws)) == 0 and ws.value == 256
    call.headDim = 96
    assert k.atbmi_pa_int8q_workspace_size(ctypes.byref(call), ctypes.byref(ws)) != 0
    call.headDim, call.numKvHeads = 128, 5
    assert k.atbmi_pa_int8q_workspace_size(ctypes.byref(call), ctypes.byref(ws)) != 0
    call.numKvHeads, call.numQueryRows = 8, 1
    assert k.atbmi_pa_int8q_workspace_size(ctypes.byref(call), ctypes.byref(ws)) != 0        # two rows asked for
    call.numQueryRows = 2
    assert k.atbmi_pa_int8q_decode(ctypes.byref(call), None, 0, stream.cuda_stream) != 0     # null tensors
    # the kernel fetches the mask as aligned 32-bit words: odd strides or row lengths, or a base off a 4-byte
    # boundary, would make it read outside the rows
    call.hasMask, call.maskLen, call.maskSeqStride, call.mask = 1, 200, 200, 4096
    assert k.atbmi_pa_int8q_workspace_size(ctypes.byref(call), ctypes.byref(ws)) == 0
    for bad in (dict(maskLen=201, maskSeqStride=202), dict(maskSeqStride=201), dict(maskHeadStride=3), dict(mask=4098)):
        for name, value in {**dict(maskLen=200, maskSeqStride=200, maskHeadStride=0, mask=4096), **bad}.items():
            setattr(call, name, value)
        assert k.atbmi_pa_int8q_workspace_size(ctypes.byref(call), ctypes.byref(ws)) != 0, bad
        assert "4-byte" in binding.last_kernel_error()


@pytest.mark.parametrize("offline,mask,dtype", [(False, "norm", torch.bfloat16), (True, None, torch.float16),
                                                (False, "alibi", torch.float16), (False, "spec", torch.float16)])
def test_paged_attention_operation_with_int8_queries(binding, oracle, dev, stream, offline, mask, dtype):
    """PagedAttentionOperation, quantType TYPE_QUANT_QKV_ONLINE (3) / OFFLINE (2), through Setup / Execute. Inputs:
    query, keyCache, valueCache, blockTables, contextLens, [mask], kDescale, vDescale, [pScale] (reference
    paged_attention_operation.cpp:408-444); the output comes in outDataType."""
    heads, kv_heads, d, block = 32, 2, 128, 128
    # "spec": MASK_TYPE_SPEC, one mask row per QUERY row [rows, maxS]: the rows of the per-sequence mask of the
    # sequences that have a context, so that the sequence behind the empty one reads row 2, not row 3
    spec = mask == "spec"
    c = _case(750 + int(offline), [3000, 300, 0, 33, 65, 1, 16, 1400, 300], heads, kv_heads, d, block, dtype,
              "norm" if spec else mask, offline)
    scale = 1.0 / math.sqrt(d)
    lens = torch.from_numpy(c["ctx"])
    ctx = binding.Context(stream)
    op = binding.OperationRunner("PagedAttentionOperation", binding.PagedAttentionParam(
        headNum=heads, kvHeadNum=kv_heads, qkScale=scale, quantType=2 if offline else 3,
        maskType={None: 0, "norm": 1, "alibi": 2, "spec": 3}[mask],
        outDataType=binding.ACL_BF16 if dtype == torch.bfloat16 else binding.ACL_FLOAT16), ctx)
    ins = [c["q8"].to(dev), c["k8"].to(dev), c["v8"].to(dev), c["tables"].to(dev), lens.to(dev)]
    if spec:
        ins.append(c["mask"][torch.from_numpy(c["ctx"] > 0)][:, 0, :].contiguous().to(dev))
    elif mask is not None:
        ins.append(c["mask"].to(dev))
    ins += [c["kd"].to(dev), c["vd"].to(dev)]
    if offline:
        ins.append(c["ps"].to(dev))
    with torch.cuda.stream(stream):
        out = torch.full((c["rows"], heads, d), 7.0, dtype=dtype, device=dev)
        op.run(ins, outputs=[out], host_inputs={4: lens})

    stream.synchronize()
    # the operation leaves the cut of long contexts to the library (equal shares of the list of tiles, see
    # library_cuts): online that moves no int8 weight, offline it does (the weights are taken against each piece's own
    # running maximum)
    cuts = library_cuts(c, torch.cuda.get_device_properties(dev).multi_processor_count)
    assert cuts
    want = _oracle(oracle, c, scale, "own", piece_cuts=cuts)
    assert_close(out, want, TOL[dtype], "operation")
    if not spec:
        assert torch.equal(out, int8q_cabi(binding, stream, dev, c, scale, piece_tiles=0))
    ok, rates = _double_golden(_oracle(oracle, c, scale, None), want, out.float().cpu().numpy(), dtype)
    assert ok, rates
    # allocated from InferShape the output has the type outDataType names
    with torch.cuda.stream(stream):
        fresh = op.run(ins, host_inputs={4: lens})[0]
    stream.synchronize()
    assert fresh.dtype == dtype and torch.equal(fresh, out)
    op.close()
    ctx.close()
