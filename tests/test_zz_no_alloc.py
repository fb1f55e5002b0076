"""The decode entry point that allocates nothing (atbmi_pa_decode_static) against atbmi_pa_decode: the
same plan and tensors through both, results equal bit for bit, on two calls in a row, the second with a
smaller input (the static scratch keeps the first call's partial rows)."""
import ctypes
import math

import numpy as np
import pytest
import torch

from pa_harness import dtype_code, random_tables

pytestmark = pytest.mark.gpu


def _decode_both(binding, stream, dev, rng, batch, heads, kv_heads, d, ctx, dtype, kv_int8=False):
    k = binding.kernels()
    block = 128
    ctx = np.asarray(ctx, dtype=np.int32)
    pool = int(((ctx.astype(np.int64) + block - 1) // block).sum()) + 3
    tables = torch.from_numpy(random_tables(rng, ctx, block, pool)).to(dev)
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(rng.integers(1 << 30)))
    q = (torch.rand((batch, heads, d), generator=gen) * 2 - 1).to(dtype).to(dev)
    if kv_int8:
        kc = torch.randint(-9, 10, (pool, block, kv_heads, d), generator=gen, dtype=torch.int8).to(dev)
        vc = torch.randint(-9, 10, (pool, block, kv_heads, d), generator=gen, dtype=torch.int8).to(dev)
        ks = (torch.rand(kv_heads * d, generator=gen) * 0.015 + 0.005).to(dev)
        vs = (torch.rand(kv_heads * d, generator=gen) * 0.015 + 0.005).to(dev)
    else:
        kc = (torch.rand((pool, block, kv_heads, d), generator=gen) * 2 - 1).to(dtype).to(dev)
        vc = (torch.rand((pool, block, kv_heads, d), generator=gen) * 2 - 1).to(dtype).to(dev)
        ks = vs = None
    shape = binding.AtbmiPaShape(
        qDtype=dtype_code(binding, q), kvDtype=dtype_code(binding, kc), numHeads=heads, numKvHeads=kv_heads,
        headDimK=d, headDimV=d, blockSize=block, numBlocks=pool, maxBlocksPerSeq=tables.shape[1], numQueryRows=batch,
        qkScale=1.0 / math.sqrt(d), kernel=binding.ATBMI_PA_KERNEL_MFMA)
    plan = ctypes.c_void_p()
    assert k.atbmi_pa_plan_create(ctypes.byref(shape), ctypes.byref(plan)) == 0, binding.last_kernel_error()
    try:
        assert k.atbmi_pa_plan_update(plan, ctx.ctypes.data, len(ctx)) == 0, binding.last_kernel_error()
        ws_bytes = k.atbmi_pa_plan_workspace_size(plan)
        outs = []
        with torch.cuda.stream(stream):
            ws = torch.empty(max(int(ws_bytes), 16), dtype=torch.uint8, device=dev)
            for static in (False, True):
                out = torch.full((batch, heads, d), 7.0, dtype=dtype, device=dev)
                t = binding.AtbmiPaTensors()
                t.query, t.keyCache, t.valueCache = q.data_ptr(), kc.data_ptr(), vc.data_ptr()
                t.blockTables, t.out = tables.data_ptr(), out.data_ptr()
                if kv_int8:
                    t.kScale, t.vScale = ks.data_ptr(), vs.data_ptr()
                if static:
                    rc = k.atbmi_pa_decode_static(plan, ctypes.byref(t), stream.cuda_stream)
                else:
                    rc = k.atbmi_pa_decode(plan, ctypes.byref(t), ws.data_ptr(), ws_bytes, stream.cuda_stream)
                assert rc == 0, binding.last_kernel_error()
                outs.append(out)
        stream.synchronize()
    finally:
        k.atbmi_pa_plan_destroy(plan)
    return outs[0], outs[1], ws_bytes


def test_static_scratch_decode_equals_workspace_decode(binding):
    assert torch.cuda.is_available(), "this test needs the MI355X"
    dev = torch.device("cuda:0")
    stream = torch.cuda.Stream(device=dev)
    k = binding.kernels()
    assert k.atbmi_pa_static_scratch_bytes() == 32 << 20
    rng = np.random.Generator(np.random.PCG64(4242))
    # first call: 24 sequences of 600..3000 tokens, rows cut by many ranges; second call: a smaller batch
    calls = [
        (24, 32, 8, 128, rng.integers(600, 3000, size=24), torch.bfloat16, False),
        (5, 32, 8, 128, [900, 33, 1500, 64, 257], torch.bfloat16, False),
        (16, 64, 8, 128, rng.integers(300, 2500, size=16), torch.float16, True),
        (1, 8, 1, 128, [96], torch.float16, False),
    ]
    for batch, heads, kv_heads, d, ctx, dtype, kv_int8 in calls:
        print("static decode: batch %d heads %d/%d d %d int8 %s" % (batch, heads, kv_heads, d, kv_int8), flush=True)
        want, got, ws_bytes = _decode_both(binding, stream, dev, rng, batch, heads, kv_heads, d, ctx, dtype, kv_int8)
        assert ws_bytes > 0, "the case must split rows over ranges, or the scratch is not exercised"
        assert torch.isfinite(want.float()).all()
        assert torch.equal(want.view(torch.int16), got.view(torch.int16))


def test_static_scratch_decode_refuses_what_does_not_fit(binding):
    assert torch.cuda.is_available(), "this test needs the MI355X"
    dev = torch.device("cuda:0")
    k = binding.kernels()
    # 128 heads x 512 channels over 256 ranges: 134 MB of partial rows
    shape = binding.AtbmiPaShape(qDtype=1, kvDtype=1, numHeads=128, numKvHeads=1, headDimK=576, headDimV=512,
                                 blockSize=128, numBlocks=4096, maxBlocksPerSeq=32, numQueryRows=64, mlaCombined=1,
                                 qkScale=0.07, kernel=binding.ATBMI_PA_KERNEL_MFMA)
    plan = ctypes.c_void_p()
    assert k.atbmi_pa_plan_create(ctypes.byref(shape), ctypes.byref(plan)) == 0
    lens = np.full(64, 3001, dtype=np.int32)
    assert k.atbmi_pa_plan_update(plan, lens.ctypes.data, 64) == 0
    big = k.atbmi_pa_plan_workspace_size(plan)
    t = binding.AtbmiPaTensors()
    dummy = torch.zeros(64, device=dev)
    t.query = t.keyCache = t.blockTables = t.out = dummy.data_ptr()
    assert big > k.atbmi_pa_static_scratch_bytes(), "the case is meant to need more partial rows than the scratch holds"
    assert k.atbmi_pa_decode_static(plan, ctypes.byref(t), None) == 1
    assert "static scratch" in binding.last_kernel_error()
    k.atbmi_pa_plan_destroy(plan)
    # a scalar-kernel plan uploads its tables: refused as well
    shape = binding.AtbmiPaShape(qDtype=0, kvDtype=0, numHeads=8, numKvHeads=8, headDimK=128, headDimV=128,
                                 blockSize=128, numBlocks=64, maxBlocksPerSeq=8, numQueryRows=2, qkScale=0.1,
                                 kernel=binding.ATBMI_PA_KERNEL_SCALAR)
    assert k.atbmi_pa_plan_create(ctypes.byref(shape), ctypes.byref(plan)) == 0
    lens = np.array([300, 700], dtype=np.int32)
    assert k.atbmi_pa_plan_update(plan, lens.ctypes.data, 2) == 0
    assert k.atbmi_pa_decode_static(plan, ctypes.byref(t), None) == 1
    assert "kernel arguments" in binding.last_kernel_error()
    k.atbmi_pa_plan_destroy(plan)
