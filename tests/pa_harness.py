"""Helpers shared by the GPU tests: run the kernels through the C ABI or the
atb::Operation layer on torch tensors, and turn tensors into oracle inputs."""
import ctypes
import os

import numpy as np
import torch


def to_oracle(t):
    """float32 numpy copy of a float tensor; int8 tensors stay int8."""
    if t is None:
        return None
    if t.dtype == torch.int8 or t.dtype == torch.int32:
        return t.cpu().numpy()
    return t.float().cpu().numpy()


def dtype_code(binding, t):
    return {torch.float16: binding.ATBMI_F16, torch.bfloat16: binding.ATBMI_BF16, torch.int8: binding.ATBMI_INT8}[t.dtype]


def pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx_host, scale, k_scale=None, k_off=None, v_scale=None,
                   v_off=None, mla_dv=0, q_scale=0.0, kernel=0, chunk_tokens=None, out=None, return_plan_info=False,
                   mask=None, mask_per_head=False, logn=None, q_lens=None, mask_rows="sequence", q_rope=None,
                   k_rope=None, lse=None, head_major=False, poison_workspace=False, fractal_nz=False, causal_rows=None):
    """atbmi_pa_plan_* + atbmi_pa_decode on `stream`; returns the output tensor.
    mask: device tensor of q's dtype shaped like one of the reference's decode
    masks; mask_per_head says that a 3-dim mask's first dim counts heads (ALIBI).
    q_rope / k_rope: the split latent layout (q and kc then hold the first 512
    channels); lse: a [rows, heads] tensor of q's dtype that receives the log-sum-exp;
    fractal_nz: kc and k_rope are [blocks, channels / 16, block size, 16]; causal_rows: True or a
    list of flags per sequence (atbmi_pa_plan_set_causal_rows)."""
    k = binding.kernels()
    rows, heads, d = q.shape
    rope = 0 if q_rope is None else q_rope.shape[2]
    d += rope
    dv = mla_dv if mla_dv else vc.shape[3]
    mask_batch_stride, mask_head_stride = mask_strides(mask, mask_per_head)
    if mask_rows != "sequence":
        mask_batch_stride, mask_head_stride = (mask.shape[1], 0) if mask is not None else (0, 0)
    shape = binding.AtbmiPaShape(
        qDtype=dtype_code(binding, q), kvDtype=dtype_code(binding, kc), numHeads=heads,
        numKvHeads=1 if fractal_nz else kc.shape[1 if head_major else 2],
        kvLayout=2 if fractal_nz else (1 if head_major else 0),
        headDimK=d, headDimV=dv, blockSize=kc.shape[2 if (head_major or fractal_nz) else 1], numBlocks=kc.shape[0], maxBlocksPerSeq=tables.shape[1],
        numQueryRows=rows, mlaCombined=1 if mla_dv else 0, hasOffset=1 if k_off is not None else 0, kernel=kernel,
        qkScale=scale, qScale=q_scale, hasMask=0 if mask is None else 1, maskBatchStride=mask_batch_stride,
        maskHeadStride=mask_head_stride, maskLen=0 if mask is None else mask.shape[-1],
        hasLogN=0 if logn is None else 1,
        descalePacked=1 if (k_scale is not None and k_scale.dtype == torch.int64) else 0,
        maskRowBy={"sequence": 0, "query": 1, "position": 2}[mask_rows], ropeDim=rope)
    old = os.environ.get("ATBMI_PA_CHUNK_TOKENS")
    if chunk_tokens is not None:
        os.environ["ATBMI_PA_CHUNK_TOKENS"] = str(chunk_tokens)
    plan = ctypes.c_void_p()
    try:
        rc = k.atbmi_pa_plan_create(ctypes.byref(shape), ctypes.byref(plan))
    finally:
        if chunk_tokens is not None:
            if old is None:
                del os.environ["ATBMI_PA_CHUNK_TOKENS"]
            else:
                os.environ["ATBMI_PA_CHUNK_TOKENS"] = old
    if rc != 0:
        raise RuntimeError("plan_create: " + binding.last_kernel_error())
    try:
        lens = np.ascontiguousarray(np.asarray(ctx_host, dtype=np.int32))
        if causal_rows is not None:
            flags = None if causal_rows is True else np.ascontiguousarray(np.asarray(causal_rows, dtype=np.int32))
            rc = k.atbmi_pa_plan_set_causal_rows(plan, 1, None if flags is None else flags.ctypes.data,
                                                 0 if flags is None else len(flags))
            if rc != 0:
                raise RuntimeError("plan_set_causal_rows: " + binding.last_kernel_error())
        if q_lens is None:
            rc = k.atbmi_pa_plan_update(plan, lens.ctypes.data, len(lens))
        else:
            qn = np.ascontiguousarray(np.asarray(q_lens, dtype=np.int32))
            rc = k.atbmi_pa_plan_update_multi(plan, lens.ctypes.data, qn.ctypes.data, len(lens))
        if rc != 0:
            raise RuntimeError("plan_update: " + binding.last_kernel_error())
        ws_bytes = k.atbmi_pa_plan_workspace_size(plan)
        with torch.cuda.stream(stream):
            ws = torch.empty(max(int(ws_bytes), 16), dtype=torch.uint8, device=q.device)
            if poison_workspace:
                ws.fill_(0xFF)  # every fp32 in it reads as NaN until a kernel writes it
            if out is None:
                out = torch.zeros((rows, heads, dv), dtype=q.dtype, device=q.device)
            t = binding.AtbmiPaTensors()
            t.query = q.data_ptr()
            t.keyCache = kc.data_ptr()
            t.valueCache = vc.data_ptr() if vc is not None else None
            t.blockTables = tables.data_ptr()
            t.kScale = k_scale.data_ptr() if k_scale is not None else None
            t.kOffset = k_off.data_ptr() if k_off is not None else None
            t.vScale = v_scale.data_ptr() if v_scale is not None else None
            t.vOffset = v_off.data_ptr() if v_off is not None else None
            t.out = out.data_ptr()
            t.mask = mask.data_ptr() if mask is not None else None
            t.logN = logn.data_ptr() if logn is not None else None
            t.queryRope = q_rope.data_ptr() if q_rope is not None else None
            t.keyRopeCache = k_rope.data_ptr() if k_rope is not None else None
            t.lse = lse.data_ptr() if lse is not None else None
            rc = k.atbmi_pa_decode(plan, ctypes.byref(t), ws.data_ptr(), ws_bytes, stream.cuda_stream)
            if rc != 0:
                raise RuntimeError("pa_decode: " + binding.last_kernel_error())
        stream.synchronize()
        info = dict(chunks=k.atbmi_pa_plan_num_chunks(plan), bytes=k.atbmi_pa_plan_algorithmic_bytes(plan),
                    workspace=ws_bytes)
    finally:
        k.atbmi_pa_plan_destroy(plan)
    return (out, info) if return_plan_info else out


def pack_descale(scale):
    """fp32 device vector -> int64 device vector with the float's bits in the low half
    (what atb::Utils::QuantParamConvert produces on the host)."""
    return scale.contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF


def mask_strides(mask, per_head):
    """(batch stride, head stride) in elements of a decode mask, by the rules of
    the reference tiling (tiling/paged_attention_tiling.cpp:36-74)."""
    if mask is None:
        return 0, 0
    assert mask.is_contiguous()
    if mask.dim() == 2:
        return 0, 0
    if mask.dim() == 3:
        assert mask.shape[1] == 1
        return (0, mask.shape[2]) if per_head else (mask.shape[2], 0)
    assert mask.dim() == 4 and mask.shape[2] == 1
    return mask.shape[1] * mask.shape[3], (0 if mask.shape[1] == 1 else mask.shape[3])


def oracle_pa(oracle, q, kc, vc, tables, ctx_host, scale, k_scale=None, k_off=None, v_scale=None, v_off=None,
              mla_dv=0, q_scale=0.0, out_init=0.0, mask=None, mask_per_head=False, logn=None, q_lens=None,
              mask_rows="sequence", lse_out=None, head_major=False, compress_kv_heads=0, razor_offset=None,
              causal_rows=None, empty_keep_rows=False):
    qd = "bf16" if q.dtype == torch.bfloat16 else "float16"
    return oracle.paged_attention(
        to_oracle(q), to_oracle(kc), to_oracle(vc), tables.cpu().numpy(), np.asarray(ctx_host), scale,
        to_oracle(k_scale), to_oracle(k_off), to_oracle(v_scale), to_oracle(v_off), mla_v_head_size=mla_dv,
        q_scale=q_scale, q_dtype=qd, out_init=out_init, mask=to_oracle(mask), logn=to_oracle(logn),
        mask_per_head=mask_per_head if (mask is not None and mask.dim() == 3) else None, q_lens=q_lens,
        mask_rows=mask_rows, lse_out=lse_out, head_major=head_major, compress_kv_heads=compress_kv_heads,
        razor_offset=to_oracle(razor_offset), causal_rows=causal_rows, empty_keep_rows=empty_keep_rows)


def assert_close(got, want, tol, what=""):
    """|got - want| <= tol + tol * |want| elementwise (rtol = atol = tol)."""
    got = got.float().cpu().numpy() if isinstance(got, torch.Tensor) else np.asarray(got, dtype=np.float32)
    want = np.asarray(want, dtype=np.float32)
    assert got.shape == want.shape, (got.shape, want.shape)
    err = np.abs(got - want)
    lim = tol + tol * np.abs(want)
    bad = err > lim
    assert not bad.any() and np.isfinite(got).all(), "%s: %d of %d outside tol %g, max err %g at %s" % (
        what, int(bad.sum()), bad.size, tol, float(err.max()), np.unravel_index(int(err.argmax()), err.shape))


def random_tables(rng, ctx, block, pool, unique=True):
    """Block tables for the given lengths; unused entries hold valid ids."""
    ctx = np.asarray(ctx, dtype=np.int64)
    nblk = (ctx + block - 1) // block
    width = max(1, int(nblk.max()))
    total = int(nblk.sum())
    ids = rng.permutation(pool)[:total] if unique else rng.integers(0, pool, size=total)
    tables = np.zeros((len(ctx), width), dtype=np.int32)
    pos = 0
    for b in range(len(ctx)):
        n = int(nblk[b])
        tables[b, :n] = ids[pos:pos + n]
        tables[b, n:] = ids[pos] if n else 0
        pos += n
    return tables
