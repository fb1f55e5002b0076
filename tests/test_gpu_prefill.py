"""GPU parity of MultiLatentAttention's prefill calcType: the HIP flash-attention kernel through the C ABI,
through atb::Operation and through the AtbMLAPreFill two-call wrappers, against the fp32 CPU oracle on the
same seeded inputs. Tolerance rtol = atol = 1e-3 for fp16 and 2e-2 for bf16. Shapes follow the reference's
own tests (tests/apitest/opstest/python/operations/multi_latent_attention/test_multi_latent_attention_prefill.py:
800-1340: 1-2 heads, 128-2048 tokens, no mask / the 512 x 512 triangular mask / the internal causal mask / a
window of 954) plus ragged batches, empty sequences, grouped KV heads and the padded key layout."""
import ctypes
import math

import numpy as np
import pytest
import torch

from pa_harness import assert_close, dtype_code

pytestmark = pytest.mark.gpu

TOL = {torch.float16: 1e-3, torch.bfloat16: 2e-2}


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return torch.device("cuda:0")


@pytest.fixture(scope="module")
def stream(dev):
    return torch.cuda.Stream(device=dev)


def _inputs(seed, dev, lens, heads, kv_heads, dtype, padded_rows=0, std=1.0):
    """query, queryRope, key, keyRope, value as device tensors; keys packed, or padded per sequence with NaN
    in the padding rows."""
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    tq = int(sum(lens))
    mk = lambda *shape: (torch.randn(shape, generator=gen) * std).to(dtype)
    q, qr = mk(tq, heads, 128), mk(tq, heads, 64)
    k, kr, v = mk(tq, kv_heads, 128), mk(tq, kv_heads, 64), mk(tq, kv_heads, 128)
    if padded_rows:
        def pad(t):
            out = torch.full((len(lens), padded_rows) + tuple(t.shape[1:]), float("nan"), dtype=dtype)
            pos = 0
            for b, n in enumerate(lens):
                out[b, :n] = t[pos:pos + n]
                pos += n
            return out.reshape(len(lens) * padded_rows, *t.shape[1:])
        k, kr, v = pad(k), pad(kr), pad(v)
    return [t.to(dev) for t in (q, qr, k, kr, v)]


def _oracle(oracle, tensors, lens, scale, mask, window=0, padded_rows=0):
    q, qr, k, kr, v = [t.float().cpu().numpy() for t in tensors]
    return oracle.mla_prefill(q, qr, k, kr, v, lens, lens, scale, mask=mask, window=window, kv_padded_rows=padded_rows)


def prefill_cabi(binding, stream, tensors, q_lens, kv_lens, heads, kv_heads, scale, mask, window=0, padded_rows=0):
    k = binding.kernels()
    q, qr, key, kr, v = tensors
    ql = np.ascontiguousarray(np.asarray(q_lens, dtype=np.int32))
    kl = np.ascontiguousarray(np.asarray(kv_lens, dtype=np.int32))
    call = binding.AtbmiMlaPrefillCall(
        dtype=dtype_code(binding, q), numHeads=heads, numKvHeads=kv_heads,
        mask={"none": 0, "causal": 1, "window": 2}[mask], windowSize=window, qkScale=scale, batch=len(ql),
        kvPaddedRows=padded_rows, hostQLens=ql.ctypes.data, hostKvLens=kl.ctypes.data)
    ws_bytes = ctypes.c_uint64(0)
    if k.atbmi_mla_prefill_workspace_size(ctypes.byref(call), ctypes.byref(ws_bytes)) != 0:
        raise RuntimeError("mla_prefill_workspace_size: " + binding.last_kernel_error())
    with torch.cuda.stream(stream):
        ws = torch.empty(max(int(ws_bytes.value), 16), dtype=torch.uint8, device=q.device)
        out = torch.full((q.shape[0], heads, 128), 7.0, dtype=q.dtype, device=q.device)
        call.query, call.queryRope, call.key = q.data_ptr(), qr.data_ptr(), key.data_ptr()
        call.keyRope, call.value, call.out = kr.data_ptr(), v.data_ptr(), out.data_ptr()
        if k.atbmi_mla_prefill(ctypes.byref(call), ws.data_ptr(), ws_bytes.value, stream.cuda_stream) != 0:
            raise RuntimeError("mla_prefill: " + binding.last_kernel_error())
    stream.synchronize()
    return out


# lens, heads, kv_heads, mask, window, dtype, padded rows
PREFILL_MATRIX = [
    ([512], 1, 1, "none", 0, torch.float16, 0),             # reference :800-853
    ([128], 1, 1, "causal", 0, torch.float16, 0),           # :856-912 (the 512 x 512 mask) and :1036-1091
    ([128], 1, 1, "none", 0, torch.bfloat16, 0),            # :915-975
    ([128, 128], 2, 1, "causal", 0, torch.bfloat16, 128),   # :1152-1207: two heads over one KV head, padded keys
    ([2048] * 2, 1, 1, "window", 954, torch.float16, 0),    # :1210-1272 (batch 16 there)
    ([2048] * 2, 1, 1, "window", 954, torch.bfloat16, 0),   # :1275-1337
    ([300, 0, 1, 129, 77, 1000], 4, 4, "causal", 0, torch.float16, 0),
    ([300, 0, 1, 129, 77, 1000], 4, 4, "none", 0, torch.bfloat16, 0),
    ([300, 0, 1, 129, 77, 1000], 4, 2, "window", 33, torch.float16, 1024),
    ([700, 31], 8, 8, "window", 1, torch.float16, 0),       # every query sees only itself
    ([257], 3, 1, "window", 5000, torch.bfloat16, 0),       # a window longer than the sequence is the causal mask
    ([1537], 16, 16, "causal", 0, torch.bfloat16, 0),
]


@pytest.mark.parametrize("case", PREFILL_MATRIX, ids=lambda c: "b%d_t%d_h%d_g%d_%s%s_%s%s" % (
    len(c[0]), sum(c[0]), c[1], c[2], c[3], c[4] or "", str(c[5]).split(".")[-1], "_padded" if c[6] else ""))
def test_mla_prefill_kernel(binding, oracle, dev, stream, case):
    lens, heads, kv_heads, mask, window, dtype, padded = case
    tensors = _inputs(500 + sum(lens) + heads, dev, lens, heads, kv_heads, dtype, padded)
    scale = 1.0 / math.sqrt(192.0)
    want = _oracle(oracle, tensors, lens, scale, mask, window, padded)
    got = prefill_cabi(binding, stream, tensors, lens, lens, heads, kv_heads, scale, mask, window, padded)
    assert_close(got, want, TOL[dtype], "prefill %s" % (case,))


def test_mla_prefill_more_keys_than_queries_and_empty_batch(binding, oracle, dev, stream):
    """Without a mask the two lengths of a sequence are independent; a batch with no query launches nothing."""
    q_lens, kv_lens = [5, 130, 0, 64], [700, 33, 50, 0]
    gen = torch.Generator(device="cpu")
    gen.manual_seed(77)
    mk = lambda *shape: torch.randn(shape, generator=gen).to(torch.float16).to(dev)
    tq, tk = sum(q_lens), sum(kv_lens)
    tensors = [mk(tq, 2, 128), mk(tq, 2, 64), mk(tk, 2, 128), mk(tk, 2, 64), mk(tk, 2, 128)]
    got = prefill_cabi(binding, stream, tensors, q_lens, kv_lens, 2, 2, 0.09, "none")
    q, qr, k, kr, v = [t.float().cpu().numpy() for t in tensors]
    want = oracle.mla_prefill(q, qr, k, kr, v, q_lens, kv_lens, 0.09)
    assert_close(got, want, 1e-3, "cross lengths")
    assert torch.equal(got[135:], torch.zeros_like(got[135:]))   # queries without keys yield zeros
    with pytest.raises(RuntimeError, match="must agree"):
        prefill_cabi(binding, stream, tensors, q_lens, kv_lens, 2, 2, 0.09, "causal")
    untouched = prefill_cabi(binding, stream, tensors, [0, 0], [0, 0], 2, 2, 0.09, "none")
    assert torch.equal(untouched, torch.full_like(untouched, 7.0))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_mla_prefill_through_operation_api(binding, oracle, dev, stream, dtype):
    """MultiLatentAttentionOperation with calcType PREFILL through InferShape / Setup / Execute for every mask
    type: inputs query, queryRope, key, keyRope, value, qSeqLen, kvSeqLen (+ mask); 3-dim and 2-dim queries,
    packed and padded keys (reference multi_latent_attention_operation.cpp:622-771)."""
    lens = [200, 37, 0, 515]
    heads = 4
    scale = 1.0 / math.sqrt(192.0)
    tensors = _inputs(900, dev, lens, heads, heads, dtype)
    lens_t = torch.tensor(lens, dtype=torch.int32)
    c = binding.Context(stream)
    tri = torch.triu(torch.full((512, 512), -10000.0 if dtype == torch.float16 else 1.0), 1).to(dtype).to(dev)
    for mask_type, kind, window in ((0, "none", 0), (2, "causal", 0), (3, "causal", 0), (4, "window", 100)):
        padded = 515 if mask_type == 3 else 0    # CAUSAL_MASK takes the keys as [batch, maxSeqLen, kvHeads * channels]
        t = _inputs(900, dev, lens, heads, heads, dtype, padded) if padded else tensors
        want = _oracle(oracle, t, lens, scale, kind, window, padded)
        ins = list(t)
        if padded:
            ins[2:5] = [x.reshape(len(lens), padded, -1) for x in ins[2:5]]
        ins += [lens_t.to(dev), lens_t.to(dev)]
        if mask_type == 2:
            ins.append(tri)
        if mask_type == 4:
            band = torch.zeros((515, 515), dtype=dtype, device=dev)
            ins.append(band)
        op = binding.OperationRunner("MultiLatentAttentionOperation", binding.MultiLatentAttentionParam(
            headNum=heads, kvHeadNum=heads, qkScale=scale, cacheMode=1, calcType=4, maskType=mask_type,
            windowSize=window), c)
        with torch.cuda.stream(stream):
            out, = op.run(ins, host_inputs={5: lens_t, 6: lens_t})
        stream.synchronize()
        assert tuple(out.shape) == (sum(lens), heads, 128) and out.dtype == dtype
        assert_close(out, want, TOL[dtype], "maskType %d" % mask_type)
        if mask_type == 0:
            # the same memory described as [tokens, heads * channels]
            flat = [ins[0].reshape(sum(lens), -1), ins[1].reshape(sum(lens), -1)] + ins[2:]
            with torch.cuda.stream(stream):
                out2, = op.run(flat, host_inputs={5: lens_t, 6: lens_t})
            stream.synchronize()
            assert tuple(out2.shape) == (sum(lens), heads * 128)
            assert torch.equal(out2.reshape(out.shape), out)
        op.close()
    c.close()


def test_mla_prefill_two_call_c_wrapper(binding, oracle, dev, stream):
    """AtbMLAPreFillGetWorkspaceSize / AtbMLAPreFill (reference include/atb/atb_acl.h:141-156) with the
    MASK_FREE mask: creates the operation, runs Setup, then Execute on what Setup bound."""
    lens = [150, 300]
    heads = 2
    scale = 0.07
    dtype = torch.float16
    tensors = _inputs(901, dev, lens, heads, heads, dtype)
    want = _oracle(oracle, tensors, lens, scale, "causal")
    lens_t = torch.tensor(lens, dtype=torch.int32)
    tri = torch.triu(torch.full((512, 512), -10000.0), 1).to(dtype).to(dev)
    out = torch.zeros((sum(lens), heads, 128), dtype=dtype, device=dev)
    lib = binding.atb()
    c = binding.Context(stream)
    handles = [binding.acl_tensor_of(t) for t in tensors] + [binding.acl_tensor_of(lens_t), binding.acl_tensor_of(lens_t),
                                                             binding.acl_tensor_of(tri), binding.acl_tensor_of(out)]
    op = ctypes.c_void_p()
    ws = ctypes.c_uint64(0)
    st = lib.AtbMLAPreFillGetWorkspaceSize(*handles[:8], heads, scale, heads, 2, 1, handles[8], ctypes.byref(ws),
                                           ctypes.byref(op), c.ptr)
    assert st == 0 and op.value
    with torch.cuda.stream(stream):
        workspace = torch.empty(max(int(ws.value), 16), dtype=torch.uint8, device=dev)
        assert lib.AtbMLAPreFill(workspace.data_ptr(), ws.value, op, c.ptr) == 0
    stream.synchronize()
    assert_close(out, want, 1e-3, "AtbMLAPreFill")
    assert lib.AtbMLAPreFill(None, 0, None, c.ptr) == binding.ERROR_CODE["ERROR_INVALID_OPERATION_ADDR"]
    lib.atb_c_destroy_operation(op)
    for h in handles:
        lib.aclDestroyTensor(h)
    c.close()


def test_mla_prefill_long_prompt_properties(binding, oracle, dev, stream):
    """A DeepSeek-shaped prompt batch (16 heads of the 128, 2 x 4096 tokens, bf16, causal): the oracle on a sample
    of rows of both sequences, and two properties that hold for every row: a row's output does not change
    when later tokens of its sequence change, and the first row of a sequence is its first value row."""
    lens = [4096, 4096]
    heads = 16
    dtype = torch.bfloat16
    scale = 1.0 / math.sqrt(192.0)
    tensors = _inputs(902, dev, lens, heads, heads, dtype, std=0.5)
    got = prefill_cabi(binding, stream, tensors, lens, lens, heads, heads, scale, "causal")
    q, qr, k, kr, v = [t.float().cpu().numpy() for t in tensors]
    rows = [0, 1, 31, 32, 127, 128, 2047, 4095, 4096, 4097, 6000, 8191]
    for r in rows:
        b0 = 0 if r < 4096 else 4096
        n = r - b0 + 1
        want = oracle.mla_prefill(q[r:r + 1], qr[r:r + 1], k[b0:b0 + n], kr[b0:b0 + n], v[b0:b0 + n], [1], [n], scale)
        assert_close(got[r:r + 1], want, 2e-2, "row %d" % r)
    assert torch.equal(got[0], tensors[4][0]) and torch.equal(got[4096], tensors[4][4096])
    changed = [t.clone() for t in tensors]
    for t in changed[2:]:
        t[3000:4096] = 0.25
        t[4096 + 1000:] = -0.5
    again = prefill_cabi(binding, stream, changed, lens, lens, heads, heads, scale, "causal")
    assert torch.equal(again[:3000], got[:3000]) and torch.equal(again[4096:4096 + 1000], got[4096:4096 + 1000])
    assert not torch.equal(again[3000:4096], got[3000:4096])
