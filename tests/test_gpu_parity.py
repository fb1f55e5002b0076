"""GPU parity tests: the HIP kernels against the CPU oracle on the same seeded
inputs. ReshapeAndCache, the slot scatter and the int8 quantised cache must be
bit-exact; attention must be within rtol = atol = 1e-3 for fp16 and 2e-2 for
bf16 / int8 caches of the fp32 oracle. Shapes follow the reference's own
kernel-test matrix (tests/apitest/kernelstest/mix/test_paged_attention_common.py,
test_paged_attention_mla.py, test_reshape_and_cache.py) plus the small
benchmark configuration."""
import math

import numpy as np
import pytest
import torch

from pa_harness import assert_close, oracle_pa, pa_decode_cabi, pack_descale, random_tables, to_oracle

pytestmark = pytest.mark.gpu

TOL = {torch.float16: 1e-3, torch.bfloat16: 2e-2}
INT8_TOL = 2e-2


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return torch.device("cuda:0")


@pytest.fixture(scope="module")
def stream(dev):
    return torch.cuda.Stream(device=dev)


def _rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


# ------------------------------------------------------------------ ReshapeAndCache
RAC_SHAPES = [
    # tokens, heads, dk, dv, block, blocks, dtype   (reference test_reshape_and_cache.py:106-260, pool scaled down)
    (100, 64, 576, 512, 128, 8, torch.int8),
    (100, 64, 320, 256, 128, 8, torch.float16),
    (100, 64, 400, 200, 128, 8, torch.bfloat16),
    (100, 64, 576, 576, 128, 8, torch.int8),
    (64, 8, 128, 128, 128, 80, torch.bfloat16),   # a decode step of the 8B-shaped config
    (7, 3, 5, 3, 16, 4, torch.int8),              # odd row sizes: byte-granular copy path
    (9, 1, 7, 9, 16, 4, torch.float16),           # 2-byte-granular copy path
]


def _rac_inputs(rng, dev, tokens, heads, dk, dv, block, blocks, dtype):
    def mk(shape, lo, hi):
        a = rng.integers(lo, hi, size=shape)
        return torch.from_numpy(a.astype(np.float32)).to(dtype).to(dev) if dtype != torch.int8 else \
            torch.from_numpy(a.astype(np.int8)).to(dev)
    key = mk((tokens, heads, dk), 1, 11)
    value = mk((tokens, heads, dv), 1, 11)
    kc = mk((blocks, block, heads, dk), 20, 30)
    vc = mk((blocks, block, heads, dv), 20, 30)
    n = blocks * block
    slots = rng.choice(np.arange(-n, n), size=tokens, replace=False).astype(np.int32)
    return key, value, kc, vc, slots


def _bits(t):
    return t.view(torch.int16) if t.dtype in (torch.float16, torch.bfloat16) else t


@pytest.mark.parametrize("shape", RAC_SHAPES, ids=lambda s: "x".join(str(v) for v in s[:6]) + str(s[6]).split(".")[-1])
def test_reshape_and_cache_bit_exact(binding, oracle, dev, stream, shape):
    rng = _rng(11)
    key, value, kc, vc, slots = _rac_inputs(rng, dev, *shape)
    want_k, want_v = oracle.reshape_and_cache(_bits(key).cpu().numpy(), _bits(value).cpu().numpy(),
                                              _bits(kc).cpu().numpy(), _bits(vc).cpu().numpy(), slots)
    ctx = binding.Context(stream)
    runner = binding.OperationRunner("ReshapeAndCacheOperation", binding.ReshapeAndCacheParam(), ctx)
    with torch.cuda.stream(stream):
        slots_d = torch.from_numpy(slots).to(dev)
        runner.run([key, value, kc, vc, slots_d], outputs=[kc, vc])
    stream.synchronize()
    assert np.array_equal(_bits(kc).cpu().numpy(), want_k)
    assert np.array_equal(_bits(vc).cpu().numpy(), want_v)
    assert (slots < 0).any()
    runner.close()
    ctx.close()


def test_reshape_and_cache_single_cache_and_out_of_range_slots(binding, oracle, dev, stream):
    rng = _rng(12)
    key, _, kc, _, slots = _rac_inputs(rng, dev, 20, 1, 576, 576, 128, 2, torch.bfloat16)
    want_k, _ = oracle.reshape_and_cache(_bits(key).cpu().numpy(), None, _bits(kc).cpu().numpy(), None, slots)
    ctx = binding.Context(stream)
    runner = binding.OperationRunner("ReshapeAndCacheOperation", binding.ReshapeAndCacheParam(kvCacheCfg=1), ctx)
    with torch.cuda.stream(stream):
        runner.run([key, kc, torch.from_numpy(slots).to(dev)], outputs=[kc])
    stream.synchronize()
    assert np.array_equal(_bits(kc).cpu().numpy(), want_k)
    # slots past the end of the cache are undefined in the reference; here they are skipped
    before = kc.clone()
    k = binding.kernels()
    with torch.cuda.stream(stream):
        far = torch.full((20,), 2 * 128 + 5, dtype=torch.int32, device=dev)
        rc = k.atbmi_reshape_and_cache(key.data_ptr(), None, kc.data_ptr(), None, far.data_ptr(), 20, 1, 576, 0,
                                       2 * 128, 2, stream.cuda_stream)
    stream.synchronize()
    assert rc == 0 and torch.equal(_bits(kc), _bits(before))
    runner.close()
    ctx.close()


# ------------------------------------------------------------------ ReshapeAndCache, fractal-NZ caches
NZ_RAC_SHAPES = [
    # tokens, heads, dk, dv, block, blocks, key dtype, value dtype
    (6144, 1, 512, 64, 128, 64, torch.int8, torch.float16),      # reference test_reshape_and_cache_nz.py:99-108
    (8192, 1, 128, 128, 128, 96, torch.int8, torch.float16),     # :110-119
    (6144, 1, 512, 64, 128, 64, torch.float16, torch.float16),   # :121-130
    (8192, 1, 128, 128, 128, 96, torch.float16, torch.float16),  # :132-141
    (4, 6, 64, 128, 64, 4, torch.int8, torch.bfloat16),          # CSV row 46: int8 key, heads * 64 / 32 pieces
    (4, 6, 128, 128, 128, 4, torch.bfloat16, torch.float16),     # CSV row 43: mixed 16-bit types
    (64, 1, 512, 64, 128, 34, torch.int8, torch.bfloat16),       # a decode step of the MLA int8 cache
    (33, 3, 32, 16, 16, 5, torch.float16, torch.bfloat16),       # smallest pieces, block size 16
]


def _nz_rac_inputs(rng, dev, tokens, heads, dk, dv, block, blocks, kdt, vdt):
    def mk(shape, dtype, lo, hi):
        a = rng.integers(lo, hi, size=shape)
        return torch.from_numpy(a.astype(np.int8)).to(dev) if dtype == torch.int8 else \
            torch.from_numpy(a.astype(np.float32)).to(dtype).to(dev)
    kl = 32 if kdt == torch.int8 else 16
    key, value = mk((tokens, heads, dk), kdt, -100, 100), mk((tokens, heads, dv), vdt, -100, 100)
    kc, vc = mk((blocks, heads * dk // kl, block, kl), kdt, 101, 120), mk((blocks, heads * dv // 16, block, 16), vdt, 101, 120)
    n = blocks * block
    # as the reference's test: unique slots from [-n, n), the negative ones are skipped, token 0 in slot 0
    slots = rng.choice(np.delete(np.arange(-n, n), n), size=tokens, replace=False).astype(np.int32)
    slots[0] = 0
    return key, value, kc, vc, slots


@pytest.mark.parametrize("shape", NZ_RAC_SHAPES, ids=lambda s: "x".join(str(v) for v in s[:6]) + "".join(
    "_" + str(t).split(".")[-1] for t in s[6:]))
def test_reshape_and_cache_nz_bit_exact(binding, oracle, dev, stream, shape):
    """kvCacheCfg K_CACHE_V_CACHE_NZ through the operation and through the C ABI, against the oracle."""
    rng = _rng(14)
    tokens, heads, dk, dv, block, blocks = shape[:6]
    key, value, kc, vc, slots = _nz_rac_inputs(rng, dev, *shape)
    kc2, vc2 = kc.clone(), vc.clone()
    want_k, want_v = oracle.reshape_and_cache_nz(_bits(key).cpu().numpy(), _bits(value).cpu().numpy(),
                                                 _bits(kc).cpu().numpy(), _bits(vc).cpu().numpy(), slots)
    ctx = binding.Context(stream)
    runner = binding.OperationRunner("ReshapeAndCacheOperation", binding.ReshapeAndCacheParam(kvCacheCfg=2), ctx)
    nz = [binding.make_tensor(binding._torch_acl_dtype(t), list(t.shape), device_ptr=t.data_ptr(), fmt="fractal_nz")
          for t in (kc, vc)]
    with torch.cuda.stream(stream):
        slots_d = torch.from_numpy(slots).to(dev)
        runner.run([key, value, nz[0], nz[1], slots_d], outputs=nz)
        rc = binding.kernels().atbmi_reshape_and_cache_nz(
            key.data_ptr(), value.data_ptr(), kc2.data_ptr(), vc2.data_ptr(), slots_d.data_ptr(), tokens, heads * dk,
            heads * dv, block, blocks, key.element_size(), value.element_size(), stream.cuda_stream)
    stream.synchronize()
    assert rc == 0, binding.last_kernel_error()
    for got in ((kc, vc), (kc2, vc2)):
        assert np.array_equal(_bits(got[0]).cpu().numpy(), want_k)
        assert np.array_equal(_bits(got[1]).cpu().numpy(), want_v)
    assert (slots < 0).any() and not np.array_equal(want_k, 0 * want_k)
    runner.close()
    ctx.close()


def test_reshape_and_cache_nz_feeds_multi_latent_attention(binding, oracle, dev, stream):
    """The step as a model runs it: latent and rotary rows written by ReshapeAndCache, read by
    MultiLatentAttention. Fractal-NZ caches (kvCacheCfg 2 -> cacheMode NZCACHE) must give the same bits as
    the token-major pair (kvCacheCfg 0 -> cacheMode KROPE_CTKV) on the same rows, and unaligned bases and
    slots past the end of the cache are handled by the C ABI as documented."""
    rng = _rng(15)
    heads, dv, dr, block, dtype = 32, 512, 64, 128, torch.float16
    ctx_lens = np.array([300, 129, 17], dtype=np.int32)
    blocks_per = 3
    blocks = 3 * blocks_per + 1
    tables = torch.from_numpy(rng.permutation(blocks)[:9].reshape(3, blocks_per).astype(np.int32)).to(dev)
    tokens = int(ctx_lens.sum())
    latent = ((torch.rand((tokens, 1, dv)) - 0.5)).to(dtype).to(dev)
    rotary = ((torch.rand((tokens, 1, dr)) - 0.5)).to(dtype).to(dev)
    slots = np.concatenate([tables.cpu().numpy()[b, np.arange(n) // block] * block + np.arange(n) % block
                            for b, n in enumerate(ctx_lens)]).astype(np.int32)
    nd = [torch.zeros((blocks, block, 1, dv), dtype=dtype, device=dev), torch.zeros((blocks, block, 1, dr), dtype=dtype, device=dev)]
    nz = [torch.zeros((blocks, dv // 16, block, 16), dtype=dtype, device=dev), torch.zeros((blocks, dr // 16, block, 16), dtype=dtype, device=dev)]
    nz_desc = [binding.make_tensor(binding._torch_acl_dtype(t), list(t.shape), device_ptr=t.data_ptr(), fmt="fractal_nz")
               for t in nz]
    c = binding.Context(stream)
    write_nd = binding.OperationRunner("ReshapeAndCacheOperation", binding.ReshapeAndCacheParam(), c)
    write_nz = binding.OperationRunner("ReshapeAndCacheOperation", binding.ReshapeAndCacheParam(kvCacheCfg=2), c)
    q = ((torch.rand((3, heads, dv + dr)) - 0.5)).to(dtype).to(dev)
    lens = torch.from_numpy(ctx_lens)
    scale = 1.0 / math.sqrt(192.0)
    outs = []
    with torch.cuda.stream(stream):
        slots_d = torch.from_numpy(slots).to(dev)
        write_nd.run([latent, rotary, nd[0], nd[1], slots_d], outputs=nd)
        write_nz.run([latent, rotary, nz_desc[0], nz_desc[1], slots_d], outputs=nz_desc)
        for mode, caches in ((1, nd), (3, nz_desc)):
            op = binding.OperationRunner("MultiLatentAttentionOperation", binding.MultiLatentAttentionParam(
                headNum=heads, kvHeadNum=1, qkScale=scale, cacheMode=mode), c)
            outs.append(op.run([q[..., :dv].contiguous(), q[..., dv:].contiguous(), caches[0], caches[1], tables,
                                lens.to(dev)], host_inputs={5: lens})[0])
            op.close()
    stream.synchronize()
    assert torch.equal(outs[0], outs[1]) and float(outs[0].float().abs().max()) > 0
    for a, b in zip(nd, nz):
        assert np.array_equal(oracle.nd_to_nz(_bits(a).cpu().numpy()[:, :, 0, :]), _bits(b).cpu().numpy())
    # the C ABI alone: bases aligned to 2 bytes only (element-wide accesses), slots past the cache skipped
    k = binding.kernels()
    store = torch.zeros(blocks * block * (dv + dr) + 64, dtype=dtype, device=dev)
    odd_k = store[1:1 + nz[0].numel()]
    odd_v = store[nz[0].numel() + 3:nz[0].numel() + 3 + nz[1].numel()]
    with torch.cuda.stream(stream):
        far = slots_d.clone()
        far[::7] = blocks * block + 5
        rc = k.atbmi_reshape_and_cache_nz(latent.data_ptr(), rotary.data_ptr(), odd_k.data_ptr(), odd_v.data_ptr(),
                                          far.data_ptr(), tokens, dv, dr, block, blocks, 2, 2, stream.cuda_stream)
    stream.synchronize()
    assert rc == 0, binding.last_kernel_error()
    kept = slots.copy()
    kept[::7] = -1
    want_k, want_v = oracle.reshape_and_cache_nz(_bits(latent).cpu().numpy(), _bits(rotary).cpu().numpy(),
                                                 np.zeros(nz[0].shape, np.int16), np.zeros(nz[1].shape, np.int16), kept)
    assert np.array_equal(_bits(odd_k).cpu().numpy().reshape(want_k.shape), want_k)
    assert np.array_equal(_bits(odd_v).cpu().numpy().reshape(want_v.shape), want_v)
    assert k.atbmi_reshape_and_cache_nz(latent.data_ptr(), rotary.data_ptr(), odd_k.data_ptr(), odd_v.data_ptr(),
                                        far.data_ptr(), tokens, dv + 8, dr, block, blocks, 2, 2, stream.cuda_stream) != 0
    write_nd.close()
    write_nz.close()
    c.close()


# ------------------------------------------------------------------ ReshapeAndCacheWithStride
STRIDED_CASES = [
    # tokens, heads, d, view builder -> (storage elements, strides, offset) per input, what it exercises
    ("unit_test_view", 2, 32, 128, lambda T, H, D: (T * H * D * 2, (H * D, D, 1), 5)),       # reference unit test: odd offset, 2-byte path
    ("fused_qkv_k", 64, 8, 128, lambda T, H, D: (T * (32 + 2 * H) * D, ((32 + 2 * H) * D, D, 1), 32 * D)),  # K slice of [T, (32+8+8)*128]
    ("padded_heads", 9, 3, 40, lambda T, H, D: (T * H * 48 + 8, (H * 48, 48, 1), 4)),        # 8-byte path
    ("channel_stride", 5, 4, 16, lambda T, H, D: (T * H * D * 3 + 7, (H * D * 3, D * 3, 3), 7)),  # channels not contiguous
    ("heads_major", 6, 4, 32, lambda T, H, D: (H * T * D, (D, T * D, 1), 0)),                # a [H, T, D] buffer viewed [T, H, D]
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", STRIDED_CASES, ids=lambda c: c[0])
def test_reshape_and_cache_with_stride_bit_exact(binding, oracle, dev, stream, case, dtype):
    """Strided key / value views through ReshapeAndCacheWithStrideOperation against the oracle's view
    + cache write (reference tests/unittest/ops/reshape_and_cache_with_stride/
    test_reshape_and_cache_with_stride.cpp:411-470: view by strides and offset, then the plain golden)."""
    name, T, H, D, view = case
    rng = _rng(31)
    block, blocks = 16, 8
    n_store, strides, offset = view(T, H, D)
    mk = lambda n, lo, hi: torch.from_numpy(rng.integers(lo, hi, size=n).astype(np.float32)).to(dtype).to(dev)
    k_store, v_store = mk(n_store, 1, 1000), mk(n_store + 16, 1, 1000)
    v_offset = offset + 16 if name != "unit_test_view" else offset
    kc = mk((blocks, block, H, D), 2000, 3000)
    vc = mk((blocks, block, H, D), 2000, 3000)
    slots = rng.choice(np.arange(-blocks * block, blocks * block), size=T, replace=False).astype(np.int32)
    slots[0] = max(slots[0], 0)
    key_view = oracle.strided_view(_bits(k_store).cpu().numpy(), (T, H, D), strides, offset)
    value_view = oracle.strided_view(_bits(v_store).cpu().numpy(), (T, H, D), strides, v_offset)
    want_k, want_v = oracle.reshape_and_cache(key_view, value_view, _bits(kc).cpu().numpy(), _bits(vc).cpu().numpy(), slots)

    acl = binding.ACL_FLOAT16 if dtype == torch.float16 else binding.ACL_BF16
    k_str, v_str = np.array(strides, dtype=np.int64), np.array(strides, dtype=np.int64)
    k_off, v_off = np.array([offset], dtype=np.int64), np.array([v_offset], dtype=np.int64)
    host = lambda a: binding.make_tensor(binding.ACL_INT64, list(a.shape), None, host_ptr=a.ctypes.data)
    ctx = binding.Context(stream)
    runner = binding.OperationRunner("ReshapeAndCacheWithStrideOperation", binding.ReshapeAndCacheWithStrideParam(), ctx)
    with torch.cuda.stream(stream):
        slots_d = torch.from_numpy(slots).to(dev)
        ins = [binding.make_tensor(acl, [T, H, D], k_store.data_ptr()), binding.make_tensor(acl, [T, H, D], v_store.data_ptr()),
               kc, vc, slots_d, host(k_str), host(v_str), host(k_off), host(v_off)]
        runner.run(ins, outputs=[kc, vc])
    stream.synchronize()
    assert np.array_equal(_bits(kc).cpu().numpy(), want_k)
    assert np.array_equal(_bits(vc).cpu().numpy(), want_v)
    runner.close()

    # single-cache form on the same view
    kc2 = mk((blocks, block, H, D), 2000, 3000)
    want_k2, _ = oracle.reshape_and_cache(key_view, None, _bits(kc2).cpu().numpy(), None, slots)
    single = binding.OperationRunner("ReshapeAndCacheWithStrideOperation",
                                     binding.ReshapeAndCacheWithStrideParam(kvCacheCfg=1), ctx)
    with torch.cuda.stream(stream):
        single.run([binding.make_tensor(acl, [T, H, D], k_store.data_ptr()), kc2, slots_d, host(k_str), host(k_off)],
                   outputs=[kc2])
    stream.synchronize()
    assert np.array_equal(_bits(kc2).cpu().numpy(), want_k2)
    single.close()
    ctx.close()


# batch, heads, head size, block, dtype, sequence lengths (lo, hi)
COMPRESS_WRITE_CASES = [
    (2, 4, 128, 128, torch.float16, (300, 700)),     # reference test_reshape_and_cache_wins.py shapes, shorter
    (5, 8, 128, 128, torch.bfloat16, (1, 400)),
    (3, 2, 64, 16, torch.int8, (50, 200)),
    (4, 8, 128, 128, torch.float16, (1024, 4096)),   # reference test_reshape_and_cache_wins_rope.py lengths
    (1, 1, 32, 16, torch.bfloat16, (17, 18)),
]


@pytest.mark.parametrize("mean_window", [False, True], ids=["keep_last", "mean_window"])
@pytest.mark.parametrize("case", COMPRESS_WRITE_CASES, ids=lambda c: "b%d_h%d_d%d_bs%d_%s" % (
    c[0], c[1], c[2], c[3], str(c[4]).split(".")[-1]))
def test_reshape_and_cache_head_compression_bit_exact(binding, oracle, dev, stream, case, mean_window):
    """ReshapeAndCacheParam::compressType KVHEAD (the last wins[i] tokens of each (sequence, head) pair) and
    KVHEAD_ROPE (a window of tokens replaced by its mean), bit for bit against the oracle; slots outside the
    pairs' stretches keep their contents."""
    batch, heads, d, block, dtype, (lo, hi) = case
    if mean_window and dtype == torch.int8:
        pytest.skip("the window mean is defined for 16-bit rows")
    rng = _rng(900 + batch + heads + d)
    seq = rng.integers(lo, hi, size=batch).astype(np.int32)
    tokens = int(seq.sum())
    pairs = batch * heads
    per_seq = np.repeat(seq, heads)
    wins = np.minimum(rng.integers(0, hi, size=pairs), per_seq).astype(np.int32)
    offs = None
    if mean_window:
        offs = np.array([rng.integers(-1, n - w + 1) for n, w in zip(per_seq, wins)], dtype=np.int32)
        offs[0] = -1
        wins[min(1, pairs - 1)] = min(1, wins[min(1, pairs - 1)])
        need = np.where((offs < 0) | (wins == 0), per_seq, per_seq - wins + 1)
    else:
        need = wins
    # every pair gets whole blocks of its own, in shuffled order; one pair is skipped
    order = rng.permutation(pairs)
    nblocks = (need + block - 1) // block
    first = np.zeros(pairs, dtype=np.int64)
    first[order] = np.concatenate([[0], np.cumsum(nblocks[order])[:-1]])
    slots = (first * block).astype(np.int32)
    if pairs > 2:
        slots[2] = -1
    blocks = int(nblocks.sum()) + 2
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(rng.integers(1 << 30)))
    if dtype == torch.int8:
        mk = lambda *shape: torch.randint(-128, 128, shape, generator=gen, dtype=torch.int8)
    else:
        mk = lambda *shape: ((torch.rand(shape, generator=gen) * 10 - 5)).to(dtype)
    key, value = mk(tokens, heads, d), mk(tokens, heads, d)
    kc0, vc0 = mk(blocks, block, 1, d), mk(blocks, block, 1, d)
    ins = [key.to(dev), value.to(dev), kc0.to(dev), vc0.to(dev), torch.from_numpy(slots).to(dev),
           torch.from_numpy(wins).to(dev), torch.from_numpy(seq).to(dev)]
    if mean_window:
        ins.append(torch.from_numpy(offs).to(dev))
    c = binding.Context(stream)
    op = binding.OperationRunner("ReshapeAndCacheOperation",
                                 binding.ReshapeAndCacheParam(compressType=2 if mean_window else 1), c)
    with torch.cuda.stream(stream):
        op.run(ins, outputs=[ins[2], ins[3]])
    stream.synchronize()
    op.close()
    c.close()
    od = {torch.float16: "float16", torch.bfloat16: "bf16", torch.int8: None}[dtype]
    want_k, want_v = oracle.reshape_and_cache_compress(
        to_oracle(key), to_oracle(value), to_oracle(kc0), to_oracle(vc0), slots, wins, seq, offs, out_dtype=od)
    for got, want, what in ((ins[2], want_k, "key"), (ins[3], want_v, "value")):
        want_t = torch.from_numpy(np.ascontiguousarray(want)).to(dtype)
        assert torch.equal(_bits(got.cpu()), _bits(want_t)), what


OMNI_CASES = [
    (1, 1, 256, 256, torch.bfloat16, (1024, 4096)),  # reference test_reshape_and_cache_omni_compress.py, one pair
    (40, 1, 96, 128, torch.float16, (200, 900)),     # its many-sequence shape (head size 96), shorter sequences
    (3, 8, 128, 128, torch.float16, (1, 700)),
    (5, 4, 64, 16, torch.bfloat16, (30, 300)),
]


@pytest.mark.parametrize("case", OMNI_CASES, ids=lambda c: "b%d_h%d_d%d_bs%d_%s" % (
    c[0], c[1], c[2], c[3], str(c[4]).split(".")[-1]))
def test_reshape_and_cache_omni_bit_exact(binding, oracle, dev, stream, case):
    """ReshapeAndCacheOmniOperation (a window of tokens per (sequence, head) pair is left out) bit for bit against
    the oracle: pairs without a window (offset -1, or a window of no tokens), windows at the start, at the end and
    past the end of their sequence, a skipped pair; slots outside the pairs' stretches keep their contents."""
    batch, heads, d, block, dtype, (lo, hi) = case
    rng = _rng(1300 + batch + heads + d)
    seq = rng.integers(lo, hi, size=batch).astype(np.int32)
    tokens = int(seq.sum())
    pairs = batch * heads
    per_seq = np.repeat(seq, heads)
    wins = np.minimum(rng.integers(0, hi, size=pairs), per_seq).astype(np.int32)
    offs = np.array([rng.integers(-1, n - w + 1) for n, w in zip(per_seq, wins)], dtype=np.int32)
    offs[0] = -1
    if pairs > 5:
        wins[1] = 0
        offs[3], wins[3] = 0, max(1, per_seq[3] // 2)               # the window opens the sequence
        offs[4] = per_seq[4] - wins[4]                               # ... ends it
        offs[5], wins[5] = per_seq[5] // 2, per_seq[5]               # ... runs past its end
    kept = np.where((offs < 0) | (wins == 0), per_seq, np.minimum(offs, per_seq) + np.maximum(per_seq - offs - wins, 0))
    order = rng.permutation(pairs)
    nblocks = (kept + block - 1) // block
    first = np.zeros(pairs, dtype=np.int64)
    first[order] = np.concatenate([[0], np.cumsum(nblocks[order])[:-1]])
    slots = (first * block).astype(np.int32)
    if pairs > 2:
        slots[2] = -1
    blocks = int(nblocks.sum()) + 2
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(rng.integers(1 << 30)))
    mk = lambda *shape: ((torch.rand(shape, generator=gen) * 10 - 5)).to(dtype)
    key, value = mk(tokens, heads, d), mk(tokens, heads, d)
    kc0, vc0 = mk(blocks, block, 1, d), mk(blocks, block, 1, d)
    ins = [key.to(dev), value.to(dev), kc0.to(dev), vc0.to(dev)] + \
          [torch.from_numpy(a).to(dev) for a in (slots, wins, seq, offs)]
    c = binding.Context(stream)
    op = binding.OperationRunner("ReshapeAndCacheOmniOperation", binding.ReshapeAndCacheOmniParam(), c)
    with torch.cuda.stream(stream):
        op.run(ins, outputs=[ins[2], ins[3]])
    stream.synchronize()
    op.close()
    c.close()
    want_k, want_v = oracle.reshape_and_cache_omni(to_oracle(key), to_oracle(value), to_oracle(kc0), to_oracle(vc0),
                                                   slots, wins, seq, offs)
    assert not np.array_equal(want_k, to_oracle(kc0))
    for got, want, what in ((ins[2], want_k, "key"), (ins[3], want_v, "value")):
        want_t = torch.from_numpy(np.ascontiguousarray(want)).to(dtype)
        assert torch.equal(_bits(got.cpu()), _bits(want_t)), what


def test_reshape_and_cache_with_stride_equals_plain_on_contiguous_input(binding, dev, stream):
    """With the strides of a contiguous tensor and offset 0 the operation is ReshapeAndCache."""
    rng = _rng(32)
    key, value, kc, vc, slots = _rac_inputs(rng, dev, 64, 8, 128, 128, 128, 80, torch.bfloat16)
    kc2, vc2 = kc.clone(), vc.clone()
    strides = np.array([8 * 128, 128, 1], dtype=np.int64)
    zero = np.zeros(1, dtype=np.int64)
    host = lambda a: binding.make_tensor(binding.ACL_INT64, list(a.shape), None, host_ptr=a.ctypes.data)
    ctx = binding.Context(stream)
    plain = binding.OperationRunner("ReshapeAndCacheOperation", binding.ReshapeAndCacheParam(), ctx)
    strided = binding.OperationRunner("ReshapeAndCacheWithStrideOperation", binding.ReshapeAndCacheWithStrideParam(), ctx)
    with torch.cuda.stream(stream):
        slots_d = torch.from_numpy(slots).to(dev)
        plain.run([key, value, kc, vc, slots_d], outputs=[kc, vc])
        strided.run([key, value, kc2, vc2, slots_d, host(strides), host(strides), host(zero), host(zero)],
                    outputs=[kc2, vc2])
    stream.synchronize()
    assert torch.equal(_bits(kc), _bits(kc2)) and torch.equal(_bits(vc), _bits(vc2))
    plain.close()
    strided.close()
    ctx.close()


# ------------------------------------------------------------------ ElewiseOperation (per-channel quantiser / dequantiser)
def test_elewise_quant_per_channel_bit_exact(binding, oracle, dev, stream):
    """ELEWISE_QUANT_PER_CHANNEL against the reference golden (fp16 division, round, offset, clamp), bit-exact:
    every finite fp16 pattern as x, the shapes of the reference's tests (scale over the trailing dimensions,
    a single scale, no offset), fp16 and bf16."""
    rng = _rng(71)
    ctx = binding.Context(stream)
    runner = binding.OperationRunner("ElewiseOperation", binding.ElewiseParam(elewiseType=17), ctx)
    bits = np.arange(65536, dtype=np.uint16).view(np.float16)
    allx = bits[np.isfinite(bits)]
    allx = np.concatenate([allx, allx[: (-len(allx)) % 1024]]).reshape(-1, 1024)
    cases = [(torch.float16, torch.from_numpy(allx.copy()), (1024,), True),
             (torch.float16, None, (32, 160), True), (torch.float16, None, (1,), True),
             (torch.float16, None, (32, 32), False), (torch.bfloat16, None, (32, 160), True),
             (torch.float16, None, (7, 9), True)]     # odd sizes: the element-wise path
    for dtype, x, scale_shape, with_offset in cases:
        if x is None:
            lead = (27,) if len(scale_shape) == 2 else (64, 1024)
            x = torch.from_numpy(rng.uniform(-300, 300, size=lead + (scale_shape if scale_shape != (1,) else ())).astype(np.float32)).to(dtype)
        scale = torch.from_numpy(rng.uniform(0.1, 3.0, size=scale_shape).astype(np.float32)).to(dtype)
        offset = torch.from_numpy(rng.integers(-10, 10, size=scale_shape).astype(np.int8)) if with_offset else \
            torch.empty((0,), dtype=torch.int8)
        # the golden converts bf16 inputs to fp16 first
        want = oracle.quant_per_channel_golden_dtype(x.to(torch.float16).numpy(), scale.to(torch.float16).numpy(),
                                                     offset.numpy() if with_offset else None)
        with torch.cuda.stream(stream):
            keep = [x.to(dev), scale.to(dev), offset.to(dev)]
            ins = [binding.tensor_of(keep[0]), binding.tensor_of(keep[1]),
                   binding.tensor_of(keep[2]) if with_offset else binding.make_tensor("int8", [0], None)]
            out = torch.empty(x.shape, dtype=torch.int8, device=dev)
            runner.run(ins, outputs=[out])
        stream.synchronize()
        assert np.array_equal(out.cpu().numpy(), want), (dtype, scale_shape, with_offset)
    runner.close()
    ctx.close()


def test_elewise_quant_special_scales_and_inputs(binding, oracle, dev, stream):
    """Scales of 0, infinity, NaN, the smallest subnormal and the largest fp16 beside ordinary ones, and x with
    infinities, NaN and signed zeros: the multiply-and-correct path of the quantiser must hand these to the
    plain division and agree with the golden (NaN quantises to 0)."""
    ctx = binding.Context(stream)
    runner = binding.OperationRunner("ElewiseOperation", binding.ElewiseParam(elewiseType=17), ctx)
    special = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 6e-8, 65504.0, 1.0, 0.5, 3.0, -2.0, 0.33, 1e-3, 100.0, 7.0, 0.1],
                       dtype=np.float16)
    xs = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 6e-8, -6e-8, 65504.0, -65504.0, 1.0, -1.0, 0.5, 1.5, 2.5, -2.5, 126.5],
                  dtype=np.float16)
    x = torch.from_numpy(np.repeat(xs[:, None], 16, axis=1).copy())        # row = x value, column = scale
    with np.errstate(all="ignore"):
        want = oracle.quant_per_channel_golden_dtype(x.numpy(), special, np.zeros(16, np.int8))
    with torch.cuda.stream(stream):
        keep = [x.to(dev), torch.from_numpy(special).to(dev), torch.zeros(16, dtype=torch.int8, device=dev)]
        out = torch.empty(x.shape, dtype=torch.int8, device=dev)
        runner.run(keep, outputs=[out])
    stream.synchronize()
    assert np.array_equal(out.cpu().numpy(), want), (out.cpu().numpy(), want)
    runner.close()
    ctx.close()


def test_elewise_dequant_per_channel_bit_exact(binding, oracle, dev, stream):
    """ELEWISE_DEQUANT_PER_CHANNEL against the reference golden, bit-exact: every int8 value against every
    offset for a set of scales that includes the saturating ones, and the shapes of the reference's tests."""
    rng = _rng(72)
    ctx = binding.Context(stream)
    runner = binding.OperationRunner("ElewiseOperation", binding.ElewiseParam(elewiseType=18), ctx)
    grid_x = np.repeat(np.arange(-128, 128, dtype=np.int8), 256).reshape(256, 256)      # row = x
    grid_o = np.tile(np.arange(-128, 128, dtype=np.int8), 256).reshape(256, 256)[:1]    # column = offset
    cases = []
    for sc in (0.37, 1.0, 300.0, -512.0, 6e-5, 65504.0):
        cases.append((torch.from_numpy(grid_x.copy()), np.full((256,), sc, np.float16), grid_o[0].copy()))
    cases.append((torch.from_numpy(rng.integers(-128, 128, size=(27, 32, 160)).astype(np.int8)),
                  rng.uniform(0.1, 1, size=(32, 160)).astype(np.float16), rng.integers(-128, 128, size=(32, 160)).astype(np.int8)))
    cases.append((torch.from_numpy(rng.integers(-128, 128, size=(64, 1024)).astype(np.int8)),
                  np.array([0.25], np.float16), np.array([-7], np.int8)))
    cases.append((torch.from_numpy(rng.integers(-128, 128, size=(10, 8192)).astype(np.int8)),
                  rng.uniform(0.1, 1, size=(8192,)).astype(np.float16), None))
    cases.append((torch.from_numpy(rng.integers(-128, 128, size=(5, 7, 9)).astype(np.int8)),
                  rng.uniform(0.1, 1, size=(7, 9)).astype(np.float16), rng.integers(-128, 128, size=(7, 9)).astype(np.int8)))
    for x, scale, offset in cases:
        want = oracle.dequant_per_channel(x.numpy(), scale, offset)
        with torch.cuda.stream(stream):
            keep = [x.to(dev), torch.from_numpy(scale).to(dev)] + ([torch.from_numpy(offset).to(dev)] if offset is not None else [])
            ins = [binding.tensor_of(keep[0]), binding.tensor_of(keep[1]),
                   binding.tensor_of(keep[2]) if offset is not None else binding.make_tensor("int8", [0], None)]
            out = torch.empty(x.shape, dtype=torch.float16, device=dev)
            runner.run(ins, outputs=[out])
        stream.synchronize()
        assert np.array_equal(out.cpu().numpy().view(np.int16), want.view(np.int16)), (tuple(x.shape), scale.shape)
    runner.close()
    ctx.close()


# ------------------------------------------------------------------ Rope
ROPE_CASES = [
    # name, q shape, k shape, table rows, head_dim, rotaryCoeff, cosFormat, seq lens, x dtype, table dtype
    ("glm_coeff4", (4, 4096), (4, 4096), 4, 128, 4, 0, [4], torch.float16, torch.float16),            # rope.csv row 1
    ("interleaved_4d", (2, 256, 32, 64), (2, 256, 32, 64), 512, 64, 64, 0, [256, 256], torch.float16, torch.float16),  # row 2
    ("gqa_half", (128, 1024), (128, 128), 128, 128, 2, 0, [128], torch.float16, torch.float16),        # row 3
    ("fp32_tables", (128, 1024), (128, 128), 128, 128, 2, 0, [128], torch.float16, torch.float32),     # test_rope_operation2.py:103-117
    ("deepseek", (3072, 8192), (3072, 64), 3072, 64, 2, 0, [3072], torch.float16, torch.float16),      # row 25
    ("coeff16_bf16", (4, 448), (4, 448), 4, 16, 16, 0, [4], torch.bfloat16, torch.bfloat16),           # row 26
    ("coeff4_positions", (9, 19264), (9, 19264), 4, 448, 4, 1, [4, 2, 3], torch.bfloat16, torch.bfloat16),  # row 40 (cosFormat 1)
    ("positions_half", (2048, 1024), (2048, 1024), 700, 128, 2, 1, [700, 1, 647, 700], torch.float16, torch.float16),  # test_rope_operation3.py:57-74
    ("llama3_8b_step", (64, 4096), (64, 1024), 64, 128, 2, 0, [1] * 64, torch.bfloat16, torch.bfloat16),  # the decode step before workload C2
]


@pytest.mark.parametrize("case", ROPE_CASES, ids=lambda c: c[0])
def test_rope_operation(binding, oracle, dev, stream, case):
    """RopeOperation against the fp32 oracle rounded once. Tolerance: one step of the 16-bit output grid
    (the kernel rounds products and sum separately in fp32 like the oracle; what is left are the ties of the
    final rounding), and under 0.1 % of the elements may differ at all."""
    name, q_shape, k_shape, rows, d, coeff, fmt, lens, dtype, tab_dtype = case
    rng = _rng(51)
    u = lambda shape, dt: torch.from_numpy(rng.uniform(-2, 2, size=shape).astype(np.float32)).to(dt)
    q, k = u(q_shape, dtype), u(k_shape, dtype)
    cos, sin = u((rows, d), tab_dtype), u((rows, d), tab_dtype)
    lens_t = torch.tensor(lens, dtype=torch.int32)
    T = q_shape[0] if len(q_shape) == 2 else q_shape[0] * q_shape[1]
    want_q, want_k = oracle.rope(q.float().numpy().reshape(T, -1), k.float().numpy().reshape(T, -1), cos.float().numpy(),
                                 sin.float().numpy(), lens, coeff, fmt, out_dtype="bf16" if dtype == torch.bfloat16 else np.float16)
    ctx = binding.Context(stream)
    runner = binding.OperationRunner("RopeOperation", binding.RopeParam(rotaryCoeff=coeff, cosFormat=fmt), ctx)
    with torch.cuda.stream(stream):
        out_q, out_k = runner.run([t.to(dev) for t in (q, k, cos, sin, lens_t)])
    stream.synchronize()
    assert tuple(out_q.shape) == q_shape and tuple(out_k.shape) == k_shape
    for got, want in ((out_q, want_q), (out_k, want_k)):
        g = got.float().cpu().numpy().reshape(T, -1)
        w = want.astype(np.float32)
        step = np.abs(w) * (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10) + 2.0 ** -24
        assert np.all(np.abs(g - w) <= step), float(np.abs(g - w).max())
        assert np.mean(g != w) < 1e-3
    runner.close()
    ctx.close()


def test_rope_in_place_and_tokens_outside_the_sequences(binding, oracle, dev, stream):
    """The C ABI with the outputs aliasing the inputs, and cosFormat 1 with more tokens than the sequences
    hold and a sequence longer than the tables: those tokens keep their values."""
    k_ = binding.kernels()
    rng = _rng(52)
    T, hq, hk, d, rows = 12, 256, 64, 64, 4
    u = lambda *shape: torch.from_numpy(rng.uniform(-2, 2, size=shape).astype(np.float32)).to(torch.float16)
    q, k, cos, sin = u(T, hq), u(T, hk), u(rows, d), u(rows, d)
    lens = [3, 6, 1]   # 10 of the 12 tokens; positions 4 and 5 of the second sequence have no table row
    pos = np.array([0, 1, 2, 0, 1, 2, 3, -1, -1, 0, -1, -1])
    live = pos >= 0
    want_q, want_k = q.numpy().copy(), k.numpy().copy()
    lq, lk = oracle.rope(q.float().numpy()[live], k.float().numpy()[live], cos.float().numpy()[pos[live]],
                         sin.float().numpy()[pos[live]], [int(live.sum())], 2, 0)
    want_q[live], want_k[live] = lq, lk
    with torch.cuda.stream(stream):
        qd, kd, cd, sd = (t.to(dev) for t in (q, k, cos, sin))
        ld = torch.tensor(lens, dtype=torch.int32, device=dev)
        rc = k_.atbmi_rope(qd.data_ptr(), kd.data_ptr(), cd.data_ptr(), sd.data_ptr(), ld.data_ptr(), qd.data_ptr(),
                           kd.data_ptr(), T, hq, hk, d, rows, len(lens), 2, 1, 0, 0, stream.cuda_stream)
    stream.synchronize()
    assert rc == 0, binding.last_kernel_error()
    for got, want in ((qd, want_q), (kd, want_k)):
        g = got.cpu().numpy().astype(np.float32)
        assert np.all(np.abs(g - want.astype(np.float32)) <= np.abs(want.astype(np.float32)) * 2.0 ** -10 + 2.0 ** -24)
        assert np.array_equal(got.cpu().numpy()[~live].view(np.int16), want[~live].view(np.int16))


# ------------------------------------------------------------------ NormRopeReshape
def _reference_standard(got, want, factor_max, factor_mean):
    """The reference's own pass criterion for this operator (tests/apitest/opstest/python/operations/
    norm_rope_reshape/test_norm_rope_reshape.py:74-85): |diff| <= factor_max * max(1, |golden|) everywhere
    and |mean(diff / max(1, |golden|))| <= factor_mean."""
    diff = np.abs(got.astype(np.float64) - want.astype(np.float64))
    scale = np.maximum(1.0, np.abs(want.astype(np.float64)))
    assert np.all(diff <= factor_max * scale), float((diff / scale).max())
    assert abs(np.mean(diff / scale)) <= factor_mean


@pytest.mark.parametrize("lo,hi", [(0.0, 1.0), (-100.0, 100.0)])
def test_norm_rope_reshape_operation_fp16(binding, oracle, dev, stream, lo, hi):
    """The reference's operation test shape (64 tokens, 512 + 64 channels, 192 blocks of 128) with its
    [0, 1) inputs, and the CSV rows' [-100, 100] range; fp16. Tolerance: the reference's fp16 standard
    2^-8 / 2^-10; on top of it every element must be within one fp16 step of the fp32 oracle rounded once."""
    rng = _rng(41)
    T, n, r, blocks, block = 64, 512, 64, 192, 128
    u = lambda *shape: torch.from_numpy(rng.uniform(lo, hi, size=shape).astype(np.float32)).to(torch.float16)
    x, gamma, rope, cos, sin = u(T, 1, n), u(n), u(T, r), u(T, r), u(T, r)
    cache = u(blocks, block, 1, n + r)
    slots = rng.choice(np.arange(-50, blocks * block), size=T, replace=False).astype(np.int32)
    slots[:3] = [-1, 0, blocks * block - 1]
    want = oracle.norm_rope_reshape(x.float().numpy(), gamma.float().numpy(), rope.float().numpy(), cos.float().numpy(),
                                    sin.float().numpy(), slots, cache.numpy(), 1e-5)
    ctx = binding.Context(stream)
    runner = binding.OperationRunner("NormRopeReshapeOperation", binding.NormRopeReshapeParam(epsilon=1e-5), ctx)
    with torch.cuda.stream(stream):
        cache_d = cache.to(dev)
        ins = [t.to(dev) for t in (x, gamma, rope, cos, sin)] + [torch.from_numpy(slots).to(dev), cache_d]
        runner.run(ins, outputs=[cache_d])
    stream.synchronize()
    got = cache_d.cpu().numpy()
    _reference_standard(got, want, 2.0 ** -8, 2.0 ** -10)
    # within one step of the 16-bit grid; rows of skipped and untouched slots are bit-identical
    step = np.abs(np.nextafter(want, np.float16(np.inf)).astype(np.float32) - want.astype(np.float32))
    assert np.all(np.abs(got.astype(np.float32) - want.astype(np.float32)) <= step)
    assert np.mean(got.view(np.int16) != want.view(np.int16)) < 0.01
    flat_got, flat_in = got.reshape(blocks * block, -1), cache.numpy().reshape(blocks * block, -1)
    untouched = np.setdiff1d(np.arange(blocks * block), slots[slots >= 0])
    assert np.array_equal(flat_got[untouched].view(np.int16), flat_in[untouched].view(np.int16))
    runner.close()
    ctx.close()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_norm_rope_reshape_kernel_many_tokens(binding, oracle, dev, stream, dtype):
    """The kernel-level test of the reference (tests/apitest/kernelstest/mix/
    test_rms_norm_and_rope_and_reshape_and_cache_bf16.py:91-130: tokens x 512 + 64 channels, inputs in
    [-100, 100], slots a random permutation, blocks of 512) through the C ABI, with 8192 tokens and
    odd row sizes as a second shape. Tolerance: the reference's standard, 2^-7 for bf16 and 2^-8 / 2^-10 for fp16."""
    k = binding.kernels()
    rng = _rng(42)
    for T, n, r, block in ((8192, 512, 64, 512), (37, 48, 16, 16), (19, 1024, 40, 16)):
        blocks = (T + 100 + block - 1) // block
        u = lambda *shape: torch.from_numpy(rng.uniform(-100, 100, size=shape).astype(np.float32)).to(dtype)
        x, gamma, rope, cos, sin = u(T, 1, n), u(n), u(T, r), u(T, r), u(T, r)
        slots = rng.permutation(T + 100)[:T].astype(np.int32)
        cache = torch.zeros((blocks, block, 1, n + r), dtype=dtype)
        is_bf16 = dtype == torch.bfloat16
        want = oracle.norm_rope_reshape(x.float().numpy(), gamma.float().numpy(), rope.float().numpy(),
                                        cos.float().numpy(), sin.float().numpy(), slots, cache.float().numpy(), 1e-5,
                                        out_dtype="bf16" if is_bf16 else np.float16)
        with torch.cuda.stream(stream):
            d = [t.to(dev) for t in (x, gamma, rope, cos, sin)]
            slots_d = torch.from_numpy(slots).to(dev)
            cache_d = cache.to(dev)
            rc = k.atbmi_norm_rope_reshape_and_cache(d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(),
                                                     d[4].data_ptr(), slots_d.data_ptr(), cache_d.data_ptr(), T, n, r,
                                                     blocks * block, 1 if is_bf16 else 0, 1e-5, stream.cuda_stream)
        stream.synchronize()
        assert rc == 0, binding.last_kernel_error()
        got = cache_d.float().cpu().numpy()
        if is_bf16:
            _reference_standard(got, want.astype(np.float32), 2.0 ** -7, 2.0 ** -7)
        else:
            _reference_standard(got, want.astype(np.float32), 2.0 ** -8, 2.0 ** -10)
        assert np.mean(got != want.astype(np.float32)) < 0.01


# ------------------------------------------------------------------ quantiser
def test_quant_all_fp16_patterns_bit_exact(binding, oracle, dev, stream):
    k = binding.kernels()
    x = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.float16)
    scales = np.array([0.005, 0.0123, 0.02, 0.37, 1.0, 3.0, 1e-4, 7.3], dtype=np.float32)
    x = x.reshape(8192, 8).to(dev)  # channel c = pattern % 8 sees scale c
    offs = np.array([0, 3, -3, 100, -100, 0, 1, -1], dtype=np.int32)
    for offset in (None, offs):
        with torch.cuda.stream(stream):
            out = torch.empty((8192, 8), dtype=torch.int8, device=dev)
            s_d = torch.from_numpy(scales).to(dev)
            o_d = torch.from_numpy(offset).to(dev) if offset is not None else None
            rc = k.atbmi_quant_per_channel(x.data_ptr(), binding.ATBMI_F16, s_d.data_ptr(),
                                           o_d.data_ptr() if o_d is not None else None, out.data_ptr(), 8192, 8,
                                           stream.cuda_stream)
        stream.synchronize()
        assert rc == 0
        want = oracle.quant_per_channel(x.float().cpu().numpy(), scales, offset)
        assert np.array_equal(out.cpu().numpy(), want)


def test_quant_bf16_bit_exact(binding, oracle, dev, stream):
    k = binding.kernels()
    x = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).reshape(4096, 16).to(dev)
    scales = _rng(13).uniform(0.005, 0.02, size=16).astype(np.float32)
    with torch.cuda.stream(stream):
        out = torch.empty((4096, 16), dtype=torch.int8, device=dev)
        s_d = torch.from_numpy(scales).to(dev)
        rc = k.atbmi_quant_per_channel(x.data_ptr(), binding.ATBMI_BF16, s_d.data_ptr(), None, out.data_ptr(), 4096, 16,
                                       stream.cuda_stream)
    stream.synchronize()
    assert rc == 0
    assert np.array_equal(out.cpu().numpy(), oracle.quant_per_channel(x.float().cpu().numpy(), scales))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_reshape_and_cache_quant_bit_exact(binding, oracle, dev, stream, dtype):
    """Fused quantise + cache write == quantiser followed by ReshapeAndCache."""
    rng = _rng(14)
    tokens, g, d, block, blocks = 128, 8, 128, 128, 6
    k = binding.kernels()
    key = torch.from_numpy(rng.standard_normal((tokens, g, d)).astype(np.float32) * 0.5).to(dtype).to(dev)
    value = torch.from_numpy(rng.standard_normal((tokens, g, d)).astype(np.float32) * 0.5).to(dtype).to(dev)
    ks = rng.uniform(0.005, 0.02, size=g * d).astype(np.float32)
    vs = rng.uniform(0.005, 0.02, size=g * d).astype(np.float32)
    kc = torch.from_numpy(rng.integers(-127, 128, size=(blocks, block, g, d)).astype(np.int8)).to(dev)
    vc = torch.from_numpy(rng.integers(-127, 128, size=(blocks, block, g, d)).astype(np.int8)).to(dev)
    n = blocks * block
    slots = rng.choice(np.arange(-n, n), size=tokens, replace=False).astype(np.int32)
    qk = oracle.quant_per_channel(key.float().cpu().numpy().reshape(tokens, -1), ks).reshape(tokens, g, d)
    qv = oracle.quant_per_channel(value.float().cpu().numpy().reshape(tokens, -1), vs).reshape(tokens, g, d)
    want_k, want_v = oracle.reshape_and_cache(qk, qv, kc.cpu().numpy(), vc.cpu().numpy(), slots)
    with torch.cuda.stream(stream):
        ks_d, vs_d, sl_d = torch.from_numpy(ks).to(dev), torch.from_numpy(vs).to(dev), torch.from_numpy(slots).to(dev)
        rc = k.atbmi_reshape_and_cache_quant(key.data_ptr(), value.data_ptr(),
                                             binding.ATBMI_BF16 if dtype == torch.bfloat16 else binding.ATBMI_F16,
                                             ks_d.data_ptr(), vs_d.data_ptr(), kc.data_ptr(), vc.data_ptr(),
                                             sl_d.data_ptr(), tokens, g, d, d, n, stream.cuda_stream)
    stream.synchronize()
    assert rc == 0
    assert np.array_equal(kc.cpu().numpy(), want_k) and np.array_equal(vc.cpu().numpy(), want_v)


# ------------------------------------------------------------------ block copy, paged cache load
# blocks, block size, heads, head size, sources, destinations, dtype
# (reference test_block_copy.py cases; an odd block size in bytes for the narrow-vector path; C2-sized blocks)
BLOCK_COPY_SHAPES = [
    (100, 2, 2, 2, 30, 30, torch.float16),
    (64, 16, 8, 128, 5, 40, torch.bfloat16),
    (37, 3, 1, 5, 4, 9, torch.int8),
    (300, 128, 8, 128, 16, 64, torch.float16),
]


@pytest.mark.parametrize("shape", BLOCK_COPY_SHAPES, ids=lambda s: "x".join(str(v) for v in s[:6]) + str(s[6]).split(".")[-1])
def test_block_copy_bit_exact(binding, oracle, dev, stream, shape):
    blocks, block, heads, d, n_src, n_dst, dtype = shape
    rng = _rng(500 + blocks)
    if dtype == torch.int8:
        kc = torch.from_numpy(rng.integers(-128, 128, size=(blocks, block, heads, d)).astype(np.int8)).to(dev)
        vc = torch.from_numpy(rng.integers(-128, 128, size=(blocks, block, heads, d)).astype(np.int8)).to(dev)
    else:
        kc = torch.from_numpy(rng.standard_normal((blocks, block, heads, d)).astype(np.float32)).to(dtype).to(dev)
        vc = torch.from_numpy(rng.standard_normal((blocks, block, heads, d)).astype(np.float32)).to(dtype).to(dev)
    perm = rng.permutation(blocks)
    src = perm[:n_src].astype(np.int32)
    dst = perm[n_src:n_src + n_dst].astype(np.int32)
    cuts = np.sort(rng.choice(np.arange(1, n_dst), size=n_src - 1, replace=False)) if n_src > 1 else np.array([], int)
    cum = np.append(cuts, n_dst).astype(np.int32)
    want_k, want_v = oracle.block_copy(_bits(kc).cpu().numpy(), _bits(vc).cpu().numpy(), src, dst, cum)
    src_d, dst_d, cum_d = (torch.from_numpy(a).to(dev) for a in (src, dst, cum))
    elem = kc.element_size()
    # through the C ABI on copies, then through the operation on the tensors themselves
    k2, v2 = kc.clone(), vc.clone()
    with torch.cuda.stream(stream):
        rc = binding.kernels().atbmi_block_copy(k2.data_ptr(), v2.data_ptr(), src_d.data_ptr(), dst_d.data_ptr(),
                                                cum_d.data_ptr(), n_src, n_dst, blocks, block * heads * d * elem,
                                                block * heads * d * elem, stream.cuda_stream)
    assert rc == 0, binding.last_kernel_error()
    stream.synchronize()
    assert np.array_equal(_bits(k2).cpu().numpy(), want_k) and np.array_equal(_bits(v2).cpu().numpy(), want_v)
    c = binding.Context(stream)
    op = binding.OperationRunner("BlockCopyOperation", binding.BlockCopyParam(), c)
    with torch.cuda.stream(stream):
        assert op.run([kc, vc, src_d, dst_d, cum_d], outputs=[]) == []
    stream.synchronize()
    assert np.array_equal(_bits(kc).cpu().numpy(), want_k) and np.array_equal(_bits(vc).cpu().numpy(), want_v)
    op.close()
    c.close()


# batch, heads, head size K, head size V, block size, blocks, dtype   (reference test_paged_cache_load_operation_nd.py:24-33)
CACHE_LOAD_SHAPES = [
    (16, 16, 144, 128, 128, 128, torch.float16),
    (16, 16, 144, 128, 128, 128, torch.int8),
    (32, 16, 192, 128, 64, 256, torch.bfloat16),
    (5, 2, 24, 8, 16, 40, torch.float16),
]


@pytest.mark.parametrize("cumsum,starts", [(True, True), (False, True), (False, False), (True, False)])
@pytest.mark.parametrize("shape", CACHE_LOAD_SHAPES, ids=lambda s: "x".join(str(v) for v in s[:6]) + str(s[6]).split(".")[-1])
def test_paged_cache_load_bit_exact(binding, oracle, dev, stream, shape, cumsum, starts):
    batch, heads, dk, dv, block, blocks, dtype = shape
    rng = _rng(520 + batch + int(cumsum) * 2 + int(starts))
    if dtype == torch.int8:
        kc = torch.from_numpy(rng.integers(-128, 128, size=(blocks, block, heads, dk)).astype(np.int8)).to(dev)
        vc = torch.from_numpy(rng.integers(-128, 128, size=(blocks, block, heads, dv)).astype(np.int8)).to(dev)
    else:
        kc = torch.from_numpy(rng.integers(1, 11, size=(blocks, block, heads, dk)).astype(np.float32)).to(dtype).to(dev)
        vc = torch.from_numpy(rng.integers(1, 11, size=(blocks, block, heads, dv)).astype(np.float32)).to(dtype).to(dev)
    lens = rng.integers(0, 1025, size=batch).astype(np.int32)
    lens[rng.integers(batch)] = 0
    max_blocks = (int(lens.max()) + block - 1) // block + 4
    tables = rng.integers(0, blocks, size=(batch, max_blocks)).astype(np.int32)
    seq_starts = (rng.integers(0, 5, size=batch) * block).astype(np.int32) if starts else np.zeros(batch, np.int32)
    total = int(lens.sum())
    key = torch.zeros((total, heads, dk), dtype=dtype, device=dev)
    value = torch.zeros((total, heads, dv), dtype=dtype, device=dev)
    arg = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32) if cumsum else lens
    want_k, want_v = oracle.paged_cache_load(_bits(kc).cpu().numpy(), _bits(vc).cpu().numpy(), tables, arg,
                                             _bits(key).cpu().numpy(), _bits(value).cpu().numpy(),
                                             seq_starts if starts else None, cumsum)
    c = binding.Context(stream)
    op = binding.OperationRunner("PagedCacheLoadOperation", binding.PagedCacheLoadParam(
        kvCacheCfg=1, isSeqLensCumsumMode=cumsum, hasSeqStarts=starts), c)
    with torch.cuda.stream(stream):
        op.run([kc, vc, torch.from_numpy(tables).to(dev), torch.from_numpy(arg).to(dev), key, value,
                torch.from_numpy(seq_starts).to(dev)], outputs=[key, value])
    stream.synchronize()
    assert np.array_equal(_bits(key).cpu().numpy(), want_k) and np.array_equal(_bits(value).cpu().numpy(), want_v)
    op.close()
    c.close()


# batch, channels K, channels V, block size, blocks, key dtype, value dtype
# (reference test_paged_cache_load_nz.py:150-260: 128-channel rows of every dtype pair; the MLA int8 cache)
NZ_LOAD_SHAPES = [
    (16, 128, 128, 128, 128, torch.float16, torch.float16),
    (16, 128, 128, 128, 128, torch.int8, torch.int8),
    (16, 128, 128, 128, 128, torch.bfloat16, torch.bfloat16),
    (16, 128, 128, 128, 128, torch.int8, torch.float16),
    (8, 512, 64, 128, 290, torch.int8, torch.bfloat16),    # CSV row 13 ("modelcase"): int8 latent + 16-bit rotary rows
    (5, 64, 32, 16, 40, torch.float16, torch.float16),
]


@pytest.mark.parametrize("shape", NZ_LOAD_SHAPES, ids=lambda s: "x".join(str(v) for v in s[:5]) + "".join(
    "_" + str(t).split(".")[-1] for t in s[5:]))
def test_paged_cache_load_nz_bit_exact(binding, oracle, dev, stream, shape):
    """kvCacheCfg K_CACHE_V_CACHE_NZ (the param's default) through the operation and the C ABI."""
    batch, ck, cv, block, blocks, kdt, vdt = shape
    rng = _rng(560 + batch + ck)

    def cache(chans, dtype):
        last = 32 if dtype == torch.int8 else 16
        a = rng.integers(-100, 100, size=(blocks, chans // last, block, last))
        return torch.from_numpy(a.astype(np.int8)).to(dev) if dtype == torch.int8 else \
            torch.from_numpy(a.astype(np.float32)).to(dtype).to(dev)
    kc, vc = cache(ck, kdt), cache(cv, vdt)
    lens = rng.integers(1, 1025, size=batch).astype(np.int32)
    lens[rng.integers(batch)] = 0
    max_blocks = (int(lens.max()) + block - 1) // block + 2
    tables = rng.integers(0, blocks, size=(batch, max_blocks)).astype(np.int32)
    total = int(lens.sum())
    key = torch.zeros((total, ck), dtype=kdt, device=dev)
    value = torch.zeros((total, cv), dtype=vdt, device=dev)
    key2, value2 = key.clone(), value.clone()
    want_k, want_v = oracle.paged_cache_load_nz(_bits(kc).cpu().numpy(), _bits(vc).cpu().numpy(), tables, lens,
                                                _bits(key).cpu().numpy(), _bits(value).cpu().numpy())
    c = binding.Context(stream)
    op = binding.OperationRunner("PagedCacheLoadOperation", binding.PagedCacheLoadParam(), c)
    nz = [binding.make_tensor(binding._torch_acl_dtype(t), list(t.shape), device_ptr=t.data_ptr(), fmt="fractal_nz")
          for t in (kc, vc)]
    with torch.cuda.stream(stream):
        tables_d, lens_d = torch.from_numpy(tables).to(dev), torch.from_numpy(lens).to(dev)
        op.run([nz[0], nz[1], tables_d, lens_d, key, value], outputs=[key, value])
        rc = binding.kernels().atbmi_paged_cache_load_nz(
            kc.data_ptr(), vc.data_ptr(), tables_d.data_ptr(), lens_d.data_ptr(), key2.data_ptr(), value2.data_ptr(),
            batch, max_blocks, block, blocks, ck * kc.element_size(), cv * vc.element_size(), 32, 32, total,
            int(lens.max()), stream.cuda_stream)
    stream.synchronize()
    assert rc == 0, binding.last_kernel_error()
    for got_k, got_v in ((key, value), (key2, value2)):
        assert np.array_equal(_bits(got_k).cpu().numpy(), want_k) and np.array_equal(_bits(got_v).cpu().numpy(), want_v)
    assert total > 0 and np.any(want_k != 0)
    op.close()
    c.close()


def test_cache_write_then_load_round_trip_at_c2_size(binding, pkg, dev, stream):
    """ReshapeAndCache followed by PagedCacheLoad returns the written rows in order (full C2 layout:
    64 sequences, 158 839 rows of 8 x 128 bf16), and BlockCopy of a sequence's blocks preserves them."""
    w = pkg.workloads
    cfg = w.config("c2")
    lay = w.layout(cfg)
    ctx, tables = lay["ctx"], lay["tables"]
    g, d, bs = cfg["kv_heads"], cfg["d"], cfg["block"]
    total = int(ctx.sum())
    gen = torch.Generator(device=dev)
    gen.manual_seed(7)
    rows_k = torch.randn((total, g, d), generator=gen, device=dev).to(torch.bfloat16)
    rows_v = torch.randn((total, g, d), generator=gen, device=dev).to(torch.bfloat16)
    kc = torch.zeros((lay["pool"], bs, g, d), dtype=torch.bfloat16, device=dev)
    vc = torch.zeros_like(kc)
    slots = np.concatenate([tables[b][np.arange(n) // bs].astype(np.int64) * bs + np.arange(n) % bs
                            for b, n in enumerate(ctx)]).astype(np.int32)
    c = binding.Context(stream)
    rac = binding.OperationRunner("ReshapeAndCacheOperation", binding.ReshapeAndCacheParam(), c)
    load = binding.OperationRunner("PagedCacheLoadOperation", binding.PagedCacheLoadParam(kvCacheCfg=1), c)
    out_k, out_v = torch.zeros_like(rows_k), torch.zeros_like(rows_v)
    tables_d = torch.from_numpy(tables).to(dev)
    with torch.cuda.stream(stream):
        rac.run([rows_k, rows_v, kc, vc, torch.from_numpy(slots).to(dev)], outputs=[kc, vc])
        load.run([kc, vc, tables_d, torch.from_numpy(ctx).to(dev), out_k, out_v,
                  torch.zeros(len(ctx), dtype=torch.int32, device=dev)], outputs=[out_k, out_v])
    stream.synchronize()
    assert torch.equal(out_k, rows_k) and torch.equal(out_v, rows_v)
    rac.close()
    load.close()
    c.close()


# ------------------------------------------------------------------ attention
def _pa_inputs(rng, dev, batch, heads, kv_heads, block, d, dv, ctx, dtype, kv_int8=False, pool_extra=4, std=1.0,
               unique=True):
    ctx = np.asarray(ctx if hasattr(ctx, "__len__") else [ctx] * batch, dtype=np.int32)
    need = int(((ctx.astype(np.int64) + block - 1) // block).sum())
    pool = need + pool_extra
    tables = random_tables(rng, ctx, block, pool, unique=unique)
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(rng.integers(1 << 30)))
    q = (torch.rand((len(ctx), heads, d), generator=gen) * 2 - 1).to(dtype).to(dev)
    if kv_int8:
        kc = torch.randint(-4, 5, (pool, block, kv_heads, d), generator=gen, dtype=torch.int8).to(dev)
        vc = torch.randint(-4, 5, (pool, block, kv_heads, dv), generator=gen, dtype=torch.int8).to(dev)
    else:
        kc = ((torch.rand((pool, block, kv_heads, d), generator=gen) * 2 - 1) * std).to(dtype).to(dev)
        vc = ((torch.rand((pool, block, kv_heads, dv), generator=gen) * 2 - 1) * std).to(dtype).to(dev)
    return q, kc, vc, torch.from_numpy(tables).to(dev), ctx


# batch, heads, kv_heads, block, d, ctx, dtype  (reference test_paged_attention_common.py case list)
PA_MATRIX = [
    (6, 32, 32, 128, 128, 819, torch.float16),
    (13, 32, 32, 128, 128, 200, torch.bfloat16),
    (13, 8, 1, 128, 128, 88, torch.float16),
    (20, 127, 1, 128, 128, 88, torch.float16),
    (18, 30, 2, 128, 128, 88, torch.float16),
    (20, 33, 33, 128, 128, 88, torch.float16),
    (4, 32, 2, 128, 128, 2048, torch.float16),
    (4, 24, 1, 16, 256, 3000, torch.float16),
    (2, 24, 1, 16, 256, 30000, torch.float16),
    (9, 40, 40, 16, 96, [3000, 300, 14000, 33, 65, 1, 16, 14000, 300], torch.float16),
    (1, 12, 1, 128, 128, 16390, torch.float16),
    (5, 8, 4, 128, 128, 13164, torch.bfloat16),
    (3, 12, 1, 128, 128, 32768, torch.bfloat16),
]


def _kernels_for(binding, d, dv, block):
    """Kernel selections to test: the scalar kernel always, the MFMA kernel where it is built."""
    return [binding.ATBMI_PA_KERNEL_SCALAR, binding.ATBMI_PA_KERNEL_AUTO]


@pytest.mark.parametrize("case", PA_MATRIX, ids=lambda c: "b%d_h%d_g%d_bs%d_d%d_%s" % (
    c[0], c[1], c[2], c[3], c[4], str(c[6]).split(".")[-1]))
def test_paged_attention_matrix(binding, oracle, dev, stream, case):
    batch, heads, kv_heads, block, d, ctx, dtype = case
    rng = _rng(hash(case[:5]) % 1000 + 20)
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, batch, heads, kv_heads, block, d, d, ctx, dtype)
    scale = 1.0 / math.sqrt(d)
    want = oracle_pa(oracle, q, kc, vc, tables, ctx, scale)
    for kernel in _kernels_for(binding, d, d, block):
        got = pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx, scale, kernel=kernel)
        assert_close(got, want, TOL[dtype], "kernel=%d" % kernel)


# Every head size that is a multiple of 32 has an MFMA build, for 16-bit caches and (from 64) for int8 caches (the
# reference's tests hold 64, 96, 128 and 256): batch, heads, kv_heads, block, d, ctx, dtype, int8 cache
HEAD_SIZES = [
    (3, 8, 2, 16, 32, [100, 700, 33], torch.float16, False),
    (2, 12, 4, 128, 160, [900, 129], torch.bfloat16, False),
    (2, 8, 8, 64, 192, [600, 2100], torch.float16, False),
    (2, 6, 2, 128, 224, [1500, 40], torch.bfloat16, False),
    (2, 10, 2, 128, 96, [513, 1300], torch.bfloat16, True),
    (2, 12, 4, 128, 160, [900, 129], torch.float16, True),
    (2, 8, 8, 64, 192, [600, 2100], torch.bfloat16, True),
    (2, 6, 2, 128, 224, [1500, 40], torch.float16, True),
]


@pytest.mark.parametrize("case", HEAD_SIZES, ids=lambda c: "d%d_%s%s" % (c[4], str(c[6]).split(".")[-1], "_int8" if c[7] else ""))
def test_mfma_kernel_on_every_multiple_of_32(binding, oracle, dev, stream, case):
    batch, heads, kv_heads, block, d, ctx, dtype, int8 = case
    rng = _rng(900 + d + int(int8))
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, batch, heads, kv_heads, block, d, d, ctx, dtype, kv_int8=int8)
    scale = 1.0 / math.sqrt(d)
    ks = ko = vs = vo = None
    if int8:
        ks = torch.from_numpy(rng.uniform(0.05, 0.5, size=kv_heads * d).astype(np.float32)).to(dev)
        vs = torch.from_numpy(rng.uniform(0.05, 0.5, size=kv_heads * d).astype(np.float32)).to(dev)
        ko = torch.from_numpy(rng.integers(-20, 20, size=kv_heads * d).astype(np.int32)).to(dev)
        vo = torch.from_numpy(rng.integers(-20, 20, size=kv_heads * d).astype(np.int32)).to(dev)
    want = oracle_pa(oracle, q, kc, vc, tables, ctx, scale, ks, ko, vs, vo)
    # asked for by name: the plan refuses a shape the MFMA kernel does not cover
    got = pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx, scale, ks, ko, vs, vo, kernel=binding.ATBMI_PA_KERNEL_MFMA)
    assert_close(got, want, INT8_TOL if int8 else TOL[dtype], "MFMA kernel, head size %d" % d)
    got = pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx, scale, ks, ko, vs, vo, kernel=binding.ATBMI_PA_KERNEL_SCALAR)
    assert_close(got, want, INT8_TOL if int8 else TOL[dtype], "scalar kernel, head size %d" % d)


# Fewer 32-token steps than the waves of a workgroup: batch, heads, kv_heads, d, ctx, dtype
TINY_PLANS = [
    (1, 8, 1, 128, [96], torch.float16),
    (1, 8, 2, 128, [64], torch.float16),
    (1, 4, 1, 64, [224], torch.bfloat16),
    (2, 16, 1, 128, [33, 70], torch.float16),
    (1, 12, 1, 256, [97], torch.float16),
    (3, 8, 1, 128, [1, 40, 129], torch.bfloat16),
]


@pytest.mark.parametrize("case", TINY_PLANS, ids=lambda c: "b%d_h%d_g%d_d%d_%s" % (
    c[0], c[1], c[2], c[3], "_".join(str(n) for n in c[4])))
def test_plans_with_fewer_steps_than_waves(binding, oracle, dev, stream, case):
    """One short sequence and few KV heads: the step space is shorter than the ranges a workgroup's waves
    could take, so some waves must idle and the merge must only see ranges that were written. The
    workspace is filled with NaN first: an unwritten partial row that is read shows up."""
    batch, heads, kv_heads, d, ctx, dtype = case
    rng = _rng(900 + heads + d + ctx[0])
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, batch, heads, kv_heads, 128, d, d, ctx, dtype)
    scale = 1.0 / math.sqrt(d)
    want = oracle_pa(oracle, q, kc, vc, tables, ctx, scale)
    for kernel in _kernels_for(binding, d, d, 128):
        got, info = pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx, scale, kernel=kernel, return_plan_info=True,
                                   poison_workspace=True)
        assert_close(got, want, TOL[dtype], "kernel=%d, %d ranges" % (kernel, info["chunks"]))


# batch, heads, kv_heads, block, d, ctx, dtype, mask kind
HEAD_MAJOR_MATRIX = [
    (16, 40, 10, 128, 128, 3000, torch.bfloat16, "norm3"),  # reference test_paged_attention_operation_BNSD.py:392-405
    (4, 32, 16, 64, 128, [100, 2000, 64, 777], torch.float16, None),  # the reference table's PagedAttentionBNSD row
    (5, 8, 8, 16, 64, [819, 12, 4000, 256, 300], torch.float16, "alibi4"),
    (3, 12, 1, 128, 256, [700, 1, 5000], torch.bfloat16, None),
    (4, 30, 2, 32, 96, [88, 1500, 3, 640], torch.float16, None),
    (2, 9, 3, 16, 80, [300, 45], torch.float16, None),
]


@pytest.mark.parametrize("case", HEAD_MAJOR_MATRIX, ids=lambda c: "b%d_h%d_g%d_bs%d_d%d_%s_%s" % (
    c[0], c[1], c[2], c[3], c[4], str(c[6]).split(".")[-1], c[7]))
def test_paged_attention_head_major_blocks(binding, oracle, dev, stream, case):
    """InputLayout TYPE_BNSD: caches [numBlocks, kvHeads, blockSize, headSize]. Against the oracle, and
    bit for bit against the same kernel on the token-major cache (the rows and their order are the same)."""
    batch, heads, kv_heads, block, d, ctx, dtype, kind = case
    rng = _rng(700 + batch + heads)
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, batch, heads, kv_heads, block, d, d, ctx, dtype)
    max_len = int(ctx.max())
    mask, per_head = (None, False) if kind is None else _mask_tensor(oracle, rng, dev, kind, ctx, heads, max_len, dtype)
    kc_hm = kc.permute(0, 2, 1, 3).contiguous()
    vc_hm = vc.permute(0, 2, 1, 3).contiguous()
    scale = 1.0 / math.sqrt(d)
    want = oracle_pa(oracle, q, kc_hm, vc_hm, tables, ctx, scale, mask=mask, mask_per_head=per_head, head_major=True)
    for kernel in _kernels_for(binding, d, d, block):
        got = pa_decode_cabi(binding, stream, q, kc_hm, vc_hm, tables, ctx, scale, kernel=kernel, mask=mask,
                             mask_per_head=per_head, head_major=True)
        assert_close(got, want, TOL[dtype], "kernel=%d" % kernel)
        same = pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx, scale, kernel=kernel, mask=mask,
                              mask_per_head=per_head)
        assert torch.equal(_bits(got), _bits(same)), "kernel=%d differs from the token-major run" % kernel


def test_head_major_blocks_through_operation_api(binding, oracle, dev, stream):
    """PagedAttentionParam::inputLayout = TYPE_BNSD with and without a mask (reference
    test_paged_attention_operation_BNSD.py:417-430: headNum 40, kvHeadNum 10, maskType 1, inputLayout 1)."""
    rng = _rng(741)
    heads, kv_heads, d, block = 40, 10, 128, 128
    ctx = np.array([3000, 300, 17, 1024, 129], dtype=np.int32)
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, len(ctx), heads, kv_heads, block, d, d, ctx, torch.bfloat16)
    kc_hm = kc.permute(0, 2, 1, 3).contiguous()
    vc_hm = vc.permute(0, 2, 1, 3).contiguous()
    lens = torch.from_numpy(ctx)
    scale = 1.0 / math.sqrt(d)
    c = binding.Context(stream)
    mask, per_head = _mask_tensor(oracle, rng, dev, "norm3", ctx, heads, 3000, torch.bfloat16)
    for mask_type, m in ((0, None), (1, mask)):
        pa = binding.OperationRunner("PagedAttentionOperation", binding.PagedAttentionParam(
            headNum=heads, kvHeadNum=kv_heads, qkScale=scale, maskType=mask_type, inputLayout=1), c)
        ins = [q, kc_hm, vc_hm, tables, lens.to(dev)] + ([m] if m is not None else [])
        with torch.cuda.stream(stream):
            out, = pa.run(ins, host_inputs={4: lens})
        stream.synchronize()
        assert tuple(out.shape) == (5, heads, d)
        want = oracle_pa(oracle, q, kc_hm, vc_hm, tables, ctx, scale, mask=m, mask_per_head=False, head_major=True)
        assert_close(out, want, TOL[torch.bfloat16], "maskType=%d" % mask_type)
        # the token-major reading of the same buffers is a different result
        assert np.abs(oracle_pa(oracle, q, kc_hm.reshape(kc.shape), vc_hm.reshape(vc.shape), tables, ctx, scale, mask=m,
                                mask_per_head=False) - want).max() > 1e-2
        pa.close()
    c.close()


# name, model batch, heads, kv heads, block, d, dtype, mask kind, int8 cache (+ offsets), razor offsets, zero lengths
COMPRESS_CASES = [
    ("plain", 5, 32, 8, 128, 128, torch.float16, None, False, False, False),
    ("norm3", 4, 32, 8, 128, 128, torch.bfloat16, "norm3", False, False, False),
    ("alibi4", 3, 40, 2, 128, 128, torch.float16, "alibi4", False, False, False),   # 20 heads per KV head: two tiles
    ("alibi4_1", 4, 16, 4, 16, 64, torch.float16, "alibi4_1", False, False, False),
    ("alibi3", 4, 32, 2, 128, 128, torch.bfloat16, "alibi3", False, False, False),
    ("int8", 6, 16, 4, 128, 128, torch.float16, None, True, False, False),
    ("int8_norm3", 3, 32, 8, 64, 128, torch.float16, "norm3", True, False, False),
    ("razor", 5, 32, 2, 128, 128, torch.bfloat16, None, False, True, False),
    ("razor_int8", 4, 8, 8, 32, 128, torch.float16, None, True, True, False),        # reference CSV shape: 8 heads, 8 KV heads
    ("zeros", 4, 32, 8, 128, 128, torch.float16, "alibi4", False, False, True),
    ("d96", 3, 12, 3, 16, 96, torch.float16, "norm3", False, False, False),
]


@pytest.mark.parametrize("forced", ["scalar", None])
@pytest.mark.parametrize("case", COMPRESS_CASES, ids=lambda c: c[0])
def test_head_compression_through_operation_api(binding, oracle, dev, stream, case, forced, monkeypatch):
    """PagedAttentionParam::compressType: caches [numBlocks, blockSize, 1, headSize], one context length and
    block-table row per (sequence, KV head) pair (reference golden test_paged_attention_common.py:292-360 and
    tiling/paged_attention_tiling.cpp:36-80,217-226); COMPRESS_TYPE_KVHEAD_ROPE adds the per-slot score offsets."""
    name, batch, heads, n, block, d, dtype, kind, kv_int8, razor, zeros = case
    rng = _rng(800 + batch + heads + n)
    if forced:
        monkeypatch.setenv("ATBMI_PA_KERNEL", forced)
    group = heads // n
    ctx = rng.integers(1, 1400, size=batch * n).astype(np.int32)
    ctx[rng.integers(0, batch * n)] = 2500
    if zeros:
        ctx[[1, 2, batch * n - 1]] = 0
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, batch * n, group, 1, block, d, d, ctx, dtype, kv_int8=kv_int8)
    q_model = q.view(batch, heads, d)
    max_len = 2500
    mask = per_head = None
    if kind is not None:
        mask, per_head = _mask_tensor(oracle, rng, dev, kind, np.full(batch, max_len), heads, max_len, dtype)
    ks = ko = vs = vo = ro = None
    if kv_int8:
        ks = torch.from_numpy(rng.uniform(0.01, 0.1, size=n * d).astype(np.float32)).to(dev)
        vs = torch.from_numpy(rng.uniform(0.01, 0.1, size=n * d).astype(np.float32)).to(dev)
        ko = torch.from_numpy(rng.integers(-20, 20, size=n * d).astype(np.int32)).to(dev)
        vo = torch.from_numpy(rng.integers(-20, 20, size=n * d).astype(np.int32)).to(dev)
    if razor:
        # like the reference generator (:469-478): mostly zero, values in [0, 20) at one offset of most blocks
        r = np.zeros((kc.shape[0], block), dtype=np.float32)
        rows = np.where(rng.random(kc.shape[0]) < 0.8)[0]
        r[rows, rng.integers(0, block, size=len(rows))] = rng.uniform(0, 20, size=len(rows)).astype(np.float32)
        ro = torch.from_numpy(r).to(dev)
    scale = 1.0 / math.sqrt(d)
    param = binding.PagedAttentionParam(
        headNum=heads, kvHeadNum=n, qkScale=scale, compressType=2 if razor else 1,
        maskType={None: 0, "norm3": 1}.get(kind, 2), quantType=1 if kv_int8 else 0, hasQuantOffset=kv_int8,
        batchRunStatusEnable=zeros)
    lens = torch.from_numpy(ctx)
    ins = [q_model, kc, vc, tables, lens.to(dev)]
    host = {4: lens}
    if mask is not None:
        ins.append(mask)
    if zeros:
        status = torch.from_numpy((ctx > 0).astype(np.int32))
        host[len(ins)] = status
        ins.append(status.to(dev))
    if kv_int8:
        ins += [ks, ko, vs, vo]
    if razor:
        ins.append(ro)
    c = binding.Context(stream)
    pa = binding.OperationRunner("PagedAttentionOperation", param, c)
    out = torch.full((batch, heads, d), 7.0, dtype=dtype, device=dev)
    with torch.cuda.stream(stream):
        pa.run(ins, outputs=[out], host_inputs=host)
    stream.synchronize()
    pa.close()
    c.close()
    want = oracle_pa(oracle, q_model, kc, vc, tables, ctx, scale, ks, ko, vs, vo, mask=mask, mask_per_head=per_head,
                     compress_kv_heads=n, razor_offset=ro, out_init=7.0)
    assert_close(out, want, INT8_TOL if kv_int8 else TOL[dtype], name)
    if razor or kind is not None:  # the offsets / the mask matter in this case
        plain = oracle_pa(oracle, q_model, kc, vc, tables, ctx, scale, ks, ko, vs, vo, compress_kv_heads=n, out_init=7.0)
        assert np.abs(want - plain).max() > 0.01


def test_compressed_write_then_compressed_attention(binding, oracle, dev, stream):
    """The two halves of head compression together: ReshapeAndCache (KVHEAD) keeps the last wins[i] tokens of
    every (sequence, KV head) pair, PagedAttention (KVHEAD) attends over them; the result is plain attention
    of each head group over its own window of the uncompressed keys and values."""
    rng = _rng(955)
    batch, heads, n, d, block = 3, 16, 4, 128, 128
    seq = rng.integers(200, 600, size=batch).astype(np.int32)
    wins = np.array([rng.integers(1, s + 1) for s in np.repeat(seq, n)], dtype=np.int32)
    nblocks = (wins + block - 1) // block
    first = np.concatenate([[0], np.cumsum(nblocks)[:-1]])
    slots = (first * block).astype(np.int32)
    blocks = int(nblocks.sum()) + 1
    tables = np.zeros((batch * n, int(nblocks.max())), dtype=np.int32)
    for i in range(batch * n):
        tables[i, :nblocks[i]] = first[i] + np.arange(nblocks[i])
    gen = torch.Generator(device="cpu")
    gen.manual_seed(9)
    mk = lambda *shape: (torch.rand(shape, generator=gen) * 2 - 1).to(torch.float16)
    key, value, q = mk(int(seq.sum()), n, d), mk(int(seq.sum()), n, d), mk(batch, heads, d)
    kc = torch.zeros((blocks, block, 1, d), dtype=torch.float16, device=dev)
    vc = torch.zeros_like(kc)
    c = binding.Context(stream)
    rac = binding.OperationRunner("ReshapeAndCacheOperation", binding.ReshapeAndCacheParam(compressType=1), c)
    scale = 1.0 / math.sqrt(d)
    pa = binding.OperationRunner("PagedAttentionOperation", binding.PagedAttentionParam(
        headNum=heads, kvHeadNum=n, qkScale=scale, compressType=1), c)
    lens = torch.from_numpy(wins)
    with torch.cuda.stream(stream):
        rac.run([key.to(dev), value.to(dev), kc, vc, torch.from_numpy(slots).to(dev), lens.to(dev),
                 torch.from_numpy(seq).to(dev)], outputs=[kc, vc])
        out, = pa.run([q.to(dev), kc, vc, torch.from_numpy(tables).to(dev), lens.to(dev)], host_inputs={4: lens})
    stream.synchronize()
    rac.close()
    pa.close()
    c.close()
    group = heads // n
    ends = np.cumsum(seq)
    want = np.zeros((batch, heads, d), dtype=np.float32)
    for i in range(batch * n):
        b, g = divmod(i, n)
        rows = slice(int(ends[b]) - int(wins[i]), int(ends[b]))
        want[b, g * group:(g + 1) * group] = oracle.attention_one(
            to_oracle(q)[b, g * group:(g + 1) * group], to_oracle(key)[rows, g:g + 1], to_oracle(value)[rows, g:g + 1],
            np.float32(scale))
    assert_close(out, want, TOL[torch.float16], "write + attention")


@pytest.mark.parametrize("forced", ["scalar", None])
def test_spec_mask_with_one_query_token_per_sequence(binding, oracle, dev, stream, forced, monkeypatch):
    """MASK_TYPE_SPEC without CALC_TYPE_SPEC: the mask [query rows, maxS] has one row per query row (the reference
    kernel library's look-ahead shape, mixkernels/pagedattention/paged_attention_operation.cpp:742-751); a sequence
    of length 0 takes neither a query row nor a mask row."""
    if forced:
        monkeypatch.setenv("ATBMI_PA_KERNEL", forced)
    rng = _rng(977)
    heads, kv_heads, d, block = 32, 8, 128, 128
    ctx = np.array([700, 0, 33, 2048, 129], dtype=np.int32)
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, len(ctx), heads, kv_heads, block, d, d, ctx, torch.float16)
    q = q[:4].contiguous()
    mask = rng.standard_normal((4, 2048)).astype(np.float32)
    mask[:, :5] = -10000.0
    mask = torch.from_numpy(mask).to(torch.float16).to(dev)
    scale = 1.0 / math.sqrt(d)
    lens = torch.from_numpy(ctx)
    status = torch.from_numpy((ctx > 0).astype(np.int32))
    c = binding.Context(stream)
    pa = binding.OperationRunner("PagedAttentionOperation", binding.PagedAttentionParam(
        headNum=heads, kvHeadNum=kv_heads, qkScale=scale, maskType=3, batchRunStatusEnable=True), c)
    with torch.cuda.stream(stream):
        out, = pa.run([q, kc, vc, tables, lens.to(dev), mask, status.to(dev)], host_inputs={4: lens, 6: status})
    stream.synchronize()
    pa.close()
    c.close()
    want = oracle_pa(oracle, q, kc, vc, tables, ctx, scale, mask=mask, mask_rows="query")
    assert_close(out, want, TOL[torch.float16], "SPEC mask, one token per sequence")
    assert np.abs(want - oracle_pa(oracle, q, kc, vc, tables, ctx, scale)).max() > 0.01


def test_c1_decode_step_through_operation_api(binding, oracle, pkg, dev, stream):
    """Benchmark configuration 1 end to end: ReshapeAndCache then PagedAttention
    through atb::Operation, fp16, rtol = atol = 1e-3."""
    w = pkg.workloads
    cfg = w.config("c1")
    step = w.make_step(cfg, dev)
    scale = w.qk_scale(cfg)
    kc0, vc0 = step["key_cache"].clone(), step["value_cache"].clone()
    want_k, want_v = oracle.reshape_and_cache(_bits(step["k_new"]).cpu().numpy(), _bits(step["v_new"]).cpu().numpy(),
                                              _bits(kc0).cpu().numpy(), _bits(vc0).cpu().numpy(),
                                              step["layout"]["slots"])
    ctx = binding.Context(stream)
    rac = binding.OperationRunner("ReshapeAndCacheOperation", binding.ReshapeAndCacheParam(), ctx)
    pa = binding.OperationRunner("PagedAttentionOperation", binding.PagedAttentionParam(
        headNum=cfg["heads"], kvHeadNum=cfg["kv_heads"], qkScale=scale), ctx)
    with torch.cuda.stream(stream):
        rac.run([step["k_new"], step["v_new"], step["key_cache"], step["value_cache"], step["slot_mapping"]],
                outputs=[step["key_cache"], step["value_cache"]])
        lens_dev = step["context_lens"].to(dev)
        out, = pa.run([step["q"], step["key_cache"], step["value_cache"], step["block_tables"], lens_dev],
                      host_inputs={4: step["context_lens"]})
    stream.synchronize()
    assert np.array_equal(_bits(step["key_cache"]).cpu().numpy(), want_k)
    assert np.array_equal(_bits(step["value_cache"]).cpu().numpy(), want_v)
    want = oracle.paged_attention(to_oracle(step["q"]), to_oracle(step["key_cache"]), to_oracle(step["value_cache"]),
                                  step["layout"]["tables"], step["layout"]["ctx"], scale)
    assert_close(out, want, 1e-3, "c1")
    # the new token is part of the context: dropping it must change the result
    short = oracle.paged_attention(to_oracle(step["q"]), to_oracle(kc0), to_oracle(vc0), step["layout"]["tables"],
                                   step["layout"]["ctx"], scale)
    assert np.abs(short - want).max() > 1e-3
    rac.close()
    pa.close()
    ctx.close()


# batch, heads, kv_heads, ctx, q dtype, with offsets   (reference :2179-2808)
INT8_MATRIX = [
    (24, 8, 8, 256, torch.float16, False),
    (16, 8, 1, 256, torch.bfloat16, False),
    (1, 24, 1, 513, torch.bfloat16, False),
    (16, 8, 1, 256, torch.float16, True),
    (1, 8, 8, 256, torch.float16, False),
    (1, 8, 8, 1780, torch.float16, True),
    (8, 64, 8, 1200, torch.float16, False),
]


@pytest.mark.parametrize("case", INT8_MATRIX, ids=lambda c: "b%d_h%d_g%d_ctx%d_%s_off%d" % (
    c[0], c[1], c[2], c[3], str(c[4]).split(".")[-1], c[5]))
def test_paged_attention_int8_cache(binding, oracle, dev, stream, case):
    batch, heads, kv_heads, ctx, dtype, with_off = case
    rng = _rng(30 + batch + heads)
    d = 128
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, batch, heads, kv_heads, 128, d, d, ctx, dtype, kv_int8=True)
    ks = torch.from_numpy(rng.uniform(0.05, 0.5, size=kv_heads * d).astype(np.float32)).to(dev)
    vs = torch.from_numpy(rng.uniform(0.05, 0.5, size=kv_heads * d).astype(np.float32)).to(dev)
    ko = torch.from_numpy(rng.integers(-20, 20, size=kv_heads * d).astype(np.int32)).to(dev) if with_off else None
    vo = torch.from_numpy(rng.integers(-20, 20, size=kv_heads * d).astype(np.int32)).to(dev) if with_off else None
    scale = 1.0 / math.sqrt(d)
    want = oracle_pa(oracle, q, kc, vc, tables, ctx, scale, ks, ko, vs, vo)
    for kernel in _kernels_for(binding, d, d, 128):
        got = pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx, scale, ks, ko, vs, vo, kernel=kernel)
        assert_close(got, want, INT8_TOL, "kernel=%d" % kernel)


def test_int8_offsets_that_cancel_the_values_on_split_rows(binding, oracle, dev, stream):
    """Values around +100 with an offset of -100: the dequantised values are small differences of large numbers.
    Rows cut across wave ranges travel as 16-bit partial rows, which the attention kernel descales before it rounds
    them, so the merged result keeps the accuracy of an unsplit row (a partial row kept in int8 units and rounded
    to 16 bits first would be off by about 2e-3 here)."""
    rng = _rng(47)
    heads, kv_heads, d = 8, 2, 128
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, 2, heads, kv_heads, 128, d, d, [3000, 1500], torch.float16, kv_int8=True)
    gen = torch.Generator(device="cpu")
    gen.manual_seed(5)
    vc = torch.randint(96, 105, tuple(vc.shape), generator=gen, dtype=torch.int8).to(dev)
    ks = torch.full((kv_heads * d,), 0.05, dtype=torch.float32, device=dev)
    vs = torch.full((kv_heads * d,), 0.05, dtype=torch.float32, device=dev)
    ko = torch.zeros(kv_heads * d, dtype=torch.int32, device=dev)
    vo = torch.full((kv_heads * d,), -100, dtype=torch.int32, device=dev)
    scale = 1.0 / math.sqrt(d)
    want = oracle_pa(oracle, q, kc, vc, tables, ctx, scale, ks, ko, vs, vo)
    assert np.abs(want).max() < 0.25  # (the values lie within +-0.2)
    got, info = pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx, scale, ks, ko, vs, vo, kernel=0,
                               return_plan_info=True)
    assert info["chunks"] > 8  # the rows are cut
    assert_close(got, want, 3e-4, "cancelling offsets")


def test_int8_through_operation_api_with_offsets(binding, oracle, dev, stream):
    rng = _rng(41)
    heads, kv_heads, d = 32, 16, 128
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, 4, heads, kv_heads, 64, d, d, [100, 2000, 64, 777], torch.float16,
                                        kv_int8=True)
    ks = torch.from_numpy(rng.uniform(0.01, 0.1, size=kv_heads * d).astype(np.float32)).to(dev)
    vs = torch.from_numpy(rng.uniform(0.01, 0.1, size=kv_heads * d).astype(np.float32)).to(dev)
    ko = torch.from_numpy(rng.integers(-20, 20, size=kv_heads * d).astype(np.int32)).to(dev)
    vo = torch.from_numpy(rng.integers(-20, 20, size=kv_heads * d).astype(np.int32)).to(dev)
    scale = 1.0 / math.sqrt(d)
    c = binding.Context(stream)
    pa = binding.OperationRunner("PagedAttentionOperation", binding.PagedAttentionParam(
        headNum=heads, kvHeadNum=kv_heads, qkScale=scale, quantType=1, hasQuantOffset=True), c)
    lens = torch.from_numpy(ctx)
    with torch.cuda.stream(stream):
        out, = pa.run([q, kc, vc, tables, lens.to(dev), ks, ko, vs, vo], host_inputs={4: lens})
    stream.synchronize()
    assert_close(out, oracle_pa(oracle, q, kc, vc, tables, ctx, scale, ks, ko, vs, vo), INT8_TOL, "dequant api")
    # the same descales uint64-packed (Utils::QuantParamConvert; reference
    # test_paged_attention_common.py:120-122,523-533): bit-identical output
    ks64, vs64 = pack_descale(ks), pack_descale(vs)
    assert ks64.dtype == torch.int64 and int(ks64.min()) >= 0
    with torch.cuda.stream(stream):
        out64, = pa.run([q, kc, vc, tables, lens.to(dev), ks64, ko, vs64, vo], host_inputs={4: lens})
    stream.synchronize()
    assert torch.equal(out64, out)
    for kernel in (binding.ATBMI_PA_KERNEL_SCALAR, binding.ATBMI_PA_KERNEL_AUTO):
        a = pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx, scale, ks, ko, vs, vo, kernel=kernel)
        b = pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx, scale, ks64, ko, vs64, vo, kernel=kernel)
        assert torch.equal(a, b)
    pa.close()
    c.close()


# batch, heads, d, dv, block, ctx, dtype   (reference test_paged_attention_mla.py:713-1137, op test :412-444)
MLA_MATRIX = [
    (20, 128, 576, 512, 128, 256, torch.float16),
    (1, 8, 576, 512, 128, 256, torch.bfloat16),
    (64, 32, 192, 128, 128, 256, torch.float16),
    (32, 8, 576, 512, 128, 819, torch.float16),
    (4, 128, 576, 512, 128, [3000, 17, 128, 1025], torch.bfloat16),
    (1, 16, 576, 512, 256, 256, torch.float16),      # block size 256: reference test_paged_attention_mla.py:1137-1152
    (3, 16, 576, 512, 256, [700, 256, 257], torch.bfloat16),
    (2, 128, 576, 512, 256, [2000, 511], torch.float16),  # ... and on the 128-head kernel
]


@pytest.mark.parametrize("case", MLA_MATRIX, ids=lambda c: "b%d_h%d_d%d_dv%d_%s" % (
    c[0], c[1], c[2], c[3], str(c[6]).split(".")[-1]))
def test_paged_attention_mla_combined_cache(binding, oracle, dev, stream, case):
    batch, heads, d, dv, block, ctx, dtype = case
    rng = _rng(50 + batch)
    q, kc, _, tables, ctx = _pa_inputs(rng, dev, batch, heads, 1, block, d, dv, ctx, dtype, std=0.5)
    scale = 1.0 / math.sqrt(d)
    want = oracle_pa(oracle, q, kc, None, tables, ctx, scale, mla_dv=dv)
    for kernel in _kernels_for(binding, d, dv, block):
        got = pa_decode_cabi(binding, stream, q, kc, None, tables, ctx, scale, mla_dv=dv, kernel=kernel)
        assert_close(got, want, TOL[dtype], "kernel=%d" % kernel)


# The 128-head kernel (combined 576/512 cache, heads a multiple of 128) has paths of its own:
# batch, heads, block, ctx, dtype, chunk_tokens, what the case is for
MLA_WIDE_MATRIX = [
    (3, 256, 128, [700, 45, 1], torch.bfloat16, None, "two head groups of 128, ragged lengths, one token"),
    (6, 128, 128, [333, 32, 31, 33, 64, 257], torch.float16, 64, "ranges of two steps: rows cut everywhere"),
    (2, 128, 16, [18000, 500], torch.bfloat16, 32768, "block size 16, one range: more block ids than the LDS table holds"),
    (2, 128, 16, [18000, 500], torch.bfloat16, None, "block size 16, many short ranges"),
    (5, 128, 32, [96, 4100, 1, 160, 2047], torch.float16, 4096, "block size 32, ranges spanning sequences"),
    (1, 128, 128, [12345], torch.float16, 320, "one long row merged from many ranges"),
    # head counts that are not a multiple of 128 (tensor-parallel ranks): waves with fewer than 32 heads, or none
    (3, 16, 128, [700, 45, 1], torch.bfloat16, None, "16 heads: half a wave"),
    (4, 32, 128, [2100, 333, 32, 64], torch.float16, None, "32 heads: one wave"),
    (3, 64, 64, [1500, 257, 31], torch.bfloat16, 64, "64 heads, rows cut everywhere"),
    (2, 40, 128, [900, 129], torch.float16, None, "40 heads: a wave and a quarter of one"),
    (2, 136, 128, [900, 129], torch.bfloat16, None, "136 heads: a second group of 8"),
    (2, 8, 16, [3000, 5], torch.float16, None, "8 heads, block size 16"),
]


@pytest.mark.parametrize("case", MLA_WIDE_MATRIX, ids=lambda c: "b%d_h%d_bs%d_%s_%s" % (
    c[0], c[1], c[2], str(c[4]).split(".")[-1], c[5]))
def test_paged_attention_mla_128_head_kernel(binding, oracle, dev, stream, case):
    """Checked against the oracle and, element by element, against the fp32 scalar kernel."""
    batch, heads, block, ctx, dtype, chunk, _ = case
    rng = _rng(300 + batch + block)
    q, kc, _, tables, ctx = _pa_inputs(rng, dev, batch, heads, 1, block, 576, 512, ctx, dtype, std=0.5)
    scale = 1.0 / math.sqrt(576)
    want = oracle_pa(oracle, q, kc, None, tables, ctx, scale, mla_dv=512)
    got, info = pa_decode_cabi(binding, stream, q, kc, None, tables, ctx, scale, mla_dv=512,
                               kernel=binding.ATBMI_PA_KERNEL_MFMA, chunk_tokens=chunk, return_plan_info=True)
    assert_close(got, want, TOL[dtype], "128-head kernel, %d ranges" % info["chunks"])
    ref = pa_decode_cabi(binding, stream, q, kc, None, tables, ctx, scale, mla_dv=512,
                         kernel=binding.ATBMI_PA_KERNEL_SCALAR)
    assert_close(got, ref.float().cpu().numpy(), TOL[dtype], "128-head kernel vs scalar kernel")
    for rep in range(3):  # same answer on relaunch: the tile buffers and the id table carry nothing over
        again = pa_decode_cabi(binding, stream, q, kc, None, tables, ctx, scale, mla_dv=512,
                               kernel=binding.ATBMI_PA_KERNEL_MFMA, chunk_tokens=chunk)
        assert torch.equal(again, got), "relaunch %d differs" % rep


# heads, block, ctx, mask row length, dtype, mask layout, ranges   (the 128-head kernel's masked build)
MLA_WIDE_MASKED = [
    (128, 128, [700, 45, 1, 2049], 2050, torch.bfloat16, "norm3", None),
    (16, 128, [333, 1000, 31], 1000, torch.float16, "norm3", None),        # rows as long as the longest context
    (40, 64, [515, 129, 2048, 4], 2048, torch.bfloat16, "norm3", 64),      # rows cut everywhere
    (32, 16, [3000, 5], 3002, torch.float16, "norm2", None),               # one row shared by all sequences
    (128, 128, [257, 130], 1026, torch.float16, "hidden", None),           # -inf over whole tiles and whole rows
]


@pytest.mark.parametrize("case", MLA_WIDE_MASKED, ids=lambda c: "h%d_bs%d_%s_%s" % (
    c[0], c[1], str(c[4]).split(".")[-1], c[5]))
def test_paged_attention_mla_128_head_kernel_with_a_mask(binding, oracle, dev, stream, case):
    """The combined-cache kernel with a mask row per sequence: against the oracle and against the fp32 scalar kernel."""
    heads, block, ctx, max_len, dtype, kind, chunk = case
    rng = _rng(400 + heads + block)
    q, kc, _, tables, ctx = _pa_inputs(rng, dev, len(ctx), heads, 1, block, 576, 512, ctx, dtype, std=0.5)
    if kind == "hidden":
        m = rng.standard_normal((len(ctx), 1, max_len)).astype(np.float32)
        m[0, 0, :64] = -np.inf        # the first two tiles of the first sequence
        m[0, 0, 100:131] = -np.inf
        m[1, 0, :] = -np.inf          # all of the second sequence: its rows come out as zeros
        mask = torch.from_numpy(m).to(dtype).to(dev).contiguous()
    else:
        mask, _ = _mask_tensor(oracle, rng, dev, kind, ctx, heads, max_len, dtype)
    scale = 1.0 / math.sqrt(576)
    with np.errstate(invalid="ignore"):
        want = oracle_pa(oracle, q, kc, None, tables, ctx, scale, mla_dv=512, mask=mask)
    if kind == "hidden":
        want[1] = 0.0  # (the oracle's softmax of a row of -inf is not a number; the kernels write zeros)
    got, info = pa_decode_cabi(binding, stream, q, kc, None, tables, ctx, scale, mla_dv=512, mask=mask,
                               kernel=binding.ATBMI_PA_KERNEL_MFMA, chunk_tokens=chunk, return_plan_info=True)
    assert_close(got, want, TOL[dtype], "128-head kernel with a mask, %d ranges" % info["chunks"])
    ref = pa_decode_cabi(binding, stream, q, kc, None, tables, ctx, scale, mla_dv=512, mask=mask,
                         kernel=binding.ATBMI_PA_KERNEL_SCALAR)
    assert_close(got, ref.float().cpu().numpy(), TOL[dtype], "128-head kernel with a mask vs scalar kernel")


def test_mla_through_operation_api_and_split_head_sizes(binding, oracle, dev, stream):
    rng = _rng(61)
    c = binding.Context(stream)
    # combined cache: 4 inputs, output width mlaVHeadSize
    q, kc, _, tables, ctx = _pa_inputs(rng, dev, 5, 16, 1, 128, 576, 512, [300, 1, 129, 128, 640], torch.bfloat16,
                                       std=0.5)
    scale = 1.0 / math.sqrt(192)
    pa = binding.OperationRunner("PagedAttentionOperation", binding.PagedAttentionParam(
        headNum=16, kvHeadNum=1, qkScale=scale, mlaVHeadSize=512), c)
    lens = torch.from_numpy(ctx)
    with torch.cuda.stream(stream):
        out, = pa.run([q, kc, tables, lens.to(dev)], host_inputs={3: lens})
    stream.synchronize()
    assert tuple(out.shape) == (5, 16, 512)
    assert_close(out, oracle_pa(oracle, q, kc, None, tables, ctx, scale, mla_dv=512), 2e-2, "mla api")
    pa.close()
    # separate caches with different K and V head sizes (reference CSV row "MLA": 128 / 96)
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, 4, 32, 16, 64, 128, 96, [64, 500, 33, 1000], torch.float16)
    pa = binding.OperationRunner("PagedAttentionOperation", binding.PagedAttentionParam(
        headNum=32, kvHeadNum=16, qkScale=0.088), c)
    lens = torch.from_numpy(ctx)
    with torch.cuda.stream(stream):
        out, = pa.run([q, kc, vc, tables, lens.to(dev)], host_inputs={4: lens})
    stream.synchronize()
    assert tuple(out.shape) == (4, 32, 96)
    assert_close(out, oracle_pa(oracle, q, kc, vc, tables, ctx, 0.088), 1e-3, "dk!=dv")
    pa.close()
    c.close()


# ------------------------------------------------------------------ masks, logN, dynamic batch
def _mask_tensor(oracle, rng, dev, kind, ctx, heads, max_len, dtype):
    """A decode mask of the given layout in q's dtype, plus whether a 3-dim one is per head.
    NORM masks hide the first i positions of sequence i with -10000 like the reference
    tests do (test_paged_attention_common.py:501-505) and carry small random values
    elsewhere, so that a wrong row or column shows; ALIBI masks are the reference's
    slope * distance rows (:489-499)."""
    batch = len(ctx)
    if kind == "norm2":
        m = rng.standard_normal((1, max_len)).astype(np.float32)
        m[0, :2] = -10000.0
    elif kind == "norm3":
        m = oracle.norm_mask(batch, max_len) + rng.standard_normal((batch, 1, max_len)).astype(np.float32)
        for i, n in enumerate(ctx):  # never hide a whole sequence
            m[i, 0, max(int(n) - 1, 0)] = 0.0
    elif kind == "alibi4":
        m = oracle.alibi_mask(ctx, heads, max_len)
    elif kind == "alibi4_1":
        m = oracle.alibi_mask(ctx, heads, max_len)[:, 3:4].copy()
    elif kind == "alibi3":
        m = oracle.alibi_mask([max_len], heads, max_len)[0]
    else:
        raise ValueError(kind)
    return torch.from_numpy(m).to(dtype).to(dev).contiguous(), kind == "alibi3"


# layout, batch, heads, kv_heads, block, d, ctx, mask row length, dtype, logN, int8 cache
# (reference test_paged_attention_common.py:725-1100: logN, alibi multi batch, norm mask with
#  long / small / ragged lengths; CSV rows PagedAttentionDequantNorm / DequantAlibi)
MASK_MATRIX = [
    ("norm3", 4, 32, 32, 128, 128, 15, 15, torch.float16, False, False),
    ("norm3", 6, 32, 32, 128, 128, 200, 256, torch.float16, False, False),
    ("norm3", 3, 40, 40, 128, 128, [30000, 77, 4099], 30001, torch.bfloat16, False, False),
    ("norm2", 5, 8, 2, 16, 128, [33, 900, 64, 1, 3000], 3000, torch.float16, False, False),
    ("alibi4", 2, 32, 32, 128, 128, 500, 500, torch.bfloat16, False, False),
    ("alibi4", 7, 30, 2, 128, 128, [88, 1500, 3, 128, 129, 640, 2000], 2002, torch.float16, True, False),
    ("alibi4_1", 4, 16, 4, 64, 96, [100, 2000, 64, 777], 2048, torch.float16, False, False),
    ("alibi3", 5, 32, 8, 128, 128, [819, 12, 4000, 256, 300], 4000, torch.float16, False, False),
    (None, 30, 32, 32, 128, 128, 69, 0, torch.bfloat16, True, False),
    ("norm3", 30, 32, 32, 128, 128, 69, 72, torch.bfloat16, True, False),
    ("norm3", 8, 64, 8, 128, 128, 1200, 1200, torch.float16, False, True),
    ("alibi4", 4, 32, 16, 64, 128, [100, 2000, 64, 777], 2000, torch.float16, False, True),
    ("norm3", 3, 24, 1, 16, 256, [3000, 5, 12000], 12000, torch.float16, False, False),
    # reference test_paged_attention_common.py:2660-2671 (bf16, ALiBi mask, 32 768 tokens, split over many ranges);
    # three of its twelve sequences, one of them at the full length
    ("alibi4", 3, 12, 1, 128, 128, [32768, 2049, 700], 32768, torch.bfloat16, False, False),
]


@pytest.mark.parametrize("case", MASK_MATRIX, ids=lambda c: "%s_b%d_h%d_g%d_d%d_%s%s%s" % (
    c[0], c[1], c[2], c[3], c[5], str(c[8]).split(".")[-1], "_logn" if c[9] else "", "_int8" if c[10] else ""))
def test_paged_attention_masks_and_logn(binding, oracle, dev, stream, case):
    kind, batch, heads, kv_heads, block, d, ctx, max_len, dtype, with_logn, kv_int8 = case
    rng = _rng(200 + batch + heads)
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, batch, heads, kv_heads, block, d, d, ctx, dtype, kv_int8=kv_int8)
    mask, per_head = (None, False) if kind is None else _mask_tensor(oracle, rng, dev, kind, ctx, heads, max_len, dtype)
    logn = torch.from_numpy(rng.uniform(1, 2, size=batch).astype(np.float32)).to(dev) if with_logn else None
    ks = ko = vs = vo = None
    if kv_int8:
        ks = torch.from_numpy(rng.uniform(0.05, 0.5, size=kv_heads * d).astype(np.float32)).to(dev)
        vs = torch.from_numpy(rng.uniform(0.05, 0.5, size=kv_heads * d).astype(np.float32)).to(dev)
    scale = 1.0 / math.sqrt(d)
    want = oracle_pa(oracle, q, kc, vc, tables, ctx, scale, ks, ko, vs, vo, mask=mask, mask_per_head=per_head,
                     logn=logn)
    plain = oracle_pa(oracle, q, kc, vc, tables, ctx, scale, ks, ko, vs, vo)
    assert np.abs(want - plain).max() > 0.01  # the mask / logN matters in this case
    tol = INT8_TOL if kv_int8 else TOL[dtype]
    for kernel in _kernels_for(binding, d, d, block):
        got = pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx, scale, ks, ko, vs, vo, kernel=kernel,
                             mask=mask, mask_per_head=per_head, logn=logn)
        assert_close(got, want, tol, "kernel=%d" % kernel)


@pytest.mark.parametrize("kernel", [1, 0])
def test_mask_rows_follow_the_sequence_index_past_empty_sequences(binding, oracle, dev, stream, kernel):
    """Empty sequences take no query row, but mask and logN rows stay indexed by
    the position in contextLens (reference test_paged_attention_common.py:311-358)."""
    rng = _rng(231)
    heads, kv_heads, d, block = 16, 4, 128, 16
    ctx = np.array([0, 37, 1, 0, 400, 16, 0], dtype=np.int32)
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, len(ctx), heads, kv_heads, block, d, d, ctx, torch.float16)
    mask, _ = _mask_tensor(oracle, rng, dev, "alibi4", ctx, heads, 401, torch.float16)
    mask += torch.from_numpy(rng.standard_normal((len(ctx), 1, 1, 401)).astype(np.float32)).to(dev).half()
    logn = torch.from_numpy(rng.uniform(1, 2, size=len(ctx)).astype(np.float32)).to(dev)
    scale = 1.0 / math.sqrt(d)
    out = torch.full((len(ctx), heads, d), 0.1, dtype=torch.float16, device=dev)
    got = pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx, scale, kernel=kernel, out=out, mask=mask, logn=logn)
    want = oracle_pa(oracle, q, kc, vc, tables, ctx, scale, out_init=0.1, mask=mask, logn=logn)
    assert_close(got, want, 1e-3, "empty+mask")


def test_four_dim_norm_mask_reads_its_first_row(binding, oracle, dev, stream):
    """MASK_TYPE_NORM with a (batch, heads, 1, maxS) mask through the operation: the reference lets the shape through
    (kernel library paged_attention_operation.cpp:760) while its tiling derives strides for the 2- and 3-dim NORM
    masks only (tiling/paged_attention_tiling.cpp:62-74), so both strides stay 0 and every sequence and head reads
    the tensor's first row. The result must equal the oracle with that row as a (1, maxS) mask, and differ from the
    reading by sequence and head."""
    rng = _rng(233)
    heads, kv_heads, d, block, dtype = 8, 2, 128, 16, torch.float16
    ctx = np.array([300, 17, 0, 129], dtype=np.int32)
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, len(ctx), heads, kv_heads, block, d, d, ctx, dtype)
    mask = torch.from_numpy((rng.standard_normal((len(ctx), heads, 1, 304)) * 2).astype(np.float32)).to(dtype).to(dev)
    scale = 1.0 / math.sqrt(d)
    lens = torch.from_numpy(ctx)
    c = binding.Context(stream)
    op = binding.OperationRunner("PagedAttentionOperation", binding.PagedAttentionParam(
        headNum=heads, kvHeadNum=kv_heads, qkScale=scale, maskType=1), c)
    with torch.cuda.stream(stream):
        out = torch.full((len(ctx), heads, d), 0.1, dtype=dtype, device=dev)
        op.run([q, kc, vc, tables, lens.to(dev), mask], outputs=[out], host_inputs={4: lens})
    stream.synchronize()
    first_row = oracle_pa(oracle, q, kc, vc, tables, ctx, scale, out_init=0.1, mask=mask[0, 0].reshape(1, -1))
    by_index = oracle_pa(oracle, q, kc, vc, tables, ctx, scale, out_init=0.1, mask=mask)
    assert np.abs(first_row - by_index).max() > 0.01
    assert_close(out, first_row, TOL[dtype], "4-dim NORM mask")
    op.close()
    c.close()


@pytest.mark.parametrize("kernel", [1, 0])
@pytest.mark.parametrize("chunk", [64, 1024])
def test_minus_infinity_mask_hides_whole_ranges(binding, oracle, dev, stream, kernel, chunk):
    """A bf16 mask of -inf over the first 300 positions: ranges of the split that
    lie wholly inside it contribute nothing, and the result is the attention over
    the rest."""
    rng = _rng(232)
    heads, kv_heads, d, block = 8, 2, 128, 16
    ctx = [1000, 301, 640]
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, 3, heads, kv_heads, block, d, d, ctx, torch.bfloat16)
    m = np.zeros((3, 1, 1000), np.float32)
    m[:, :, :300] = -np.inf
    mask = torch.from_numpy(m).to(torch.bfloat16).to(dev)
    scale = 1.0 / math.sqrt(d)
    got = pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx, scale, kernel=kernel, chunk_tokens=chunk, mask=mask)
    want = oracle_pa(oracle, q, kc, vc, tables, ctx, scale, mask=mask, mask_per_head=False)
    assert_close(got, want, TOL[torch.bfloat16], "-inf mask")


def test_mla_with_norm_mask(binding, oracle, dev, stream):
    """The combined-cache variant takes a NORM mask (not ALIBI, not logN) in the
    reference; 128 heads, so the kernel choice with and without mask differs."""
    rng = _rng(233)
    batch, heads, d, dv, block = 3, 128, 576, 512, 128
    ctx = np.array([700, 33, 1500], dtype=np.int32)
    q, kc, _, tables, ctx = _pa_inputs(rng, dev, batch, heads, 1, block, d, d, ctx, torch.bfloat16, std=0.5)
    mask, _ = _mask_tensor(oracle, rng, dev, "norm3", ctx, heads, 1500, torch.bfloat16)
    want = oracle_pa(oracle, q, kc, None, tables, ctx, 0.05, mla_dv=dv, mask=mask, mask_per_head=False)
    for kernel in (binding.ATBMI_PA_KERNEL_SCALAR, binding.ATBMI_PA_KERNEL_AUTO):
        got = pa_decode_cabi(binding, stream, q, kc, None, tables, ctx, 0.05, mla_dv=dv, kernel=kernel, mask=mask)
        assert_close(got, want, TOL[torch.bfloat16], "mla mask kernel=%d" % kernel)


def test_masks_logn_and_dynamic_batch_through_operation_api(binding, oracle, dev, stream):
    """Input order of the operation: q, caches, tables, lens, mask, batchRunStatus, ..., logN
    (reference paged_attention_operation.cpp:408-444). With a dynamic batch the
    query holds one row per running sequence only."""
    rng = _rng(234)
    heads, kv_heads, d, block = 32, 16, 128, 64
    ctx = np.array([100, 0, 2000, 64, 0, 777], dtype=np.int32)
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, len(ctx), heads, kv_heads, block, d, d, ctx, torch.float16)
    q = q[:4].contiguous()
    status = torch.from_numpy((ctx > 0).astype(np.int32))
    lens = torch.from_numpy(ctx)
    logn = torch.from_numpy(rng.uniform(1, 2, size=len(ctx)).astype(np.float32)).to(dev)
    scale = 1.0 / math.sqrt(d)
    c = binding.Context(stream)
    for kind, mask_type in (("norm3", 1), ("alibi4", 2), ("alibi3", 2)):
        mask, per_head = _mask_tensor(oracle, rng, dev, kind, ctx, heads, 2048, torch.float16)
        pa = binding.OperationRunner("PagedAttentionOperation", binding.PagedAttentionParam(
            headNum=heads, kvHeadNum=kv_heads, qkScale=scale, maskType=mask_type, batchRunStatusEnable=True,
            scaleType=1), c)
        with torch.cuda.stream(stream):
            out, = pa.run([q, kc, vc, tables, lens.to(dev), mask, status.to(dev), logn],
                          host_inputs={4: lens, 6: status})
        stream.synchronize()
        assert tuple(out.shape) == (4, heads, d)
        want = oracle_pa(oracle, q, kc, vc, tables, ctx, scale, mask=mask, mask_per_head=per_head, logn=logn)
        assert_close(out, want, 1e-3, kind)
        pa.close()
    # int8 cache with offsets and a mask: the descale tensors follow the mask
    q8, kc8, vc8, tables8, ctx8 = _pa_inputs(rng, dev, 4, heads, kv_heads, block, d, d, [100, 2000, 64, 777],
                                             torch.float16, kv_int8=True)
    ks = torch.from_numpy(rng.uniform(0.01, 0.1, size=kv_heads * d).astype(np.float32)).to(dev)
    vs = torch.from_numpy(rng.uniform(0.01, 0.1, size=kv_heads * d).astype(np.float32)).to(dev)
    ko = torch.from_numpy(rng.integers(-20, 20, size=kv_heads * d).astype(np.int32)).to(dev)
    vo = torch.from_numpy(rng.integers(-20, 20, size=kv_heads * d).astype(np.int32)).to(dev)
    mask, _ = _mask_tensor(oracle, rng, dev, "norm3", ctx8, heads, 2000, torch.float16)
    pa = binding.OperationRunner("PagedAttentionOperation", binding.PagedAttentionParam(
        headNum=heads, kvHeadNum=kv_heads, qkScale=scale, quantType=1, hasQuantOffset=True, maskType=1), c)
    lens8 = torch.from_numpy(ctx8)
    with torch.cuda.stream(stream):
        out, = pa.run([q8, kc8, vc8, tables8, lens8.to(dev), mask, ks, ko, vs, vo], host_inputs={4: lens8})
    stream.synchronize()
    assert_close(out, oracle_pa(oracle, q8, kc8, vc8, tables8, ctx8, scale, ks, ko, vs, vo, mask=mask,
                                mask_per_head=False), INT8_TOL, "dequant + mask")
    pa.close()
    c.close()


# ------------------------------------------------------------------ split latent layout, log-sum-exp output
# batch, heads, ctx, q_lens (None: one token each), dtype, chunk override
# (reference test_multi_latent_attention.py / _lse.py / _mtp.py: heads 8..128, block 128, 512 + 64 channels)
SPLIT_MATRIX = [
    (32, 32, 256, None, torch.float16, None),
    (4, 128, [3000, 17, 128, 1025], None, torch.bfloat16, None),
    (20, 128, 256, None, torch.float16, 64),
    (3, 128, [700, 0, 1500], [2, 3, 4], torch.bfloat16, None),
    (5, 8, [819, 12, 4000, 256, 300], None, torch.float16, None),
    (6, 64, 515, [1, 2, 1, 3, 1, 1], torch.bfloat16, None),
]


@pytest.mark.parametrize("case", SPLIT_MATRIX, ids=lambda c: "b%d_h%d_%s%s%s" % (
    c[0], c[1], str(c[4]).split(".")[-1], "_multi" if c[3] else "", "_chunk%d" % c[5] if c[5] else ""))
def test_split_latent_layout_and_lse(binding, oracle, dev, stream, case):
    """Query and cache rows given as 512 + 64 channels in two tensors each give bit-for-bit what the
    576-channel rows give (same kernels, two sources), and both match the oracle; the log-sum-exp
    output matches the oracle's within the output tolerance."""
    batch, heads, ctx, q_lens, dtype, chunk = case
    rng = _rng(400 + batch + heads)
    d, dv, block = 576, 512, 128
    _, kc, _, tables, ctx = _pa_inputs(rng, dev, batch, heads, 1, block, d, d, ctx, dtype, std=0.5)
    rows = int(sum((1 if q_lens is None else q_lens[i]) for i in range(batch) if ctx[i] > 0))
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(rng.integers(1 << 30)))
    q = (torch.rand((rows, heads, d), generator=gen) * 2 - 1).to(dtype).to(dev)
    q_nope, q_rope = q[..., :dv].contiguous(), q[..., dv:].contiguous()
    k_nope, k_rope = kc[..., :dv].contiguous(), kc[..., dv:].contiguous()
    scale = 1.0 / math.sqrt(192.0)
    want_lse = np.zeros((rows, heads), np.float32)
    want = oracle_pa(oracle, q, kc, None, tables, ctx, scale, mla_dv=dv, q_lens=q_lens, lse_out=want_lse)
    for kernel in (binding.ATBMI_PA_KERNEL_SCALAR, binding.ATBMI_PA_KERNEL_AUTO):
        lse = torch.zeros((rows, heads), dtype=dtype, device=dev)
        got = pa_decode_cabi(binding, stream, q_nope, k_nope, None, tables, ctx, scale, mla_dv=dv, kernel=kernel,
                             q_lens=q_lens, q_rope=q_rope, k_rope=k_rope, lse=lse, chunk_tokens=chunk)
        assert_close(got, want, TOL[dtype], "split kernel=%d" % kernel)
        assert_close(lse, want_lse, TOL[dtype], "lse kernel=%d" % kernel)
        lse2 = torch.zeros_like(lse)
        combined = pa_decode_cabi(binding, stream, q, kc, None, tables, ctx, scale, mla_dv=dv, kernel=kernel,
                                  q_lens=q_lens, lse=lse2, chunk_tokens=chunk)
        assert torch.equal(got, combined) and torch.equal(lse, lse2)
        # the same caches in the fractal-NZ layout [blocks, channels / 16, block, 16]: other addresses, same values
        nz_nope = torch.from_numpy(oracle.nd_to_nz(k_nope.view(torch.int16).cpu().numpy()[:, :, 0, :])).to(dev).view(dtype)
        nz_rope = torch.from_numpy(oracle.nd_to_nz(k_rope.view(torch.int16).cpu().numpy()[:, :, 0, :])).to(dev).view(dtype)
        assert tuple(nz_nope.shape) == (kc.shape[0], 32, block, 16) and tuple(nz_rope.shape) == (kc.shape[0], 4, block, 16)
        lse3 = torch.zeros_like(lse)
        from_nz = pa_decode_cabi(binding, stream, q_nope, nz_nope, None, tables, ctx, scale, mla_dv=dv, kernel=kernel,
                                 q_lens=q_lens, q_rope=q_rope, k_rope=nz_rope, lse=lse3, chunk_tokens=chunk,
                                 fractal_nz=True)
        assert torch.equal(got, from_nz) and torch.equal(lse, lse3), "fractal-NZ caches, kernel=%d" % kernel


@pytest.mark.parametrize("heads,dtype", [(128, torch.bfloat16), (32, torch.float16), (8, torch.float16)])
def test_multi_latent_attention_operation(binding, oracle, dev, stream, heads, dtype):
    """MultiLatentAttentionOperation, cacheMode KROPE_CTKV, through Setup / Execute: plain decode, with
    the log-sum-exp output (CALC_TYPE_RING), several query tokens with the SPEC mask (CALC_TYPE_SPEC) and
    both (CALC_TYPE_SPEC_AND_RING). Inputs: query, queryRope, kvCache, kvCacheRope, blockTables,
    contextLens, [mask], [qSeqlen] (reference multi_latent_attention_operation.cpp:245-266). With 128 heads the
    reference runs a job per query token over the context up to that token and does not read the mask
    (tiling/mla_tiling.cpp:139-144, mla_tiling_dependency.cpp:292-316): the oracle then takes causal rows and no
    mask, although the (randomly biased) mask tensor is handed over."""
    rng = _rng(440 + heads)
    d, dv, block = 576, 512, 128
    ctx = np.array([700, 33, 1500, 128], dtype=np.int32)
    _, kc, _, tables, ctx = _pa_inputs(rng, dev, 4, heads, 1, block, d, d, ctx, dtype, std=0.5)
    k_nope, k_rope = kc[..., :dv].contiguous(), kc[..., dv:].contiguous()
    q_lens = np.array([2, 1, 3, 1], dtype=np.int32)
    scale = 1.0 / math.sqrt(192.0)
    lens, qn = torch.from_numpy(ctx), torch.from_numpy(q_lens)
    c = binding.Context(stream)
    for calc in (0, 2, 1, 3):
        multi, ring = calc in (1, 3), calc in (2, 3)
        rows = int(q_lens.sum()) if multi else 4
        q = (torch.rand((rows, heads, d)) * 2 - 1).to(dtype).to(dev)
        ins = [q[..., :dv].contiguous(), q[..., dv:].contiguous(), k_nope, k_rope, tables, lens.to(dev)]
        host = {5: lens}
        mask = None
        if multi:
            mask = _spec_mask(rng, dev, "query", ctx, q_lens, dtype)
            ins += [mask, qn.to(dev)]
            host[7] = qn
        op = binding.OperationRunner("MultiLatentAttentionOperation", binding.MultiLatentAttentionParam(
            headNum=heads, kvHeadNum=1, qkScale=scale, cacheMode=1, calcType=calc, maskType=1 if multi else 0), c)
        with torch.cuda.stream(stream):
            outs = op.run(ins, host_inputs=host)
        stream.synchronize()
        assert len(outs) == (2 if ring else 1) and tuple(outs[0].shape) == (rows, heads, dv)
        want_lse = np.zeros((rows, heads), np.float32)
        per_token = multi and heads == 128
        want = oracle_pa(oracle, q, kc, None, tables, ctx, scale, mla_dv=dv, mask=None if per_token else mask,
                         q_lens=q_lens if multi else None, mask_rows="query" if multi else "sequence",
                         lse_out=want_lse, causal_rows=True if per_token else None)
        assert_close(outs[0], want, TOL[dtype], "calcType %d" % calc)
        if ring:
            assert tuple(outs[1].shape) == (rows, heads, 1) and outs[1].dtype == dtype
            assert_close(outs[1][..., 0], want_lse, TOL[dtype], "lse calcType %d" % calc)
        op.close()
        # cacheMode NZCACHE: the caches as [blocks, channels / 16, 128, 16] in the fractal-NZ format
        # (reference test_multi_latent_attention_int8nz.py:633-636,767-797)
        nz = [torch.from_numpy(oracle.nd_to_nz(t.view(torch.int16).cpu().numpy()[:, :, 0, :])).to(dev).view(dtype)
              for t in (k_nope, k_rope)]
        ins[2:4] = [binding.make_tensor(binding._torch_acl_dtype(t), list(t.shape), device_ptr=t.data_ptr(),
                                        fmt="fractal_nz") for t in nz]
        op = binding.OperationRunner("MultiLatentAttentionOperation", binding.MultiLatentAttentionParam(
            headNum=heads, kvHeadNum=1, qkScale=scale, cacheMode=3, calcType=calc, maskType=1 if multi else 0), c)
        with torch.cuda.stream(stream):
            outs_nz = op.run(ins, host_inputs=host)
        stream.synchronize()
        assert len(outs_nz) == len(outs) and all(torch.equal(a, b) for a, b in zip(outs, outs_nz)), "NZCACHE %d" % calc
        op.close()
    c.close()


@pytest.mark.parametrize("heads", [128, 32])
def test_multi_latent_attention_empty_context_keeps_its_rows(binding, oracle, dev, stream, heads):
    """A sequence without context in the middle of a batch with several query tokens: its query rows stay its own
    (nothing is written to their outputs) and the rows of the sequences behind it do not move up, as the reference's
    tiling lays them out (tiling/mla_tiling.cpp:146-149: beginQ moves on by qSeqLen whatever kvSeqLen is). With the
    SPEC mask on 32 heads (one mask row per query row, the empty sequence's included) and on the job-per-token path of
    128 heads, both with the log-sum-exp output."""
    rng = _rng(470 + heads)
    d, dv, block, dtype = 576, 512, 128, torch.float16
    ctx = np.array([700, 0, 300, 0], dtype=np.int32)
    q_lens = np.array([2, 3, 1, 2], dtype=np.int32)
    rows = int(q_lens.sum())
    _, kc, _, tables, _ = _pa_inputs(rng, dev, 4, heads, 1, block, d, d, np.maximum(ctx, 1), dtype, std=0.5)
    k_nope, k_rope = kc[..., :dv].contiguous(), kc[..., dv:].contiguous()
    scale = 1.0 / math.sqrt(192.0)
    lens, qn = torch.from_numpy(ctx), torch.from_numpy(q_lens)
    q = (torch.rand((rows, heads, d)) * 2 - 1).to(dtype).to(dev)
    mask = torch.from_numpy(np.where(np.arange(700)[None, :] < 690, rng.standard_normal((rows, 700)), -10000.0)
                            .astype(np.float32)).to(dtype).to(dev)
    c = binding.Context(stream)
    op = binding.OperationRunner("MultiLatentAttentionOperation", binding.MultiLatentAttentionParam(
        headNum=heads, kvHeadNum=1, qkScale=scale, cacheMode=1, calcType=3, maskType=1), c)
    out = torch.full((rows, heads, dv), 0.25, dtype=dtype, device=dev)
    lse = torch.full((rows, heads, 1), 7.0, dtype=dtype, device=dev)
    with torch.cuda.stream(stream):
        op.run([q[..., :dv].contiguous(), q[..., dv:].contiguous(), k_nope, k_rope, tables, lens.to(dev), mask, qn.to(dev)],
               outputs=[out, lse], host_inputs={5: lens, 7: qn})
    stream.synchronize()
    per_token = heads == 128
    want_lse = np.full((rows, heads), 7.0, np.float32)
    want = oracle_pa(oracle, q, kc, None, tables, ctx, scale, mla_dv=dv, mask=None if per_token else mask, q_lens=q_lens,
                     mask_rows="query", lse_out=want_lse, causal_rows=True if per_token else None, out_init=0.25,
                     empty_keep_rows=True)
    assert_close(out, want, TOL[dtype], "empty context in the middle, %d heads" % heads)
    assert_close(lse[..., 0], want_lse, TOL[dtype], "its log-sum-exp")
    assert torch.all(out[2:5] == 0.25) and torch.all(out[6:] == 0.25) and torch.all(lse[2:5] == 7.0)
    op.close()
    c.close()


@pytest.mark.parametrize("kernel", [1, 2])
def test_causal_rows_through_the_c_abi(binding, oracle, dev, stream, kernel):
    """atbmi_pa_plan_set_causal_rows: the t-th of n query rows attends to the first ctx - n + t + 1 tokens, per
    sequence when flags are given; on the generic kernels (GQA, where query tokens would otherwise share a pass)
    and on the MLA kernels (16 and 128 heads), whole rows and rows cut into ranges."""
    rng = _rng(480 + kernel)
    for heads, kv_heads, d, dv, ctx, q_lens, flags, dtype, chunk in (
            (32, 8, 128, 0, [1000, 0, 2300, 130, 4], [2, 3, 4, 1, 4], None, torch.bfloat16, None),
            (32, 8, 128, 0, [1000, 0, 2300, 130, 4], [2, 3, 4, 1, 4], [1, 1, 0, 1, 0], torch.float16, 256),
            (16, 1, 576, 512, [300, 1200], [2, 4], None, torch.float16, None),
            (128, 1, 576, 512, [700, 33, 1500], [2, 1, 3], [0, 1, 1], torch.bfloat16, None)):
        q_lens_np = np.asarray(q_lens, np.int32)
        _, kc, vc, tables, ctx = _pa_inputs(rng, dev, len(ctx), heads, kv_heads, 128, d, dv or d, ctx, dtype, std=0.5)
        rows = int(sum(n for n, c in zip(q_lens, ctx) if c > 0))
        q = (torch.rand((rows, heads, d)) * 2 - 1).to(dtype).to(dev)
        scale = 1.0 / math.sqrt(d)
        lse = torch.zeros((rows, heads), dtype=dtype, device=dev)
        got = pa_decode_cabi(binding, stream, q, kc, None if dv else vc, tables, ctx, scale, mla_dv=dv, kernel=kernel,
                             q_lens=q_lens_np, lse=lse, chunk_tokens=chunk,
                             causal_rows=True if flags is None else flags)
        want_lse = np.zeros((rows, heads), np.float32)
        want = oracle_pa(oracle, q, kc, None if dv else vc, tables, ctx, scale, mla_dv=dv, q_lens=q_lens_np,
                         lse_out=want_lse, causal_rows=True if flags is None else flags)
        assert_close(got, want, TOL[dtype], "causal rows heads=%d kernel=%d" % (heads, kernel))
        assert_close(lse, want_lse, TOL[dtype], "causal rows lse heads=%d kernel=%d" % (heads, kernel))


def test_multi_latent_attention_causal_mask_types(binding, oracle, dev, stream):
    """MultiLatentAttentionOperation with several query tokens and no mask tensor to read: MASK_TYPE_CAUSAL_MASK (any
    head count), MASK_TYPE_MASK_FREE on 128 heads with maskUseStatus flags per sequence (reference golden
    test_multi_latent_attention_mtp.py:160-180,582-633: the look-ahead rows, or the whole context where the flag
    is 0), and 128 heads with no mask type at all (the reference's job per query token)."""
    rng = _rng(490)
    d, dv, block, dtype = 576, 512, 128, torch.float16
    ctx = np.array([700, 33, 1500, 128], dtype=np.int32)
    q_lens = np.array([2, 1, 3, 2], dtype=np.int32)
    rows = int(q_lens.sum())
    scale = 1.0 / math.sqrt(192.0)
    lens, qn = torch.from_numpy(ctx), torch.from_numpy(q_lens)
    c = binding.Context(stream)
    for heads, calc, mask_type, flags in ((32, 1, 3, None), (128, 3, 2, [1, 0, 1, 1]), (128, 3, 2, None),
                                          (128, 1, 0, None)):
        _, kc, _, tables, _ = _pa_inputs(rng, dev, 4, heads, 1, block, d, d, ctx, dtype, std=0.5)
        k_nope, k_rope = kc[..., :dv].contiguous(), kc[..., dv:].contiguous()
        q = (torch.rand((rows, heads, d)) * 2 - 1).to(dtype).to(dev)
        ins = [q[..., :dv].contiguous(), q[..., dv:].contiguous(), k_nope, k_rope, tables, lens.to(dev)]
        host = {5: lens}
        if mask_type == 2:   # the template of the reference's mask-free tests ([125 + 2 q, 128]); not read on this path
            ins.append(torch.from_numpy(np.triu(np.full((131, 128), -10000.0, np.float32), -1)).to(dtype).to(dev))
        host[len(ins)] = qn
        ins.append(qn.to(dev))
        if flags is not None:
            host[len(ins)] = torch.tensor(flags, dtype=torch.int32)
            ins.append(host[len(ins)].to(dev))
        op = binding.OperationRunner("MultiLatentAttentionOperation", binding.MultiLatentAttentionParam(
            headNum=heads, kvHeadNum=1, qkScale=scale, cacheMode=1, calcType=calc, maskType=mask_type,
            maskUseStatusType=0 if flags is None else 1), c)
        with torch.cuda.stream(stream):
            outs = op.run(ins, host_inputs=host)
        stream.synchronize()
        want_lse = np.zeros((rows, heads), np.float32)
        want = oracle_pa(oracle, q, kc, None, tables, ctx, scale, mla_dv=dv, q_lens=q_lens, lse_out=want_lse,
                         causal_rows=True if flags is None else flags)
        assert_close(outs[0], want, TOL[dtype], "heads %d calcType %d maskType %d" % (heads, calc, mask_type))
        if calc == 3:
            assert_close(outs[1][..., 0], want_lse, TOL[dtype], "lse heads %d" % heads)
        op.close()
    c.close()


def test_mask_free_template_expansion_and_operation(binding, oracle, dev, stream):
    """MASK_TYPE_MASK_FREE with fewer than 128 heads: atbmi_mla_mask_free_expand reproduces the oracle's reading of the
    template bit for bit (the reference's template, a random one, one per sequence; contexts that end early in a
    128-token tile, so that the triangle reaches into the tile before), and MultiLatentAttentionOperation run on it
    equals the oracle with those mask rows."""
    import ctypes
    k = binding.kernels()
    rng = _rng(495)
    ctx = np.array([700, 33, 1500, 128, 129, 258, 0, 5], dtype=np.int32)
    q_lens = np.array([2, 1, 3, 2, 4, 4, 2, 5], dtype=np.int32)
    rows = int(q_lens.sum())   # (the sequence without context keeps its two rows: zeros)
    mask_len = 1504
    for dtype in (torch.float16, torch.bfloat16):
        standard = np.triu(np.full((125 + 2 * 5, 128), -10000.0, np.float32), 2 - 5)
        random = (rng.standard_normal((135, 128)) * 3).astype(np.float32)
        per_seq = np.stack([standard if b % 2 == 0 else random for b in range(len(ctx))])
        for template in (standard, random, per_seq):
            tmpl = torch.from_numpy(template).to(dtype).to(dev)
            call = binding.AtbmiMlaMaskFreeCall(
                batch=len(ctx), numQueryRows=rows, templateBatch=len(ctx) if template.ndim == 3 else 0,
                templateRows=template.shape[-2], maskLen=mask_len, hostContextLens=ctx.ctypes.data,
                hostQueryLens=q_lens.ctypes.data)
            ws_bytes = ctypes.c_uint64(0)
            assert k.atbmi_mla_mask_free_workspace_size(ctypes.byref(call), ctypes.byref(ws_bytes)) == 0
            assert ws_bytes.value == rows * 16
            with torch.cuda.stream(stream):
                ws = torch.empty(ws_bytes.value, dtype=torch.uint8, device=dev)
                out = torch.full((rows, mask_len), 7.0, dtype=dtype, device=dev)
                call.maskTemplate, call.outMask = tmpl.data_ptr(), out.data_ptr()
                rc = k.atbmi_mla_mask_free_expand(ctypes.byref(call), ws.data_ptr(), ws_bytes.value, stream.cuda_stream)
                assert rc == 0, binding.last_kernel_error()
            stream.synchronize()
            want = oracle.mla_mask_free_rows(tmpl.float().cpu().numpy(), ctx, q_lens, mask_len)
            assert np.array_equal(out.float().cpu().numpy(), want)
    # a template without the rows a sequence reads is refused
    call = binding.AtbmiMlaMaskFreeCall(batch=len(ctx), numQueryRows=rows, templateBatch=0, templateRows=100, maskLen=mask_len,
                                        hostContextLens=ctx.ctypes.data, hostQueryLens=q_lens.ctypes.data)
    assert k.atbmi_mla_mask_free_workspace_size(ctypes.byref(call), ctypes.byref(ws_bytes)) != 0

    # through the operation: 32 and 16 heads, the reference's template and a template per sequence with one all-zero
    d, dv, block, dtype = 576, 512, 128, torch.float16
    ctx, q_lens = ctx[:6].copy(), np.full(6, 4, dtype=np.int32)   # (the reference's template is made for one q)
    rows = int(q_lens.sum())
    scale = 1.0 / math.sqrt(192.0)
    lens, qn = torch.from_numpy(ctx), torch.from_numpy(q_lens)
    c = binding.Context(stream)
    standard = np.triu(np.full((125 + 2 * 4, 128), -10000.0, np.float32), 2 - 4)
    per_seq = np.stack([standard if b != 2 else np.zeros_like(standard) for b in range(6)])
    for heads, calc, template in ((32, 1, standard), (16, 3, per_seq)):
        _, kc, _, tables, _ = _pa_inputs(rng, dev, 6, heads, 1, block, d, d, ctx, dtype, std=0.5)
        q = (torch.rand((rows, heads, d)) * 2 - 1).to(dtype).to(dev)
        tmpl = torch.from_numpy(template).to(dtype).to(dev)
        ins = [q[..., :dv].contiguous(), q[..., dv:].contiguous(), kc[..., :dv].contiguous(), kc[..., dv:].contiguous(),
               tables, lens.to(dev), tmpl, qn.to(dev)]
        op = binding.OperationRunner("MultiLatentAttentionOperation", binding.MultiLatentAttentionParam(
            headNum=heads, kvHeadNum=1, qkScale=scale, cacheMode=1, calcType=calc, maskType=2), c)
        with torch.cuda.stream(stream):
            outs = op.run(ins, host_inputs={5: lens, 7: qn})
        stream.synchronize()
        mask = torch.from_numpy(oracle.mla_mask_free_rows(tmpl.float().cpu().numpy(), ctx, q_lens, int(ctx.max())))
        want_lse = np.zeros((rows, heads), np.float32)
        want = oracle_pa(oracle, q, kc, None, tables, ctx, scale, mla_dv=dv, q_lens=q_lens, mask=mask, mask_rows="query",
                         lse_out=want_lse)
        assert_close(outs[0], want, TOL[dtype], "mask-free heads %d" % heads)
        if calc == 3:
            assert_close(outs[1][..., 0], want_lse, TOL[dtype], "mask-free lse heads %d" % heads)
        if template.ndim == 2:   # the reference's template is the causal rule
            causal = oracle_pa(oracle, q, kc, None, tables, ctx, scale, mla_dv=dv, q_lens=q_lens, causal_rows=True)
            assert_close(outs[0], causal, TOL[dtype], "mask-free equals causal rows, heads %d" % heads)
        op.close()
    c.close()


def test_two_call_c_wrappers_run_the_operations(binding, oracle, dev, stream):
    """AtbMLAGetWorkspaceSize + AtbMLA and AtbPagedCacheLoadGetWorkspaceSize + AtbPagedCacheLoad on
    aclTensor handles (reference include/atb/atb_acl.h:99-116,251-267): plain decode, the log-sum-exp
    output, several query tokens with the mask; results against the oracle."""
    import ctypes
    lib = binding.atb()
    rng = _rng(470)
    heads, d, dv, block, dtype = 128, 576, 512, 128, torch.bfloat16
    ctx_lens = np.array([700, 33, 1500, 128], dtype=np.int32)
    _, kc, _, tables, ctx_lens = _pa_inputs(rng, dev, 4, heads, 1, block, d, d, ctx_lens, dtype, std=0.5)
    k_nope, k_rope = kc[..., :dv].contiguous(), kc[..., dv:].contiguous()
    q_lens = np.array([2, 1, 3, 1], dtype=np.int32)
    scale = 1.0 / math.sqrt(192.0)
    lens_host, qn_host = torch.from_numpy(ctx_lens), torch.from_numpy(q_lens)
    c = binding.Context(stream)
    A = binding.acl_tensor_of
    for calc in (0, 2, 1):
        multi, ring = calc == 1, calc == 2
        rows = int(q_lens.sum()) if multi else 4
        with torch.cuda.stream(stream):
            q = (torch.rand((rows, heads, d)) * 2 - 1).to(dtype).to(dev)
            qn_, qr_ = q[..., :dv].contiguous(), q[..., dv:].contiguous()
            out = torch.zeros((rows, heads, dv), dtype=dtype, device=dev)
            lse = torch.zeros((rows, heads, 1), dtype=dtype, device=dev)
            mask = _spec_mask(rng, dev, "query", ctx_lens, q_lens, dtype) if multi else None
        stream.synchronize()
        handles = [A(qn_), A(qr_), A(k_nope), A(k_rope), A(tables), A(lens_host), A(mask) if multi else None,
                   A(qn_host) if multi else None, A(out), A(lse) if ring else None]
        ws, op = ctypes.c_uint64(0), ctypes.c_void_p()
        st = lib.AtbMLAGetWorkspaceSize(*handles[:8], None, None, heads, scale, 1, 1 if multi else 0, calc, 1, handles[8],
                                        handles[9], ctypes.byref(ws), ctypes.byref(op), c.ptr)
        assert st == 0 and op.value, binding.ERROR_NAMES[st]
        with torch.cuda.stream(stream):
            work = torch.empty(max(int(ws.value), 1), dtype=torch.uint8, device=dev)
            st = lib.AtbMLA(work.data_ptr(), ws.value, op, c.ptr)
        stream.synchronize()
        assert st == 0, binding.ERROR_NAMES[st]
        want_lse = np.zeros((rows, heads), np.float32)
        # (128 heads: a job per query token, the mask tensor is not read)
        want = oracle_pa(oracle, q, kc, None, tables, ctx_lens, scale, mla_dv=dv, mask=None,
                         q_lens=q_lens if multi else None, lse_out=want_lse, causal_rows=True if multi else None)
        assert_close(out, want, TOL[dtype], "AtbMLA calcType %d" % calc)
        if ring:
            assert_close(lse[..., 0], want_lse, TOL[dtype], "AtbMLA lse")
        lib.atb_c_destroy_operation(op)
        for h in handles:
            if h:
                lib.aclDestroyTensor(h)

    # PagedCacheLoad through its wrapper
    heads_kv, hd, blocks, bs = 4, 64, 12, 16
    lens = np.array([20, 5, 33], dtype=np.int32)
    tables_np = rng.permutation(blocks)[:9].reshape(3, 3).astype(np.int32)
    with torch.cuda.stream(stream):
        kcache = torch.from_numpy(rng.integers(-100, 100, size=(blocks, bs, heads_kv, hd)).astype(np.float32)).to(torch.float16).to(dev)
        vcache = torch.from_numpy(rng.integers(-100, 100, size=(blocks, bs, heads_kv, hd)).astype(np.float32)).to(torch.float16).to(dev)
        key = torch.zeros((int(lens.sum()), heads_kv, hd), dtype=torch.float16, device=dev)
        value = torch.zeros_like(key)
        t_d, l_d = torch.from_numpy(tables_np).to(dev), torch.from_numpy(lens).to(dev)
        starts = torch.zeros(3, dtype=torch.int32, device=dev)
    stream.synchronize()
    want_k, want_v = oracle.paged_cache_load(_bits(kcache).cpu().numpy(), _bits(vcache).cpu().numpy(), tables_np, lens,
                                             _bits(key).cpu().numpy(), _bits(value).cpu().numpy(), np.zeros(3, np.int32))
    handles = [A(kcache), A(vcache), A(t_d), A(l_d), A(key), A(value), A(starts)]
    ws, op = ctypes.c_uint64(0), ctypes.c_void_p()
    st = lib.AtbPagedCacheLoadGetWorkspaceSize(*handles, 1, False, True, ctypes.byref(ws), ctypes.byref(op), c.ptr)
    assert st == 0 and op.value, binding.ERROR_NAMES[st]
    st = lib.AtbPagedCacheLoad(None, 0, op, c.ptr)
    stream.synchronize()
    assert st == 0, binding.ERROR_NAMES[st]
    assert np.array_equal(_bits(key).cpu().numpy(), want_k) and np.array_equal(_bits(value).cpu().numpy(), want_v)
    lib.atb_c_destroy_operation(op)
    for h in handles:
        lib.aclDestroyTensor(h)
    c.close()


def test_lse_output_of_plain_and_masked_decode(binding, oracle, dev, stream):
    """The log-sum-exp output is not tied to the latent layouts: separate K and V caches, a mask, rows
    split over ranges and rows written directly."""
    rng = _rng(420)
    heads, kv_heads, d, block = 32, 8, 128, 128
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, 5, heads, kv_heads, block, d, d, [3000, 40, 0, 129, 1000],
                                        torch.float16)
    mask, _ = _mask_tensor(oracle, rng, dev, "alibi4", ctx, heads, 3000, torch.float16)
    scale = 1.0 / math.sqrt(d)
    want_lse = np.zeros((5, heads), np.float32)
    want = oracle_pa(oracle, q, kc, vc, tables, ctx, scale, mask=mask, lse_out=want_lse)
    for kernel in (binding.ATBMI_PA_KERNEL_SCALAR, binding.ATBMI_PA_KERNEL_AUTO):
        lse = torch.zeros((5, heads), dtype=torch.float16, device=dev)
        got = pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx, scale, kernel=kernel, mask=mask, lse=lse)
        assert_close(got, want, 1e-3, "out kernel=%d" % kernel)
        assert_close(lse[:4], want_lse[:4], 2e-3, "lse kernel=%d" % kernel)  # |lse| ~ 8: fp16 spacing 4e-3..8e-3
        assert torch.all(lse[4] == 0)


# ------------------------------------------------------------------ several query tokens per sequence
def _spec_mask(rng, dev, kind, ctx, q_lens, dtype):
    """The masks of the reference's multi-token tests: "query" — one row per query row, the
    causal triangle of -10000 over the last q positions of its sequence
    (test_paged_attention_mla_mtp.py:220-231); "position" — the square causal mask
    (test_paged_attention_operation_parallel_decoding_910B.py:157-160); both with a random
    bias added where they are zero."""
    max_len = int(max(ctx))
    if kind == "position":
        m = np.triu(np.ones((max_len, max_len), np.float32), 1) * -10000.0
    else:
        rows = int(sum(n for n, c in zip(q_lens, ctx) if c > 0))
        m = np.zeros((rows, max_len), np.float32)
        row = 0
        for n, c in zip(q_lens, ctx):
            if c == 0:
                continue
            m[row:row + n, c - n:c] = np.triu(np.ones((n, n), np.float32), 1) * -10000.0
            row += n
    # a random bias on the visible positions, so that a wrong row shows even where the triangle is small
    m = np.where(m == 0, rng.standard_normal(m.shape).astype(np.float32), m)
    return torch.from_numpy(m).to(dtype).to(dev)


# heads, kv_heads, block, d, dv (0: same as d; > 0 with kv_heads 1 and d 576: MLA), ctx, q_lens, mask, dtype
# (reference parallel-decoding test: q [1, 15, 30, 6] over k [10, 64, 64, 64]; MLA MTP tests: 2..4 tokens)
SPEC_MATRIX = [
    (32, 32, 128, 128, 0, [10, 64, 64, 64], [1, 15, 30, 6], "query", torch.float16),
    (32, 32, 128, 128, 0, [10, 64, 64, 64], [1, 15, 30, 6], "position", torch.float16),
    (32, 8, 128, 128, 0, [1000, 0, 2300, 130, 4], [2, 3, 4, 1, 4], "query", torch.bfloat16),
    (30, 2, 16, 128, 0, [700, 33, 1500], [3, 2, 4], "position", torch.float16),
    (16, 4, 64, 96, 0, [513, 800], [4, 0], "query", torch.float16),
    (128, 1, 128, 576, 512, [700, 33, 1500], [2, 1, 3], None, torch.bfloat16),
    (32, 1, 128, 576, 512, [300, 1200], [2, 4], "query", torch.float16),
]


@pytest.mark.parametrize("case", SPEC_MATRIX, ids=lambda c: "h%d_g%d_d%d_%s_%s" % (
    c[0], c[1], c[3], c[7], str(c[8]).split(".")[-1]))
def test_paged_attention_several_query_tokens(binding, oracle, dev, stream, case):
    heads, kv_heads, block, d, mla_dv, ctx, q_lens, kind, dtype = case
    rng = _rng(300 + heads + len(ctx))
    dv = mla_dv if mla_dv else d
    _, kc, vc, tables, ctx = _pa_inputs(rng, dev, len(ctx), heads, kv_heads, block, d, d, ctx, dtype,
                                        std=0.5 if mla_dv else 1.0)
    if mla_dv:
        vc = None
    rows = int(sum(n for n, c in zip(q_lens, ctx) if c > 0))
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(rng.integers(1 << 30)))
    q = (torch.rand((rows + 1, heads, d), generator=gen) * 2 - 1).to(dtype).to(dev)
    mask = None if kind is None else _spec_mask(rng, dev, kind, ctx, q_lens, dtype)
    scale = 1.0 / math.sqrt(d)
    mode = kind or "sequence"
    want = oracle_pa(oracle, q, kc, vc, tables, ctx, scale, mla_dv=mla_dv, out_init=0.25, mask=mask, q_lens=q_lens,
                     mask_rows=mode)
    if kind is not None:
        unmasked = oracle_pa(oracle, q, kc, vc, tables, ctx, scale, mla_dv=mla_dv, out_init=0.25, q_lens=q_lens)
        assert np.abs(want - unmasked).max() > 0.01
    for kernel in (binding.ATBMI_PA_KERNEL_SCALAR, binding.ATBMI_PA_KERNEL_AUTO):
        out = torch.full((rows + 1, heads, dv), 0.25, dtype=dtype, device=dev)
        got = pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx, scale, mla_dv=mla_dv, kernel=kernel, out=out,
                             mask=mask, q_lens=q_lens, mask_rows=mode)
        assert_close(got, want, TOL[dtype], "kernel=%d" % kernel)


# heads, block, ctx, q_lens, mask, dtype, chunk override: the 128-head kernel takes the query tokens of a sequence
# as more heads of one pass, 128 / heads of them (at most 8) at a time
MLA_WIDE_TOKENS = [
    (16, 128, [700, 33, 1500], [2, 1, 3], "query", torch.bfloat16, None),
    (16, 128, [900, 40, 300], [8, 11, 5], "query", torch.float16, None),       # 8 a pass, then the rest
    (16, 64, [2100, 64], [4, 2], "query", torch.bfloat16, 128),                # partial rows of every token
    (8, 128, [515, 1030], [9, 3], "position", torch.float16, None),            # 8 tokens fill half the rows
    (48, 16, [1200, 77, 300], [2, 2, 1], "query", torch.bfloat16, 256),        # 96 rows: a wave without any
    (40, 128, [640, 1300], [3, 3], None, torch.float16, None),                 # 120 rows, a pass of one token behind
    (64, 128, [513, 4000], [2, 2], "sequence", torch.bfloat16, None),          # one mask row for both tokens
    (32, 128, [3000, 3000, 3000, 3000], [4, 4, 4, 4], None, torch.bfloat16, 512),
    (16, 128, [700, 0, 300, 64, 2], [3, 2, 0, 5, 2], "query", torch.float16, None),   # no context, no query tokens
]


@pytest.mark.parametrize("case", MLA_WIDE_TOKENS, ids=lambda c: "h%d_bs%d_q%s_%s_%s%s" % (
    c[0], c[1], "-".join(map(str, c[3])), c[4], str(c[5]).split(".")[-1], "_chunk%d" % c[6] if c[6] else ""))
def test_paged_attention_mla_128_head_kernel_with_several_query_tokens(binding, oracle, dev, stream, case):
    """Several query tokens per sequence over the combined cache, with the log-sum-exp output: against the oracle and
    against the fp32 scalar kernel."""
    heads, block, ctx, q_lens, kind, dtype, chunk = case
    rng = _rng(700 + heads + block + len(ctx))
    _, kc, _, tables, ctx = _pa_inputs(rng, dev, len(ctx), heads, 1, block, 576, 576, ctx, dtype, std=0.5)
    rows = int(sum(n for n, c in zip(q_lens, ctx) if c > 0))
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(rng.integers(1 << 30)))
    q = (torch.rand((rows + 1, heads, 576), generator=gen) * 2 - 1).to(dtype).to(dev)
    if kind == "sequence":
        mask, _ = _mask_tensor(oracle, rng, dev, "norm3", ctx, heads, int(max(ctx)), dtype)
    else:
        mask = None if kind is None else _spec_mask(rng, dev, kind, ctx, q_lens, dtype)
    mode = kind or "sequence"
    scale = 1.0 / math.sqrt(192.0)
    want_lse = np.zeros((rows + 1, heads), np.float32)
    want = oracle_pa(oracle, q, kc, None, tables, ctx, scale, mla_dv=512, out_init=0.25, mask=mask, q_lens=q_lens,
                     mask_rows=mode, lse_out=want_lse)
    results = []
    for kernel in (binding.ATBMI_PA_KERNEL_MFMA, binding.ATBMI_PA_KERNEL_SCALAR):
        out = torch.full((rows + 1, heads, 512), 0.25, dtype=dtype, device=dev)
        lse = torch.zeros((rows + 1, heads), dtype=dtype, device=dev)
        got = pa_decode_cabi(binding, stream, q, kc, None, tables, ctx, scale, mla_dv=512, kernel=kernel, out=out,
                             mask=mask, q_lens=q_lens, mask_rows=mode, lse=lse, chunk_tokens=chunk)
        assert_close(got, want, TOL[dtype], "kernel=%d" % kernel)
        assert_close(lse[:rows], want_lse[:rows], TOL[dtype], "lse kernel=%d" % kernel)
        results.append(got.float().cpu().numpy())
    assert_close(results[0], results[1], TOL[dtype], "128-head kernel vs scalar kernel")


def test_several_query_tokens_through_operation_api(binding, oracle, dev, stream):
    """calcType = CALC_TYPE_SPEC: inputs q, caches, tables, contextLens, mask, qSeqLens
    (reference paged_attention_operation.cpp:408-426), both lengths with hostData."""
    rng = _rng(320)
    heads, kv_heads, d, block = 32, 8, 128, 128
    ctx = np.array([10, 64, 640, 64], dtype=np.int32)
    q_lens = np.array([1, 15, 30, 6], dtype=np.int32)
    _, kc, vc, tables, ctx = _pa_inputs(rng, dev, 4, heads, kv_heads, block, d, d, ctx, torch.float16)
    q = (torch.rand((52, heads, d)) * 2 - 1).half().to(dev)
    scale = 1.0 / math.sqrt(d)
    lens, qn = torch.from_numpy(ctx), torch.from_numpy(q_lens)
    c = binding.Context(stream)
    for kind, mask_type in (("query", 3), ("position", 1)):
        mask = _spec_mask(rng, dev, kind, ctx, q_lens, torch.float16)
        pa = binding.OperationRunner("PagedAttentionOperation", binding.PagedAttentionParam(
            headNum=heads, kvHeadNum=kv_heads, qkScale=scale, maskType=mask_type, calcType=1), c)
        with torch.cuda.stream(stream):
            out, = pa.run([q, kc, vc, tables, lens.to(dev), mask, qn.to(dev)], host_inputs={4: lens, 6: qn})
        stream.synchronize()
        assert tuple(out.shape) == (52, heads, d)
        want = oracle_pa(oracle, q, kc, vc, tables, ctx, scale, mask=mask, q_lens=q_lens, mask_rows=kind)
        assert_close(out, want, 1e-3, kind)
        pa.close()
    c.close()


def test_decode_step_through_torch_atb(pkg, oracle, dev):
    """A decode step the way a torch_atb user writes it: Operation(param).forward([...]) with the
    context lengths as a CPU tensor, on torch's current stream."""
    ta = pkg.torch_atb
    rng = _rng(600)
    heads, kv_heads, d, block = 32, 8, 128, 128
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, 4, heads, kv_heads, block, d, d, [300, 17, 1025, 128], torch.float16)
    new_k = (torch.rand((4, kv_heads, d)) * 2 - 1).half().to(dev)
    new_v = (torch.rand((4, kv_heads, d)) * 2 - 1).half().to(dev)
    last = ctx.astype(np.int64) - 1
    t = tables.cpu().numpy()
    slots = torch.from_numpy((t[np.arange(4), last // block].astype(np.int64) * block + last % block).astype(np.int32))
    want_k, want_v = oracle.reshape_and_cache(_bits(new_k).cpu().numpy(), _bits(new_v).cpu().numpy(),
                                              _bits(kc).cpu().numpy(), _bits(vc).cpu().numpy(), slots.numpy())
    rac = ta.Operation(ta.ReshapeAndCacheParam())
    outs = rac.forward([new_k, new_v, kc, vc, slots.to(dev)])
    assert outs[0] is kc and outs[1] is vc
    assert np.array_equal(_bits(kc).cpu().numpy(), want_k) and np.array_equal(_bits(vc).cpu().numpy(), want_v)
    scale = 1.0 / math.sqrt(d)
    pa = ta.Operation(ta.PagedAttentionParam(head_num=heads, kv_head_num=kv_heads, qk_scale=scale))
    out, = pa.forward([q, kc, vc, tables, torch.from_numpy(ctx)])
    assert_close(out, oracle_pa(oracle, q, kc, vc, tables, ctx, scale), 1e-3, "torch_atb")
    rac.close()
    pa.close()


# ------------------------------------------------------------------ edge semantics
@pytest.mark.parametrize("kernel", [1, 0])
def test_empty_sequences_garbage_rows_and_shared_blocks(binding, oracle, dev, stream, kernel):
    rng = _rng(70)
    heads, kv_heads, d, block = 16, 4, 128, 16
    ctx = np.array([0, 37, 1, 0, 400, 16, 0], dtype=np.int32)
    # blocks may be shared between sequences and repeat inside one (read-only)
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, len(ctx), heads, kv_heads, block, d, d, ctx, torch.float16,
                                        unique=False)
    # poison every cache row no sequence may read
    used = np.zeros((kc.shape[0], block), dtype=bool)
    t = tables.cpu().numpy()
    for b, n in enumerate(ctx):
        j = np.arange(n)
        used[t[b][j // block], j % block] = True
    mask = torch.from_numpy(~used).to(dev)
    kc[mask] = float("nan")
    vc[mask] = float("nan")
    # block-table entries past the last used block must never be dereferenced
    t2 = t.copy()
    for b, n in enumerate(ctx):
        t2[b, (n + block - 1) // block:] = 0x3FFFFFF
    tables2 = torch.from_numpy(t2).to(dev)
    scale = 1.0 / math.sqrt(d)
    out = torch.full((len(ctx), heads, d), 0.1, dtype=torch.float16, device=dev)
    got = pa_decode_cabi(binding, stream, q, kc, vc, tables2, ctx, scale, kernel=kernel, out=out)
    kc_o, vc_o = kc.clone(), vc.clone()
    kc_o[mask] = 0
    vc_o[mask] = 0
    want = oracle_pa(oracle, q, kc_o, vc_o, tables, ctx, scale, out_init=0.1)
    # rows 0..3 belong to the four non-empty sequences, rows 4..6 are never written
    assert_close(got, want, 1e-3, "edge")
    assert torch.all(got[4:] == torch.tensor(0.1, dtype=torch.float16))


@pytest.mark.parametrize("kernel", [1, 0])
@pytest.mark.parametrize("chunk", [128, 256, 1024, 100000])
def test_split_kv_chunking_does_not_change_the_result(binding, oracle, dev, stream, kernel, chunk):
    rng = _rng(80)
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, 3, 32, 8, 128, 128, 128, [5000, 129, 2049], torch.bfloat16)
    scale = 1.0 / math.sqrt(128)
    got, info = pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx, scale, kernel=kernel, chunk_tokens=chunk,
                               return_plan_info=True)
    assert_close(got, oracle_pa(oracle, q, kc, vc, tables, ctx, scale), 2e-2, "chunk=%d" % chunk)
    # scalar kernel: chunks per sequence; MFMA kernel: equal ranges of the whole batch
    if chunk == 128:
        assert info["chunks"] >= (40 + 2 + 17 if kernel == 1 else 50)
    if chunk == 100000:
        assert info["chunks"] == (3 if kernel == 1 else 1)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_q_scale_premultiply(binding, oracle, dev, stream, dtype):
    rng = _rng(90)
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, 4, 8, 8, 128, 128, 128, [300, 64, 512, 9], dtype)
    for kernel in (1, 0):
        got = pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx, 0.2, q_scale=0.7, kernel=kernel)
        assert_close(got, oracle_pa(oracle, q, kc, vc, tables, ctx, 0.2, q_scale=0.7), TOL[dtype], "qScale")


def test_operation_runs_on_the_stream_its_id_names(binding, oracle, dev, stream):
    """A context with two execute streams: the operation with stream id 1 launches on the second one (the first is
    held busy by a long copy queued before, and the result is complete once the second stream alone has been waited for)."""
    rng = _rng(96)
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, 4, 32, 8, 128, 128, 128, [700, 1500, 128, 3000], torch.float16)
    scale = 1.0 / math.sqrt(128)
    second = torch.cuda.Stream(device=dev)
    c = binding.Context(stream)
    assert c.set_streams([stream, second]) == 0
    pa = binding.OperationRunner("PagedAttentionOperation", binding.PagedAttentionParam(
        headNum=32, kvHeadNum=8, qkScale=scale), c)
    assert pa.op.set_stream_id(1) == 0 and pa.op.get_stream_id() == 1
    lens = torch.from_numpy(ctx)
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        big = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        for _ in range(60):  # some ten milliseconds of work on the first stream
            big.fill_(1)
    with torch.cuda.stream(second):
        out, = pa.run([q, kc, vc, tables, lens.to(dev)], host_inputs={4: lens})
    second.synchronize()
    busy = not stream.query()
    assert_close(out, oracle_pa(oracle, q, kc, vc, tables, ctx, scale), 1e-3, "stream 1")
    stream.synchronize()
    assert busy, "the first stream was meant to be still busy when the second one had finished"
    pa.close()
    c.close()


def test_repeated_execute_and_changing_lengths(binding, oracle, dev, stream):
    """One operation, Setup + Execute repeatedly with growing context lengths, no sync in between."""
    rng = _rng(95)
    heads, kv_heads, d, block = 32, 8, 128, 128
    base = np.array([700, 1500, 128, 3000], dtype=np.int32)
    q, kc, vc, tables, _ = _pa_inputs(rng, dev, 4, heads, kv_heads, block, d, d, base + 8, torch.float16)
    scale = 1.0 / math.sqrt(d)
    c = binding.Context(stream)
    pa = binding.OperationRunner("PagedAttentionOperation", binding.PagedAttentionParam(
        headNum=heads, kvHeadNum=kv_heads, qkScale=scale), c)
    outs = []
    with torch.cuda.stream(stream):
        for step in range(8):
            lens = torch.from_numpy(base + step)
            out, = pa.run([q, kc, vc, tables, lens.to(dev)], host_inputs={4: lens})
            outs.append(out)
    stream.synchronize()
    for step in (0, 3, 7):
        assert_close(outs[step], oracle_pa(oracle, q, kc, vc, tables, base + step, scale), 1e-3, "step %d" % step)
    pa.close()
    c.close()


@pytest.mark.parametrize("charged", [3, 12, 40])
@pytest.mark.parametrize("ctx", [[33, 700, 5, 64, 1500, 90, 2100], [4000, 40, 40, 40, 3000, 1]],
                         ids=["mixed", "long_and_tiny"])
def test_ranges_that_hold_only_the_steps_charged_for_a_row_start(binding, oracle, dev, stream, monkeypatch, ctx, charged):
    """The planner charges the start of every row some steps of its own; with the charge raised
    (ATBMI_PA_ROW_START_STEPS) above the length of a wave range, whole ranges fall into charged steps and leave
    empty partial rows (zeros, log-sum-exp -inf), which the merge must weigh as nothing. The result stays the
    oracle's and within rounding of the default plan's."""
    rng = _rng(98)
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, len(ctx), 32, 8, 128, 128, 128, ctx, torch.float16)
    scale = 1.0 / math.sqrt(128)
    want = oracle_pa(oracle, q, kc, vc, tables, ctx, scale)
    plain = pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx, scale, kernel=0)
    monkeypatch.setenv("ATBMI_PA_ROW_START_STEPS", str(charged))
    for rep in range(3):  # (reused workspace: the empty rows must be written every time)
        got = pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx, scale, kernel=0, poison_workspace=rep == 1)
        assert_close(got, want, 1e-3, "charged %d, repetition %d" % (charged, rep))
        assert_close(got, plain.float().cpu().numpy(), 1e-3, "against the default plan")


@pytest.mark.parametrize("heads,kv_heads", [(30, 2), (8, 2), (8, 4), (32, 8), (16, 1)])
def test_rows_spanning_wave_ranges_merge_consistently(binding, oracle, dev, stream, heads, kv_heads):
    """Rows cut across several wave ranges leave partial rows in the workspace, written by CUs of
    different XCDs and read back by the merge kernel that follows on the stream. Repeated launches
    on reused workspace addresses must all give the oracle's rows."""
    rng = _rng(97)
    q, kc, vc, tables, ctx = _pa_inputs(rng, dev, 18, heads, kv_heads, 128, 128, 128, 88, torch.float16)
    scale = 1.0 / math.sqrt(128)
    want = oracle_pa(oracle, q, kc, vc, tables, ctx, scale)
    for rep in range(12):
        got = pa_decode_cabi(binding, stream, q, kc, vc, tables, ctx, scale, kernel=0)
        assert_close(got, want, 1e-3, "repetition %d" % rep)
