"""Full-size benchmark configurations (C2-C5) on the GPU, through atb::Operation.

At these sizes parity is checked three ways: (1) the oracle on every sequence of the batch,
each given only its own blocks (a few seconds of numpy for all five configurations); (2) the two independent GPU
implementations - MFMA kernel and fp32 scalar kernel - must agree on every output
row; (3) the cache write is checked exhaustively on the GPU: written slots hold the
new rows (quantised bit-exactly for the int8 cache), every other byte is unchanged.
Tolerances: 1e-3 fp16, 2e-2 bf16 / int8-KV (rtol = atol)."""
import numpy as np
import pytest
import torch

from pa_harness import assert_close, pa_decode_cabi

pytestmark = pytest.mark.gpu

TOL = {"c2": 2e-2, "c2_fp16": 1e-3, "c3": 2e-2, "c4": 1e-3, "c5": 2e-2}


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return torch.device("cuda:0")


@pytest.fixture(scope="module")
def stream(dev):
    return torch.cuda.Stream(device=dev)


def _sample_rows(oracle, step, cfg, scale, rows):
    """Oracle output for the given sequences, each from its own blocks only."""
    out = {}
    tables = step["layout"]["tables"]
    ctx = step["layout"]["ctx"]
    kc, vc = step["key_cache"], step["value_cache"]
    ks = step["k_scale"].cpu().numpy() if "k_scale" in step else None
    vs = step["v_scale"].cpu().numpy() if "v_scale" in step else None
    for b in rows:
        n = int(ctx[b])
        nblk = (n + cfg["block"] - 1) // cfg["block"]
        ids = torch.from_numpy(tables[b, :nblk].astype(np.int64)).to(kc.device)
        kb = kc[ids].cpu()
        vb = vc[ids].cpu() if vc is not None else None
        kb = kb.numpy() if kb.dtype == torch.int8 else kb.float().numpy()
        if vb is not None:
            vb = vb.numpy() if vb.dtype == torch.int8 else vb.float().numpy()
        q = step["q"][b:b + 1].float().cpu().numpy()
        out[b] = oracle.paged_attention(q, kb, vb, np.arange(nblk, dtype=np.int32)[None, :], np.array([n]), scale,
                                        ks, None, vs, None, mla_v_head_size=cfg["dv"] if cfg.get("mla") else 0)[0]
    return out


@pytest.mark.parametrize("name", ["c2", "c2_fp16", "c3", "c4", "c5"])
def test_full_size_decode_step(binding, oracle, pkg, dev, stream, name):
    w = pkg.workloads
    cfg = w.config(name)
    step = w.make_step(cfg, dev)
    scale = w.qk_scale(cfg)
    int8 = cfg["kv"] == "int8"
    mla = bool(cfg.get("mla"))
    ctx_lens = step["layout"]["ctx"]
    slots = torch.from_numpy(step["layout"]["slots"].astype(np.int64)).to(dev)
    b, h, g, d, dv = cfg["batch"], cfg["heads"], cfg["kv_heads"], cfg["d"], cfg["dv"]

    # ---- cache write
    kc_before = step["key_cache"].clone()
    vc_before = None if mla else step["value_cache"].clone()
    c = binding.Context(stream)
    k = binding.kernels()
    with torch.cuda.stream(stream):
        if int8:
            rc = k.atbmi_reshape_and_cache_quant(
                step["k_new"].data_ptr(), step["v_new"].data_ptr(), binding.ATBMI_F16, step["k_scale"].data_ptr(),
                step["v_scale"].data_ptr(), step["key_cache"].data_ptr(), step["value_cache"].data_ptr(),
                step["slot_mapping"].data_ptr(), b, g, d, dv, cfg["block"] * step["layout"]["pool"],
                stream.cuda_stream)
            assert rc == 0, binding.last_kernel_error()
        elif mla:
            rac = binding.OperationRunner("ReshapeAndCacheOperation", binding.ReshapeAndCacheParam(kvCacheCfg=1), c)
            rac.run([step["k_new"], step["key_cache"], step["slot_mapping"]], outputs=[step["key_cache"]])
        else:
            rac = binding.OperationRunner("ReshapeAndCacheOperation", binding.ReshapeAndCacheParam(), c)
            rac.run([step["k_new"], step["v_new"], step["key_cache"], step["value_cache"], step["slot_mapping"]],
                    outputs=[step["key_cache"], step["value_cache"]])
    stream.synchronize()

    def check_cache(cache, before, new_rows, scales, dim):
        flat = cache.view(-1, g * dim)
        if int8:
            want = torch.from_numpy(oracle.quant_per_channel(
                new_rows.float().cpu().numpy().reshape(b, -1), scales.cpu().numpy())).to(dev)
        else:
            want = new_rows.reshape(b, -1)
        assert torch.equal(flat[slots].view(torch.int8), want.view(torch.int8)), "written rows differ"
        # everything else is untouched: put the old rows back and compare whole caches
        restored = cache.clone()
        restored.view(-1, g * dim)[slots] = before.view(-1, g * dim)[slots]
        assert torch.equal(restored.view(torch.int8), before.view(torch.int8)), "a row outside the slot mapping changed"

    check_cache(step["key_cache"], kc_before, step["k_new"], step.get("k_scale"), d)
    if not mla:
        check_cache(step["value_cache"], vc_before, step["v_new"], step.get("v_scale"), dv)
    del kc_before, vc_before

    # ---- attention through the operator API (MFMA kernel)
    param = binding.PagedAttentionParam(headNum=h, kvHeadNum=g, qkScale=scale, quantType=1 if int8 else 0,
                                        mlaVHeadSize=dv if mla else 0)
    pa = binding.OperationRunner("PagedAttentionOperation", param, c)
    lens = step["context_lens"]
    with torch.cuda.stream(stream):
        lens_dev = lens.to(dev)
        if mla:
            ins, host_idx = [step["q"], step["key_cache"], step["block_tables"], lens_dev], 3
        else:
            ins, host_idx = [step["q"], step["key_cache"], step["value_cache"], step["block_tables"], lens_dev], 4
            if int8:
                ins += [step["k_scale"], step["v_scale"]]
        out, = pa.run(ins, host_inputs={host_idx: lens})
    stream.synchronize()
    assert tuple(out.shape) == (b, h, dv) and bool(torch.isfinite(out.float()).all())

    # (1) the oracle on every sequence of the batch
    rows = list(range(b))
    for r, want in _sample_rows(oracle, step, cfg, scale, rows).items():
        assert_close(out[r], want, TOL[name], "%s sequence %d (ctx %d)" % (name, r, ctx_lens[r]))

    # (2) the fp32 scalar kernel, an independent implementation, on the whole batch
    ref = pa_decode_cabi(binding, stream, step["q"], step["key_cache"], step["value_cache"], step["block_tables"],
                         ctx_lens, scale, step.get("k_scale"), None, step.get("v_scale"), None,
                         mla_dv=dv if mla else 0, kernel=binding.ATBMI_PA_KERNEL_SCALAR)
    assert_close(out, ref.float().cpu().numpy(), TOL[name], name + " mfma vs scalar")
    pa.close()
    c.close()
