#!/usr/bin/env python3
"""Times the cache-side operations at the size of benchmark workload C2 on one MI355X and
prints one JSON line per operation: BlockCopy (512 blocks of 256 KB copied in each cache),
PagedCacheLoad (all 158 839 cached rows of the 64 sequences gathered) and NormRopeReshape (the
producer of the combined MLA cache, at the 65 536 tokens of the reference's kernel test) and Rope
(8 192 tokens of a Llama-3-8B-shaped layer) and the per-channel quantiser / dequantiser of
ElewiseOperation (3 072 x 16 384) and the head-compressed forms of ReshapeAndCache and ReshapeAndCacheOmni
(4 sequences of 4 000 tokens, windows of 1 501), through
atb::Operation (Setup + Execute per call; NormRopeReshape, Rope and Elewise: Setup once). All are HBM-bound; `roofline.achieved` is their
algorithmic bytes (every source byte read once, every destination byte written once) over the
mean kernel time between HIP events on the launch stream.

    python3 ascend-transformer-boost_amd/bench_cache_ops.py [--steps 50] [--warmup 5]
"""
import argparse
import importlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
HBM_PEAK_GBPS = 8000.0


def timed(fn, stream, steps, warmup):
    import torch
    with torch.cuda.stream(stream):
        for _ in range(warmup):
            fn()
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        start.record(stream)
        for _ in range(steps):
            fn()
        stop.record(stream)
    stream.synchronize()
    return start.elapsed_time(stop) / steps


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    args = ap.parse_args()
    import torch
    pkg = importlib.import_module(os.path.basename(HERE))
    b, w = pkg.binding, pkg.workloads
    if not torch.cuda.is_available():
        sys.exit("bench_cache_ops.py: no GPU visible")
    dev = torch.device("cuda:0")
    cfg = w.config("c2")
    lay = w.layout(cfg)
    g, d, bs, pool = cfg["kv_heads"], cfg["d"], cfg["block"], lay["pool"]
    stream = torch.cuda.Stream(device=dev)
    ctx = b.Context(stream)
    kc = torch.randn((pool, bs, g, d), device=dev).to(torch.bfloat16)
    vc = torch.randn((pool, bs, g, d), device=dev).to(torch.bfloat16)
    block_bytes = bs * g * d * 2

    # ---- BlockCopy: 256 sources, two destinations each
    rng = np.random.Generator(np.random.PCG64(11))
    perm = rng.permutation(pool)
    src, dst = perm[:256].astype(np.int32), perm[256:768].astype(np.int32)
    cum = (np.arange(1, 257) * 2).astype(np.int32)
    src_d, dst_d, cum_d = (torch.from_numpy(a).to(dev) for a in (src, dst, cum))
    copy = b.OperationRunner("BlockCopyOperation", b.BlockCopyParam(), ctx)
    ms = timed(lambda: copy.run([kc, vc, src_d, dst_d, cum_d], outputs=[]), stream, args.steps, args.warmup)
    alg = 2 * (len(src) + len(dst)) * block_bytes
    print(json.dumps({"operation": "BlockCopyOperation", "workload": "C2 caches: 256 source blocks of 256 KB to 512 "
                      "destination blocks, in the key and in the value cache", "ms_per_call": ms,
                      "roofline": {"bound": "hbm", "achieved": alg / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS,
                                   "unit": "GB/s", "frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                                   "algorithmic_bytes": alg}}))
    copy.close()

    # ---- PagedCacheLoad: every cached row of the batch
    lens = lay["ctx"]
    total = int(lens.sum())
    key = torch.empty((total, g, d), dtype=torch.bfloat16, device=dev)
    value = torch.empty_like(key)
    tables_d = torch.from_numpy(lay["tables"]).to(dev)
    lens_d = torch.from_numpy(lens).to(dev)
    starts_d = torch.zeros(len(lens), dtype=torch.int32, device=dev)
    load = b.OperationRunner("PagedCacheLoadOperation", b.PagedCacheLoadParam(kvCacheCfg=1), ctx)
    ms = timed(lambda: load.run([kc, vc, tables_d, lens_d, key, value, starts_d], outputs=[key, value]), stream,
               args.steps, args.warmup)
    alg = 2 * 2 * total * g * d * 2
    print(json.dumps({"operation": "PagedCacheLoadOperation", "workload": "C2: %d rows of %d B gathered from each "
                      "cache into contiguous key / value" % (total, g * d * 2), "ms_per_call": ms,
                      "roofline": {"bound": "hbm", "achieved": alg / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS,
                                   "unit": "GB/s", "frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                                   "algorithmic_bytes": alg}}))
    load.close()

    # ---- the same rows through fractal-NZ caches [blocks, channels / 16, blockSize, 16]: written by
    # ReshapeAndCache (kvCacheCfg 2) from contiguous rows, gathered back by PagedCacheLoad (kvCacheCfg 0)
    chans = g * d
    nz_caches = [torch.zeros((pool, chans // 16, bs, 16), dtype=torch.bfloat16, device=dev) for _ in range(2)]
    nz_desc = [b.make_tensor(b._torch_acl_dtype(t), list(t.shape), device_ptr=t.data_ptr(), fmt="fractal_nz")
               for t in nz_caches]
    slots = np.concatenate([lay["tables"][i][np.arange(n) // bs].astype(np.int64) * bs + np.arange(n) % bs
                            for i, n in enumerate(lens)]).astype(np.int32)
    slots_d = torch.from_numpy(slots).to(dev)
    rows_k = torch.randn((total, g, d), device=dev).to(torch.bfloat16)
    rows_v = torch.randn((total, g, d), device=dev).to(torch.bfloat16)
    write = b.OperationRunner("ReshapeAndCacheOperation", b.ReshapeAndCacheParam(kvCacheCfg=2), ctx)
    ms = timed(lambda: write.run([rows_k, rows_v, nz_desc[0], nz_desc[1], slots_d], outputs=nz_desc), stream, args.steps,
               args.warmup)
    print(json.dumps({"operation": "ReshapeAndCacheOperation (fractal-NZ caches)", "workload": "C2 as a prefill: %d rows "
                      "of %d B scattered into each cache in 32-byte pieces" % (total, chans * 2), "ms_per_call": ms,
                      "roofline": {"bound": "hbm", "achieved": alg / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS,
                                   "unit": "GB/s", "frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                                   "algorithmic_bytes": alg}}))
    write.close()
    key2 = torch.empty((total, chans), dtype=torch.bfloat16, device=dev)
    value2 = torch.empty_like(key2)
    load = b.OperationRunner("PagedCacheLoadOperation", b.PagedCacheLoadParam(), ctx)
    ms = timed(lambda: load.run([nz_desc[0], nz_desc[1], tables_d, lens_d, key2, value2], outputs=[key2, value2]), stream,
               args.steps, args.warmup)
    stream.synchronize()
    if not (torch.equal(key2.view(total, g, d), rows_k) and torch.equal(value2.view(total, g, d), rows_v)):
        sys.exit("bench_cache_ops.py: rows written to the fractal-NZ caches did not come back")
    print(json.dumps({"operation": "PagedCacheLoadOperation (fractal-NZ caches)", "workload": "C2: %d rows of %d B "
                      "gathered from each cache (32-byte pieces) into contiguous key / value" % (total, chans * 2),
                      "ms_per_call": ms,
                      "roofline": {"bound": "hbm", "achieved": alg / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS,
                                   "unit": "GB/s", "frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                                   "algorithmic_bytes": alg}}))
    load.close()
    del nz_caches, rows_k, rows_v, key2, value2

    # ---- NormRopeReshape: 65 536 tokens of 512 + 64 channels into a cache of 512-token blocks
    tokens, n, r, block = 65536, 512, 64, 512
    blocks = (tokens + 100 + block - 1) // block
    x = torch.rand((tokens, 1, n), device=dev).to(torch.float16)
    gamma = torch.rand((n,), device=dev).to(torch.float16)
    rope, cos, sin = (torch.rand((tokens, r), device=dev).to(torch.float16) for _ in range(3))
    slots = torch.from_numpy(rng.permutation(tokens + 100)[:tokens].astype(np.int32)).to(dev)
    cache = torch.zeros((blocks, block, 1, n + r), dtype=torch.float16, device=dev)
    fused = b.OperationRunner("NormRopeReshapeOperation", b.NormRopeReshapeParam(epsilon=1e-5), ctx)
    # The kernel takes less time than Setup + Execute take on the host from Python: Setup once, then Execute
    # per call, so that the events bracket a stream the host keeps full.
    ins = [b.tensor_of(t) for t in (x, gamma, rope, cos, sin, slots, cache)]
    outs = [b.tensor_of(cache)]
    st, ws = fused.op.setup(ins, outs, ctx)
    assert st == 0 and ws == 0

    def execute():
        assert fused.op.execute(ins, outs, None, 0, ctx) == 0
    ms = timed(execute, stream, args.steps, args.warmup)
    alg = tokens * ((n + 3 * r) * 2 + 4 + (n + r) * 2) + n * 2
    print(json.dumps({"operation": "NormRopeReshapeOperation", "workload": "%d tokens: RMSNorm of %d channels + rotary "
                      "embedding of %d channels written into the combined cache, fp16 (Setup once, Execute per call)" % (tokens, n, r),
                      "ms_per_call": ms,
                      "roofline": {"bound": "hbm", "achieved": alg / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS,
                                   "unit": "GB/s", "frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                                   "algorithmic_bytes": alg}}))
    fused.close()

    # ---- Rope: 8 192 tokens of a Llama-3-8B-shaped layer (32 query heads, 8 KV heads, head size 128), bf16
    tokens, hq, hk, d = 8192, 32 * 128, 8 * 128, 128
    q = torch.rand((tokens, hq), device=dev).to(torch.bfloat16)
    k = torch.rand((tokens, hk), device=dev).to(torch.bfloat16)
    cos, sin = (torch.rand((tokens, d), device=dev).to(torch.bfloat16) for _ in range(2))
    lens_r = torch.tensor([tokens], dtype=torch.int32, device=dev)
    q_out, k_out = torch.empty_like(q), torch.empty_like(k)
    rope = b.OperationRunner("RopeOperation", b.RopeParam(rotaryCoeff=2), ctx)
    ins = [b.tensor_of(t) for t in (q, k, cos, sin, lens_r)]
    outs = [b.tensor_of(q_out), b.tensor_of(k_out)]
    st, ws = rope.op.setup(ins, outs, ctx)
    assert st == 0 and ws == 0

    def execute_rope():
        assert rope.op.execute(ins, outs, None, 0, ctx) == 0
    ms = timed(execute_rope, stream, args.steps, args.warmup)
    alg = tokens * ((hq + hk) * 2 * 2 + 2 * d * 2)
    print(json.dumps({"operation": "RopeOperation", "workload": "%d tokens, query rows of %d and key rows of %d channels, "
                      "head size %d, rotaryCoeff 2, bf16 (Setup once, Execute per call)" % (tokens, hq, hk, d),
                      "ms_per_call": ms,
                      "roofline": {"bound": "hbm", "achieved": alg / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS,
                                   "unit": "GB/s", "frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                                   "algorithmic_bytes": alg}}))
    rope.close()

    # ---- Elewise per-channel quantiser / dequantiser: 3 072 rows of 16 384 channels (a CSV row of the reference)
    rows, ch = 3072, 16384
    x = (torch.rand((rows, ch), device=dev) * 200 - 100).to(torch.float16)
    scale = (torch.rand((ch,), device=dev) * 0.9 + 0.1).to(torch.float16)
    offset = torch.randint(-10, 10, (ch,), dtype=torch.int8, device=dev)
    xq = torch.empty((rows, ch), dtype=torch.int8, device=dev)
    xd = torch.empty((rows, ch), dtype=torch.float16, device=dev)
    for name, etype, src, dst in (("quantiser", b.ElewiseParam.ELEWISE_QUANT_PER_CHANNEL, x, xq),
                                  ("dequantiser", b.ElewiseParam.ELEWISE_DEQUANT_PER_CHANNEL, xq, xd)):
        op = b.OperationRunner("ElewiseOperation", b.ElewiseParam(elewiseType=etype), ctx)
        ins = [b.tensor_of(t) for t in (src, scale, offset)]
        outs = [b.tensor_of(dst)]
        st, ws = op.op.setup(ins, outs, ctx)
        assert st == 0 and ws == 0

        def execute_elewise():
            assert op.op.execute(ins, outs, None, 0, ctx) == 0
        ms = timed(execute_elewise, stream, args.steps, args.warmup)
        alg = rows * ch * 3 + ch * 3
        print(json.dumps({"operation": "ElewiseOperation (per-channel %s)" % name,
                          "workload": "%d x %d fp16 <-> int8, scale and offset per channel (Setup once, Execute per call)"
                          % (rows, ch), "ms_per_call": ms,
                          "roofline": {"bound": "hbm", "achieved": alg / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS,
                                       "unit": "GB/s", "frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                                       "algorithmic_bytes": alg}}))
        op.close()
    # ---- ReshapeAndCache under head compression: 4 sequences of 4 000 tokens, 8 KV heads of 128 channels, bf16;
    # windows of 1 501 tokens per (sequence, head) pair (the sizes of the reference's kernel test)
    batch, heads, d, block, length, win = 4, 8, 128, 128, 4000, 1501
    pairs = batch * heads
    key = torch.randn((batch * length, heads, d), device=dev).to(torch.bfloat16)
    value = torch.randn_like(key)
    seq_d = torch.full((batch,), length, dtype=torch.int32, device=dev)
    wins_d = torch.full((pairs,), win, dtype=torch.int32, device=dev)
    for name, compress, rows_out in (("keep-last windows", 1, win), ("mean windows", 2, length - win + 1),
                                     ("dropped windows", 3, length - win)):
        per_pair = (rows_out + block - 1) // block
        cache_k = torch.zeros((pairs * per_pair, block, 1, d), dtype=torch.bfloat16, device=dev)
        cache_v = torch.zeros_like(cache_k)
        slots_d = (torch.arange(pairs, dtype=torch.int32, device=dev) * (per_pair * block)).contiguous()
        tensors = [key, value, cache_k, cache_v, slots_d, wins_d, seq_d]
        if compress >= 2:
            tensors.append(torch.from_numpy(rng.integers(0, length - win + 1, size=pairs).astype(np.int32)).to(dev))
        if compress == 3:  # the operation of its own that leaves the window out altogether
            op = b.OperationRunner("ReshapeAndCacheOmniOperation", b.ReshapeAndCacheOmniParam(), ctx)
        else:
            op = b.OperationRunner("ReshapeAndCacheOperation", b.ReshapeAndCacheParam(compressType=compress), ctx)
        ins = [b.tensor_of(t) for t in tensors]
        outs = [b.tensor_of(cache_k), b.tensor_of(cache_v)]
        st, ws = op.op.setup(ins, outs, ctx)
        assert st == 0 and ws == 0

        def execute_compress():
            assert op.op.execute(ins, outs, None, 0, ctx) == 0
        ms = timed(execute_compress, stream, args.steps, args.warmup)
        rows_in = win if compress == 1 else (length if compress == 2 else rows_out)
        alg = 2 * pairs * (rows_in + rows_out) * d * 2
        print(json.dumps({"operation": ("ReshapeAndCacheOmniOperation (%s)" if compress == 3 else
                                        "ReshapeAndCacheOperation (head compression, %s)") % name,
                          "workload": "%d sequences of %d tokens, %d heads of %d channels, windows of %d tokens, bf16 "
                          "(Setup once, Execute per call)" % (batch, length, heads, d, win), "ms_per_call": ms,
                          "roofline": {"bound": "hbm", "achieved": alg / (ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS,
                                       "unit": "GB/s", "frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                                       "algorithmic_bytes": alg}}))
        op.close()
    ctx.close()


if __name__ == "__main__":
    main()
