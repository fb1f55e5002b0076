#!/usr/bin/env python3
"""Decode-step benchmark: ReshapeAndCache + PagedAttention through atb::Operation
on one MI355X, synthetic data of the named configuration.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2]

Prints ONE JSON line: whole-step throughput (tokens/s = sequences decoded per
second, inputs resident in HBM), the attention kernel's achieved HBM bandwidth
against the 8 TB/s roofline (algorithmic bytes / mean kernel time from HIP
events on the launch stream), and the CPU oracle timed on a bounded sample of
the same workload.
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
PKG = "ascend-transformer-boost_amd"
HBM_PEAK_GBPS = 8000.0

# HBM bytes one attention launch moves, from rocprofv3 FETCH_SIZE / WRITE_SIZE counter runs of this
# script, scaled by what the same counters read for a 256 MiB copy (--calibrate-copy); the runs and the
# scale factors are written up in the profiles/ summaries of each workload. Keyed by workload and its
# algorithmic bytes, so a changed workload reports null instead of a stale figure.
MEASURED_TRAFFIC = {("c2", 651658484): 658.7e6, ("c2_alibi", 661824180): 669.5e6, ("c2_mtp4", 656075180): 683.6e6,
                    ("c3", 1364204576): 1379.2e6, ("c5", 253384304): 388.7e6,
                    ("c5_split", 253384304): 378.4e6}

DESCRIPTIONS = {
    "c1": "C1 small fp16 decode: batch 4, 8 q heads, 8 kv heads, d128, block 128, ctx U[64,512]",
    "c2": "C2 Llama-3-8B-shaped bf16 decode: batch 64, 32 q heads, 8 kv heads, d128, block 128, ctx U[1024,4096]",
    "c2_fp16": "C2 shape in fp16: batch 64, 32 q heads, 8 kv heads, d128, block 128, ctx U[1024,4096]",
    "c2_alibi": "C2 with an ALiBi mask [batch, heads, 1, maxS]: batch 64, 32 q heads, 8 kv heads, d128, block 128, "
                "ctx U[1024,4096], bf16",
    "c2_norm": "C2 with a NORM mask [batch, 1, maxS]: batch 64, 32 q heads, 8 kv heads, d128, block 128, "
               "ctx U[1024,4096], bf16",
    "c2_bnsd": "C2 over head-major caches [blocks, kv heads, block, d] (inputLayout TYPE_BNSD), attention only: batch 64, "
               "32 q heads, 8 kv heads, d128, block 128, ctx U[1024,4096], bf16",
    "c2_mtp4": "C2 with 4 query tokens per sequence (CALC_TYPE_SPEC, MASK_TYPE_SPEC mask [256, maxS]): batch 64, "
               "32 q heads, 8 kv heads, d128, block 128, ctx U[1024,4096], bf16",
    "c3": "C3 int8-KV 70B-shaped decode: batch 128, 64 q heads, 8 kv heads, d128, block 128, ctx U[2048,8192], fp16 q",
    "c4": "C4 skewed long-context fp16 decode: batch 16, 32 q heads, 8 kv heads, d128, ctx lognormal(median 8k) in [256,32768]",
    "c5_split": "C5 through MultiLatentAttentionOperation (cacheMode KROPE_CTKV: 512 latent + 64 rotary channels in "
                "two caches): batch 64, 128 q heads, block 128, ctx U[2048,4096], bf16",
    "c5": "C5 MLA bf16 decode: batch 64, 128 q heads, 1 latent kv head, d576/dv512, block 128, ctx U[2048,4096]",
}


def cpu_baseline(pkg, step, cfg, scale, budget_s=10.0):
    """Times the numpy oracle on the sequences of the batch, taken in order and
    again from the first once all are done, until about `budget_s` seconds of CPU
    work are spent; returns tokens/s (one token per sequence) on that sample."""
    import numpy as np
    oracle = importlib.import_module("oracle.atb_oracle")
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
    except Exception:
        threads = 1
    ctx = step["layout"]["ctx"]
    tables = step["layout"]["tables"]
    dev_q = step["q"]
    kc = step["key_cache"]
    vc = step["value_cache"]
    ks = step.get("k_scale")
    vs = step.get("v_scale")
    ks = ks.cpu().numpy() if ks is not None else None
    vs = vs.cpu().numpy() if vs is not None else None
    mask = step["mask"].float().cpu().numpy() if step.get("mask") is not None else None
    done, spent, tokens = 0, 0.0, 0
    q_len = int(cfg.get("q_len", 1))
    import torch
    b = 0
    while spent < budget_s:  # cycles over the batch until the budget is spent
        n = int(ctx[b])
        nblk = (n + cfg["block"] - 1) // cfg["block"]
        ids = torch.from_numpy(tables[b, :nblk].astype("int64")).to(kc.device)
        # only this sequence's blocks travel to the host
        kb = kc[ids].cpu()
        vb = vc[ids].cpu() if vc is not None else None
        kb = kb.numpy() if kb.dtype == torch.int8 else kb.float().numpy()
        if vb is not None:
            vb = vb.numpy() if vb.dtype == torch.int8 else vb.float().numpy()
        q = dev_q[b * q_len:(b + 1) * q_len].float().cpu().numpy()
        local = np.arange(nblk, dtype=np.int32)[None, :]
        rows_mask = None if mask is None else (mask[b * q_len:(b + 1) * q_len] if q_len > 1 else mask[b:b + 1])
        t0 = time.perf_counter()
        oracle.paged_attention(q, kb, vb, local, np.array([n]), scale, ks, None, vs, None,
                               mla_v_head_size=cfg["dv"] if cfg.get("mla") else 0, mask=rows_mask,
                               mask_per_head=False, q_lens=np.array([q_len]) if q_len > 1 else None,
                               mask_rows="query" if q_len > 1 else "sequence")
        spent += time.perf_counter() - t0
        done += q_len
        tokens += n
        b = (b + 1) % len(ctx)
    return {
        "value": done / spent if spent > 0 else 0.0,
        "unit": "tokens/s",
        "cores": threads,
        "kind": "port",
        "sample": "numpy oracle on %d query tokens of sequences drawn in order from the batch of %d "
                  "(%d context tokens), attention only, %.1f s" % (done, len(ctx), tokens, spent),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default="c2", choices=sorted(DESCRIPTIONS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--attention-only", action="store_true", help="leave ReshapeAndCache out of the step")
    ap.add_argument("--no-kernel-events", action="store_true", help="do not bracket the attention kernel with events")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device copy, as the known-size reference for hardware counters")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU; --gpus %d is not supported" % args.gpus)

    import torch
    pkg = importlib.import_module(PKG)
    b, w = pkg.binding, pkg.workloads
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    cfg = w.config(args.config)
    step = w.make_step(cfg, dev)
    scale = w.qk_scale(cfg)
    stream = torch.cuda.Stream(device=dev)
    ctx = b.Context(stream)
    int8 = cfg["kv"] == "int8"
    mla = bool(cfg.get("mla"))

    mask_type = {None: 0, "norm": 1, "alibi": 2, "spec": 3}[cfg.get("mask")]
    q_len = int(cfg.get("q_len", 1))
    rows = cfg["batch"] * q_len  # query tokens of one step
    pa_param = b.PagedAttentionParam(headNum=cfg["heads"], kvHeadNum=cfg["kv_heads"], qkScale=scale,
                                     quantType=1 if int8 else 0, mlaVHeadSize=cfg["dv"] if mla else 0,
                                     maskType=mask_type, calcType=1 if q_len > 1 else 0,
                                     inputLayout=1 if cfg.get("bnsd") else 0)
    if cfg.get("bnsd"):
        args.attention_only = True
    split = bool(cfg.get("split"))
    if split:
        pa = b.OperationRunner("MultiLatentAttentionOperation", b.MultiLatentAttentionParam(
            headNum=cfg["heads"], kvHeadNum=1, qkScale=scale, cacheMode=1), ctx)
    else:
        pa = b.OperationRunner("PagedAttentionOperation", pa_param, ctx)
    rac = None
    k = b.kernels()
    lens_host = step["context_lens"]
    host_inputs = {}
    with torch.cuda.stream(stream):
        lens_dev = lens_host.to(dev)
        if split:
            dv = cfg["dv"]
            nope, rope = step["key_cache"][..., :dv].contiguous(), step["key_cache"][..., dv:].contiguous()
            pa_in = [step["q"][..., :dv].contiguous(), step["q"][..., dv:].contiguous(), nope, rope,
                     step["block_tables"], lens_dev]
            host_idx = 5
            # the latent and rotary rows of the new token go to their caches as the K and V of one cache write
            rac = b.OperationRunner("ReshapeAndCacheOperation", b.ReshapeAndCacheParam(), ctx)
            rac_in = [step["k_new"][..., :dv].contiguous(), step["k_new"][..., dv:].contiguous(), nope, rope,
                      step["slot_mapping"]]
            rac_out = [nope, rope]  # (the combined copy stays for the CPU baseline, which concatenates anyway)
        elif mla:
            pa_in = [step["q"], step["key_cache"], step["block_tables"], lens_dev]
            host_idx = 3
            rac = b.OperationRunner("ReshapeAndCacheOperation", b.ReshapeAndCacheParam(kvCacheCfg=1), ctx)
            rac_in = [step["k_new"], step["key_cache"], step["slot_mapping"]]
            rac_out = [step["key_cache"]]
        else:
            pa_in = [step["q"], step["key_cache"], step["value_cache"], step["block_tables"], lens_dev]
            if cfg.get("bnsd"):
                pa_in[1] = step["key_cache"].permute(0, 2, 1, 3).contiguous()
                pa_in[2] = step["value_cache"].permute(0, 2, 1, 3).contiguous()
            host_idx = 4
            if mask_type:
                pa_in.append(step["mask"])
            if q_len > 1:
                host_inputs[len(pa_in)] = step["q_lens"]
                pa_in.append(step["q_lens"].to(dev))
            if int8:
                pa_in += [step["k_scale"], step["v_scale"]]
            else:
                rac = b.OperationRunner("ReshapeAndCacheOperation", b.ReshapeAndCacheParam(), ctx)
                rac_in = [step["k_new"], step["v_new"], step["key_cache"], step["value_cache"], step["slot_mapping"]]
                rac_out = [step["key_cache"], step["value_cache"]]
        host_inputs[host_idx] = lens_host
        out = torch.empty((rows, cfg["heads"], cfg["dv"]), dtype=step["q"].dtype, device=dev)
    slots = cfg["block"] * step["layout"]["pool"]

    def one_step():
        if not args.attention_only:
            if int8:
                # the quantised cache write: fp16 rows -> int8 slots
                rc = k.atbmi_reshape_and_cache_quant(
                    step["k_new"].data_ptr(), step["v_new"].data_ptr(), b.ATBMI_F16, step["k_scale"].data_ptr(),
                    step["v_scale"].data_ptr(), step["key_cache"].data_ptr(), step["value_cache"].data_ptr(),
                    step["slot_mapping"].data_ptr(), rows, cfg["kv_heads"], cfg["d"], cfg["dv"], slots,
                    stream.cuda_stream)
                assert rc == 0, b.last_kernel_error()
            else:
                rac.run(rac_in, outputs=rac_out)
        pa.run(pa_in, outputs=[out], host_inputs=host_inputs)

    if args.calibrate_copy:
        with torch.cuda.stream(stream):
            src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
            dst = torch.empty_like(src)
            dst.copy_(src)
        stream.synchronize()
    with torch.cuda.stream(stream):
        for _ in range(args.warmup):
            one_step()
        stream.synchronize()
        torch.cuda.synchronize()
        # every 4th attention launch is bracketed with HIP events on the launch stream
        k.atbmi_timing_enable(0 if args.no_kernel_events else 4)
        t0 = time.perf_counter()
        for _ in range(args.steps):
            one_step()
        stream.synchronize()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
    import ctypes
    total_ms = ctypes.c_double(0)
    launches = ctypes.c_int64(0)
    k.atbmi_timing_read(ctypes.byref(total_ms), ctypes.byref(launches))
    k.atbmi_timing_enable(0)

    ms_per_step = (t1 - t0) * 1e3 / args.steps
    alg_bytes = w.algorithmic_bytes(cfg, step["layout"]["ctx"])
    kernel_ms = total_ms.value / max(1, launches.value)
    achieved = alg_bytes / (kernel_ms * 1e-3) / 1e9 if kernel_ms > 0 else 0.0
    result = {
        "metric": "paged_attention_decode_tokens_per_s",
        "value": rows / (ms_per_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8" if int8 else cfg["dtype"],
        "data": "synthetic",
        "config": {"workload": DESCRIPTIONS[args.config], "step": ("%s only" if args.attention_only else "ReshapeAndCache + %s (Setup + Execute each)") % (
                       "MultiLatentAttention" if split else "PagedAttention"),
                   "context_tokens": int(step["layout"]["ctx"].sum())},
        "roofline": {"bound": "hbm", "kernel": "paged attention decode", "achieved": achieved,
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
                     "traffic": MEASURED_TRAFFIC.get((args.config, alg_bytes)),
                     "algorithmic_bytes": alg_bytes, "kernel_ms": kernel_ms, "launches": launches.value},
        "step_hbm_gbps": alg_bytes / (ms_per_step * 1e-3) / 1e9,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(pkg, step, cfg, scale)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
