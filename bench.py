#!/usr/bin/env python3
"""Decode-step benchmark: ReshapeAndCache + PagedAttention through atb::Operation
on one MI355X, synthetic data of the named configuration.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c2]

Prints ONE JSON line: whole-step throughput (tokens/s = sequences decoded per
second, inputs resident in HBM; --warmup untimed steps, then exactly --steps
timed ones between two synchronisations, no events inside), the attention
kernel's achieved HBM bandwidth against the 8 TB/s roofline, and the CPU oracle
timed on a bounded sample of the same workload. The kernel figures come from two
more passes over the same inputs, attention only, at least 100 launches each:
one with HIP events on the launch stream around every attention kernel (mean,
median, 10th and 90th percentile of its duration), one with events around every
whole call, attention kernel + merge kernel, nothing between them
(`frac_with_merge`). Run without --config, the line describes the bf16
8B-shaped step (C2) and carries, under "configs", the same measurements of the
other workloads of the benchmark (C2 in fp16, C3 int8-KV, C4 skewed, C5 MLA) and,
under "reference_perf_rows", the three shapes the reference publishes its own
timings for.
"""
import argparse
import hashlib
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

# The sources each workload's attention and merge kernels are compiled from: a traffic figure is tied to the hash
# of exactly these, so an edit elsewhere leaves it standing and an edit here withdraws it.
_COMMON = ["atbmi_common.h", "pa_internal.h", "pa_host.hip", "pa_reduce.hip"]
_MFMA = _COMMON + ["pa_mfma_kernel.h", "pa_mfma.hip", "pa_mfma_dispatch.inc"]
_MLA = _MFMA + ["pa_mla_kernel.h", "pa_mla.hip"]
WORKLOAD_SOURCES = {
    "c2": _MFMA + ["pa_mfma_bf16.hip"], "c2_alibi": _MFMA + ["pa_mfma_bf16.hip"], "c2_norm": _MFMA + ["pa_mfma_bf16.hip"],
    "c2_mtp4": _MFMA + ["pa_mfma_bf16.hip"], "c2_bnsd": _MFMA + ["pa_mfma_bf16.hip"],
    "c1": _MFMA + ["pa_mfma_f16.hip"], "c2_fp16": _MFMA + ["pa_mfma_f16.hip"], "c4": _MFMA + ["pa_mfma_f16.hip"],
    "c3": _MFMA + ["pa_mfma_int8.hip"],
    "c5": _MLA, "c5_split": _MLA, "c5_nz": _MLA, "c5_h16": _MLA, "c5_h32": _MLA,
    "c5_int8": ["atbmi_common.h", "pa_internal.h", "mla_int8.hip"],
    "c3_int8q": ["atbmi_common.h", "pa_internal.h", "pa_int8q.hip"],
}

# HBM bytes one attention call moves (attention kernel + its merge kernel), from rocprofv3 FETCH_SIZE /
# WRITE_SIZE counter runs of this script, scaled by what the same counters read for a 256 MiB copy
# (--calibrate-copy). Each figure names the profile summary it comes from and the hash of its workload's kernel
# sources at the time it was measured: a changed workload or changed kernels report null, not a stale figure.
MEASURED_TRAFFIC = {
    # (workload, algorithmic bytes): (HBM bytes, summary under profiles/, source hash of the workload)
    ("c2", 651658484): (659493149, "pa_mfma_bf16_d128_c2_trace_and_traffic.md", "39ccea2a1dcb"),
    ("c2_fp16", 651658484): (659489879, "pa_mfma_fp16_d128_c2_fp16_trace_and_traffic.md", "81b016f9ec73"),
    ("c3", 1364204576): (1381768462, "pa_mfma_int8_d128_c3_trace_and_traffic.md", "61638a628ebd"),
    ("c3_int8q", 1363148320): (1379036066, "pa_int8q_d128_c3_sizes_trace_counters_traffic.md", "f19d2f9626c2"),
    ("c4", 722875880): (728783707, "pa_mfma_fp16_d128_c4_trace_and_traffic.md", "81b016f9ec73"),
    ("c5_h16", 237786736): (249995659, "pa_mla_bf16_d576_c5_16_heads_trace_and_traffic.md", "af5ed28e4ff4"),
    ("c5", 253384304): (342817654, "pa_mla_bf16_d576_c5_trace_and_traffic.md", "af5ed28e4ff4"),
}
OTHER_WORKLOADS = ["c2_fp16", "c3", "c3_int8q", "c4", "c5"]  # timed in the same run as the headline workload
MIN_KERNEL_LAUNCHES = 100  # launches behind every kernel figure, whatever --steps says
MALL_BYTES = 256 << 20     # memory-side cache of the MI355X


def kernel_source_hash(workload):
    """Short hash of the sources `workload`'s attention and merge kernels are built from."""
    h = hashlib.sha256()
    for name in WORKLOAD_SOURCES[workload]:
        with open(os.path.join(ROOT, PKG, "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:12]


def cpu_description():
    """(logical cores of the host, model string) as the kernel reports them."""
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return os.cpu_count() or 1, model


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
    "c3_int8q": "C3 with int8 queries (quantType TYPE_QUANT_QKV_ONLINE: int8 q, k, v, one descale per query head; random "
                "int8 contents), attention only: batch 128, 64 q heads, 8 kv heads, d128, block 128, ctx U[2048,8192], "
                "fp16 out",
    "c4": "C4 skewed long-context fp16 decode: batch 16, 32 q heads, 8 kv heads, d128, ctx lognormal(median 8k) in [256,32768]",
    "c5_split": "C5 through MultiLatentAttentionOperation (cacheMode KROPE_CTKV: 512 latent + 64 rotary channels in "
                "two caches): batch 64, 128 q heads, block 128, ctx U[2048,4096], bf16",
    "c5_nz": "C5 through MultiLatentAttentionOperation with cacheMode NZCACHE (fractal-NZ caches [blocks, 32 | 4, 128, 16]), "
             "attention only: batch 64, 128 q heads, block 128, ctx U[2048,4096], bf16",
    "c5_int8": "C5 through MultiLatentAttentionOperation with cacheMode INT8_NZCACHE (int8 query and latent cache, "
               "fractal-NZ, bf16 rotary parts; random int8 contents), attention only: batch 64, 128 q heads, block 128, "
               "ctx U[2048,4096]",
    "c5": "C5 MLA bf16 decode: batch 64, 128 q heads, 1 latent kv head, d576/dv512, block 128, ctx U[2048,4096]",
    "c5_h16": "C5 on one of eight tensor-parallel ranks (16 of the 128 q heads, the whole latent cache): batch 64, "
              "d576/dv512, block 128, ctx U[2048,4096], bf16",
    "c5_h32": "C5 on one of four tensor-parallel ranks (32 of the 128 q heads, the whole latent cache): batch 64, "
              "d576/dv512, block 128, ctx U[2048,4096], bf16",
}


def cpu_baseline(pkg, step, cfg, scale, budget_s=10.0):
    """Times the numpy oracle on the sequences of the batch, taken in order and
    again from the first once all are done, until about `budget_s` seconds of CPU
    work are spent; returns tokens/s (one token per sequence) on that sample."""
    import numpy as np
    oracle = importlib.import_module("oracle.atb_oracle")
    # threads numpy's BLAS may use (the oracle's matrix products are the only parallel part)
    try:
        from threadpoolctl import threadpool_info
        threads = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
    except ImportError:
        threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
    host_cores, cpu_model = cpu_description()
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
        "host_cores": host_cores,
        "cpu_model": cpu_model,
        "kind": "port",
        "sample": "numpy oracle on %d query tokens of sequences drawn in order from the batch of %d "
                  "(%d context tokens), attention only, %.1f s" % (done, len(ctx), tokens, spent),
    }


def run_workload(pkg, name, steps, warmup, attention_only=False, kernel_events=True, calibrate_copy=False,
                 want_cpu_baseline=False):
    """Sets one workload up on cuda:0, times `steps` decode steps after `warmup` untimed ones and returns
    the measurements (and, on request, the CPU baseline on the same inputs)."""
    import ctypes
    import torch
    b, w = pkg.binding, pkg.workloads
    dev = torch.device("cuda:0")
    cfg = w.config(name)
    step = w.make_step(cfg, dev)
    scale = w.qk_scale(cfg)
    stream = torch.cuda.Stream(device=dev)
    ctx = b.Context(stream)
    int8 = cfg["kv"] == "int8"
    mla = bool(cfg.get("mla"))

    mask_type = {None: 0, "norm": 1, "alibi": 2, "spec": 3}[cfg.get("mask")]
    q_len = int(cfg.get("q_len", 1))
    rows = cfg["batch"] * q_len  # query tokens of one step
    int8q = bool(cfg.get("int8q"))
    pa_param = b.PagedAttentionParam(headNum=cfg["heads"], kvHeadNum=cfg["kv_heads"], qkScale=scale,
                                     quantType=3 if int8q else (1 if int8 else 0),
                                     outDataType=b.ACL_FLOAT16 if int8q else 0, mlaVHeadSize=cfg["dv"] if mla else 0,
                                     maskType=mask_type, calcType=1 if q_len > 1 else 0,
                                     inputLayout=1 if cfg.get("bnsd") else 0)
    nz = bool(cfg.get("nz"))
    if cfg.get("bnsd") or nz or int8q:
        attention_only = True
    split = bool(cfg.get("split"))
    if split:
        pa = b.OperationRunner("MultiLatentAttentionOperation", b.MultiLatentAttentionParam(
            headNum=cfg["heads"], kvHeadNum=1, qkScale=scale,
            cacheMode=2 if cfg.get("int8nz") else (3 if nz else 1)), ctx)
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
            if nz:
                # [blocks, block, 1, channels] -> [blocks, channels / 16, block, 16], described in the fractal-NZ format
                nz_caches = [t[:, :, 0, :].reshape(t.shape[0], t.shape[1], -1, 16).permute(0, 2, 1, 3).contiguous()
                             for t in (nope, rope)]
                if cfg.get("int8nz"):
                    # int8 latent parts with random contents, slabs of 32 channels; one descale per head each
                    nz_caches[0] = torch.randint(-5, 6, (nope.shape[0], dv // 32, nope.shape[1], 32), dtype=torch.int8,
                                                 device=dev)
                    pa_in[0] = torch.randint(-5, 6, tuple(pa_in[0].shape), dtype=torch.int8, device=dev)
                    descales = [torch.rand(cfg["heads"], device=dev) * 0.04 + 0.001 for _ in range(2)]
                    pa_in += descales
                pa_in[2:4] = [b.make_tensor(b._torch_acl_dtype(t), list(t.shape), device_ptr=t.data_ptr(),
                                            fmt="fractal_nz") for t in nz_caches]
        elif mla:
            pa_in = [step["q"], step["key_cache"], step["block_tables"], lens_dev]
            host_idx = 3
            if mask_type:
                pa_in.append(step["mask"])
            if q_len > 1:
                host_inputs[len(pa_in)] = step["q_lens"]
                pa_in.append(step["q_lens"].to(dev))
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
            if int8q:
                pa_in[0] = torch.randint(-5, 6, tuple(step["q"].shape), dtype=torch.int8, device=dev)
                pa_in += [torch.rand(cfg["heads"], device=dev) * 0.04 + 0.001 for _ in range(2)]
            elif int8:
                pa_in += [step["k_scale"], step["v_scale"]]
            else:
                rac = b.OperationRunner("ReshapeAndCacheOperation", b.ReshapeAndCacheParam(), ctx)
                rac_in = [step["k_new"], step["v_new"], step["key_cache"], step["value_cache"], step["slot_mapping"]]
                rac_out = [step["key_cache"], step["value_cache"]]
        host_inputs[host_idx] = lens_host
        out = torch.empty((rows, cfg["heads"], cfg["dv"]), dtype=step["q"].dtype, device=dev)
        # A working set that fits the 256 MB memory-side cache would be served from there when every step reads
        # the same tensors: such a workload gets copies of its caches, enough for 768 MB, and the steps go
        # round them, so that a step's rows were last touched at least 512 MB of traffic ago.
        pools = [(pa_in, rac_in if rac is not None else None, rac_out if rac is not None else None)]
        caches = []        # (an object of the lists above, what makes a copy of it, the bytes the attention reads of it)
        alive = []         # tensors behind the descriptors of copies
        size = lambda t: t.numel() * t.element_size()
        if split:
            caches += [(t, t.clone, 0 if nz else size(t)) for t in (nope, rope)]
            if nz:
                def described_copy(t):
                    alive.append(t.clone())
                    return b.make_tensor(b._torch_acl_dtype(alive[-1]), list(alive[-1].shape),
                                         device_ptr=alive[-1].data_ptr(), fmt="fractal_nz")
                caches += [(pa_in[2 + i], (lambda t=t: described_copy(t)), size(t)) for i, t in enumerate(nz_caches)]
        elif not int8 and not cfg.get("bnsd"):
            caches += [(step[n], step[n].clone, size(step[n])) for n in ("key_cache", "value_cache")
                       if step.get(n) is not None]
        cache_bytes = sum(c[2] for c in caches)
        if 0 < cache_bytes < MALL_BYTES * 2:
            for _ in range(-(-MALL_BYTES * 3 // cache_bytes) - 1):
                copies = {id(obj): copy() for obj, copy, _ in caches}
                swap = lambda ts: None if ts is None else [copies.get(id(t), t) for t in ts]
                pools.append((swap(pa_in), swap(pools[0][1]), swap(pools[0][2])))
    slots = cfg["block"] * step["layout"]["pool"]
    turn = [0]

    def next_pool():
        turn[0] += 1
        return pools[turn[0] % len(pools)]

    def one_step():
        pa_in, rac_in, rac_out = next_pool()
        if not attention_only:
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

    if calibrate_copy:
        with torch.cuda.stream(stream):
            src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
            dst = torch.empty_like(src)
            dst.copy_(src)
        stream.synchronize()
    import numpy as np

    def timed_pass(count, whole):
        """`count` attention calls on the same inputs, every one bracketed with HIP events on the launch stream:
        around the attention kernel (whole = False) or around attention + merge as one interval (whole = True).
        Returns the durations in milliseconds."""
        k.atbmi_timing_whole_calls(1 if whole else 0)
        k.atbmi_timing_enable(1)
        for _ in range(count):
            pa.run(next_pool()[0], outputs=[out], host_inputs=host_inputs)
        stream.synchronize()
        first = (ctypes.c_float * count)()
        second = (ctypes.c_float * count)()
        got = ctypes.c_int64(0)
        rc = k.atbmi_timing_read_samples(first, second, count, ctypes.byref(got))
        k.atbmi_timing_enable(0)
        k.atbmi_timing_whole_calls(0)
        assert rc == 0, b.last_kernel_error()
        return np.array((second if whole else first)[:got.value], dtype=np.float64)

    with torch.cuda.stream(stream):
        for _ in range(warmup):
            one_step()
        stream.synchronize()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            one_step()
        stream.synchronize()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        kernel_samples = with_merge_samples = np.zeros(0)
        if kernel_events:
            launches_wanted = max(steps, MIN_KERNEL_LAUNCHES)
            kernel_samples = timed_pass(launches_wanted, whole=False)
            with_merge_samples = timed_pass(launches_wanted, whole=True)

    def spread(samples):
        if len(samples) == 0:
            return {"mean": 0.0, "median": 0.0, "p10": 0.0, "p90": 0.0}
        return {"mean": float(samples.mean()), "median": float(np.median(samples)),
                "p10": float(np.percentile(samples, 10)), "p90": float(np.percentile(samples, 90))}

    ms_per_step = (t1 - t0) * 1e3 / steps
    alg_bytes = w.algorithmic_bytes(cfg, step["layout"]["ctx"])
    kernel_stats, with_merge_stats = spread(kernel_samples), spread(with_merge_samples)
    kernel_ms, with_merge_ms = kernel_stats["mean"], with_merge_stats["mean"]
    achieved = alg_bytes / (kernel_ms * 1e-3) / 1e9 if kernel_ms > 0 else 0.0
    with_merge = alg_bytes / (with_merge_ms * 1e-3) / 1e9 if with_merge_ms > 0 else 0.0
    traffic, source = None, None
    entry = MEASURED_TRAFFIC.get((name, alg_bytes))
    if entry is not None:
        if entry[2] == kernel_source_hash(name):
            traffic, source = entry[0], "profiles/" + entry[1]
        else:
            source = "none: the kernels of this workload changed since profiles/%s was taken" % entry[1]
    measured = {
        "workload": DESCRIPTIONS[name],
        "step": ("%s only" if attention_only else "ReshapeAndCache + %s (Setup + Execute each)") % (
            "MultiLatentAttention" if split else "PagedAttention"),
        "context_tokens": int(step["layout"]["ctx"].sum()),
        "cache_copies": len(pools),  # > 1: the steps go round copies of the caches (see run_workload)
        "rows": rows,
        "dtype": "int8" if int8 else cfg["dtype"],
        "steps": steps,
        "ms_per_step": ms_per_step,
        "tokens_per_s": rows / (ms_per_step * 1e-3),
        "roofline": {"bound": "hbm", "kernel": "paged attention decode", "achieved": achieved,
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
                     "frac_with_merge": with_merge / HBM_PEAK_GBPS, "traffic": traffic, "traffic_source": source,
                     "algorithmic_bytes": alg_bytes, "kernel_ms": kernel_ms, "kernel_ms_spread": kernel_stats,
                     "kernel_with_merge_ms": with_merge_ms, "kernel_with_merge_ms_spread": with_merge_stats,
                     "launches": int(len(kernel_samples)),
                     "method": "HIP events on the launch stream around every attention kernel of %d attention-only calls; "
                               "frac_with_merge from a second pass of as many calls with one interval around attention + "
                               "merge kernel" % len(kernel_samples)},
        "step_hbm_gbps": alg_bytes / (ms_per_step * 1e-3) / 1e9,
        "kernel_source_hash": kernel_source_hash(name),
    }
    baseline = cpu_baseline(pkg, step, cfg, scale) if want_cpu_baseline else None
    if rac is not None:
        rac.close()
    pa.close()
    ctx.close()
    del step, out, pa_in
    torch.cuda.empty_cache()
    return measured, baseline


def reference_perf_rows(pkg, calls=200, warmup=20):
    """The three shapes the reference keeps timings for (its QA baselines: one whole operator call each, on an
    Ascend NPU it does not name): Setup + Execute + stream synchronisation per call here, microseconds. Reference:
    tests/high_level_test/PagedAttentionOperation/Performance/PagedAttentionOperation_Perf_TestCase.csv:2 with
    PagedAttentionOperation_BaseLine.csv:2, and tests/high_level_test/ReshapeAndCacheOperation/Performance/
    ReshapeAndCacheOperation_Perf_TestCase.csv:2-3 with ReshapeAndCacheOperation_BaseLine.csv:2-3."""
    import numpy as np
    import torch
    b = pkg.binding
    dev = torch.device("cuda:0")
    stream = torch.cuda.Stream(device=dev)
    ctx = b.Context(stream)
    gen = torch.Generator(device=dev).manual_seed(7)
    rows = []

    def time_calls(call):
        with torch.cuda.stream(stream):
            for _ in range(warmup):
                call()
                stream.synchronize()
            samples = []
            for _ in range(calls):
                t0 = time.perf_counter()
                call()
                stream.synchronize()
                samples.append((time.perf_counter() - t0) * 1e6)
        samples = np.array(samples)
        return {"median_us": float(np.median(samples)), "p10_us": float(np.percentile(samples, 10)),
                "p90_us": float(np.percentile(samples, 90)), "calls": calls}

    with torch.cuda.stream(stream):
        caches = [torch.randn((4, 128, 1, 128), generator=gen, device=dev, dtype=torch.float16) for _ in range(2)]
        # PagedAttentionOperation1: q [1, 8, 128], caches [4, 128, 1, 128], block table [1, 4], 8 heads over 1 KV head
        q = torch.randn((1, 8, 128), generator=gen, device=dev, dtype=torch.float16)
        tables = torch.arange(4, dtype=torch.int32, device=dev).reshape(1, 4)
        lens = torch.tensor([512], dtype=torch.int32)
        out = torch.empty((1, 8, 128), dtype=torch.float16, device=dev)
        pa = b.OperationRunner("PagedAttentionOperation",
                               b.PagedAttentionParam(headNum=8, kvHeadNum=1, qkScale=0.0883883461356163), ctx)
        pa_in = [q, caches[0], caches[1], tables, lens.to(dev)]
    measured = time_calls(lambda: pa.run(pa_in, outputs=[out], host_inputs={4: lens}))
    rows.append(dict(measured, case="PagedAttentionOperation1", shape="q [1,8,128], caches [4,128,1,128], table [1,4], "
                     "context 512 (the dump's own length is not in the table: the longest the block table holds)",
                     reference_us=200.555))
    pa.close()
    for case, tokens, ref_us in (("ReshapeAndCacheOperation1", 256, 206.315), ("ReshapeAndCacheOperation2", 1, 187.805)):
        with torch.cuda.stream(stream):
            key = torch.randn((tokens, 1, 128), generator=gen, device=dev, dtype=torch.float16)
            value = torch.randn((tokens, 1, 128), generator=gen, device=dev, dtype=torch.float16)
            slots = torch.randperm(512, generator=gen, device=dev)[:tokens].to(torch.int32)
            rac = b.OperationRunner("ReshapeAndCacheOperation", b.ReshapeAndCacheParam(), ctx)
            rac_in = [key, value, caches[0], caches[1], slots]
        measured = time_calls(lambda: rac.run(rac_in, outputs=[caches[0], caches[1]]))
        rows.append(dict(measured, case=case, shape="key / value [%d,1,128], caches [4,128,1,128]" % tokens,
                         reference_us=ref_us))
        rac.close()
    ctx.close()
    return {"what": "Setup + Execute + stream synchronisation of one operator call, host clock, fp16; reference_us is the "
                    "reference's own QA baseline for the same shape on an unnamed Ascend NPU (context, not a comparison "
                    "on equal hardware)",
            "rows": rows}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default=None, choices=sorted(DESCRIPTIONS),
                    help="time this workload alone (default: c2, followed by the benchmark's other workloads)")
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
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    headline = args.config or "c2"
    m, baseline = run_workload(pkg, headline, args.steps, args.warmup, attention_only=args.attention_only,
                               kernel_events=not args.no_kernel_events, calibrate_copy=args.calibrate_copy,
                               want_cpu_baseline=not args.no_cpu_baseline)
    result = {
        "metric": "paged_attention_decode_tokens_per_s",
        "value": m["tokens_per_s"],
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": m["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": m["dtype"],
        "data": "synthetic",
        "config": {"workload": m["workload"], "step": m["step"], "context_tokens": m["context_tokens"],
                   "cache_copies": m["cache_copies"]},
        "roofline": m["roofline"],
        "step_hbm_gbps": m["step_hbm_gbps"],
        "kernel_source_hash": m["kernel_source_hash"],
    }
    if baseline is not None:
        result["cpu_baseline"] = baseline
    if args.config is None:
        # the other workloads of the benchmark, same procedure; the timed steps are capped so that the
        # whole run stays within a few minutes whatever --steps asks of the headline workload
        others = {}
        for name in OTHER_WORKLOADS:
            om, _ = run_workload(pkg, name, min(args.steps, 100), min(args.warmup, 10),
                                 kernel_events=not args.no_kernel_events)
            others[name] = om
        result["configs"] = others
        result["reference_perf_rows"] = reference_perf_rows(pkg)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
