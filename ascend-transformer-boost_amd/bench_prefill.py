#!/usr/bin/env python3
"""Times MultiLatentAttentionOperation with calcType PREFILL on one MI355X and prints one JSON line per
workload: DeepSeek-V3-shaped prompts (128 heads of 128 + 64 query / key channels and 128 value channels, bf16)
with the causal mask, without a mask and with a sliding window, through atb::Operation (Setup + Execute per
call). The kernel is bound by the matrix cores: `roofline.achieved` is the algorithmic flops (2 x (192 + 128)
per visible (query, key) pair and head) over the mean time of a call between HIP events on the launch stream,
against the dense bf16 MFMA peak.

    python3 ascend-transformer-boost_amd/bench_prefill.py [--steps 20] [--warmup 3] [--only INDEX]
"""
import argparse
import importlib
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
MFMA_PEAK_TFLOPS = 2500.0

WORKLOADS = [
    # name, sequence lengths, heads, maskType, window
    ("causal, 4 prompts of 4 096 tokens", [4096] * 4, 128, 3, 0),
    ("causal, 1 prompt of 16 384 tokens", [16384], 128, 3, 0),
    ("causal, ragged prompts (8 of 300 .. 6 000 tokens)", [300, 6000, 1500, 4096, 777, 2048, 5000, 129], 128, 3, 0),
    ("no mask, 2 prompts of 4 096 tokens", [4096] * 2, 128, 0, 0),
    ("sliding window of 1 024, 2 prompts of 8 192 tokens", [8192] * 2, 128, 4, 1024),
]


def visible_pairs(lens, mask_type, window):
    total = 0
    for n in lens:
        if mask_type == 0:
            total += n * n
        elif mask_type == 4:
            total += sum(min(i + 1, window) for i in range(n))
        else:
            total += n * (n + 1) // 2
    return total


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--only", type=int, default=None, help="time only the workload with this index")
    args = ap.parse_args()
    import torch
    pkg = importlib.import_module(os.path.basename(HERE))
    b = pkg.binding
    if not torch.cuda.is_available():
        sys.exit("bench_prefill.py: no GPU visible")
    dev = torch.device("cuda:0")
    stream = torch.cuda.Stream(device=dev)
    ctx = b.Context(stream)
    scale = 1.0 / (192.0 ** 0.5)
    for name, lens, heads, mask_type, window in (WORKLOADS if args.only is None else [WORKLOADS[args.only]]):
        tokens, longest = sum(lens), max(lens)
        with torch.cuda.stream(stream):
            mk = lambda *shape: (torch.randn(shape, device=dev) * 0.5).to(torch.bfloat16)
            q, qr = mk(tokens, heads, 128), mk(tokens, heads, 64)
            if mask_type == 3:  # CAUSAL_MASK takes the keys padded per sequence
                k, kr, v = (mk(len(lens), longest, heads * c) for c in (128, 64, 128))
            else:
                k, kr, v = mk(tokens, heads, 128), mk(tokens, heads, 64), mk(tokens, heads, 128)
            out = torch.empty((tokens, heads, 128), dtype=torch.bfloat16, device=dev)
        lens_t = torch.tensor(lens, dtype=torch.int32)
        ins = [q, qr, k, kr, v, lens_t.to(dev), lens_t.to(dev)]
        if mask_type == 4:
            ins.append(torch.zeros((longest, longest), dtype=torch.bfloat16, device=dev))
        op = b.OperationRunner("MultiLatentAttentionOperation", b.MultiLatentAttentionParam(
            headNum=heads, kvHeadNum=heads, qkScale=scale, cacheMode=1, calcType=4, maskType=mask_type,
            windowSize=window), ctx)
        host = {5: lens_t, 6: lens_t}
        with torch.cuda.stream(stream):
            for _ in range(args.warmup):
                op.run(ins, outputs=[out], host_inputs=host)
            start = torch.cuda.Event(enable_timing=True)
            stop = torch.cuda.Event(enable_timing=True)
            start.record(stream)
            for _ in range(args.steps):
                op.run(ins, outputs=[out], host_inputs=host)
            stop.record(stream)
        stream.synchronize()
        ms = start.elapsed_time(stop) / args.steps
        flops = visible_pairs(lens, mask_type, window) * heads * 2 * (192 + 128)
        achieved = flops / (ms * 1e-3) / 1e12
        print(json.dumps({"operation": "MultiLatentAttentionOperation (calcType PREFILL)",
                          "workload": "%s, %d heads, bf16" % (name, heads), "ms_per_call": ms,
                          "tokens_per_s": tokens / (ms * 1e-3),
                          "roofline": {"bound": "mfma", "achieved": achieved, "peak": MFMA_PEAK_TFLOPS,
                                       "unit": "TFLOP/s", "frac": achieved / MFMA_PEAK_TFLOPS,
                                       "algorithmic_flops": flops}}), flush=True)
        op.close()
        del q, qr, k, kr, v, out, ins
        torch.cuda.empty_cache()
    ctx.close()


if __name__ == "__main__":
    main()
