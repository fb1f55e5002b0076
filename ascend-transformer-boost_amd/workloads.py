"""Seeded synthetic decode-step workloads (the five benchmark configurations).

Each workload is one decode step: new K/V rows for every sequence, the paged
caches, block tables, context lengths (the new token is the last position),
slot mapping and the query. Lengths, tables and slots come from a numpy
PCG64 generator (seed 1000 + config number) so they are identical everywhere;
tensor contents come from a torch generator on the target device with the
same seed.
"""
import math

import numpy as np

CONFIGS = {
    # name: batch, heads, kv_heads, d, dv, block, ctx range, dtype, kv dtype, distribution, value scale
    "c1": dict(batch=4, heads=8, kv_heads=8, d=128, dv=128, block=128, ctx=(64, 512), dtype="float16",
               kv="float16", dist="uniform", std=1.0, pool=64),
    "c2": dict(batch=64, heads=32, kv_heads=8, d=128, dv=128, block=128, ctx=(1024, 4096), dtype="bf16",
               kv="bf16", dist="uniform", std=0.5, pool=None),
    "c2_fp16": dict(batch=64, heads=32, kv_heads=8, d=128, dv=128, block=128, ctx=(1024, 4096), dtype="float16",
                    kv="float16", dist="uniform", std=0.5, pool=None),
    # C2 with the additive masks of the reference's decode tests: ALiBi rows per (sequence, head),
    # and a per-sequence NORM row that hides the first i positions of sequence i
    "c2_alibi": dict(batch=64, heads=32, kv_heads=8, d=128, dv=128, block=128, ctx=(1024, 4096), dtype="bf16",
                     kv="bf16", dist="uniform", std=0.5, pool=None, mask="alibi"),
    "c2_norm": dict(batch=64, heads=32, kv_heads=8, d=128, dv=128, block=128, ctx=(1024, 4096), dtype="bf16",
                    kv="bf16", dist="uniform", std=0.5, pool=None, mask="norm"),
    # C2 as a multi-token (speculative / MTP) decode step: 4 query tokens per sequence, the last 4
    # positions of its context, with the per-query-row causal mask of the reference's tests
    "c2_mtp4": dict(batch=64, heads=32, kv_heads=8, d=128, dv=128, block=128, ctx=(1024, 4096), dtype="bf16",
                    kv="bf16", dist="uniform", std=0.5, pool=None, mask="spec", q_len=4),
    "c3": dict(batch=128, heads=64, kv_heads=8, d=128, dv=128, block=128, ctx=(2048, 8192), dtype="float16",
               kv="int8", dist="uniform", std=1.0, pool=None),
    "c4": dict(batch=16, heads=32, kv_heads=8, d=128, dv=128, block=128, ctx=(256, 32768), dtype="float16",
               kv="float16", dist="lognormal", std=1.0, pool=None),
    "c5": dict(batch=64, heads=128, kv_heads=1, d=576, dv=512, block=128, ctx=(2048, 4096), dtype="bf16",
               kv="bf16", dist="uniform", std=0.3, pool=None, mla=True),
}
# C2 over head-major caches [blocks, kv heads, block, d] (InputLayout TYPE_BNSD); attention only: the reference
# has no cache write for this layout
CONFIGS["c2_bnsd"] = dict(CONFIGS["c2"], bnsd=True)
# C5 as MultiLatentAttentionOperation sees it: the same rows, 512 latent + 64 rotary channels in two
# tensors each for the query and the cache.
CONFIGS["c5_split"] = dict(CONFIGS["c5"], split=True)
CONFIGS["c5_nz"] = dict(CONFIGS["c5"], split=True, nz=True)
CONFIGS["c5_int8"] = dict(CONFIGS["c5"], split=True, nz=True, int8nz=True)
# C5 as one of eight / four tensor-parallel ranks sees it: the same cache, 16 / 32 of the 128 query heads
CONFIGS["c5_h16"] = dict(CONFIGS["c5"], heads=16)
CONFIGS["c5_h32"] = dict(CONFIGS["c5"], heads=32)
# C3 with int8 queries as well (PagedAttentionParam quantType QKV online): the same int8 caches, one descale per query head
CONFIGS["c3_int8q"] = dict(CONFIGS["c3"], int8q=True)

SEEDS = {"c1": 1001, "c2": 1002, "c2_fp16": 1002, "c2_alibi": 1002, "c2_norm": 1002, "c2_mtp4": 1002, "c2_bnsd": 1002, "c3": 1003, "c4": 1004, "c5": 1005, "c5_split": 1005, "c5_nz": 1005, "c5_int8": 1005, "c5_h16": 1005, "c5_h32": 1005, "c3_int8q": 1003}


def config(name, **overrides):
    cfg = dict(CONFIGS[name])
    cfg["name"] = name
    cfg.setdefault("mla", False)
    cfg.update(overrides)
    return cfg


def qk_scale(cfg):
    # DeepSeek-V3 MLA scales by the un-absorbed head size (128 nope + 64 rope).
    return 1.0 / math.sqrt(192.0) if cfg.get("mla") else 1.0 / math.sqrt(cfg["d"])


def draw_lengths(cfg, rng):
    lo, hi = cfg["ctx"]
    b = cfg["batch"]
    if cfg["dist"] == "lognormal":
        # median 8192, sigma 1.0, clipped to the configured range
        x = np.exp(rng.normal(math.log(8192.0), 1.0, size=b))
        return np.clip(np.rint(x), lo, hi).astype(np.int32)
    return rng.integers(lo, hi + 1, size=b, dtype=np.int64).astype(np.int32)


def layout(cfg, seed=None):
    """Host-side structure of a step: lengths, block tables, slot mapping."""
    rng = np.random.Generator(np.random.PCG64(SEEDS.get(cfg["name"], 1) if seed is None else seed))
    ctx = draw_lengths(cfg, rng)
    bs = cfg["block"]
    blocks_per_seq = (ctx.astype(np.int64) + bs - 1) // bs
    total = int(blocks_per_seq.sum())
    pool = cfg["pool"] if cfg.get("pool") else int(math.ceil(total * 1.1))
    max_blocks = int(blocks_per_seq.max())
    perm = rng.permutation(pool)[:total]  # drawn without replacement: every block has one owner
    tables = np.zeros((cfg["batch"], max_blocks), dtype=np.int32)
    pos = 0
    for b in range(cfg["batch"]):
        n = int(blocks_per_seq[b])
        tables[b, :n] = perm[pos:pos + n]
        tables[b, n:] = perm[pos]  # unused entries stay valid block ids
        pos += n
    # the new tokens are the last q_len positions of each context (one for a plain decode step)
    n = int(cfg.get("q_len", 1))
    pos = (ctx.astype(np.int64)[:, None] - n + np.arange(n)[None, :]).reshape(-1)
    seq = np.repeat(np.arange(cfg["batch"]), n)
    slots = (tables[seq, pos // bs].astype(np.int64) * bs + pos % bs).astype(np.int32)
    return dict(ctx=ctx, tables=tables, slots=slots, pool=pool, max_blocks=max_blocks,
                q_lens=np.full(cfg["batch"], n, dtype=np.int32))


def torch_dtype(name):
    import torch
    return {"float16": torch.float16, "bf16": torch.bfloat16, "int8": torch.int8}[name]


def alibi_slopes(heads):
    """2^(-8 k / n), k = 1..n, n the largest power of two <= heads, then 2^(-4 k / n) for odd k
    (reference tests/apitest/kernelstest/mix/test_paged_attention_common.py:74-83)."""
    n = 1 << (int(heads).bit_length() - 1)
    return [2.0 ** (-8.0 * k / n) for k in range(1, n + 1)] + \
           [2.0 ** (-4.0 * k / n) for k in range(1, 1 + 2 * (heads - n), 2)]


def make_mask(cfg, ctx, device):
    """The additive mask of a masked workload, in the query dtype, rows padded to a
    multiple of the block size. "alibi": [batch, heads, 1, maxS], slope_h * (j - ctx_i + 1)
    on the valid positions (reference :489-499); "norm": [batch, 1, maxS], -10000 on the
    first i positions of sequence i (reference :501-505); "spec": [batch * q_len, maxS], for
    the t-th query token of a sequence -10000 on the q_len - 1 - t positions after its own
    (reference tests/apitest/kernelstest/mix/test_paged_attention_mla_mtp.py:220-231)."""
    import torch
    bs = cfg["block"]
    max_s = (int(max(ctx)) + bs - 1) // bs * bs
    lens = torch.as_tensor(np.asarray(ctx), device=device, dtype=torch.float32)
    pos = torch.arange(max_s, device=device, dtype=torch.float32)
    if cfg["mask"] == "alibi":
        slopes = torch.tensor(alibi_slopes(cfg["heads"]), device=device, dtype=torch.float32)
        dist = pos[None, :] - lens[:, None] + 1.0                       # [batch, maxS]
        m = slopes[None, :, None] * torch.where(dist <= 0, dist, torch.zeros_like(dist))[:, None, :]
        return m[:, :, None, :].to(torch_dtype(cfg["dtype"])).contiguous()
    if cfg["mask"] == "spec":
        n = int(cfg["q_len"])
        own = (lens[:, None] - n + torch.arange(n, device=device, dtype=torch.float32)[None, :]).reshape(-1, 1)
        end = lens.repeat_interleave(n)[:, None]
        hidden = (pos[None, :] > own) & (pos[None, :] < end)
        m = torch.where(hidden, torch.full((1, 1), -10000.0, device=device), torch.zeros((1, 1), device=device))
        return m.to(torch_dtype(cfg["dtype"])).contiguous()
    row = torch.arange(len(ctx), device=device, dtype=torch.float32)
    m = torch.where(pos[None, :] < row[:, None], torch.full((1, 1), -10000.0, device=device),
                    torch.zeros((1, 1), device=device))
    return m[:, None, :].to(torch_dtype(cfg["dtype"])).contiguous()


def make_step(cfg, device, seed=None):
    """Tensors of one decode step on `device` (torch). Returns a dict:
    q, k_new, v_new (query dtype), key_cache, value_cache (kv dtype; value_cache
    is None for MLA), k_scale/v_scale (fp32, int8 caches only), block_tables,
    slot_mapping (int32, device), context_lens and q_lens (int32, CPU), mask (query
    dtype, or None) and cfg/layout."""
    import torch
    lay = layout(cfg, seed)
    gen = torch.Generator(device=device)
    gen.manual_seed(SEEDS.get(cfg["name"], 1) if seed is None else seed)
    qdt = torch_dtype(cfg["dtype"])
    b, h, g, d, dv, bs = cfg["batch"], cfg["heads"], cfg["kv_heads"], cfg["d"], cfg["dv"], cfg["block"]
    b *= int(cfg.get("q_len", 1))  # query / new K,V rows: one per query token
    pool = lay["pool"]
    std = cfg["std"]

    def normal(shape, s):
        return torch.randn(shape, generator=gen, device=device, dtype=torch.float32) * s

    out = dict(cfg=cfg, layout=lay)
    out["q"] = normal((b, h, d), 1.0 if cfg["kv"] == "int8" else std).to(qdt)
    if cfg["kv"] == "int8":
        out["k_scale"] = torch.rand((g * d,), generator=gen, device=device) * 0.015 + 0.005
        out["v_scale"] = torch.rand((g * dv,), generator=gen, device=device) * 0.015 + 0.005
        out["key_cache"] = torch.randint(-127, 128, (pool, bs, g, d), generator=gen, device=device,
                                         dtype=torch.int8)
        out["value_cache"] = torch.randint(-127, 128, (pool, bs, g, dv), generator=gen, device=device,
                                           dtype=torch.int8)
        out["k_new"] = normal((b, g, d), 0.5).to(qdt)
        out["v_new"] = normal((b, g, dv), 0.5).to(qdt)
    else:
        # generated block-wise so the fp32 staging buffer stays small
        kc = torch.empty((pool, bs, g, d), device=device, dtype=qdt)
        step = max(1, (1 << 26) // (bs * g * d))
        for i in range(0, pool, step):
            n = min(step, pool - i)
            kc[i:i + n] = normal((n, bs, g, d), std).to(qdt)
        out["key_cache"] = kc
        if cfg.get("mla"):
            out["value_cache"] = None
        else:
            vc = torch.empty((pool, bs, g, dv), device=device, dtype=qdt)
            for i in range(0, pool, step):
                n = min(step, pool - i)
                vc[i:i + n] = normal((n, bs, g, dv), std).to(qdt)
            out["value_cache"] = vc
        out["k_new"] = normal((b, g, d), std).to(qdt)
        out["v_new"] = None if cfg.get("mla") else normal((b, g, dv), std).to(qdt)
    out["block_tables"] = torch.from_numpy(lay["tables"]).to(device)
    out["slot_mapping"] = torch.from_numpy(lay["slots"]).to(device)
    out["context_lens"] = torch.from_numpy(lay["ctx"].copy())
    out["mask"] = make_mask(cfg, lay["ctx"], device) if cfg.get("mask") else None
    out["q_lens"] = torch.from_numpy(lay["q_lens"].copy())
    return out


def algorithmic_bytes(cfg, ctx):
    """HBM bytes a decode-attention call must move: valid K/V rows + q + out +
    block-table entries + context lengths (+ scale vectors for an int8 cache, + the
    mask rows over the valid positions). With several query tokens per sequence K and V
    still count once per sequence; q, out and the mask count per query row."""
    kv = 1 if cfg["kv"] == "int8" else 2
    g, d, dv, h, bs = cfg["kv_heads"], cfg["d"], cfg["dv"], cfg["heads"], cfg["block"]
    ctx = np.asarray(ctx, dtype=np.int64)
    per_tok = g * (d if cfg.get("mla") else d + dv) * kv
    n = int(cfg.get("q_len", 1))
    rows = int((ctx > 0).sum()) * n
    total = int(ctx.sum()) * per_tok + rows * h * (d + dv) * 2
    if cfg.get("int8q"):  # int8 query rows, 16-bit output rows, two descales per query head instead of per channel
        total = int(ctx.sum()) * per_tok + rows * h * (d + dv * 2) + 2 * h * 4 - g * (d + dv) * 4
    if cfg.get("int8nz"):  # 512 int8 + 64 16-bit channels per cache row; 512 int8 + 64 16-bit per query row and head
        total = int(ctx.sum()) * (512 + 64 * 2) + rows * h * (512 + 64 * 2 + dv * 2) + 2 * h * 4
    total += int(((ctx + bs - 1) // bs).sum()) * 4 + len(ctx) * 4
    if cfg["kv"] == "int8":
        total += g * (d + dv) * 4
    if cfg.get("mask"):
        total += int(ctx.sum()) * n * (h if cfg["mask"] == "alibi" else 1) * 2
    if n > 1:
        total += len(ctx) * 4  # the query lengths
    return total
