"""CPU oracle for the PagedAttention-decode / ReshapeAndCache path.

TEST INFRASTRUCTURE ONLY. This is the checker the GPU kernels are compared
against; nothing in the product may import it (only tests/, the smoke entry
and the benchmark's cpu_baseline leg do).

It restates, in numpy, the reference's own CPU goldens for these operators.
The reference itself cannot be built here (its host code needs the CANN
toolkit and the MKI library, its device code the AscendC compiler), and its
Python test files import torch_npu at module level, so nothing of it is
executed; every function below follows the cited reference lines and is
pinned by tests/test_oracle.py against closed forms, fp64 brute force and
the invariants of the mathematics (no function is left "parity unpinned"):

  reshape_and_cache   tests/apitest/kernelstest/mix/test_reshape_and_cache.py:45-65
  reshape_and_cache_nz
                      tests/apitest/kernelstest/mix/test_reshape_and_cache_nz.py:45-66 (fractal-NZ caches
                      [blocks, channels / last, block_size, last], last = 32 for int8 keys, else 16); pinned by
                      element loops over flat addresses and by nz_to_nd of the result = the plain write
  reshape_and_cache_compress
                      tests/apitest/kernelstest/mix/test_reshape_and_cache_wins.py:61-88 (the last wins[i]
                      tokens of every (sequence, head) pair) and test_reshape_and_cache_wins_rope.py:78-131 (a
                      window replaced by its mean); pinned by element loops over flat addresses, the slot
                      counts, a one-token window = plain copy, and the float64 mean
  reshape_and_cache_omni
                      tests/framework/python/CsvOpsTestTool/data_generation.py:9797-9846 and
                      tests/apitest/kernelstest/mix/test_reshape_and_cache_omni_compress.py:80-116 (a window of
                      tokens per (sequence, head) pair is left out); pinned by element loops over flat addresses
                      with an index list built another way, the slot counts, no window = the plain write of one
                      head, and mean-window's result with its mean slot taken out
  dequant_per_channel tests/apitest/opstest/python/operations/elewise/test_elewise_dequant.py:23-31
  strided_view        tests/unittest/ops/reshape_and_cache_with_stride/test_reshape_and_cache_with_stride.cpp:
                      219-245 (element [i0, i1, i2] of the view is storage[offset + sum(i_k * stride_k)]),
                      :411-433 (the view then goes through the plain reshape_and_cache golden)
  rope                tests/apitest/opstest/python/operations/rope/test_rope_operation2.py:120-218 (the general
                      form: rows cut into units of the table row size, a unit into rotaryCoeff / 2 chunks, in a
                      chunk first half <- -second half, second half <- first half, times sin, plus x times
                      cos), :86-101 (fp32 arithmetic, one rounding), test_rope_operation3.py:29-55 (cosFormat 1:
                      table row = position inside the token's sequence)
  norm_rope_reshape   tests/apitest/opstest/python/operations/norm_rope_reshape/test_norm_rope_reshape.py:21-71
                      and tests/apitest/kernelstest/mix/test_rms_norm_and_rope_and_reshape_and_cache_bf16.py:24-74
                      (rms = 1 / sqrt(mean(x^2) + eps); x * rms * gamma; r * cos + rotate_half(r) * sin with
                      rotate_half = concat(-second half, first half); both written side by side into the slot)
  quant_per_channel   tests/apitest/opstest/python/operations/elewise/test_elewise_quant.py:24-32,
                      tests/apitest/kernelstest/elewise/test_quant_per_channel.py:22-40
  paged_attention     tests/apitest/kernelstest/mix/test_paged_attention_common.py:85-118 (grouped
                      matmul, int8 dequant (q + offset) * scale per channel g*D + d), :132-139
                      (softmax), :229-276 (the fp32 "out_high" branch; :252-254 the mask is added
                      in fp32 after the scale), :278-365 (paged gather, zero-length sequences are
                      skipped and take no query row; :311-313,347-349 logN multiplies the scale of
                      sequence i; :353-358 a 4-dim mask is sliced [i, :, :, :ctx], a 3-dim one
                      [i, :, :ctx], with i the index into context_lens); :74-83 (ALiBi slopes),
                      :488-505 (the masks the reference tests feed);
                      head-major caches: test_paged_attention_operation_BNSD.py:369-373 (pinned by flat
                      addresses); head compression: test_paged_attention_common.py:292-360 with :85-101 and
                      :249-252 (pinned against ordinary attention on the rearranged cache, loop version);
                      several query tokens per sequence (calcType SPEC): tests/apitest/opstest/python/
                      operations/paged_attention/test_paged_attention_operation_parallel_decoding_910B.py:
                      75-121 (sequence i owns q_lens[i] consecutive query rows, every one attends to
                      all k_lens[i] tokens; mask rows [k - q : k] of the square causal mask, or rows
                      [cu : cu + q] of the per-query-row mask), tests/apitest/kernelstest/mix/
                      test_paged_attention_mla_mtp.py:120-166 (the same for the MLA cache, fp32 branch);
                      MultiLatentAttention: tests/apitest/opstest/python/operations/multi_latent_attention/
                      test_multi_latent_attention_lse.py:122-130 (lse = row max + log(row sum)), :148-182,
                      :386-388 (query and cache split [512, 64] along the channels);
                      MLA: tests/apitest/opstest/python/operations/paged_attention/
                      test_paged_attention_operation_mla.py:229-262 (V = K[..., :head_size_vo])
  nd_to_nz, nz_to_nd  tests/apitest/opstest/python/operations/multi_latent_attention/
                      test_multi_latent_attention_int8nz.py:24-44 (shape_nd_to_nz, convert_nd_to_nz),
                      :633-636 (a cache [blocks, block_size, channels] becomes [blocks, channels / 16,
                      block_size, 16]); the NZCACHE operator is paged_attention over nz_to_nd of its
                      caches (:767-797 feed the same golden as the ND test); pinned by flat addresses,
                      the round trip and the reference's two-step reshape / permute written with torch
  paged_attention_int8q
                      tests/apitest/kernelstest/mix/test_paged_attention_common.py:104-110 (exact int32 products of
                      the int8 query and the int8 key rows, times a descale per query head), :147-168
                      (softmax_quant_numpy: the weights of a tile quantised to int8, online against the tile's
                      largest weight or offline with a given factor per head), :171-229 (tiles joined by online
                      rescaling), :256-276 (scale, mask, and the whole context as one tile as the high-precision
                      golden). As for mla_int8_decode the tile length is a parameter of the golden, not of the
                      operator (:3026-3227 run it with the Ascend kernel's block size and split). Pinned by an
                      independent float64 loop version, by exactly representable cases where quantisation loses
                      nothing (= float attention over the dequantised tensors), by tile invariance in those cases,
                      by agreement with mla_int8_decode on a shared case, and, for contexts cut into pieces
                      (:176-229), by running every piece as a sequence of its own and joining them in float64
                      by their log-sum-exps
  mla_int8_decode     tests/apitest/opstest/python/operations/multi_latent_attention/
                      test_multi_latent_attention_int8nz.py:115-121 (exact int32 products of the int8 query and
                      cache, times a per-head descale), :276-286 (the 64 rotary channels in fp32, added before
                      the scale; mask after it), :179-196 (softmax_quant_torch: weights exp(s - running max)
                      quantised to int8 against the largest weight of the tile: rint(fp16(w / (wmax / 127)))),
                      :198-262 (softmax_quant_numpy_online: per tile, exact int32 products of the int8 weights
                      and the int8 values times pvDescale * wmax / 127, tiles joined by the usual online
                      rescaling; lse = log(sum) + max). The tile length is a parameter of the golden, not a
                      property of the operator: its own tests run 128 tokens for 32 and for 128 heads
                      (:668-766) and 512 for 128 heads (:845-1104), and compare by the double-golden
                      criterion of tests/apitest/opstest/python/operations/precision_calcu.py:111-140 against
                      the whole context as one tile. Pinned by an independent float64 loop version, by the
                      limit of fine descales (-> ordinary attention over the dequantised tensors), and by
                      closed forms of the quantiser
  causal_rows (paged_attention, mla_int8_decode)
                      src/kernels/mixkernels/multi_latent_attention/tiling/mla_tiling.cpp:139-144 and
                      mla_tiling_dependency.cpp:292-316 (128 heads, or an int8 cache with several query tokens: one
                      job per query token over kvSeqlen - qSeqLen + its index + 1 tokens, the mask type dropped, a
                      maskUseStatus of 0 keeping the whole context), test_multi_latent_attention_int8nz.py:356-364
                      (the golden does the same); pinned against every row run alone on its shortened context,
                      against the -inf look-ahead mask, and per sequence
  mla_mask_free_rows  src/kernels/mixkernels/multi_latent_attention/op_kernel/mla.cce:3719-3750 with 2581-2592 (which
                      rows of the compressed mask the kernel adds to the last two 128-token tiles),
                      test_multi_latent_attention_mtp.py:342-368 (the template); pinned by the closed form: the
                      reference's template read this way is "token > k - q + i" for every context length and q
  mla_prefill         tests/apitest/opstest/python/operations/multi_latent_attention/
                      test_multi_latent_attention_prefill.py:519-700 (gen_out_tensor: per sequence and head
                      score = q . k^T * tor over the 128 + 64 channels, + mask, fp32 softmax over the keys,
                      times v; the fp32 "out_true" branch), :301-316 and :373-391 (the masks: strictly upper
                      triangle hidden, with a window also everything at or below the diagonal shifted down
                      by the window), :707-716 (query and key split [128, 64] along the channels);
                      pinned by torch's scaled_dot_product_attention (plain, is_causal, explicit band
                      mask), float64 loops and closed forms
  block_copy          tests/apitest/opstest/python/operations/block_copy/test_block_copy.py (golden_calc:
                      source i goes to the destinations dst[cum_sum[i-1] : cum_sum[i]], one after the other)
  paged_cache_load    tests/apitest/opstest/python/operations/paged_cache_load/
                      test_paged_cache_load_operation_nd.py:57-170 (token j of sequence i comes from block
                      table[i][seq_starts[i] // block_size + j // block_size], offset j % block_size; lengths
                      or their running sums. The golden also skips negative block ids, moving later rows up;
                      its own tests never draw one (ids come from [0, num_blocks)), so that branch fixes no
                      behaviour of the kernel: here such rows are skipped in place, see paged_cache_load)
  paged_cache_load_nz tests/apitest/kernelstest/mix/test_paged_cache_load_nz.py:72-131 (the same gather from
                      fractal-NZ caches, the pieces of a row put back side by side); pinned by flat addresses,
                      by paged_cache_load over nz_to_nd of the caches and by the round trip through
                      reshape_and_cache_nz
  merge_partials      src/kernels/mixkernels/pagedattention/op_kernel/
                      paged_attention_decoder_nd_common.cce:6568-6760,7959-7975 (split-KV combine)

Arithmetic is fp32 throughout ("fp32-accumulated golden"); inputs arrive as
float32 arrays holding fp16/bf16-representable values, or int8 caches.
"""
import numpy as np


def bf16_round(x):
    """Rounds float32 values to the nearest bfloat16 (ties to even), returned as float32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    rounded = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    out = rounded.astype(np.uint32).view(np.float32).reshape(x.shape)
    return np.where(np.isnan(x), x, out)


def round_to(x, dtype):
    """Rounds float32 values to `dtype` ("float16" | "bf16" | "float32"), returned as float32."""
    if dtype == "float16":
        return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)
    if dtype == "bf16":
        return bf16_round(x)
    return np.asarray(x, dtype=np.float32)


def reshape_and_cache(key, value, key_cache, value_cache, slot_mapping):
    """Returns updated copies of the caches: for token i with slot s >= 0 the row
    key[i] ([heads, head_size_k]) lands in key_cache[s // block, s % block] and
    value[i] in value_cache likewise; negative slots are skipped. value /
    value_cache may be None (single-cache form). Pure data movement."""
    kc = np.array(key_cache, copy=True)
    vc = None if value_cache is None else np.array(value_cache, copy=True)
    block_size = kc.shape[1]
    for i, slot in enumerate(np.asarray(slot_mapping).tolist()):
        if slot < 0:
            continue
        kc[slot // block_size, slot % block_size] = key[i]
        if vc is not None:
            vc[slot // block_size, slot % block_size] = value[i]
    return kc, vc


def reshape_and_cache_nz(key, value, key_cache, value_cache, slot_mapping):
    """KV-cache write into fractal-NZ caches [blocks, heads * head_size / last, block_size, last] (copies are
    returned): token i's key row, flattened to heads * head_size elements, is cut into pieces of `last` elements
    (the cache's last dim: 32 for int8 keys, 16 otherwise; 16 for values) and piece k lands in
    key_cache[s // block_size, k, s % block_size, :], s = slot_mapping[i]; negative slots are skipped. Follows the
    reference golden tests/apitest/kernelstest/mix/test_reshape_and_cache_nz.py:45-66 (also
    tests/framework/python/CsvOpsTestTool/data_generation.py:4385-4420). Pure data movement."""
    kc = np.array(key_cache, copy=True)
    vc = np.array(value_cache, copy=True)
    block_size = kc.shape[2]
    for i, slot in enumerate(np.asarray(slot_mapping).tolist()):
        if slot < 0:
            continue
        for cache, row in ((kc, key[i]), (vc, value[i])):
            last = cache.shape[3]
            cache[slot // block_size, :, slot % block_size, :] = np.asarray(row).reshape(-1, last)
    return kc, vc


def reshape_and_cache_compress(key, value, key_cache, value_cache, slot_mapping, wins, seq_lens, offset_index=None,
                               out_dtype=None):
    """KV-cache write under head compression; caches [blocks, block, 1, D] (copied and returned).
    Pair i = b * heads + h owns the slots from slot_mapping[i] on (negative: skipped); sequence b is
    the seq_lens[b] rows of key / value [tokens, heads, D] after those of the sequences before it.
    offset_index None (COMPRESS_TYPE_KVHEAD; reference golden
    tests/apitest/kernelstest/mix/test_reshape_and_cache_wins.py:61-88): the last wins[i] tokens of
    the sequence, head h, in order.
    offset_index given (COMPRESS_TYPE_KVHEAD_ROPE; golden test_reshape_and_cache_wins_rope.py:78-131):
    o = offset_index[i] == -1 copies the whole sequence; otherwise the tokens before o, one slot
    with the mean of the wins[i] tokens from o on, then the tokens after the window (wins[i] == 0:
    everything is copied). The mean is an fp32 sum in token order divided by wins[i]; the golden
    keeps it in fp32, the reference's device kernel rounds it to the cache dtype, nearest even
    (src/kernels/mixkernels/reshape_and_cache/op_kernel/reshape_and_cache_compress_rope.cpp:92-100):
    out_dtype ("float16" / "bf16") applies that rounding, None leaves the fp32 value."""
    kc = np.array(key_cache, copy=True)
    vc = np.array(value_cache, copy=True)
    heads = key.shape[1]
    block = kc.shape[1]
    ends = np.cumsum(np.asarray(seq_lens, dtype=np.int64))
    starts = ends - np.asarray(seq_lens, dtype=np.int64)

    def put(slot, k_row, v_row):
        kc[slot // block, slot % block, 0] = k_row
        vc[slot // block, slot % block, 0] = v_row

    for i, slot in enumerate(np.asarray(slot_mapping).tolist()):
        if slot < 0:
            continue
        b, h = divmod(i, heads)
        win = int(wins[i])
        if offset_index is None:
            for j in range(win):
                tok = int(ends[b]) - win + j
                put(slot + j, key[tok, h], value[tok, h])
            continue
        off = int(offset_index[i])
        for j in range(int(seq_lens[b])):
            tok = int(starts[b]) + j
            if off == -1 or j < off or (win == 0 and j >= off):
                put(slot, key[tok, h], value[tok, h])
                slot += 1
            elif j == off:
                k_sum = np.zeros(key.shape[2], dtype=np.float32)
                v_sum = np.zeros(value.shape[2], dtype=np.float32)
                for t in range(tok, tok + win):
                    k_sum = k_sum + key[t, h].astype(np.float32)
                    v_sum = v_sum + value[t, h].astype(np.float32)
                k_mean = k_sum / np.float32(win)
                v_mean = v_sum / np.float32(win)
                if out_dtype is not None:
                    k_mean, v_mean = round_to(k_mean, out_dtype), round_to(v_mean, out_dtype)
                put(slot, k_mean, v_mean)
                slot += 1
            elif j >= off + win:
                put(slot, key[tok, h], value[tok, h])
                slot += 1
    return kc, vc


def reshape_and_cache_omni(key, value, key_cache, value_cache, slot_mapping, wins, seq_lens, offset_index):
    """KV-cache write of ReshapeAndCacheOmniOperation; caches [blocks, block, 1, D] (copied and returned),
    pairs and sequences as in reshape_and_cache_compress. Token j of the pair's sequence goes to the pair's
    next free slot when o = offset_index[i] is -1, when j < o, or when j >= o + wins[i]: the window
    [o, o + wins[i]) leaves nothing behind (reference goldens
    tests/framework/python/CsvOpsTestTool/data_generation.py:9797-9846 and
    tests/apitest/kernelstest/mix/test_reshape_and_cache_omni_compress.py:80-116; the device kernel,
    src/kernels/mixkernels/reshape_and_cache/op_kernel/reshape_and_cache_omni_compress.cpp:87-110 with
    reshape_and_cache_base.h:276-289, copies [0, o) and then [o + w, seqLen), and takes w == 0 as no window).
    wins[i] < 0 is outside the reference's domain (its kernel reads the count as unsigned, its golden
    would skip slots); it is taken as no window here."""
    kc = np.array(key_cache, copy=True)
    vc = np.array(value_cache, copy=True)
    heads = key.shape[1]
    block = kc.shape[1]
    ends = np.cumsum(np.asarray(seq_lens, dtype=np.int64))
    starts = ends - np.asarray(seq_lens, dtype=np.int64)
    for i, slot in enumerate(np.asarray(slot_mapping).tolist()):
        if slot < 0:
            continue
        b, h = divmod(i, heads)
        off = int(offset_index[i])
        win = max(int(wins[i]), 0)
        for j in range(int(seq_lens[b])):
            tok = int(starts[b]) + j
            if off == -1 or j < off or j >= off + win:
                kc[slot // block, slot % block, 0] = key[tok, h]
                vc[slot // block, slot % block, 0] = value[tok, h]
                slot += 1
    return kc, vc


def strided_view(storage, shape, strides, offset):
    """The [tokens, heads, head_size] view that ReshapeAndCacheWithStride reads: element
    (t, h, d) is storage.flat[offset + t * strides[0] + h * strides[1] + d * strides[2]],
    strides and offset in elements. Returns a contiguous copy."""
    flat = np.asarray(storage).reshape(-1)
    idx = np.full(tuple(shape), int(offset), dtype=np.int64)
    for axis, (n, st) in enumerate(zip(shape, strides)):
        ext = [1] * len(shape)
        ext[axis] = n
        idx += (np.arange(n, dtype=np.int64) * int(st)).reshape(ext)
    return flat[idx]


def rope(q, k, cos, sin, seq_lens, rotary_coeff, cos_format=0, out_dtype=np.float16):
    """Rotary embedding of q [tokens, hidden_q] and k [tokens, hidden_k] with tables [rows, head_dim]:
    out = x * cos + rotated(x) * sin, where inside every chunk of 2 * (head_dim / rotary_coeff) channels
    rotated(x) = concat(-second half, first half). Table row of token t: t itself (cos_format 0) or its
    position inside its sequence (cos_format 1; seq_lens gives the sequences). fp32 arithmetic, rounded
    once to out_dtype (np.float16, or "bf16" for bfloat16 values kept in float32). Returns (q_out, k_out)."""
    cos = np.asarray(cos, dtype=np.float32)
    sin = np.asarray(sin, dtype=np.float32)
    head_dim = cos.shape[1]
    stride = head_dim // rotary_coeff
    tokens = np.asarray(q).shape[0]
    if cos_format == 0:
        rows = np.arange(tokens)
    else:
        rows = np.concatenate([np.arange(n) for n in np.asarray(seq_lens).tolist()])[:tokens]

    def one(x):
        x = np.asarray(x, dtype=np.float32)
        units = x.reshape(tokens, -1, head_dim // (2 * stride), 2, stride)  # token, unit, chunk, half, channel
        rotated = np.stack((-units[:, :, :, 1], units[:, :, :, 0]), axis=3).reshape(tokens, -1, head_dim)
        c = cos[rows][:, None, :]
        s_ = sin[rows][:, None, :]
        out = (x.reshape(tokens, -1, head_dim) * c + rotated * s_).reshape(x.shape)
        return bf16_round(out) if out_dtype == "bf16" else out.astype(out_dtype)
    return one(q), one(k)


def norm_rope_reshape(x, gamma, key_rope, cos, sin, slot_mapping, key_cache, epsilon, out_dtype=np.float16):
    """Returns an updated copy of key_cache [blocks, block, 1, norm_dim + rope_dim]: for token i with
    slot s >= 0, the RMS-normalised x[i] (times gamma) followed by the rotated key_rope[i]. fp32
    arithmetic, rounded once to out_dtype (np.float16, or "bf16" for round-to-nearest-even bfloat16 values
    kept in float32)."""
    xf = np.asarray(x, dtype=np.float32)
    mean_sq = np.sum(np.square(xf), axis=-1, keepdims=True) / np.float32(xf.shape[-1])
    rms = np.float32(1.0) / np.sqrt(mean_sq + np.float32(epsilon))
    normed = rms * xf * np.asarray(gamma, dtype=np.float32)
    r = np.asarray(key_rope, dtype=np.float32)
    first, second = np.split(r, 2, axis=1)
    rotated = np.concatenate((-second, first), axis=1)
    roped = r * np.asarray(cos, dtype=np.float32) + rotated * np.asarray(sin, dtype=np.float32)
    rows = np.concatenate((normed.reshape(normed.shape[0], -1), roped), axis=-1)
    rows = bf16_round(rows) if out_dtype == "bf16" else rows.astype(out_dtype)
    kc = np.array(key_cache, copy=True)
    block_size = kc.shape[1]
    for i, slot in enumerate(np.asarray(slot_mapping).tolist()):
        if slot < 0:
            continue
        kc[slot // block_size, slot % block_size, 0] = rows[i]
    return kc


def block_copy(key_cache, value_cache, src_blocks, dst_blocks, cum_sum):
    """Returns copies of the caches in which block src_blocks[i] has been copied onto the blocks
    dst_blocks[cum_sum[i-1] : cum_sum[i]] (cum_sum[-1] = 0), sources taken in order, as the
    reference golden does: a destination written earlier is seen by a later copy that reads it."""
    kc = np.array(key_cache, copy=True)
    vc = np.array(value_cache, copy=True)
    start = 0
    for i, src in enumerate(np.asarray(src_blocks).tolist()):
        end = int(cum_sum[i])
        for j in range(start, end):
            dst = int(dst_blocks[j])
            kc[dst] = kc[src]
            vc[dst] = vc[src]
        start = end
    return kc, vc


def paged_cache_load(key_cache, value_cache, block_tables, seq_lens, key, value, seq_starts=None, cumsum_mode=False):
    """Returns copies of key [tokens, heads, Dk] and value [tokens, heads, Dv] with the cached rows of
    every sequence written one after the other. seq_lens holds the lengths, or with cumsum_mode their
    running sums starting at 0 (one entry more). Token j of sequence i always owns output row
    (tokens of the sequences before i) + j; where its block id is negative that row keeps its input."""
    key = np.array(key, copy=True)
    value = np.array(value, copy=True)
    block_size = key_cache.shape[1]
    lens = np.diff(np.asarray(seq_lens)) if cumsum_mode else np.asarray(seq_lens)
    row = 0
    for i, n in enumerate(lens.tolist()):
        first = 0 if seq_starts is None else int(seq_starts[i]) // block_size
        for j in range(int(n)):
            block = int(block_tables[i][first + j // block_size])
            if block >= 0:
                key[row] = key_cache[block][j % block_size]
                value[row] = value_cache[block][j % block_size]
            row += 1
    return key, value


def paged_cache_load_nz(key_cache, value_cache, block_tables, seq_lens, key, value):
    """The gather from fractal-NZ caches [blocks, channels / last, block_size, last]: returns copies of key
    [tokens, channels_k] and value [tokens, channels_v] where row (tokens of the sequences before i) + j is the
    cache row of token j of sequence i, its pieces put back side by side (reference golden
    tests/apitest/kernelstest/mix/test_paged_cache_load_nz.py:72-131). A negative block id leaves its row as it
    is (the golden would move the later rows up; its tests draw ids from [0, num_blocks) only)."""
    key = np.array(key, copy=True)
    value = np.array(value, copy=True)
    block_size = key_cache.shape[2]
    row = 0
    for i, n in enumerate(np.asarray(seq_lens).tolist()):
        for j in range(int(n)):
            block = int(block_tables[i][j // block_size])
            if block >= 0:
                key[row] = key_cache[block, :, j % block_size, :].reshape(-1)
                value[row] = value_cache[block, :, j % block_size, :].reshape(-1)
            row += 1
    return key, value


def quant_per_channel(x, scale, offset=None):
    """int8 = clip(round_half_even(x / scale) (+ offset), -128, 127) with the
    division in IEEE fp32; scale/offset broadcast over the trailing (channel)
    axis. NaN quantises to 0. The reference golden divides in the tensor's own
    dtype (fp16) and is compared with atol=1; this is its fp32 form, which is
    the one a bit-exact quantised cache is defined by."""
    x = np.asarray(x, dtype=np.float32)
    s = np.asarray(scale, dtype=np.float32)
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        r = np.rint(x / s)
    if offset is not None:
        r = r + np.asarray(offset, dtype=np.float32)
    r = np.where(np.isnan(r), np.float32(0), r)
    return np.clip(r, -128, 127).astype(np.int8)


def quant_per_channel_golden_dtype(x_fp16, scale_fp16, offset=None):
    """The golden exactly as the reference test writes it: fp16 / fp16 division."""
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        r = np.round(np.asarray(x_fp16, dtype=np.float16) / np.asarray(scale_fp16, dtype=np.float16))
    if offset is not None:
        r = r + offset
    r = np.where(np.isnan(r), 0, r)
    return np.clip(r, -128, 127).astype(np.int8)


def dequant_per_channel(x_int8, scale_fp16, offset=None):
    """ElewiseOperation's per-channel dequantiser as the reference golden writes it (tests/apitest/opstest/
    python/operations/elewise/test_elewise_dequant.py:23-31): (fp16(x) - fp16(offset)) * scale in fp16
    arithmetic, clipped to the largest finite fp16 values. scale / offset broadcast over the trailing
    dimensions of x."""
    y = np.asarray(x_int8).astype(np.float16)
    with np.errstate(over="ignore", invalid="ignore"):
        if offset is not None:
            y = y - np.asarray(offset).astype(np.float16)
        out = y * np.asarray(scale_fp16, dtype=np.float16)
    return np.clip(out, np.float16(-65504), np.float16(65504)).astype(np.float16)


def softmax_rows(sim):
    """Row softmax in fp32, max-subtracted (reference softmax_numpy)."""
    row_max = np.max(sim, axis=-1, keepdims=True)
    e = np.exp(sim - row_max)
    return e / np.sum(e, axis=-1, keepdims=True)


def _dequant(rows_i8, scale, offset, g, dim):
    """(int8 + offset) * scale with the per-(kv head, channel) vectors sliced at g*dim."""
    f = rows_i8.astype(np.float32)
    if offset is not None:
        f = f + np.asarray(offset[g * dim:(g + 1) * dim], dtype=np.float32)
    return f * np.asarray(scale[g * dim:(g + 1) * dim], dtype=np.float32)


def nd_to_nz(x, n0=16):
    """[..., rows, channels] -> [..., channels / n0, rows, n0]: the fractal-NZ layout of a matrix whose
    row count is a multiple of 16 and whose channel count is a multiple of n0 (16 for 16-bit elements,
    32 for int8). Channel c of row r moves to [c // n0, r, c % n0]."""
    x = np.asarray(x)
    rows, channels = x.shape[-2], x.shape[-1]
    if rows % 16 or channels % n0:
        raise ValueError("fractal-NZ needs rows % 16 == 0 and channels % n0 == 0")
    lead = x.shape[:-2]
    return np.ascontiguousarray(np.moveaxis(x.reshape(lead + (rows, channels // n0, n0)), -2, -3))


def nz_to_nd(x):
    """Inverse of nd_to_nz: [..., channels / n0, rows, n0] -> [..., rows, channels]."""
    x = np.asarray(x)
    n1, rows, n0 = x.shape[-3:]
    return np.ascontiguousarray(np.moveaxis(x, -3, -2)).reshape(x.shape[:-3] + (rows, n1 * n0))


def gather_rows(cache, block_table, context_len):
    """Rows 0..context_len-1 of one sequence: token j lives in block
    block_table[j // block_size] at offset j % block_size. -> [ctx, kv_heads, dim]"""
    block_size = cache.shape[1]
    j = np.arange(context_len)
    return cache[np.asarray(block_table)[j // block_size], j % block_size]


def attention_one(q, keys, values, scale, k_descale=None, k_offset=None, v_descale=None, v_offset=None,
                  bias=None, lse_out=None, descale_head=None, score_offset=None):
    """One query token against gathered rows. q [heads, D] float32; keys
    [ctx, kv_heads, D]; values [ctx, kv_heads, Dv] (float32 or int8); bias None
    or broadcastable to [heads, ctx], added to the scaled scores.
    Returns float32 [heads, Dv]: softmax(scale * q k^T + bias) v per GQA group.
    lse_out, a float32 [heads] array, receives the natural-log log-sum-exp of the
    scaled and biased scores (row max + log of the row sum of exp(score - max)).
    descale_head: the slice of the descale vectors to use instead of the KV head's
    index (the reference golden's razor_mod, test_paged_attention_common.py:85-101,341-347).
    score_offset: float32 [ctx], added to q k^T before the scale (its razor_offset_list, :249-252)."""
    if bias is not None:
        bias = np.broadcast_to(np.asarray(bias, dtype=np.float32), (q.shape[0], keys.shape[0]))
    heads = q.shape[0]
    kv_heads = keys.shape[1]
    group = heads // kv_heads
    out = np.empty((heads, values.shape[2]), dtype=np.float32)
    for g in range(kv_heads):
        k = keys[:, g, :]
        v = values[:, g, :]
        if k.dtype == np.int8:
            k = _dequant(k, k_descale, k_offset, g if descale_head is None else descale_head, keys.shape[2])
            v = _dequant(v, v_descale, v_offset, g if descale_head is None else descale_head, values.shape[2])
        k = k.astype(np.float32)
        v = v.astype(np.float32)
        qg = q[g * group:(g + 1) * group].astype(np.float32)
        sim = qg @ k.T
        if score_offset is not None:
            sim = sim + np.asarray(score_offset, dtype=np.float32)[None, :]
        sim = sim * np.float32(scale)
        if bias is not None:
            sim = sim + bias[g * group:(g + 1) * group]
        p = softmax_rows(sim)
        out[g * group:(g + 1) * group] = p @ v
        if lse_out is not None:
            row_max = np.max(sim, axis=-1)
            lse_out[g * group:(g + 1) * group] = row_max + np.log(np.sum(np.exp(sim - row_max[:, None]), axis=-1))
    return out


def alibi_slopes(n_heads):
    """Per-head ALiBi slopes as the reference tests build them: 2^(-8 k / n) for
    k = 1..n with n the largest power of two <= n_heads, then 2^(-4 k / n) for
    odd k to fill up."""
    n = 1 << (int(n_heads).bit_length() - 1)
    slopes = [2.0 ** (-8.0 * k / n) for k in range(1, n + 1)]
    slopes += [2.0 ** (-4.0 * k / n) for k in range(1, 1 + 2 * (n_heads - n), 2)]
    return np.asarray(slopes, dtype=np.float32)


def alibi_mask(context_lens, n_heads, max_len):
    """[batch, heads, 1, max_len] float32: slope_h * (j - ctx_i + 1) for j < ctx_i, else 0."""
    mask = np.zeros((len(context_lens), n_heads, 1, max_len), dtype=np.float32)
    slopes = alibi_slopes(n_heads)
    for i, ctx in enumerate(context_lens):
        pos = np.arange(ctx, dtype=np.float32) - np.float32(ctx) + 1
        mask[i, :, 0, :ctx] = slopes[:, None] * pos[None, :]
    return mask


def norm_mask(batch, max_len, value=-10000.0):
    """[batch, 1, max_len] float32: row i hides its first i positions."""
    mask = np.zeros((batch, 1, max_len), dtype=np.float32)
    for i in range(batch):
        mask[i, :, :i] = value
    return mask


def paged_attention(query, key_cache, value_cache, block_tables, context_lens, scale, k_descale=None,
                    k_offset=None, v_descale=None, v_offset=None, mla_v_head_size=0, q_scale=0.0,
                    q_dtype="float32", out_init=0.0, mask=None, logn=None, mask_per_head=None, q_lens=None,
                    mask_rows="sequence", lse_out=None, head_major=False, compress_kv_heads=0, razor_offset=None,
                    causal_rows=None, empty_keep_rows=False):
    """Decode attention over paged caches.

    query [rows, heads, D] float32; key_cache [blocks, block, kv_heads, D];
    value_cache [blocks, block, kv_heads, Dv], or None with mla_v_head_size > 0
    (V is then the first mla_v_head_size channels of the key rows).
    Sequence i with context_lens[i] == 0 is skipped and consumes no query row:
    the n-th non-empty sequence uses query row n and writes output row n.
    Rows never written keep `out_init`. q_scale not in {0, 1} pre-multiplies the
    query and rounds it to q_dtype, as the reference's separate multiply node does.
    mask (float32 values of the mask tensor's dtype) is added to the scaled scores
    of sequence i (its index in context_lens, empty ones counted): a 4-dim mask
    [batch, heads | 1, 1, max_len] is sliced [i, :, 0, :ctx], a 3-dim mask whose
    first dim is the batch [i, 0, :ctx] for every head, a 3-dim mask
    [heads, 1, max_len] (mask_per_head=True, or left to its size when heads !=
    batch), or a 2-dim [1, max_len] one, is shared by all sequences.
    logn [batch] multiplies the scale of sequence i.
    q_lens [batch] gives sequence i that many consecutive query rows (none when
    its context is empty), each attending to all context_lens[i] tokens; the
    2-dim mask then has one row per query row (mask_rows="query") or is the
    square causal mask, of which the t-th query token of a sequence with n of
    them uses row ctx - n + t (mask_rows="position").
    causal_rows (True, or a [batch] array of flags): the t-th of a sequence's n
    query rows attends to its first ctx - n + t + 1 tokens only, which is how
    the reference's MLA kernel makes several query tokens causal when it runs
    one job per query token (128 heads, or an int8 cache with more than one
    query token: src/kernels/mixkernels/multi_latent_attention/tiling/
    mla_tiling.cpp:139-144, mla_tiling_dependency.cpp:292-316; a sequence whose
    maskUseStatus entry is 0 keeps the whole context for every row).
    lse_out, a float32 [rows, heads] array, receives the log-sum-exp of every
    written row (see attention_one); other rows are left alone.
    The split latent layout of MultiLatentAttention (query / cache rows given as
    512 + 64 channels in two tensors) is the same computation on the rows
    concatenated along the channel axis, which is what the reference golden
    does the other way round (it splits the concatenated tensors).
    head_major: the caches are [blocks, kv_heads, block, D] (InputLayout TYPE_BNSD);
    the reference golden computes on the token-major cache and hands the
    operation its (0, 2, 1, 3) permutation
    (tests/apitest/opstest/python/operations/paged_attention/test_paged_attention_operation_BNSD.py:369-373),
    so this is the same computation after permuting back.
    compress_kv_heads = n > 0 (PagedAttentionParam::compressType; reference golden
    test_paged_attention_common.py:292-360): the caches hold one head per block,
    [blocks * n, block, 1, D], and block_tables / context_lens one row per
    (sequence, KV head) pair; query [tokens, heads, D] is read as
    [tokens * n, heads / n, D] and pair i takes the descale slices of KV head
    i % n. A 4-dim mask [batch, heads, 1, max_len] is read as
    [batch * n, heads / n, 1, max_len], a 3-dim mask has one row per sequence
    (pair i uses row i // n). razor_offset, float32 [blocks * n, block], is added
    to q k^T of the token in that cache slot before the scale.
    empty_keep_rows: a sequence without context still owns its q_lens[i] (or one) query rows, which
    are neither read nor written, and the rows of the sequences behind it stay where they are. This is
    what the reference's MultiLatentAttention tiling does (it moves on by qSeqLen whatever kvSeqLen
    is: src/kernels/mixkernels/multi_latent_attention/tiling/mla_tiling.cpp:146-149; its golden for
    several query tokens does the same, tests/apitest/opstest/python/operations/multi_latent_attention/
    test_multi_latent_attention_mtp.py:145-151), whereas PagedAttention gives such a sequence no row.
    Returns float32 [rows, heads, Dv]."""
    query = np.asarray(query, dtype=np.float32)
    if compress_kv_heads > 0:
        n = compress_kv_heads
        tokens, heads, d = query.shape
        if mask is not None and np.ndim(mask) == 4:
            mask = np.asarray(mask, dtype=np.float32)
            if mask.shape[1] == 1:  # one row per sequence, shared by its heads
                mask = np.repeat(mask, n, axis=0)
            else:
                mask = mask.reshape(mask.shape[0] * n, mask.shape[1] // n, 1, mask.shape[3])
        elif mask is not None and np.ndim(mask) == 3 and mask_per_head:
            # [heads, 1, max_len], shared by all sequences: the 4-dim form with the batch axis broadcast
            mask = np.asarray(mask, dtype=np.float32)
            pairs = len(context_lens)
            mask = np.broadcast_to(mask[None], (pairs // n,) + mask.shape).reshape(pairs, heads // n, 1, mask.shape[2])
        elif mask is not None and np.ndim(mask) == 3:
            mask = np.repeat(np.asarray(mask, dtype=np.float32), n, axis=0)
        out = _paged_attention_compressed(query.reshape(tokens * n, heads // n, d), key_cache, value_cache, block_tables,
                                          context_lens, scale, k_descale, k_offset, v_descale, v_offset, out_init, mask,
                                          n, razor_offset)
        return out.reshape(tokens, heads, out.shape[2])
    if head_major:
        key_cache = np.transpose(key_cache, (0, 2, 1, 3))
        value_cache = None if value_cache is None else np.transpose(value_cache, (0, 2, 1, 3))
    if mla_v_head_size > 0:
        dv = mla_v_head_size
    else:
        dv = value_cache.shape[3]
    out = np.full((query.shape[0], query.shape[1], dv), out_init, dtype=np.float32)
    if q_scale not in (0.0, 1.0):
        query = round_to(query * np.float32(q_scale), q_dtype)
    row = 0
    for i, ctx in enumerate(np.asarray(context_lens).tolist()):
        if ctx == 0:
            if empty_keep_rows:
                row += 1 if q_lens is None else int(q_lens[i])
            continue
        keys = gather_rows(key_cache, block_tables[i], ctx)
        values = keys[..., :dv] if mla_v_head_size > 0 else gather_rows(value_cache, block_tables[i], ctx)
        seq_scale = np.float32(scale) if logn is None else np.float32(scale) * np.float32(logn[i])
        n_rows = 1 if q_lens is None else int(q_lens[i])
        for t in range(n_rows):
            if mask is None:
                bias = None
            elif mask_rows == "query":
                bias = np.asarray(mask, dtype=np.float32)[row:row + 1, :ctx]
            elif mask_rows == "position":
                bias = np.asarray(mask, dtype=np.float32)[ctx - int(q_lens[i]) + t][None, :ctx]
            else:
                bias = _mask_slice(mask, i, ctx, query.shape[1], len(context_lens), mask_per_head)
            seen = _causal_row_length(ctx, n_rows, t, i, causal_rows)
            out[row] = attention_one(query[row], keys[:seen], values[:seen], seq_scale, k_descale, k_offset, v_descale,
                                     v_offset, None if bias is None else bias[..., :seen],
                                     None if lse_out is None else lse_out[row])
            row += 1
    return out


def _causal_row_length(ctx, n_rows, t, seq, causal_rows):
    """Tokens the t-th of a sequence's n_rows query rows attends to (see paged_attention's causal_rows)."""
    if causal_rows is None or causal_rows is False:
        return ctx
    if causal_rows is not True and not int(np.asarray(causal_rows)[seq]):
        return ctx
    return ctx - n_rows + t + 1


def _paged_attention_compressed(query, key_cache, value_cache, block_tables, context_lens, scale, k_descale, k_offset,
                                v_descale, v_offset, out_init, mask, n, razor_offset):
    """paged_attention over (sequence, KV head) pairs; see its compress_kv_heads."""
    out = np.full((query.shape[0], query.shape[1], value_cache.shape[3]), out_init, dtype=np.float32)
    block_size = key_cache.shape[1]
    row = 0
    for i, ctx in enumerate(np.asarray(context_lens).tolist()):
        if ctx == 0:
            continue
        keys = gather_rows(key_cache, block_tables[i], ctx)
        values = gather_rows(value_cache, block_tables[i], ctx)
        offsets = None
        if razor_offset is not None:
            j = np.arange(ctx)
            offsets = np.asarray(razor_offset, dtype=np.float32)[np.asarray(block_tables[i])[j // block_size],
                                                                  j % block_size]
        bias = None
        if mask is not None:
            m = np.asarray(mask, dtype=np.float32)
            bias = m[i, :, 0, :ctx] if m.ndim == 4 else (m[i, :, :ctx] if m.ndim == 3 else m[:1, :ctx])
        out[row] = attention_one(query[row], keys, values, np.float32(scale), k_descale, k_offset, v_descale, v_offset,
                                 bias, descale_head=i % n, score_offset=offsets)
        row += 1
    return out


def _mask_slice(mask, i, ctx, heads, batch, per_head=None):
    """The [heads | 1, ctx] slice of `mask` that sequence i sees (see paged_attention).
    per_head says whether a 3-dim mask's first dim counts heads (ALIBI) or
    sequences (NORM); None decides by its size and refuses the ambiguous case."""
    mask = np.asarray(mask, dtype=np.float32)
    if mask.ndim == 4:
        return mask[i, :, 0, :ctx]
    if mask.ndim == 3:
        if per_head is None:
            if heads == batch and mask.shape[0] == batch:
                raise ValueError("3-dim mask with heads == batch: say per_head")
            per_head = mask.shape[0] != batch
        return mask[:, 0, :ctx] if per_head else mask[i, :, :ctx]
    return mask[:1, :ctx]


def paged_attention_loops(query, key_cache, value_cache, block_tables, context_lens, scale, dense_bias=None,
                          logn=None):
    """The same computation written as plain Python loops in float64, for tiny
    inputs only: an independent check of the vectorised version (no numpy
    matmul, no broadcasting, no shared helper). dense_bias[i][h][j] is added to
    the scaled score of sequence i, head h, token j; logn[i] multiplies the scale."""
    import math
    rows, heads, d = query.shape
    _, block_size, kv_heads, _ = key_cache.shape
    dv = value_cache.shape[3]
    group = heads // kv_heads
    out = [[[0.0] * dv for _ in range(heads)] for _ in range(rows)]
    row = 0
    for i in range(len(context_lens)):
        ctx = int(context_lens[i])
        if ctx == 0:
            continue
        for h in range(heads):
            g = h // group
            scores = []
            for j in range(ctx):
                blk = int(block_tables[i][j // block_size])
                off = j % block_size
                s = 0.0
                for c in range(d):
                    s += float(query[row][h][c]) * float(key_cache[blk][off][g][c])
                s = s * float(scale) * (float(logn[i]) if logn is not None else 1.0)
                if dense_bias is not None:
                    s += float(dense_bias[i][h][j])
                scores.append(s)
            m = max(scores)
            w = [math.exp(s - m) for s in scores]
            z = sum(w)
            for c in range(dv):
                acc = 0.0
                for j in range(ctx):
                    blk = int(block_tables[i][j // block_size])
                    off = j % block_size
                    acc += w[j] * float(value_cache[blk][off][g][c])
                out[row][h][c] = acc / z
        row += 1
    return np.array(out, dtype=np.float64)


def mla_mask_free_rows(template, context_lens, q_lens, mask_len):
    """One mask row per query token from MultiLatentAttention's compressed decode mask (MASK_TYPE_MASK_FREE), as
    the reference's kernel reads it (src/kernels/mixkernels/multi_latent_attention/op_kernel/mla.cce:3719-3750,
    2581-2592): template [rows, 128] or [batch, rows, 128]; for a sequence of k tokens whose last 128-token tile
    holds n of them, query token i of q adds template row n - 1 + i to the last tile and, when n < q - 1 and there
    is a tile before it, row n + 127 + i to that one. A sequence of length 0 keeps its q rows, all zeros (see
    paged_attention's empty_keep_rows). Returns float32 [query rows, mask_len]; rows the template lacks read as 0."""
    template = np.asarray(template, np.float32)
    rows = []
    for b, (k, q) in enumerate(zip(np.asarray(context_lens).tolist(), np.asarray(q_lens).tolist())):
        if k == 0:
            rows += [np.zeros(mask_len, np.float32) for _ in range(q)]
            continue
        tmpl = template[b] if template.ndim == 3 else template
        last = (k - 1) // 128
        n = k - last * 128
        for i in range(q):
            row = np.zeros(mask_len, np.float32)
            if n - 1 + i < tmpl.shape[0]:
                row[last * 128:k] = tmpl[n - 1 + i, :n]
            if last >= 1 and n < q - 1 and n + 127 + i < tmpl.shape[0]:
                row[(last - 1) * 128:last * 128] = tmpl[n + 127 + i, :]
            rows.append(row)
    return np.stack(rows) if rows else np.zeros((0, mask_len), np.float32)


def quantise_weights(w):
    """int8 weights of one tile and head (reference softmax_quant_torch): w / (max(w) / 127) in fp32, rounded
    to fp16, then to the nearest integer (ties to even). Returns (int8 array, max(w))."""
    w = np.asarray(w, np.float32)
    wmax = np.float32(w.max()) if w.size else np.float32(0)
    if not wmax > 0:
        return np.zeros(w.shape, np.int8), np.float32(0)
    step = np.float32(wmax / np.float32(127.0))
    return np.rint((w / step).astype(np.float16)).astype(np.int8), wmax


def mla_int8_decode(q_int8, q_rope, kv_int8, k_rope, block_tables, context_lens, qk_descale, pv_descale, scale,
                    tile=128, mask=None, q_lens=None, lse_out=None, causal_rows=None):
    """Decode attention of MultiLatentAttention's int8 cache mode over token-major views of the caches:
    q_int8 [T, H, 512] int8, q_rope [T, H, 64] float, kv_int8 [blocks, block_size, 1, 512] int8 (keys and
    values), k_rope [blocks, block_size, 1, 64] float, qk_descale / pv_descale [H] float32. The weights of
    every `tile` consecutive tokens are quantised to int8 on their own. causal_rows as in paged_attention: the
    reference golden gives the j-th of q query rows context + j - q + 1 tokens unless the sequence's entry of
    batch_list is 0 (test_multi_latent_attention_int8nz.py:356-364). mask: None or [T, >= max context]
    added to the scaled scores of its query row; q_lens: query rows per sequence (default one). Returns
    float32 [T, H, 512]; lse_out [T, H] receives log(sum exp) of the scaled scores."""
    q_int8 = np.asarray(q_int8)
    rows, heads = q_int8.shape[0], q_int8.shape[1]
    out = np.zeros((rows, heads, 512), np.float32)
    qk_descale = np.asarray(qk_descale, np.float32)
    pv_descale = np.asarray(pv_descale, np.float32)
    row = 0
    for b, ctx in enumerate(np.asarray(context_lens)):
        ctx = int(ctx)
        n_rows = 1 if q_lens is None else int(q_lens[b])
        if ctx == 0:
            # the sequence keeps its query rows, untouched (see paged_attention's empty_keep_rows)
            row += n_rows
            continue
        keys = gather_rows(np.asarray(kv_int8), block_tables[b], ctx)[:, 0].astype(np.int32)     # [ctx, 512]
        rope = gather_rows(np.asarray(k_rope, np.float32), block_tables[b], ctx)[:, 0]             # [ctx, 64]
        all_keys, all_rope, whole = keys, rope, ctx
        for r in range(row, row + n_rows):
            ctx = _causal_row_length(whole, n_rows, r - row, b, causal_rows)
            keys, rope = all_keys[:ctx], all_rope[:ctx]
            prod = (q_int8[r].astype(np.int32) @ keys.T).astype(np.float32) * qk_descale[:, None]  # [H, ctx]
            s = (prod + np.asarray(q_rope[r], np.float32) @ rope.T) * np.float32(scale)
            if mask is not None:
                s = s + np.asarray(mask[r, :ctx], np.float32)[None, :]
            s = s.astype(np.float32)
            for h in range(heads):
                gm = gl = go = None
                for t0 in range(0, ctx, tile):
                    st = s[h, t0:t0 + tile]
                    hm = np.float32(st.max()) if gm is None else np.maximum(gm, np.float32(st.max()))
                    w = np.exp(st - hm).astype(np.float32) if np.isfinite(hm) else np.zeros_like(st)
                    p8, wmax = quantise_weights(w)
                    lo = (p8.astype(np.int32) @ keys[t0:t0 + tile]).astype(np.float32) * \
                        np.float32(pv_descale[h] * wmax / np.float32(127.0))
                    ll = np.float32(w.sum(dtype=np.float32))
                    if gm is None:
                        gl, go = ll, lo
                    else:
                        keep = np.float32(np.exp(gm - hm)) if np.isfinite(gm) else np.float32(0)
                        gl, go = gl * keep + ll, go * keep + lo
                    gm = hm
                out[r, h] = go / gl if gl > 0 else 0
                if lse_out is not None:
                    lse_out[r, h] = np.log(gl) + gm if gl > 0 else -np.inf
        row += n_rows
    return out


def paged_attention_int8q(q_int8, key_cache, value_cache, block_tables, context_lens, k_descale, v_descale, scale,
                          p_scale=None, tile=128, mask=None, mask_per_head=None, out_init=0.0, piece_tiles=None, piece_unit=None,
                          piece_cuts=None):
    """Decode attention with int8 queries over int8 caches (PagedAttentionParam quantType QKV online / offline;
    reference golden tests/apitest/kernelstest/mix/test_paged_attention_common.py:104-110 (exact int32 products
    times a descale per QUERY head), :256-263 (then the scale, then the mask), :147-168 (softmax_quant_numpy: weights
    exp(s - running max); online they are quantised against the tile's largest weight, rint(fp16(w / (wmax / 127)))
    with value descale v_descale * wmax / 127; offline with the given factor, rint(fp16(w * p_scale[h])) with value
    descale v_descale), :171-216 (tiles joined by the usual online rescaling, the denominator adds up the
    unquantised weights), :176-229 (the context cut into pieces that start from scratch and are joined by their
    log-sum-exps: out = sum_p exp(lse_p - L) out_p, L = log sum_p exp(lse_p)).
    q_int8 [rows, H, D] int8; key_cache / value_cache [blocks, block_size, G, D] int8; k_descale, v_descale, p_scale
    [H] float32 (p_scale None: online). The weights of every `tile` consecutive tokens are quantised on their own;
    tile=None takes the whole context as one tile, the reference's high-precision golden (:264-270). piece_tiles = c
    cuts a context of n units into ceil(n / c) pieces of ceil(n / pieces) units each, a unit being piece_unit tokens
    (a multiple of the tile; by default the tile itself); piece_cuts = {sequence: [tokens]} names the cuts of a
    sequence outright (multiples of the tile). (Online the cut changes nothing
    but the order of a few fp32 operations; offline the weights are taken against the running maximum, which starts
    anew in every piece, so the int8 weights themselves depend on the cut.) mask as in paged_attention with one query
    token per sequence. A sequence of length 0 takes no query row; rows never written keep out_init. Returns float32
    [rows, H, D]."""
    q_int8 = np.asarray(q_int8)
    rows, heads, d = q_int8.shape
    kv_heads = key_cache.shape[2]
    group = heads // kv_heads
    out = np.full((rows, heads, d), out_init, np.float32)
    k_descale = np.asarray(k_descale, np.float32)
    v_descale = np.asarray(v_descale, np.float32)
    row = 0
    for b, ctx in enumerate(np.asarray(context_lens).tolist()):
        if ctx == 0:
            continue
        keys = gather_rows(np.asarray(key_cache), block_tables[b], ctx).astype(np.int32)      # [ctx, G, D]
        values = gather_rows(np.asarray(value_cache), block_tables[b], ctx).astype(np.int32)
        bias = None if mask is None else _mask_slice(mask, b, ctx, heads, len(context_lens), mask_per_head)
        step = ctx if tile is None else tile
        bounds = [0, ctx]
        if piece_tiles is not None and tile is not None:
            unit = tile if piece_unit is None else piece_unit
            assert unit % tile == 0
            n = (ctx + unit - 1) // unit
            parts = (n + piece_tiles - 1) // piece_tiles
            each = (n + parts - 1) // parts
            bounds = [min(ctx, i * each * unit) for i in range(parts)] + [ctx]
        if piece_cuts is not None and tile is not None:
            cuts = sorted(piece_cuts.get(b, []))
            assert all(0 < t < ctx and t % tile == 0 for t in cuts)
            bounds = [0] + cuts + [ctx]
        for h in range(heads):
            g = h // group
            prod = (keys[:, g, :] @ q_int8[row, h].astype(np.int32)).astype(np.float32)       # [ctx]
            s = prod * k_descale[h] * np.float32(scale)
            if bias is not None:
                s = s + np.asarray(bias[h if bias.shape[0] > 1 else 0], np.float32)
            s = s.astype(np.float32)
            outs, lses = [], []
            for lo_tok, hi_tok in zip(bounds[:-1], bounds[1:]):
                gm = gl = go = None
                for t0 in range(lo_tok, hi_tok, step):
                    st = s[t0:min(t0 + step, hi_tok)]
                    hm = np.float32(st.max()) if gm is None else np.maximum(gm, np.float32(st.max()))
                    w = np.exp(st - hm).astype(np.float32) if np.isfinite(hm) else np.zeros_like(st)
                    if p_scale is None:
                        p8, wmax = quantise_weights(w)
                        vs = np.float32(v_descale[h] * wmax / np.float32(127.0))
                    else:
                        p8 = np.rint((w * np.float32(p_scale[h])).astype(np.float16)).astype(np.int8)
                        vs = v_descale[h]
                    lo = (p8.astype(np.int32) @ values[t0:t0 + len(st), g, :]).astype(np.float32) * vs
                    ll = np.float32(w.sum(dtype=np.float32))
                    if gm is None:
                        gl, go = ll, lo
                    else:
                        keep = np.float32(np.exp(gm - hm)) if np.isfinite(gm) else np.float32(0)
                        gl, go = gl * keep + ll, go * keep + lo
                    gm = hm
                outs.append(go / gl if gl > 0 else np.zeros(d, np.float32))
                lses.append(np.float32(np.log(gl) + gm) if gl > 0 else np.float32(-np.inf))
            if len(outs) == 1:
                out[row, h] = outs[0]
            else:
                lses = np.array(lses, np.float32)
                top = lses.max()
                wts = np.where(np.isfinite(lses), np.exp(lses - top), 0).astype(np.float32) if np.isfinite(top) \
                    else np.zeros_like(lses)
                total = np.float32(wts.sum(dtype=np.float32))
                out[row, h] = (wts[:, None] * np.array(outs, np.float32)).sum(0) / total if total > 0 else 0
        row += 1
    return out


def mla_prefill(q_nope, q_rope, k_nope, k_rope, value, q_lens, kv_lens, scale, mask="none", window=0,
                kv_padded_rows=0):
    """Prefill attention of MultiLatentAttention (calcType PREFILL): sequence b owns q_lens[b] consecutive
    query rows and kv_lens[b] key / value rows (consecutive, or rows [b * kv_padded_rows, ...) when the keys
    come padded per sequence); head h of a query attends over KV head h // (heads // kv_heads).
    q_nope [T, H, 128], q_rope [T, H, 64], k_nope [Tk, G, 128], k_rope [Tk, G, 64], value [Tk, G, 128].
    mask: "none" (every query sees every key), "causal" (query i sees keys j <= i) or "window" (j <= i and
    j > i - window). Returns float32 [T, H, 128]."""
    q = np.concatenate([np.asarray(q_nope, np.float32), np.asarray(q_rope, np.float32)], axis=-1)
    k = np.concatenate([np.asarray(k_nope, np.float32), np.asarray(k_rope, np.float32)], axis=-1)
    v = np.asarray(value, np.float32)
    heads, kv_heads = q.shape[1], k.shape[1]
    group = heads // kv_heads
    out = np.zeros((q.shape[0], heads, v.shape[2]), np.float32)
    q0 = k0 = 0
    for b, (nq, nk) in enumerate(zip(q_lens, kv_lens)):
        nq, nk = int(nq), int(nk)
        if kv_padded_rows:
            k0 = b * kv_padded_rows
        if nq > 0 and nk > 0:
            i = np.arange(nq)[:, None]
            j = np.arange(nk)[None, :]
            hidden = np.zeros((nq, nk), bool)
            if mask in ("causal", "window"):
                hidden |= j > i
            if mask == "window":
                hidden |= j <= i - window
            for h in range(heads):
                g = h // group
                score = (q[q0:q0 + nq, h] @ k[k0:k0 + nk, g].T) * np.float32(scale)
                score = np.where(hidden, -np.inf, score).astype(np.float32)
                out[q0:q0 + nq, h] = softmax_rows(score) @ v[k0:k0 + nk, g]
        q0 += nq
        k0 += nk
    return out


def partial_attention(q, keys, values, scale):
    """Attention over a KV sub-range, in the form a split produces: the
    normalised output [heads, Dv] and the natural-log log-sum-exp [heads]."""
    heads = q.shape[0]
    kv_heads = keys.shape[1]
    group = heads // kv_heads
    out = np.empty((heads, values.shape[2]), dtype=np.float32)
    lse = np.empty((heads,), dtype=np.float32)
    for g in range(kv_heads):
        qg = q[g * group:(g + 1) * group].astype(np.float32)
        sim = (qg @ keys[:, g, :].astype(np.float32).T) * np.float32(scale)
        m = sim.max(axis=-1, keepdims=True)
        e = np.exp(sim - m)
        l = e.sum(axis=-1, keepdims=True)
        out[g * group:(g + 1) * group] = (e @ values[:, g, :].astype(np.float32)) / l
        lse[g * group:(g + 1) * group] = (np.log(l) + m)[:, 0]
    return out, lse


def merge_partials(outs, lses):
    """Split-KV combine: M = max lse; L = log(sum exp(lse - M)) + M;
    O = sum exp(lse_s - L) O_s. outs [splits, heads, Dv], lses [splits, heads];
    an empty split carries lse = -inf and weighs nothing."""
    outs = np.asarray(outs, dtype=np.float32)
    lses = np.asarray(lses, dtype=np.float32)
    m = lses.max(axis=0)
    with np.errstate(invalid="ignore"):
        big_l = np.log(np.exp(lses - m).sum(axis=0)) + m
        w = np.exp(lses - big_l)
    w = np.where(np.isneginf(lses), np.float32(0), w)
    return (w[:, :, None] * outs).sum(axis=0)
