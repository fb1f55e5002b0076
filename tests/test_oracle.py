"""Pins the CPU oracle (oracle/atb_oracle.py) without running any reference code:
closed forms, exact special cases, an independent float64 loop implementation,
torch's scaled_dot_product_attention on densely gathered rows, and the
invariants of paged attention. A plausible oracle mistake (wrong channel
index for the descale, a missing scale, a transposed operand, advancing the
query row over an empty sequence) fails at least one test here."""
import math

import numpy as np
import pytest
import torch


def _rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def _paged_case(rng, batch=3, heads=4, kv_heads=2, d=16, dv=16, block=4, pool=24, max_ctx=14, dtype=np.float32):
    ctx = rng.integers(1, max_ctx + 1, size=batch)
    nblk = (ctx + block - 1) // block
    perm = rng.permutation(pool)
    tables = np.zeros((batch, int(nblk.max())), dtype=np.int32)
    pos = 0
    for b in range(batch):
        tables[b, :nblk[b]] = perm[pos:pos + nblk[b]]
        tables[b, nblk[b]:] = perm[pos]
        pos += nblk[b]
    q = rng.standard_normal((batch, heads, d)).astype(dtype)
    kc = rng.standard_normal((pool, block, kv_heads, d)).astype(dtype)
    vc = rng.standard_normal((pool, block, kv_heads, dv)).astype(dtype)
    return q, kc, vc, tables, ctx.astype(np.int32)


# ---------------------------------------------------------------- reshape_and_cache
@pytest.mark.parametrize("dtype,dk,dv", [(np.float16, 8, 8), (np.int8, 12, 6), (np.float32, 5, 9)])
def test_reshape_and_cache_closed_form(oracle, dtype, dk, dv):
    rng = _rng(1)
    tokens, heads, blocks, block = 10, 3, 6, 4
    key = rng.integers(1, 11, size=(tokens, heads, dk)).astype(dtype)
    value = rng.integers(1, 11, size=(tokens, heads, dv)).astype(dtype)
    kc0 = rng.integers(20, 30, size=(blocks, block, heads, dk)).astype(dtype)
    vc0 = rng.integers(20, 30, size=(blocks, block, heads, dv)).astype(dtype)
    # unique slots drawn from [-N, N): negatives must be skipped
    slots = rng.choice(np.arange(-blocks * block, blocks * block), size=tokens, replace=False).astype(np.int32)
    kc, vc = oracle.reshape_and_cache(key, value, kc0, vc0, slots)
    ek = kc0.copy().reshape(blocks * block, heads * dk)
    ev = vc0.copy().reshape(blocks * block, heads * dv)
    keep = slots >= 0
    ek[slots[keep]] = key[keep].reshape(-1, heads * dk)
    ev[slots[keep]] = value[keep].reshape(-1, heads * dv)
    assert np.array_equal(kc.reshape(ek.shape), ek)
    assert np.array_equal(vc.reshape(ev.shape), ev)
    assert (slots < 0).any() and keep.any()
    # inputs are not modified, untouched slots keep their content
    untouched = np.setdiff1d(np.arange(blocks * block), slots[keep])
    assert np.array_equal(kc.reshape(ek.shape)[untouched], kc0.reshape(ek.shape)[untouched])


def test_reshape_and_cache_single_cache(oracle):
    key = np.arange(2 * 1 * 4, dtype=np.float32).reshape(2, 1, 4)
    kc0 = np.zeros((2, 2, 1, 4), dtype=np.float32)
    kc, vc = oracle.reshape_and_cache(key, None, kc0, None, np.array([3, -1], dtype=np.int32))
    assert vc is None
    assert np.array_equal(kc[1, 1, 0], key[0, 0]) and kc.sum() == key[0].sum()


@pytest.mark.parametrize("key_dtype,value_dtype,heads,dk,dv", [(np.int8, np.float16, 1, 64, 32),
                                                              (np.float16, np.float16, 3, 32, 16),
                                                              (np.int8, np.float32, 2, 48, 24)])
def test_reshape_and_cache_nz_by_flat_addresses(oracle, key_dtype, value_dtype, heads, dk, dv):
    """Element c of token i's flattened row must sit at flat address
    ((block * pieces + c // last) * block_size + offset) * last + c % last of the cache (reference
    test_reshape_and_cache_nz.py:45-66 spelled out per element), and un-tiling the result must give the
    plain token-major write."""
    rng = _rng(7)
    tokens, blocks, block = 9, 3, 16
    kl = 32 if key_dtype == np.int8 else 16
    key = rng.integers(-100, 100, size=(tokens, heads, dk)).astype(key_dtype)
    value = rng.integers(-100, 100, size=(tokens, heads, dv)).astype(value_dtype)
    kc0 = rng.integers(-9, 9, size=(blocks, heads * dk // kl, block, kl)).astype(key_dtype)
    vc0 = rng.integers(-9, 9, size=(blocks, heads * dv // 16, block, 16)).astype(value_dtype)
    slots = rng.choice(np.arange(-blocks * block, blocks * block), size=tokens, replace=False).astype(np.int32)
    slots[0] = 5
    kc, vc = oracle.reshape_and_cache_nz(key, value, kc0, vc0, slots)
    for cache, cache0, rows, last in ((kc, kc0, key.reshape(tokens, -1), kl), (vc, vc0, value.reshape(tokens, -1), 16)):
        expect = cache0.copy().reshape(-1)
        pieces = rows.shape[1] // last
        for i, s in enumerate(slots.tolist()):
            if s < 0:
                continue
            for c in range(rows.shape[1]):
                expect[((s // block * pieces + c // last) * block + s % block) * last + c % last] = rows[i, c]
        assert np.array_equal(cache.reshape(-1), expect)
        plain, _ = oracle.reshape_and_cache(rows[:, None, :], None, oracle.nz_to_nd(cache0)[:, :, None, :], None, slots)
        assert np.array_equal(oracle.nz_to_nd(cache), plain[:, :, 0, :])
    assert (slots < 0).any() and not np.array_equal(kc, kc0) and np.array_equal(kc0, kc0.copy())


def test_quant_golden_dtype_exact_rational(oracle):
    """The ElewiseOperation form (16-bit scale, quotient rounded to fp16, then to an integer) against exact
    rational arithmetic: the fp16 nearest to x / s (ties to even), then the integer nearest to that."""
    from fractions import Fraction
    import math
    bits = np.arange(0, 65536, 53, dtype=np.uint16)
    x = bits.view(np.float16)
    x = x[np.isfinite(x)]

    def nearest_fp16(q):
        f = np.float16(float(q))            # double -> fp16 rounds the double; the double of q may itself be rounded,
        lo, hi = np.nextafter(f, np.float16(-np.inf)), np.nextafter(f, np.float16(np.inf))
        best = min((c for c in (lo, f, hi) if np.isfinite(c)), key=lambda c: abs(Fraction(float(c)) - q), default=f)
        return best                          # so take the closest of the neighbours by exact distance

    for s in [np.float16(0.1), np.float16(0.337), np.float16(1.0), np.float16(3.0)]:
        got = oracle.quant_per_channel_golden_dtype(x, s, np.int8(5))
        for xi, gi in zip(x.tolist(), got.tolist()):
          with np.errstate(over="ignore"):   # quotients past the fp16 range are meant to overflow here
              q = Fraction(xi) / Fraction(float(s))
              h = nearest_fp16(q)
              if not np.isfinite(h) or abs(q) >= 65520:
                  want = 127 if q > 0 else -128
              else:
                  hf = Fraction(float(h))
                  r = math.floor(hf)
                  frac = hf - r
                  r = r + 1 if frac > Fraction(1, 2) or (frac == Fraction(1, 2) and r % 2 == 1) else r
                  want = max(-128, min(127, r + 5))
              # (a quotient exactly between two fp16 values is the one case the neighbour search cannot order; skip it)
              lo, hi = np.nextafter(h, np.float16(-np.inf)), np.nextafter(h, np.float16(np.inf))
              if np.isfinite(lo) and np.isfinite(hi) and abs(Fraction(float(h)) - q) in (abs(Fraction(float(lo)) - q), abs(Fraction(float(hi)) - q)):
                  continue
              assert gi == want, (xi, float(s), gi, want)


# ---------------------------------------------------------------- dequant_per_channel
def test_dequant_per_channel_exact_products_and_saturation(oracle):
    """Every (x - offset) is an integer in [-255, 255] and a scale has 11 significant bits, so the exact
    product fits a double: the fp16 result must be that product rounded once, or +-65504 past the range."""
    from fractions import Fraction
    rng = _rng(61)
    x = rng.integers(-128, 128, size=(5, 4, 8)).astype(np.int8)
    scale = rng.uniform(0.1, 1.0, size=(4, 8)).astype(np.float16)
    scale[0, 0], scale[0, 1], scale[0, 2] = np.float16(300.0), np.float16(-512.0), np.float16(6e-5)
    offset = rng.integers(-128, 128, size=(4, 8)).astype(np.int8)
    got = oracle.dequant_per_channel(x, scale, offset)
    assert got.dtype == np.float16 and got.shape == x.shape
    exact = (x.astype(np.float64) - offset.astype(np.float64)) * scale.astype(np.float64)
    want = np.clip(exact, -65504, 65504).astype(np.float16)   # float64 -> fp16 is one rounding of an exact value
    assert np.array_equal(got.view(np.int16), want.view(np.int16))
    assert np.isfinite(got).all() and (np.abs(exact) > 65504).any()
    assert Fraction(float(got[1, 1, 3])) == Fraction(float(np.float16(float(
        (int(x[1, 1, 3]) - int(offset[1, 3])) * Fraction(float(scale[1, 3]))))))
    # no offset, and a single scale for everything
    assert np.array_equal(oracle.dequant_per_channel(x, scale), np.clip(x.astype(np.float64) * scale.astype(np.float64), -65504, 65504).astype(np.float16))
    one = oracle.dequant_per_channel(x, np.array([0.5], np.float16), np.array([3], np.int8))
    assert np.array_equal(one, ((x.astype(np.float32) - 3) * 0.5).astype(np.float16))


# ---------------------------------------------------------------- strided_view
def test_strided_view_matches_library_views_and_loops(oracle):
    """Against numpy's and torch's own strided views, against the element loop of the reference's unit
    test, and on a closed form (storage[i] = i makes every element its own address)."""
    import torch
    rng = _rng(5)
    storage = rng.standard_normal(9000).astype(np.float32)
    cases = [((2, 32, 128), (32 * 128, 128, 1), 5),    # the reference unit test's view (overlapping tokens, odd offset)
             ((3, 4, 8), (4 * 16 * 3, 16, 1), 16),     # the K slice of a fused [T, 3, H, D] projection
             ((3, 4, 8), (100, 24, 3), 7),             # channels not contiguous
             ((2, 3, 4), (12, 4, 1), 0)]               # a plain contiguous tensor
    for shape, strides, offset in cases:
        got = oracle.strided_view(storage, shape, strides, offset)
        lib = np.lib.stride_tricks.as_strided(storage[offset:], shape=shape, strides=[4 * st for st in strides])
        assert np.array_equal(got, lib)
        assert np.array_equal(got, torch.as_strided(torch.from_numpy(storage), shape, strides, offset).numpy())
        addr = oracle.strided_view(np.arange(9000), shape, strides, offset)
        t, h, d = 1, shape[1] - 1, shape[2] - 2
        assert addr[t, h, d] == offset + t * strides[0] + h * strides[1] + d * strides[2]
    shape, strides, offset = cases[2]
    got = oracle.strided_view(storage, shape, strides, offset)
    for t in range(shape[0]):
        for h in range(shape[1]):
            for d in range(shape[2]):
                assert got[t, h, d] == storage[offset + t * strides[0] + h * strides[1] + d * strides[2]]


# ---------------------------------------------------------------- rope
def _rotate_half(x):
    x0, x1 = x.chunk(2, -1)
    return __import__("torch").cat((-x1, x0), dim=-1)


def test_rope_against_the_three_forms_the_reference_tests_use(oracle):
    """rotaryCoeff 2 against x * cos + rotate_half(x) * sin over whole heads, 4 against the same applied to
    the two halves of a head separately, rotaryCoeff = head size against the interleaved-pair form; then
    the rotation as a complex multiplication, and the positions of cosFormat 1."""
    import torch
    rng = _rng(23)
    T, heads_q, heads_k, d = 7, 6, 2, 16
    q = torch.from_numpy(rng.standard_normal((T, heads_q * d)).astype(np.float32))
    k = torch.from_numpy(rng.standard_normal((T, heads_k * d)).astype(np.float32))
    cos = torch.from_numpy(rng.standard_normal((T, d)).astype(np.float32))
    sin = torch.from_numpy(rng.standard_normal((T, d)).astype(np.float32))
    lens = np.array([T], dtype=np.int32)
    f32 = dict(out_dtype=np.float32)
    # coefficient 2: whole heads
    for x, got in zip((q, k), oracle.rope(q.numpy(), k.numpy(), cos.numpy(), sin.numpy(), lens, 2, **f32)):
        xh = x.view(T, -1, d)
        want = xh * cos[:, None] + _rotate_half(xh) * sin[:, None]
        np.testing.assert_allclose(got, want.reshape(T, -1).numpy(), rtol=1e-6, atol=1e-6)
    # coefficient 4: the halves of a head, each with its half of the tables
    for x, got in zip((q, k), oracle.rope(q.numpy(), k.numpy(), cos.numpy(), sin.numpy(), lens, 4, **f32)):
        x0, x1 = x.view(T, -1, d).chunk(2, -1)
        c0, c1 = cos[:, None].chunk(2, -1)
        s0, s1 = sin[:, None].chunk(2, -1)
        want = torch.cat([x0 * c0 + _rotate_half(x0) * s0, x1 * c1 + _rotate_half(x1) * s1], dim=-1)
        np.testing.assert_allclose(got, want.reshape(T, -1).numpy(), rtol=1e-6, atol=1e-6)
    # coefficient = head size: neighbouring channels pair up; tables repeat every entry once
    half = torch.from_numpy(rng.standard_normal((T, d // 2)).astype(np.float32))
    half_s = torch.from_numpy(rng.standard_normal((T, d // 2)).astype(np.float32))
    cos_r, sin_r = half.repeat_interleave(2, dim=1), half_s.repeat_interleave(2, dim=1)
    for x, got in zip((q, k), oracle.rope(q.numpy(), k.numpy(), cos_r.numpy(), sin_r.numpy(), lens, d, **f32)):
        xs = x.view(T, -1, d // 2, 2)
        c, s_ = half[:, None], half_s[:, None]
        want = torch.stack([xs[..., 0] * c - xs[..., 1] * s_, xs[..., 1] * c + xs[..., 0] * s_], -1)
        np.testing.assert_allclose(got, want.reshape(T, -1).numpy(), rtol=1e-6, atol=1e-6)
    # a rotation: with cos / sin of one angle per pair, (x[i] + j x[i + d/2]) turns by that angle
    theta = rng.uniform(0, 2 * np.pi, size=(T, d // 2))
    ct = np.concatenate([np.cos(theta), np.cos(theta)], axis=1).astype(np.float32)
    st = np.concatenate([np.sin(theta), np.sin(theta)], axis=1).astype(np.float32)
    got, _ = oracle.rope(q.numpy(), k.numpy(), ct, st, lens, 2, **f32)
    qh = q.numpy().reshape(T, heads_q, d).astype(np.float64)
    z = (qh[..., :d // 2] + 1j * qh[..., d // 2:]) * np.exp(1j * theta)[:, None]
    np.testing.assert_allclose(got.reshape(T, heads_q, d), np.concatenate([z.real, z.imag], axis=-1), rtol=1e-5, atol=1e-5)
    # cosFormat 1: row = position inside the sequence; the same as cosFormat 0 with the rows gathered by hand
    seq = np.array([3, 1, 3], dtype=np.int32)
    pos = np.array([0, 1, 2, 0, 0, 1, 2])
    table_c, table_s = cos.numpy()[:4], sin.numpy()[:4]
    a = oracle.rope(q.numpy(), k.numpy(), table_c, table_s, seq, 2, cos_format=1, **f32)
    b = oracle.rope(q.numpy(), k.numpy(), table_c[pos], table_s[pos], seq, 2, cos_format=0, **f32)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    # 16-bit results are the fp32 ones rounded once
    h = oracle.rope(q.numpy(), k.numpy(), cos.numpy(), sin.numpy(), lens, 2)
    assert h[0].dtype == np.float16
    assert np.array_equal(h[0], oracle.rope(q.numpy(), k.numpy(), cos.numpy(), sin.numpy(), lens, 2, **f32)[0].astype(np.float16))


# ---------------------------------------------------------------- norm_rope_reshape
def test_norm_rope_reshape_closed_forms_and_library_routines(oracle):
    """RMSNorm against torch's own rms_norm and two closed forms; the rotation against complex
    multiplication (channel i and i + half are the real and imaginary part of one number turned by
    the angle whose cosine / sine the tables hold); slot placement against direct indexing."""
    import torch
    rng = _rng(21)
    T, n, r, blocks, block = 9, 64, 16, 3, 8
    x = rng.standard_normal((T, 1, n)).astype(np.float32)
    gamma = rng.standard_normal(n).astype(np.float32)
    rope = rng.standard_normal((T, r)).astype(np.float32)
    theta = rng.uniform(0, 2 * np.pi, size=(T, r // 2))
    cos = np.concatenate([np.cos(theta), np.cos(theta)], axis=1).astype(np.float32)
    sin = np.concatenate([np.sin(theta), np.sin(theta)], axis=1).astype(np.float32)
    cache0 = rng.standard_normal((blocks, block, 1, n + r)).astype(np.float32)
    slots = rng.choice(np.arange(-blocks * block, blocks * block), size=T, replace=False).astype(np.int32)
    slots[:2] = [5, -3]
    eps = 1e-5
    got = oracle.norm_rope_reshape(x, gamma, rope, cos, sin, slots, cache0, eps, out_dtype=np.float32)
    want_norm = torch.nn.functional.rms_norm(torch.from_numpy(x).double(), (n,), torch.from_numpy(gamma).double(),
                                             eps).numpy().reshape(T, n)
    z = (rope[:, :r // 2].astype(np.float64) + 1j * rope[:, r // 2:]) * np.exp(1j * theta)
    want_rope = np.concatenate([z.real, z.imag], axis=1)
    flat = got.reshape(blocks * block, n + r)
    flat0 = cache0.reshape(blocks * block, n + r)
    for i, s in enumerate(slots.tolist()):
        if s >= 0:
            np.testing.assert_allclose(flat[s, :n], want_norm[i], rtol=2e-6, atol=2e-6)
            np.testing.assert_allclose(flat[s, n:], want_rope[i], rtol=2e-6, atol=2e-6)
            # a rotation keeps the length of every (i, i + half) pair
            np.testing.assert_allclose(flat[s, n:n + r // 2] ** 2 + flat[s, n + r // 2:] ** 2,
                                       rope[i, :r // 2] ** 2 + rope[i, r // 2:] ** 2, rtol=1e-5)
    untouched = np.setdiff1d(np.arange(blocks * block), slots[slots >= 0])
    assert np.array_equal(flat[untouched], flat0[untouched]) and (slots < 0).any()
    # closed forms: a constant row normalises to sign(c) * gamma (up to epsilon); a row with one non-zero
    # channel a to a / sqrt(a^2 / n + eps) there; angle 0 leaves the rotary row alone, a quarter turn maps
    # (first, second) to (-second, first)
    xc = np.full((1, 1, n), -3.0, dtype=np.float32)
    one = np.ones((1, r), np.float32)
    zero = np.zeros((1, r), np.float32)
    out = oracle.norm_rope_reshape(xc, gamma, rope[:1], one, zero, [0], cache0, eps, out_dtype=np.float32)
    np.testing.assert_allclose(out[0, 0, 0, :n], -gamma / np.sqrt(1 + eps / 9), rtol=1e-6)
    assert np.array_equal(out[0, 0, 0, n:], rope[0])
    xh = np.zeros((1, 1, n), np.float32)
    xh[0, 0, 7] = 4.0
    out = oracle.norm_rope_reshape(xh, np.ones(n, np.float32), rope[:1], zero, one, [1], cache0, eps, out_dtype=np.float32)
    assert abs(out[0, 1, 0, 7] - 4.0 / np.sqrt(16.0 / n + eps)) < 1e-5 and np.count_nonzero(out[0, 1, 0, :n]) == 1
    assert np.array_equal(out[0, 1, 0, n:], np.concatenate([-rope[0, r // 2:], rope[0, :r // 2]]))
    # the 16-bit results are the fp32 ones rounded once
    h = oracle.norm_rope_reshape(x, gamma, rope, cos, sin, slots, cache0.astype(np.float16), eps)
    assert h.dtype == np.float16 and np.array_equal(h[0, 5, 0], got[0, 5, 0].astype(np.float16))
    b = oracle.norm_rope_reshape(x, gamma, rope, cos, sin, slots, cache0, eps, out_dtype="bf16")
    assert np.array_equal(b[0, 5, 0], oracle.bf16_round(got[0, 5, 0]))


# ---------------------------------------------------------------- quantiser
def test_quant_special_cases(oracle):
    s = np.float32(0.5)
    x = np.array([0.25, 0.75, 1.25, -0.25, -0.75, -1.25, 0.0, -0.0, 1000.0, -1000.0, np.inf, -np.inf, np.nan,
                  63.5, 63.75, -64.0, -64.25, 6e-8], dtype=np.float32)
    #            0.5->0 1.5->2 2.5->2 -0.5->0 -1.5->-2 -2.5->-2
    want = np.array([0, 2, 2, 0, -2, -2, 0, 0, 127, -128, 127, -128, 0, 127, 127, -128, -128, 0], dtype=np.int8)
    assert np.array_equal(oracle.quant_per_channel(x, s), want)
    # offset is added after rounding and before the clamp
    assert np.array_equal(oracle.quant_per_channel(x[:3], s, np.array([3, -3, 126])), np.array([3, -1, 127], np.int8))


def test_quant_exact_rational(oracle):
    """x/s rounded to fp32 then to the nearest-even integer, checked against exact
    rational arithmetic for every fp16 x on a few scales."""
    from fractions import Fraction
    bits = np.arange(0, 65536, 37, dtype=np.uint16)  # a stride through all patterns, both signs
    x = bits.view(np.float16)
    x = x[np.isfinite(x)]
    for s in [np.float32(0.005), np.float32(0.0123), np.float32(0.02), np.float32(1.0), np.float32(3.0)]:
        got = oracle.quant_per_channel(x.astype(np.float32), s)
        for xi, gi in zip(x.tolist(), got.tolist()):
            quot = Fraction(xi) / Fraction(float(s))
            f32 = np.float32(float(quot))  # double then single: both roundings checked below
            # guard against double rounding: the exact quotient must not sit on an fp32 tie
            lo, hi = np.nextafter(f32, np.float32(-np.inf)), np.nextafter(f32, np.float32(np.inf))
            assert abs(quot - Fraction(float(f32))) <= min(abs(quot - Fraction(float(lo))),
                                                           abs(quot - Fraction(float(hi))))
            fr = Fraction(float(f32))
            fl = math.floor(fr)
            rem = fr - fl
            r = fl if rem < Fraction(1, 2) else fl + 1 if rem > Fraction(1, 2) else (fl if fl % 2 == 0 else fl + 1)
            assert gi == max(-128, min(127, r)), (xi, float(s))


def test_quant_all_fp16_patterns_vs_golden_dtype(oracle):
    """The reference golden divides in fp16 and is accepted with atol=1; the fp32
    form must stay within that band for every finite fp16 input, and be monotone."""
    x = np.arange(65536, dtype=np.uint16).view(np.float16)
    x = x[np.isfinite(x)]
    for s in [0.1, 0.37, 1.0]:
        a = oracle.quant_per_channel(x.astype(np.float32), np.float32(np.float16(s))).astype(np.int32)
        b = oracle.quant_per_channel_golden_dtype(x, np.float16(s)).astype(np.int32)
        assert np.abs(a - b).max() <= 1
        order = np.argsort(x.astype(np.float32), kind="stable")
        assert (np.diff(a[order]) >= 0).all()


def test_quant_per_channel_axis(oracle):
    x = np.ones((3, 4), dtype=np.float32)
    s = np.array([1.0, 0.5, 0.25, 0.125], dtype=np.float32)
    assert np.array_equal(oracle.quant_per_channel(x, s), np.tile(np.array([1, 2, 4, 8], np.int8), (3, 1)))


# ---------------------------------------------------------------- block_copy, paged_cache_load
def test_block_copy_closed_form(oracle):
    """With disjoint sources and destinations every destination j ends up holding the block of the
    source whose cumSum interval contains j, and every other block is untouched."""
    rng = _rng(60)
    blocks = 40
    kc = rng.integers(-100, 100, size=(blocks, 4, 2, 8)).astype(np.int8)
    vc = rng.integers(-100, 100, size=(blocks, 4, 2, 8)).astype(np.int8)
    perm = rng.permutation(blocks)
    src, dst = perm[:5].astype(np.int32), perm[5:5 + 17].astype(np.int32)
    cum = np.array([3, 3, 9, 10, 17], np.int32)   # source 1 has no destination
    got_k, got_v = oracle.block_copy(kc, vc, src, dst, cum)
    owner = np.searchsorted(cum, np.arange(17), side="right")
    want_k, want_v = kc.copy(), vc.copy()
    want_k[dst] = kc[src[owner]]
    want_v[dst] = vc[src[owner]]
    assert np.array_equal(got_k, want_k) and np.array_equal(got_v, want_v)
    untouched = np.setdiff1d(np.arange(blocks), dst)
    assert np.array_equal(got_k[untouched], kc[untouched])
    # nothing to do
    same_k, _ = oracle.block_copy(kc, vc, src[:0], dst[:0], cum[:0])
    assert np.array_equal(same_k, kc)


@pytest.mark.parametrize("cumsum,starts", [(False, False), (True, False), (False, True), (True, True)])
def test_paged_cache_load_is_the_concatenation_of_gathered_rows(oracle, cumsum, starts):
    rng = _rng(61)
    blocks, block, heads, dk, dv = 30, 4, 2, 6, 3
    kc = rng.standard_normal((blocks, block, heads, dk)).astype(np.float32)
    vc = rng.standard_normal((blocks, block, heads, dv)).astype(np.float32)
    lens = np.array([5, 0, 13, 4, 1], np.int32)
    tables = rng.integers(0, blocks, size=(5, 8)).astype(np.int32)
    seq_starts = (rng.integers(0, 4, size=5) * block).astype(np.int32) if starts else None
    total = int(lens.sum())
    key0 = np.full((total + 2, heads, dk), 9.0, np.float32)
    val0 = np.full((total + 2, heads, dv), 9.0, np.float32)
    arg = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32) if cumsum else lens
    got_k, got_v = oracle.paged_cache_load(kc, vc, tables, arg, key0, val0, seq_starts, cumsum)
    want_k, want_v = [], []
    for i, n in enumerate(lens):
        shift = 0 if seq_starts is None else seq_starts[i] // block
        want_k.append(oracle.gather_rows(kc, tables[i][shift:], n))
        want_v.append(oracle.gather_rows(vc, tables[i][shift:], n))
    assert np.array_equal(got_k[:total], np.concatenate(want_k)) and np.array_equal(got_v[:total], np.concatenate(want_v))
    assert np.all(got_k[total:] == 9.0) and np.all(got_v[total:] == 9.0)
    # it undoes reshape_and_cache: rows written to their slots come back in order
    slots = np.concatenate([tables[i][(0 if seq_starts is None else seq_starts[i] // block) + np.arange(n) // block]
                            * block + np.arange(n) % block for i, n in enumerate(lens)])
    if len(np.unique(slots)) == len(slots):
        new_k = rng.standard_normal((total, heads, dk)).astype(np.float32)
        new_v = rng.standard_normal((total, heads, dv)).astype(np.float32)
        kc2, vc2 = oracle.reshape_and_cache(new_k, new_v, kc, vc, slots.astype(np.int32))
        back_k, back_v = oracle.paged_cache_load(kc2, vc2, tables, arg, key0, val0, seq_starts, cumsum)
        assert np.array_equal(back_k[:total], new_k) and np.array_equal(back_v[:total], new_v)


def test_paged_cache_load_negative_block_ids_leave_their_rows(oracle):
    kc = np.arange(2 * 2 * 1 * 1, dtype=np.float32).reshape(2, 2, 1, 1) + 1
    tables = np.array([[1, -1, 0]], np.int32)
    k, v = oracle.paged_cache_load(kc, kc, tables, np.array([5], np.int32), np.zeros((5, 1, 1), np.float32),
                                   np.zeros((5, 1, 1), np.float32))
    assert k[:, 0, 0].tolist() == [3.0, 4.0, 0.0, 0.0, 1.0] and np.array_equal(k, v)


@pytest.mark.parametrize("key_dtype,value_dtype", [(np.int8, np.int8), (np.int8, np.float16), (np.float16, np.float16)])
def test_paged_cache_load_nz_by_flat_addresses_and_round_trip(oracle, key_dtype, value_dtype):
    rng = _rng(62)
    blocks, block, ck, cv = 7, 16, 64, 32
    kl, vl = (32 if key_dtype == np.int8 else 16), (32 if value_dtype == np.int8 else 16)
    kc = rng.integers(-100, 100, size=(blocks, ck // kl, block, kl)).astype(key_dtype)
    vc = rng.integers(-100, 100, size=(blocks, cv // vl, block, vl)).astype(value_dtype)
    lens = np.array([17, 0, 40, 1], np.int32)
    tables = rng.integers(0, blocks, size=(4, 3)).astype(np.int32)
    total = int(lens.sum())
    key0 = np.full((total + 1, ck), 9, key_dtype)
    val0 = np.full((total + 1, cv), 9, value_dtype)
    got_k, got_v = oracle.paged_cache_load_nz(kc, vc, tables, lens, key0, val0)
    # element by element over the flat cache
    for cache, got, last in ((kc, got_k, kl), (vc, got_v, vl)):
        flat, chans, row = cache.reshape(-1), got.shape[1], 0
        for i, n in enumerate(lens):
            for j in range(n):
                blk = tables[i][j // block]
                for c in range(chans):
                    assert got[row, c] == flat[((blk * (chans // last) + c // last) * block + j % block) * last + c % last]
                row += 1
        assert row == total and np.all(got[total:] == 9)
    # the token-major gather over the un-tiled caches
    nd_k, nd_v = oracle.paged_cache_load(oracle.nz_to_nd(kc)[:, :, None, :], oracle.nz_to_nd(vc)[:, :, None, :], tables, lens,
                                         key0[:, None, :], val0[:, None, :])
    assert np.array_equal(nd_k[:, 0, :], got_k) and np.array_equal(nd_v[:, 0, :], got_v)
    # it undoes reshape_and_cache_nz (value caches written by that operator are 16-bit, pieces of 16)
    if vl == 16:
        tables = rng.permutation(blocks)[:6].reshape(2, 3).astype(np.int32)
        lens = np.array([33, 48], np.int32)
        slots = np.concatenate([tables[i][np.arange(n) // block] * block + np.arange(n) % block for i, n in enumerate(lens)])
        new_k = rng.integers(-100, 100, size=(81, 1, ck)).astype(key_dtype)
        new_v = rng.integers(-100, 100, size=(81, 1, cv)).astype(value_dtype)
        kc2, vc2 = oracle.reshape_and_cache_nz(new_k, new_v, kc, vc, slots.astype(np.int32))
        back_k, back_v = oracle.paged_cache_load_nz(kc2, vc2, tables, lens, np.zeros((81, ck), key_dtype), np.zeros((81, cv), value_dtype))
        assert np.array_equal(back_k, new_k[:, 0, :]) and np.array_equal(back_v, new_v[:, 0, :])


# ---------------------------------------------------------------- cache write under head compression
def _compress_case(rng, batch=3, heads=4, d=32, block=16, dtype=np.float16):
    seq = rng.integers(20, 60, size=batch).astype(np.int32)
    tokens = int(seq.sum())
    key = rng.integers(-8, 9, size=(tokens, heads, d)).astype(dtype)
    value = rng.integers(-8, 9, size=(tokens, heads, d)).astype(dtype)
    return seq, key, value


def test_compress_keep_last_by_flat_addresses(oracle):
    """COMPRESS_TYPE_KVHEAD against element-wise loops over flat addresses of key and cache."""
    rng = _rng(41)
    batch, heads, d, block = 3, 4, 32, 16
    seq, key, value = _compress_case(rng, batch, heads, d, block)
    wins = rng.integers(0, 20, size=batch * heads).astype(np.int32)
    starts_of = np.concatenate([[0], np.cumsum((wins + block - 1) // block)[:-1]]) * block
    slots = starts_of.astype(np.int32)
    slots[5] = -1
    blocks = int(((wins + block - 1) // block).sum()) + 1
    kc0 = np.full((blocks, block, 1, d), 77, dtype=np.float16)
    kc, vc = oracle.reshape_and_cache_compress(key, value, kc0, kc0, slots, wins, seq)
    want_k, want_v = kc0.ravel().copy(), kc0.ravel().copy()
    kf, vf = key.ravel(), value.ravel()
    ends = np.cumsum(seq)
    for i in range(batch * heads):
        if slots[i] < 0:
            continue
        for j in range(int(wins[i])):
            tok = int(ends[i // heads]) - int(wins[i]) + j
            for c in range(d):
                want_k[(slots[i] + j) * d + c] = kf[(tok * heads + i % heads) * d + c]
                want_v[(slots[i] + j) * d + c] = vf[(tok * heads + i % heads) * d + c]
    assert np.array_equal(kc.ravel(), want_k) and np.array_equal(vc.ravel(), want_v)
    assert np.array_equal(kc0, np.full_like(kc0, 77))  # the inputs are not written


def test_compress_mean_window_invariants(oracle):
    """COMPRESS_TYPE_KVHEAD_ROPE: a pair fills seqLen - win + 1 slots (seqLen with no window); a window of one
    token is that token, so the result equals the plain copy; the window's slot holds the mean of its
    tokens (float64 mean as the yardstick) and its neighbours the tokens next to the window."""
    rng = _rng(42)
    batch, heads, d, block = 3, 2, 32, 16
    seq, key, value = _compress_case(rng, batch, heads, d, block, np.float32)
    key = key + rng.standard_normal(key.shape).astype(np.float32)
    pairs = batch * heads
    stride = 64  # slots per pair, generous
    slots = (np.arange(pairs) * stride).astype(np.int32)
    blocks = pairs * stride // block
    marker = np.float32(-555.0)
    kc0 = np.full((blocks, block, 1, d), marker, dtype=np.float32)
    wins = np.array([5, 1, 0, 7, 20, 3], dtype=np.int32)
    offs = np.array([3, 4, 2, -1, 0, int(seq[2]) - 3], dtype=np.int32)  # last: the window ends the sequence
    kc, vc = oracle.reshape_and_cache_compress(key, value, kc0, kc0, slots, wins, seq, offs)
    flat = kc.reshape(-1, d)
    starts = np.cumsum(seq) - seq
    for i in range(pairs):
        b, h = divmod(i, heads)
        n = int(seq[b]) if offs[i] == -1 or wins[i] == 0 else int(seq[b]) - int(wins[i]) + 1
        used = flat[slots[i]:slots[i] + stride]
        assert (used[:n] != marker).all() and (used[n:] == marker).all(), i
        rows = key[starts[b]:starts[b] + seq[b], h]
        if offs[i] == -1 or wins[i] <= 1:
            assert np.array_equal(used[:n], rows), i
            continue
        o, w = int(offs[i]), int(wins[i])
        assert np.array_equal(used[:o], rows[:o]) and np.array_equal(used[o + 1:n], rows[o + w:]), i
        np.testing.assert_allclose(used[o], rows[o:o + w].astype(np.float64).mean(axis=0), rtol=1e-5, atol=1e-6)
    # rounding to the cache dtype, nearest even, is what the device kernel stores
    k16 = key.astype(np.float16)
    kc16, _ = oracle.reshape_and_cache_compress(k16, k16, kc0.astype(np.float16), kc0.astype(np.float16), slots, wins,
                                                seq, offs, out_dtype="float16")
    kc32, _ = oracle.reshape_and_cache_compress(k16, k16, kc0, kc0, slots, wins, seq, offs)
    assert np.array_equal(kc16, kc32.astype(np.float16))


def test_omni_drop_window_by_flat_addresses_and_relations(oracle):
    """ReshapeAndCacheOmni: (1) against element loops over flat addresses whose token list is built another way
    (np.delete of the window from the sequence's token numbers); (2) a pair fills seqLen - win slots (seqLen
    without a window) and nothing else; (3) with no window anywhere the result is the plain cache write of each
    head's rows; (4) it is mean-window's result with the mean's slot taken out."""
    rng = _rng(43)
    batch, heads, d, block = 3, 2, 32, 16
    seq, key, value = _compress_case(rng, batch, heads, d, block)
    pairs = batch * heads
    stride = 64
    slots = (np.arange(pairs) * stride).astype(np.int32)
    slots[4] = -1
    blocks = pairs * stride // block
    marker = np.float16(-555.0)
    kc0 = np.full((blocks, block, 1, d), marker, dtype=np.float16)
    wins = np.array([5, 1, 0, 7, 20, 3], dtype=np.int32)
    offs = np.array([3, 0, 2, -1, 0, int(seq[2]) - 3], dtype=np.int32)  # last: the window ends the sequence
    kc, vc = oracle.reshape_and_cache_omni(key, value, kc0, kc0, slots, wins, seq, offs)
    assert np.array_equal(kc0, np.full_like(kc0, marker))  # the inputs are not written
    starts = np.cumsum(seq) - seq
    want_k, want_v = kc0.ravel().copy(), kc0.ravel().copy()
    kf, vf = key.ravel(), value.ravel()
    counts = []
    for i in range(pairs):
        b, h = divmod(i, heads)
        toks = np.arange(starts[b], starts[b] + seq[b])
        if offs[i] != -1:
            toks = np.delete(toks, np.arange(offs[i], offs[i] + wins[i]))
        counts.append(len(toks))
        if slots[i] < 0:
            continue
        for n, tok in enumerate(toks.tolist()):
            for c in range(d):
                want_k[(slots[i] + n) * d + c] = kf[(tok * heads + h) * d + c]
                want_v[(slots[i] + n) * d + c] = vf[(tok * heads + h) * d + c]
    assert np.array_equal(kc.ravel(), want_k) and np.array_equal(vc.ravel(), want_v)
    per_seq = np.repeat(seq, heads)
    assert counts == np.where(offs == -1, per_seq, per_seq - wins).tolist()
    # (3) no window: every head's rows through the plain write
    none = np.full(pairs, -1, dtype=np.int32)
    kc_all, vc_all = oracle.reshape_and_cache_omni(key, value, kc0, kc0, slots, wins, seq, none)
    for i in range(pairs):
        if slots[i] < 0:
            continue
        b, h = divmod(i, heads)
        rows = slice(int(starts[b]), int(starts[b] + seq[b]))
        plain_k, plain_v = oracle.reshape_and_cache(key[rows, h:h + 1], value[rows, h:h + 1], kc0, kc0,
                                                    np.arange(slots[i], slots[i] + seq[b], dtype=np.int32))
        mine = slice(int(slots[i]), int(slots[i]) + stride)
        assert np.array_equal(kc_all.reshape(-1, d)[mine], plain_k.reshape(-1, d)[mine])
        assert np.array_equal(vc_all.reshape(-1, d)[mine], plain_v.reshape(-1, d)[mine])
    zero_win, _ = oracle.reshape_and_cache_omni(key, value, kc0, kc0, slots, np.zeros(pairs, np.int32), seq, offs)
    assert np.array_equal(zero_win, kc_all)
    # (4) mean-window keeps one slot for the window, this one none
    mean_k, _ = oracle.reshape_and_cache_compress(key, value, kc0, kc0, slots, wins, seq, offs, out_dtype="float16")
    for i in range(pairs):
        if slots[i] < 0:
            continue
        mine = kc.reshape(-1, d)[slots[i]:slots[i] + stride]
        other = mean_k.reshape(-1, d)[slots[i]:slots[i] + stride]
        if offs[i] == -1 or wins[i] == 0:
            assert np.array_equal(mine, other), i
        else:
            assert np.array_equal(mine[:stride - 1], np.delete(other, offs[i], axis=0)), i


# ---------------------------------------------------------------- attention
def test_attention_matches_independent_loops(oracle):
    rng = _rng(2)
    q, kc, vc, tables, ctx = _paged_case(rng)
    scale = 1.0 / math.sqrt(q.shape[2])
    got = oracle.paged_attention(q, kc, vc, tables, ctx, scale)
    want = oracle.paged_attention_loops(q, kc, vc, tables, ctx, scale)
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-6)


def test_attention_head_major_blocks_by_flat_addresses(oracle):
    """TYPE_BNSD caches: element (block b, head g, offset o, channel c) sits at flat address
    ((b * heads + g) * block + o) * D + c. The token-major cache is rebuilt from those addresses
    one row at a time and run through the loop version."""
    rng = _rng(23)
    heads, kv_heads, d, dv, block, pool = 6, 3, 16, 8, 4, 19
    ctx = np.array([9, 0, 4, 13], dtype=np.int32)
    tables = rng.permutation(pool)[:16].reshape(4, 4).astype(np.int32)
    q = rng.standard_normal((3, heads, d)).astype(np.float32)
    kc_hm = rng.standard_normal((pool, kv_heads, block, d)).astype(np.float32)
    vc_hm = rng.standard_normal((pool, kv_heads, block, dv)).astype(np.float32)

    def token_major(hm, width):
        flat = hm.ravel()
        tm = np.empty((pool, block, kv_heads, width), dtype=np.float32)
        for b in range(pool):
            for o in range(block):
                for g in range(kv_heads):
                    at = ((b * kv_heads + g) * block + o) * width
                    tm[b, o, g] = flat[at:at + width]
        return tm

    got = oracle.paged_attention(q, kc_hm, vc_hm, tables, ctx, 0.3, head_major=True)
    want = oracle.paged_attention_loops(q, token_major(kc_hm, d), token_major(vc_hm, dv), tables, ctx, 0.3)
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-6)
    # and it is not the token-major reading of the same buffer
    other = oracle.paged_attention(q, kc_hm.reshape(pool, block, kv_heads, d), vc_hm.reshape(pool, block, kv_heads, dv),
                                   tables, ctx, 0.3)
    assert np.abs(other - got).max() > 1e-2


def _compressed_twin(kc, vc, tables, ctx, n):
    """The head-compressed form of an ordinary paged cache: block b * n + g holds head g of block b,
    and pair (sequence s, head g) gets the table row of s mapped the same way."""
    pool, block = kc.shape[:2]
    kc_c = np.ascontiguousarray(kc.transpose(0, 2, 1, 3)).reshape(pool * n, block, 1, kc.shape[3])
    vc_c = np.ascontiguousarray(vc.transpose(0, 2, 1, 3)).reshape(pool * n, block, 1, vc.shape[3])
    tables_c = (np.repeat(tables, n, axis=0) * n + np.tile(np.arange(n), len(tables))[:, None]).astype(np.int32)
    return kc_c, vc_c, tables_c, np.repeat(ctx, n).astype(np.int32)


@pytest.mark.parametrize("mask_kind", [None, "norm3", "alibi4", "alibi4_1", "alibi3", "razor"])
def test_head_compression_equals_ordinary_attention_on_the_twin_cache(oracle, mask_kind):
    """With equal lengths for all KV heads of a sequence, attention over (sequence, KV head) pairs is
    ordinary GQA attention on a rearranged cache: checked against the loop version on the ordinary
    cache, masks and the per-slot score offsets (as a dense bias of offset * scale) included."""
    rng = _rng(31)
    heads, n, d, dv, block, pool = 6, 3, 16, 8, 4, 23
    ctx = np.array([9, 0, 4, 13], dtype=np.int32)
    tables = rng.permutation(pool)[:16].reshape(4, 4).astype(np.int32)
    q = rng.standard_normal((3, heads, d)).astype(np.float32)
    kc = rng.standard_normal((pool, block, n, d)).astype(np.float32)
    vc = rng.standard_normal((pool, block, n, dv)).astype(np.float32)
    kc_c, vc_c, tables_c, ctx_c = _compressed_twin(kc, vc, tables, ctx, n)
    max_len, scale = 16, 0.3
    mask = razor = None
    dense = np.zeros((4, heads, max_len), dtype=np.float32)
    per_head = None
    if mask_kind == "norm3":
        mask = rng.standard_normal((4, 1, max_len)).astype(np.float32)
        dense[:] = mask
    elif mask_kind == "alibi4":
        mask = rng.standard_normal((4, heads, 1, max_len)).astype(np.float32)
        dense[:] = mask[:, :, 0]
    elif mask_kind == "alibi4_1":
        mask = rng.standard_normal((4, 1, 1, max_len)).astype(np.float32)
        dense[:] = mask[:, :, 0]
    elif mask_kind == "alibi3":
        mask = rng.standard_normal((heads, 1, max_len)).astype(np.float32)
        dense[:] = mask[None, :, 0]
        per_head = True
    elif mask_kind == "razor":
        razor = rng.uniform(0, 20, size=(pool * n, block)).astype(np.float32)
        for i in range(4):
            for h in range(heads):
                for j in range(int(ctx[i])):
                    dense[i, h, j] = razor[tables[i, j // block] * n + h // (heads // n), j % block] * scale
    got = oracle.paged_attention(q, kc_c, vc_c, tables_c, ctx_c, scale, mask=mask, mask_per_head=per_head,
                                 compress_kv_heads=n, razor_offset=razor)
    want = oracle.paged_attention_loops(q, kc, vc, tables, ctx, scale, dense_bias=dense)
    np.testing.assert_allclose(got, want, rtol=3e-5, atol=3e-6)


def test_head_compression_int8_takes_the_descale_slice_of_its_kv_head(oracle):
    rng = _rng(32)
    heads, n, d, block, pool = 8, 2, 16, 4, 9
    ctx = np.array([7, 16], dtype=np.int32)
    tables = rng.permutation(pool)[:8].reshape(2, 4).astype(np.int32)
    q = rng.standard_normal((2, heads, d)).astype(np.float32)
    kc = rng.integers(-5, 6, size=(pool, block, n, d)).astype(np.int8)
    vc = rng.integers(-5, 6, size=(pool, block, n, d)).astype(np.int8)
    ks, vs = (rng.uniform(0.1, 1.0, size=n * d).astype(np.float32) for _ in range(2))
    ko, vo = (rng.integers(-3, 4, size=n * d).astype(np.int32) for _ in range(2))
    kc_c, vc_c, tables_c, ctx_c = _compressed_twin(kc, vc, tables, ctx, n)
    got = oracle.paged_attention(q, kc_c, vc_c, tables_c, ctx_c, 0.25, ks, ko, vs, vo, compress_kv_heads=n)
    want = oracle.paged_attention(q, kc, vc, tables, ctx, 0.25, ks, ko, vs, vo)  # pinned by its own tests
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)


def test_attention_matches_torch_sdpa(oracle):
    """Gathering the rows densely reduces the op to textbook attention."""
    rng = _rng(3)
    q, kc, vc, tables, ctx = _paged_case(rng, batch=4, heads=6, kv_heads=3, d=32, dv=24, block=8, pool=40, max_ctx=50)
    scale = 0.37
    got = oracle.paged_attention(q, kc, vc, tables, ctx, scale)
    group = q.shape[1] // kc.shape[2]
    for b in range(len(ctx)):
        j = np.arange(ctx[b])
        k = kc[tables[b][j // 8], j % 8]  # [ctx, G, D]
        v = vc[tables[b][j // 8], j % 8]
        kt = torch.from_numpy(np.repeat(k, group, axis=1)).double().permute(1, 0, 2)  # [H, ctx, D]
        vt = torch.from_numpy(np.repeat(v, group, axis=1)).double().permute(1, 0, 2)
        qt = torch.from_numpy(q[b]).double().unsqueeze(1)  # [H, 1, D]
        ref = torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, scale=scale).squeeze(1).numpy()
        np.testing.assert_allclose(got[b], ref, rtol=2e-5, atol=2e-6)


def test_attention_block_permutation_invariance(oracle):
    rng = _rng(4)
    q, kc, vc, tables, ctx = _paged_case(rng)
    base = oracle.paged_attention(q, kc, vc, tables, ctx, 0.25)
    perm = rng.permutation(kc.shape[0])
    inv = np.empty_like(perm)
    inv[perm] = np.arange(len(perm))
    moved = oracle.paged_attention(q, kc[perm], vc[perm], inv[tables].astype(np.int32), ctx, 0.25)
    assert np.array_equal(base, moved)


def test_attention_ctx1_returns_value_row(oracle):
    rng = _rng(5)
    q, kc, vc, tables, _ = _paged_case(rng)
    ctx = np.ones(len(tables), dtype=np.int32)
    out = oracle.paged_attention(q, kc, vc, tables, ctx, 0.3)
    group = q.shape[1] // kc.shape[2]
    for b in range(len(ctx)):
        assert np.array_equal(out[b], np.repeat(vc[tables[b, 0], 0], group, axis=0))


def test_attention_equal_keys_gives_mean_of_values(oracle):
    rng = _rng(6)
    q, kc, vc, tables, ctx = _paged_case(rng)
    kc[:] = kc[0, 0]
    out = oracle.paged_attention(q, kc, vc, tables, ctx, 0.3)
    group = q.shape[1] // kc.shape[2]
    for b in range(len(ctx)):
        j = np.arange(ctx[b])
        mean = vc[tables[b][j // 4], j % 4].mean(axis=0)
        np.testing.assert_allclose(out[b], np.repeat(mean, group, axis=0), rtol=1e-5, atol=1e-6)


def test_attention_gqa_equals_replicated_mha(oracle):
    rng = _rng(7)
    q, kc, vc, tables, ctx = _paged_case(rng, heads=6, kv_heads=2)
    gqa = oracle.paged_attention(q, kc, vc, tables, ctx, 0.2)
    mha = oracle.paged_attention(q, np.repeat(kc, 3, axis=2), np.repeat(vc, 3, axis=2), tables, ctx, 0.2)
    np.testing.assert_allclose(gqa, mha, rtol=1e-5, atol=1e-6)


def test_attention_scale_is_applied_to_scores(oracle):
    rng = _rng(8)
    q, kc, vc, tables, ctx = _paged_case(rng)
    a = oracle.paged_attention(q, kc, vc, tables, ctx, 0.5)
    b = oracle.paged_attention(q * 0.5, kc, vc, tables, ctx, 1.0)
    np.testing.assert_allclose(a, b, rtol=1e-5, atol=1e-6)
    assert np.abs(a - oracle.paged_attention(q, kc, vc, tables, ctx, 1.0)).max() > 1e-3


def test_attention_ignores_rows_past_context_and_unused_blocks(oracle):
    rng = _rng(9)
    q, kc, vc, tables, ctx = _paged_case(rng)
    base = oracle.paged_attention(q, kc, vc, tables, ctx, 0.25)
    kc2, vc2 = kc.copy(), vc.copy()
    used = np.zeros(kc.shape[:2], dtype=bool)
    for b in range(len(ctx)):
        j = np.arange(ctx[b])
        used[tables[b][j // 4], j % 4] = True
    kc2[~used] = np.nan
    vc2[~used] = np.nan
    out = oracle.paged_attention(q, kc2, vc2, tables, ctx, 0.25)
    assert np.array_equal(base, out) and (~used).any()


def test_attention_empty_sequences_take_no_query_row(oracle):
    rng = _rng(10)
    q, kc, vc, tables, ctx = _paged_case(rng, batch=4)
    dense = oracle.paged_attention(q, kc, vc, tables, ctx, 0.25)
    ctx2 = ctx.copy()
    ctx2[1] = 0
    out = oracle.paged_attention(q, kc, vc, tables, ctx2, 0.25, out_init=0.1)
    # sequences 0,2,3 use query rows 0,1,2; row 3 is never written
    assert np.array_equal(out[0], dense[0])
    want1 = oracle.paged_attention(q[1:2], kc, vc, tables[2:3], ctx[2:3], 0.25)[0]
    assert np.array_equal(out[1], want1)
    assert np.all(out[3] == np.float32(0.1))


def test_attention_empty_sequences_keep_their_rows_on_request(oracle):
    """empty_keep_rows (MultiLatentAttention; reference tiling/mla_tiling.cpp:146-149): the query rows of a sequence
    without context are left alone and every other sequence stays at the running sum of ALL query lengths; the mask
    of a query row is the one at its own index. Each sequence is checked against itself run alone."""
    rng = _rng(11)
    _, kc, vc, tables, ctx = _paged_case(rng, batch=4, heads=4, kv_heads=1, max_ctx=40)
    ctx = np.array([max(int(ctx[0]), 3), 0, max(int(ctx[2]), 2), 0], np.int32)
    q_lens = np.array([2, 3, 1, 2], np.int32)
    q = rng.standard_normal((8, 4, kc.shape[3])).astype(np.float32)
    mask = (rng.standard_normal((8, 40)) * 2).astype(np.float32)
    lse = np.full((8, 4), 7.0, np.float32)
    out = oracle.paged_attention(q, kc, vc, tables, ctx, 0.25, q_lens=q_lens, mask=mask, mask_rows="query",
                                 out_init=0.1, lse_out=lse, empty_keep_rows=True)
    starts = np.concatenate([[0], np.cumsum(q_lens)])
    for b in range(4):
        rows = slice(int(starts[b]), int(starts[b + 1]))
        if ctx[b] == 0:
            assert np.all(out[rows] == np.float32(0.1)) and np.all(lse[rows] == 7.0)
            continue
        alone_lse = np.zeros((q_lens[b], 4), np.float32)
        alone = oracle.paged_attention(q[rows], kc, vc, tables[b:b + 1], ctx[b:b + 1], 0.25, q_lens=q_lens[b:b + 1],
                                       mask=mask[rows], mask_rows="query", lse_out=alone_lse)
        assert np.array_equal(out[rows], alone) and np.array_equal(lse[rows], alone_lse)
    # without the option the same call packs the rows (PagedAttention's rule)
    packed = oracle.paged_attention(q, kc, vc, tables, ctx, 0.25, q_lens=q_lens, out_init=0.1)
    assert np.array_equal(packed[2], oracle.paged_attention(q[2:3], kc, vc, tables[2:3], ctx[2:3], 0.25)[0])
    assert np.all(packed[3:] == np.float32(0.1))


# ---------------------------------------------------------------- masks and logN
def _with_empty(ctx, at):
    ctx = ctx.copy()
    ctx[at] = 0
    return ctx


def test_masked_attention_matches_independent_loops(oracle):
    """Every mask layout against the float64 loops on a densely expanded bias, with an
    empty sequence in the middle: the mask and logN rows go by the index into
    context_lens, the query rows by the count of non-empty sequences before."""
    rng = _rng(30)
    q, kc, vc, tables, ctx = _paged_case(rng, batch=5, heads=4, kv_heads=2, max_ctx=11)
    ctx = _with_empty(ctx, 2)
    batch, heads, max_len = 5, 4, 13
    logn = rng.uniform(1, 2, size=batch).astype(np.float32)
    layouts = {
        "norm2": (rng.standard_normal((1, max_len)), None, lambda m, i, h: m[0]),
        "norm3": (rng.standard_normal((batch, 1, max_len)), False, lambda m, i, h: m[i, 0]),
        "alibi3": (rng.standard_normal((heads, 1, max_len)), True, lambda m, i, h: m[h, 0]),
        "alibi4": (rng.standard_normal((batch, heads, 1, max_len)), None, lambda m, i, h: m[i, h, 0]),
        "alibi4_1": (rng.standard_normal((batch, 1, 1, max_len)), None, lambda m, i, h: m[i, 0, 0]),
    }
    for name, (mask, per_head, row) in layouts.items():
        mask = mask.astype(np.float32)
        dense = np.stack([np.stack([row(mask, i, h) for h in range(heads)]) for i in range(batch)])
        got = oracle.paged_attention(q, kc, vc, tables, ctx, 0.3, mask=mask, mask_per_head=per_head, logn=logn)
        want = oracle.paged_attention_loops(q, kc, vc, tables, ctx, 0.3, dense_bias=dense, logn=logn)
        np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-6, err_msg=name)


def test_mask_matches_torch_sdpa_attn_mask(oracle):
    rng = _rng(31)
    q, kc, vc, tables, ctx = _paged_case(rng, batch=3, heads=6, kv_heads=6, d=32, dv=32, block=8, pool=30, max_ctx=40)
    mask = rng.standard_normal((3, 6, 1, 40)).astype(np.float32)
    out = oracle.paged_attention(q, kc, vc, tables, ctx, 0.21, mask=mask)
    for i in range(3):
        keys = oracle.gather_rows(kc, tables[i], ctx[i])
        vals = oracle.gather_rows(vc, tables[i], ctx[i])
        want = torch.nn.functional.scaled_dot_product_attention(
            torch.from_numpy(q[i])[:, None, :].double(), torch.from_numpy(keys).permute(1, 0, 2).double(),
            torch.from_numpy(vals).permute(1, 0, 2).double(),
            attn_mask=torch.from_numpy(mask[i, :, :, :ctx[i]]).double(), scale=0.21)
        np.testing.assert_allclose(out[i], want[:, 0, :].numpy(), rtol=2e-5, atol=2e-6)


def test_mask_two_token_closed_form(oracle):
    """q = 0: the weights are softmax(bias) alone, sigma(b0 - b1) for two tokens."""
    kc = np.zeros((1, 4, 1, 4), np.float32)
    vc = np.zeros((1, 4, 1, 2), np.float32)
    vc[0, 0, 0] = [1.0, 10.0]
    vc[0, 1, 0] = [3.0, -10.0]
    q = np.zeros((1, 1, 4), np.float32)
    mask = np.array([[[0.5, -1.5, 99.0, 99.0]]], np.float32)
    out = oracle.paged_attention(q, kc, vc, np.zeros((1, 1), np.int32), np.array([2], np.int32), 1.0, mask=mask,
                                 mask_per_head=False)
    w = 1.0 / (1.0 + math.exp(-2.0))
    np.testing.assert_allclose(out[0, 0], [w * 1 + (1 - w) * 3, w * 10 - (1 - w) * 10], rtol=1e-6)


def test_mask_hiding_positions_equals_attention_over_the_rest(oracle):
    """-inf, and the reference tests' -10000, on the first k positions leave exactly
    the attention over the remaining tokens."""
    rng = _rng(32)
    q, kc, vc, tables, ctx = _paged_case(rng, batch=4, heads=4, kv_heads=2, block=4, max_ctx=14)
    ctx = np.maximum(ctx, 5)
    tables = np.tile(np.arange(4, dtype=np.int32), (4, 1)) + 4 * np.arange(4, dtype=np.int32)[:, None]
    for value, tol in ((-np.inf, 1e-6), (-10000.0, 1e-6)):
        mask = oracle.norm_mask(4, 16, value)
        out = oracle.paged_attention(q, kc, vc, tables, ctx, 0.4, mask=mask, mask_per_head=False)
        for i in range(4):
            keys = oracle.gather_rows(kc, tables[i], ctx[i])[i:]
            vals = oracle.gather_rows(vc, tables[i], ctx[i])[i:]
            np.testing.assert_allclose(out[i], oracle.attention_one(q[i], keys, vals, 0.4), rtol=tol, atol=tol)


def test_mask_constant_along_a_row_changes_nothing(oracle):
    rng = _rng(33)
    q, kc, vc, tables, ctx = _paged_case(rng, batch=3, heads=4, kv_heads=2)
    base = oracle.paged_attention(q, kc, vc, tables, ctx, 0.25)
    mask = np.broadcast_to(rng.standard_normal((3, 4, 1, 1)).astype(np.float32), (3, 4, 1, 14)).copy()
    np.testing.assert_allclose(oracle.paged_attention(q, kc, vc, tables, ctx, 0.25, mask=mask), base,
                               rtol=1e-5, atol=1e-6)
    zero = np.zeros((4, 1, 14), np.float32)
    assert np.array_equal(oracle.paged_attention(q, kc, vc, tables, ctx, 0.25, mask=zero, mask_per_head=True), base)


def test_alibi_slopes_and_mask_closed_form(oracle):
    # the published ALiBi slopes: 8 heads -> 1/2 .. 1/256; 12 heads add 2^-0.5, 2^-1.5, 2^-2.5, 2^-3.5
    np.testing.assert_allclose(oracle.alibi_slopes(8), [2.0 ** -k for k in range(1, 9)], rtol=1e-7)
    np.testing.assert_allclose(oracle.alibi_slopes(12)[8:], [2.0 ** -0.5, 2.0 ** -1.5, 2.0 ** -2.5, 2.0 ** -3.5],
                               rtol=1e-7)
    assert len(oracle.alibi_slopes(40)) == 40
    m = oracle.alibi_mask([3, 0, 5], 8, 6)
    assert m.shape == (3, 8, 1, 6)
    assert np.array_equal(m[0, 0, 0], [-1.0, -0.5, 0.0, 0.0, 0.0, 0.0])   # slope 1/2, distances 2, 1, 0
    assert np.array_equal(m[2, 1, 0], [-1.0, -0.75, -0.5, -0.25, 0.0, 0.0])  # slope 1/4
    assert not m[1].any()
    n = oracle.norm_mask(3, 4)
    assert np.array_equal(n[:, 0], [[0, 0, 0, 0], [-10000, 0, 0, 0], [-10000, -10000, 0, 0]])


def test_logn_is_a_per_sequence_factor_on_the_scale(oracle):
    rng = _rng(34)
    q, kc, vc, tables, ctx = _paged_case(rng, batch=4)
    ctx = _with_empty(ctx, 1)
    logn = np.array([1.25, 7.0, 1.5, 2.0], np.float32)
    out = oracle.paged_attention(q, kc, vc, tables, ctx, 0.25, logn=logn)
    row = 0
    for i in range(4):
        if ctx[i] == 0:
            continue
        want = oracle.paged_attention(q[row:row + 1], kc, vc, tables[i:i + 1], ctx[i:i + 1],
                                      np.float32(0.25) * logn[i])
        assert np.array_equal(out[row], want[0])
        row += 1
    assert np.array_equal(oracle.paged_attention(q, kc, vc, tables, ctx, 0.25, logn=np.ones(4, np.float32)),
                          oracle.paged_attention(q, kc, vc, tables, ctx, 0.25))


# ---------------------------------------------------------------- several query tokens per sequence
def _expand_rows(tables, ctx, q_lens):
    """One single-token sequence per query row: (tables, ctx, owner sequence, token index)."""
    owner = [i for i, n in enumerate(q_lens) if ctx[i] > 0 for _ in range(n)]
    token = [t for i, n in enumerate(q_lens) if ctx[i] > 0 for t in range(n)]
    return tables[owner], ctx[owner], np.array(owner), np.array(token)


@pytest.mark.parametrize("mode", ["query", "position", None])
def test_multi_token_queries_match_loops_on_expanded_rows(oracle, mode):
    """Sequence i owns q_lens[i] consecutive query rows that all see its whole context; the
    float64 loops get one single-token sequence per query row and the mask rows spelled out."""
    rng = _rng(40)
    q, kc, vc, tables, ctx = _paged_case(rng, batch=5, heads=4, kv_heads=2, max_ctx=12)
    ctx = np.maximum(ctx, 4)
    ctx[3] = 0
    q_lens = np.array([2, 1, 4, 3, 3], np.int32)
    rows = int(q_lens[ctx > 0].sum())
    query = rng.standard_normal((rows + 1, 4, 16)).astype(np.float32)
    tables_x, ctx_x, owner, token = _expand_rows(tables, ctx, q_lens)
    max_len = 12
    if mode == "query":
        mask = rng.standard_normal((rows, max_len)).astype(np.float32)
        dense = np.repeat(mask[:, None, :], 4, axis=1)
    elif mode == "position":
        mask = rng.standard_normal((max_len, max_len)).astype(np.float32)
        pick = ctx[owner] - q_lens[owner] + token
        dense = np.repeat(mask[pick][:, None, :], 4, axis=1)
    else:
        mask, dense = None, None
    got = oracle.paged_attention(query, kc, vc, tables, ctx, 0.3, mask=mask, q_lens=q_lens,
                                 mask_rows=mode or "sequence", out_init=0.5)
    want = oracle.paged_attention_loops(query[:rows], kc, vc, tables_x, ctx_x, 0.3, dense_bias=dense)
    np.testing.assert_allclose(got[:rows], want, rtol=2e-5, atol=2e-6)
    assert np.all(got[rows] == np.float32(0.5))


def test_multi_token_causal_mask_equals_growing_contexts(oracle):
    """With the square causal mask the t-th of n query tokens sees the first ctx - n + t + 1 tokens."""
    rng = _rng(41)
    q, kc, vc, tables, ctx = _paged_case(rng, batch=3, heads=4, kv_heads=2, max_ctx=14)
    ctx = np.maximum(ctx, 5)
    q_lens = np.array([3, 1, 5], np.int32)
    query = rng.standard_normal((9, 4, 16)).astype(np.float32)
    causal = np.triu(np.full((14, 14), -np.inf, np.float32), 1)
    got = oracle.paged_attention(query, kc, vc, tables, ctx, 0.3, mask=causal, q_lens=q_lens, mask_rows="position")
    tables_x, ctx_x, owner, token = _expand_rows(tables, ctx, q_lens)
    seen = (ctx_x - q_lens[owner] + token + 1).astype(np.int32)
    want = oracle.paged_attention(query, kc, vc, tables_x, seen, 0.3)
    np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-6)
    # one query token per sequence is the plain decode step
    assert np.array_equal(oracle.paged_attention(q, kc, vc, tables, ctx, 0.3, q_lens=np.ones(3, np.int32)),
                          oracle.paged_attention(q, kc, vc, tables, ctx, 0.3))


def test_causal_rows_equal_the_look_ahead_mask_and_growing_contexts(oracle):
    """causal_rows: the t-th of n query rows sees ctx - n + t + 1 tokens. Pinned three ways: against every row
    run as a sequence of its own with the shortened context (what the reference's per-token jobs are), against
    the -inf look-ahead mask, and per sequence (a flag of 0 keeps the whole context)."""
    rng = _rng(43)
    q, kc, vc, tables, ctx = _paged_case(rng, batch=3, heads=4, kv_heads=2, max_ctx=14)
    ctx = np.maximum(ctx, 5)
    q_lens = np.array([3, 1, 5], np.int32)
    query = rng.standard_normal((9, 4, 16)).astype(np.float32)
    lse = np.zeros((9, 4), np.float32)
    got = oracle.paged_attention(query, kc, vc, tables, ctx, 0.3, q_lens=q_lens, causal_rows=True, lse_out=lse)
    tables_x, ctx_x, owner, token = _expand_rows(tables, ctx, q_lens)
    seen = (ctx_x - q_lens[owner] + token + 1).astype(np.int32)
    lse_x = np.zeros((9, 4), np.float32)
    want = oracle.paged_attention(query, kc, vc, tables_x, seen, 0.3, lse_out=lse_x)
    assert np.array_equal(got, want) and np.array_equal(lse, lse_x)
    look_ahead = np.zeros((9, 14), np.float32)
    for r in range(9):
        look_ahead[r, seen[r]:] = -np.inf
    masked = oracle.paged_attention(query, kc, vc, tables, ctx, 0.3, q_lens=q_lens, mask=look_ahead, mask_rows="query")
    np.testing.assert_allclose(got, masked, rtol=1e-6, atol=1e-6)
    # flags per sequence: sequence 0 keeps its whole context, the others are cut
    flags = np.array([0, 1, 1], np.int32)
    part = oracle.paged_attention(query, kc, vc, tables, ctx, 0.3, q_lens=q_lens, causal_rows=flags)
    full = oracle.paged_attention(query, kc, vc, tables, ctx, 0.3, q_lens=q_lens)
    assert np.array_equal(part[:3], full[:3]) and np.array_equal(part[3:], got[3:])
    assert not np.array_equal(got[:2], full[:2])           # (the cut changes rows that lose tokens)
    assert np.array_equal(got[2], full[2])                 # (the last row of a sequence loses none)


def test_mask_free_template_rows_are_the_look_ahead_triangle(oracle):
    """The reference's mask-free template (test_multi_latent_attention_mtp.py:342-358: -10000 where column - row >=
    2 - q, 125 + 2 q rows) read the way the kernel reads it gives query token i of q the mask "token > k - q + i",
    whatever the context length: last tile only, or reaching back into the tile before it; a template per sequence
    masks only the sequences whose template does."""
    for q in (1, 2, 3, 5):
        template = np.triu(np.full((125 + 2 * q, 128), -10000.0, np.float32), 2 - q)
        ctx = [k for k in (q, q + 1, 7, 127, 128, 129, 130, 131, 255, 256, 257, 260, 1000) if k >= q]
        got = oracle.mla_mask_free_rows(template, ctx, [q] * len(ctx), 1024)
        row = 0
        for k in ctx:
            for i in range(q):
                want = np.where(np.arange(1024) > k - q + i, -10000.0, 0.0).astype(np.float32)
                want[k:] = 0.0   # (past the context nothing is read)
                assert np.array_equal(got[row], want), (q, k, i)
                row += 1
    per_seq = np.stack([np.triu(np.full((129, 128), -10000.0, np.float32), 0), np.zeros((129, 128), np.float32)])
    got = oracle.mla_mask_free_rows(per_seq, [130, 130], [2, 2], 256)
    assert got[0, 129] == -10000.0 and got[1, 129] == 0.0 and not got[2:].any()
    got = oracle.mla_mask_free_rows(per_seq, [0, 5], [2, 1], 8)   # an empty sequence keeps its rows, all zeros
    assert got.shape == (3, 8) and not got[:2].any() and np.array_equal(got[2], per_seq[1, 4, :8] * (np.arange(8) < 5))


# ---------------------------------------------------------------- log-sum-exp output
def test_lse_closed_forms_and_logsumexp(oracle):
    from scipy.special import logsumexp
    rng = _rng(50)
    q, kc, vc, tables, ctx = _paged_case(rng, batch=4, heads=4, kv_heads=2, max_ctx=13)
    ctx[2] = 0
    mask = rng.standard_normal((4, 4, 1, 13)).astype(np.float32)
    lse = np.full((4, 4), 77.0, np.float32)
    oracle.paged_attention(q, kc, vc, tables, ctx, 0.3, mask=mask, lse_out=lse)
    row = 0
    for i in range(4):
        if ctx[i] == 0:
            continue
        keys = oracle.gather_rows(kc, tables[i], ctx[i]).astype(np.float64)
        for h in range(4):
            scores = keys[:, h // 2, :] @ q[row, h].astype(np.float64) * 0.3 + mask[i, h, 0, :ctx[i]]
            assert abs(lse[row, h] - logsumexp(scores)) < 1e-5
        row += 1
    assert np.all(lse[3] == 77.0)  # only three rows are written
    # one token: the score itself; n equal keys: the score plus log n
    one = np.zeros(2, np.float32)
    k1 = rng.standard_normal((1, 1, 8)).astype(np.float32)
    q1 = rng.standard_normal((2, 8)).astype(np.float32)
    oracle.attention_one(q1, k1, k1, 0.5, lse_out=one)
    np.testing.assert_allclose(one, (q1 @ k1[0, 0]) * 0.5, rtol=1e-6)
    oracle.attention_one(q1, np.repeat(k1, 7, axis=0), np.repeat(k1, 7, axis=0), 0.5, lse_out=one)
    np.testing.assert_allclose(one, (q1 @ k1[0, 0]) * 0.5 + math.log(7.0), rtol=1e-6)


def test_lse_of_a_split_context_is_logaddexp_of_the_parts(oracle):
    rng = _rng(51)
    qv = rng.standard_normal((4, 16)).astype(np.float32)
    keys = rng.standard_normal((40, 2, 16)).astype(np.float32)
    vals = rng.standard_normal((40, 2, 8)).astype(np.float32)
    whole, a, b = (np.zeros(4, np.float32) for _ in range(3))
    o = oracle.attention_one(qv, keys, vals, 0.3, lse_out=whole)
    oa = oracle.attention_one(qv, keys[:17], vals[:17], 0.3, lse_out=a)
    ob = oracle.attention_one(qv, keys[17:], vals[17:], 0.3, lse_out=b)
    np.testing.assert_allclose(whole, np.logaddexp(a, b), rtol=1e-6)
    wa = np.exp(a - whole)[:, None]
    np.testing.assert_allclose(o, wa * oa + (1 - wa) * ob, rtol=1e-5, atol=1e-6)


def test_int8_dequant_channel_indexing_and_identity(oracle):
    rng = _rng(11)
    q, _, _, tables, ctx = _paged_case(rng, heads=4, kv_heads=2, d=8, dv=8)
    kc8 = rng.integers(-20, 21, size=(24, 4, 2, 8)).astype(np.int8)
    vc8 = rng.integers(-20, 21, size=(24, 4, 2, 8)).astype(np.int8)
    # scale 1, offset 0 equals the float path on integer-valued caches
    ones = np.ones(16, dtype=np.float32)
    a = oracle.paged_attention(q, kc8, vc8, tables, ctx, 0.1, ones, None, ones, None)
    b = oracle.paged_attention(q, kc8.astype(np.float32), vc8.astype(np.float32), tables, ctx, 0.1)
    assert np.array_equal(a, b)
    # per-(kv head, channel) vectors: channel index is g*D + d
    ks = rng.uniform(0.5, 2.0, size=16).astype(np.float32)
    vs = rng.uniform(0.5, 2.0, size=16).astype(np.float32)
    ko = rng.integers(-5, 6, size=16).astype(np.int32)
    vo = rng.integers(-5, 6, size=16).astype(np.int32)
    got = oracle.paged_attention(q, kc8, vc8, tables, ctx, 0.1, ks, ko, vs, vo)
    kf = (kc8.astype(np.float32) + ko.reshape(2, 8)) * ks.reshape(2, 8)
    vf = (vc8.astype(np.float32) + vo.reshape(2, 8)) * vs.reshape(2, 8)
    want = oracle.paged_attention(q, kf, vf, tables, ctx, 0.1)
    np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-6)
    # a key offset shifts every score of a head equally and so cannot change the output
    nok = oracle.paged_attention(q, kc8, vc8, tables, ctx, 0.1, ks, None, vs, vo)
    np.testing.assert_allclose(got, nok, rtol=1e-4, atol=1e-5)


def test_mla_equals_generic_with_materialised_values(oracle):
    rng = _rng(12)
    q, kc, _, tables, ctx = _paged_case(rng, heads=8, kv_heads=1, d=24, dv=16)
    a = oracle.paged_attention(q, kc, None, tables, ctx, 0.2, mla_v_head_size=16)
    b = oracle.paged_attention(q, kc, np.ascontiguousarray(kc[..., :16]), tables, ctx, 0.2)
    assert np.array_equal(a, b) and a.shape == (3, 8, 16)


@pytest.mark.parametrize("n0", [16, 32])
def test_fractal_nz_layout_by_flat_addresses_and_round_trip(oracle, n0):
    """Channel c of row r of block b lands at flat element b*rows*channels + (c // n0)*rows*n0 + r*n0 + c % n0;
    the permutation written the reference's way (rows cut into 16s first, then the four axes permuted,
    test_multi_latent_attention_int8nz.py:38-44) gives the same array; nz_to_nd undoes it."""
    rng = _rng(120 + n0)
    blocks, rows, channels = 3, 32, 4 * n0
    x = rng.integers(-1000, 1000, size=(blocks, rows, channels)).astype(np.int16)
    nz = oracle.nd_to_nz(x, n0)
    assert nz.shape == (blocks, channels // n0, rows, n0) and nz.flags["C_CONTIGUOUS"]
    flat = nz.reshape(-1)
    for b in range(blocks):
        for r in range(rows):
            for c in range(channels):
                assert flat[b * rows * channels + (c // n0) * rows * n0 + r * n0 + c % n0] == x[b, r, c]
    t = torch.from_numpy(x).reshape(blocks, rows // 16, 16, channels // n0, n0).permute(0, 3, 1, 2, 4)
    assert np.array_equal(t.reshape(blocks, channels // n0, rows, n0).numpy(), nz)
    assert np.array_equal(oracle.nz_to_nd(nz), x)
    with pytest.raises(ValueError):
        oracle.nd_to_nz(x[:, :8], n0)


def _int8_case(rng, ctx, heads=4, block=16, q_lens=None):
    ctx = np.asarray(ctx, np.int32)
    nblk = (ctx + block - 1) // block
    pool = int(nblk.sum()) + 2
    perm = rng.permutation(pool)
    tables = np.zeros((len(ctx), max(1, int(nblk.max()))), np.int32)
    pos = 0
    for b in range(len(ctx)):
        tables[b, :nblk[b]] = perm[pos:pos + nblk[b]]
        pos += nblk[b]
    rows = int(sum((1 if q_lens is None else q_lens[b]) for b in range(len(ctx))))  # (empty sequences keep theirs)
    q8 = rng.integers(-5, 6, size=(rows, heads, 512)).astype(np.int8)
    qr = rng.uniform(-5, 5, size=(rows, heads, 64)).astype(np.float16).astype(np.float32)
    kv8 = rng.integers(-5, 6, size=(pool, block, 1, 512)).astype(np.int8)
    kr = rng.uniform(-5, 5, size=(pool, block, 1, 64)).astype(np.float16).astype(np.float32)
    qd = rng.uniform(1 / 127, 5 / 127, size=heads).astype(np.float32)
    pd = rng.uniform(-5 / 127, 5 / 127, size=heads).astype(np.float32)
    return q8, qr, kv8, kr, tables, ctx, qd, pd


def test_int8_weight_quantiser_closed_forms(oracle):
    """w / (max / 127) rounded to fp16, then to the nearest integer, ties to even (reference
    test_multi_latent_attention_int8nz.py:191-194)."""
    p8, wmax = oracle.quantise_weights(np.array([1.0, 0.5, 0.25, 0.0, 3 / 254], np.float32))
    assert wmax == 1.0 and p8.tolist() == [127, 64, 32, 0, 2]      # 63.5 -> 64, 31.75 -> 32, 1.5 -> 2
    p8, wmax = oracle.quantise_weights(np.array([0.02, 0.01, 0.02], np.float32))
    assert p8.tolist() == [127, 64, 127] and wmax == np.float32(0.02)
    # fp16 keeps 11 bits: 2047 / 2048 of the maximum is 126.94 -> fp16 126.9375 -> 127
    assert oracle.quantise_weights(np.array([1.0, 2047 / 2048], np.float32))[0].tolist() == [127, 127]
    assert oracle.quantise_weights(np.zeros(3, np.float32))[0].tolist() == [0, 0, 0]


@pytest.mark.parametrize("tile", [16, 48, 1000])
def test_int8_decode_matches_independent_loops(oracle, tile):
    """Token by token in Python integers and float64, every tile's weights quantised by their own maximum."""
    rng = _rng(140 + tile)
    q8, qr, kv8, kr, tables, ctx, qd, pd = _int8_case(rng, [37, 0, 5, 96], heads=3, q_lens=[2, 1, 1, 1])
    mask = (rng.standard_normal((5, 96)) * 2).astype(np.float32)
    lse = np.zeros((5, 3), np.float32)
    got = oracle.mla_int8_decode(q8, qr, kv8, kr, tables, ctx, qd, pd, 0.04, tile=tile, mask=mask, q_lens=[2, 1, 1, 1],
                                 lse_out=lse)
    row = 0
    for b, n in enumerate(ctx):
        if n == 0:
            # the sequence without context keeps its query row (reference tiling/mla_tiling.cpp:146-149): nothing is
            # written there, and the rows behind it do not move up
            assert not got[row].any() and not lse[row].any()
            row += [2, 1, 1, 1][b]
            continue
        for _ in range([2, 1, 1, 1][b]):
            for h in range(3):
                s = []
                for t in range(n):
                    blk, off = tables[b, t // 16], t % 16
                    prod = sum(int(a) * int(c) for a, c in zip(q8[row, h], kv8[blk, off, 0]))
                    rope = float(np.dot(qr[row, h].astype(np.float64), kr[blk, off, 0]))
                    s.append(np.float32((np.float32(np.float32(prod) * qd[h]) + np.float32(rope)) * np.float32(0.04)) +
                             mask[row, t])
                s = np.array(s, np.float64)
                num, den, ref = np.zeros(512), 0.0, None
                for t0 in range(0, n, tile):
                    st = s[t0:t0 + tile]
                    new = st.max() if ref is None else max(ref, st.max())
                    if ref is not None:
                        num, den = num * math.exp(ref - new), den * math.exp(ref - new)
                    ref = new
                    w = np.exp(st - ref)
                    p8 = np.rint((w.astype(np.float32) / np.float32(np.float32(w.max()) / np.float32(127))).astype(np.float16))
                    for i, t in enumerate(range(t0, min(n, t0 + tile))):
                        blk, off = tables[b, t // 16], t % 16
                        num += p8[i] * kv8[blk, off, 0].astype(np.float64) * (float(pd[h]) * float(np.float32(w.max())) / 127)
                    den += w.sum()
                np.testing.assert_allclose(got[row, h], num / den, rtol=2e-5, atol=2e-6)
                np.testing.assert_allclose(lse[row, h], math.log(den) + ref, rtol=1e-5, atol=1e-5)
            row += 1


def test_int8_decode_causal_rows_are_shortened_contexts(oracle):
    """The reference golden runs the j-th of q query rows over context + j - q + 1 tokens
    (test_multi_latent_attention_int8nz.py:356-364): causal_rows equals that row run alone as a sequence with the
    shortened context (tiles and all), and a sequence flagged 0 keeps the whole context."""
    rng = _rng(147)
    q_lens = [3, 1, 2]
    q8, qr, kv8, kr, tables, ctx, qd, pd = _int8_case(rng, [37, 5, 96], heads=3, q_lens=q_lens)
    lse = np.zeros((6, 3), np.float32)
    got = oracle.mla_int8_decode(q8, qr, kv8, kr, tables, ctx, qd, pd, 0.04, tile=16, q_lens=q_lens, causal_rows=True,
                                 lse_out=lse)
    row = 0
    for b, n in enumerate(q_lens):
        for j in range(n):
            one_lse = np.zeros((1, 3), np.float32)
            alone = oracle.mla_int8_decode(q8[row:row + 1], qr[row:row + 1], kv8, kr, tables[b:b + 1],
                                           [ctx[b] + j - n + 1], qd, pd, 0.04, tile=16, lse_out=one_lse)
            assert np.array_equal(got[row], alone[0]) and np.array_equal(lse[row], one_lse[0])
            row += 1
    full = oracle.mla_int8_decode(q8, qr, kv8, kr, tables, ctx, qd, pd, 0.04, tile=16, q_lens=q_lens)
    part = oracle.mla_int8_decode(q8, qr, kv8, kr, tables, ctx, qd, pd, 0.04, tile=16, q_lens=q_lens,
                                  causal_rows=[0, 1, 1])
    assert np.array_equal(part[:3], full[:3]) and np.array_equal(part[3:], got[3:])
    assert not np.array_equal(got[0], full[0]) and np.array_equal(got[2], full[2])


def test_int8_decode_limits_and_closed_forms(oracle):
    rng = _rng(150)
    q8, qr, kv8, kr, tables, ctx, qd, pd = _int8_case(rng, [1, 64, 33], heads=2)
    lse = np.zeros((3, 2), np.float32)
    got = oracle.mla_int8_decode(q8, qr, kv8, kr, tables, ctx, qd, pd, 0.05, tile=16, lse_out=lse)
    # one token: its weight is 127 of 127, the output is its value row times the head's descale
    np.testing.assert_allclose(got[0], kv8[tables[0, 0], 0, 0][None, :] * pd[:, None], rtol=1e-6)
    # 127 levels per tile: within about half a level of ordinary attention over the dequantised tensors, and
    # the log-sum-exp (which adds up the unquantised weights) agrees to float precision
    q = np.concatenate([q8.astype(np.float32) * qd[None, :, None], qr], -1)
    kc = np.concatenate([kv8.astype(np.float32), kr], -1)
    plain_lse = np.zeros((3, 2), np.float32)
    plain = oracle.paged_attention(q, kc, None, tables, ctx, 0.05, mla_v_head_size=512, lse_out=plain_lse)
    plain = plain * pd[None, :, None]
    assert np.abs(got - plain).max() <= 0.012 * np.abs(kv8).max() * np.abs(pd).max() * 4
    assert np.abs(got - plain).max() > 0                     # (it is not the unquantised computation)
    np.testing.assert_allclose(lse, plain_lse, rtol=1e-5, atol=1e-5)
    # equal scores: every weight is 127, the output is the mean of the value rows
    q0 = np.zeros_like(q8[:1])
    flat = oracle.mla_int8_decode(q0, np.zeros_like(qr[:1]), kv8, kr, tables[1:2], ctx[1:2], qd, pd, 0.05, tile=16)
    rows = kv8[tables[1, np.arange(64) // 16], np.arange(64) % 16, 0].astype(np.float64)
    np.testing.assert_allclose(flat[0], rows.mean(0)[None, :] * pd[:, None], rtol=1e-5, atol=1e-6)


def _int8q_case(rng, ctx, heads=4, kv_heads=2, d=64, block=16):
    ctx = np.asarray(ctx, np.int32)
    nblk = (ctx + block - 1) // block
    pool = int(nblk.sum()) + 2
    perm = rng.permutation(pool)
    tables = np.zeros((len(ctx), max(1, int(nblk.max()))), np.int32)
    pos = 0
    for b in range(len(ctx)):
        tables[b, :nblk[b]] = perm[pos:pos + nblk[b]]
        pos += nblk[b]
    rows = int((ctx > 0).sum())
    q8 = rng.integers(-5, 6, size=(rows, heads, d)).astype(np.int8)
    k8 = rng.integers(-5, 6, size=(pool, block, kv_heads, d)).astype(np.int8)
    v8 = rng.integers(-5, 6, size=(pool, block, kv_heads, d)).astype(np.int8)
    kd = rng.uniform(-5 / 127, 5 / 127, size=heads).astype(np.float32)
    vd = rng.uniform(-5 / 127, 5 / 127, size=heads).astype(np.float32)
    ps = rng.uniform(20, 127, size=heads).astype(np.float32)
    return q8, k8, v8, tables, ctx, kd, vd, ps


@pytest.mark.parametrize("tile,offline", [(16, False), (48, False), (None, False), (16, True), (1000, True)])
def test_int8q_attention_matches_independent_loops(oracle, tile, offline):
    """Token by token in Python integers and float64: descale per query head, the mask after the scale, every
    tile's weights quantised by their own maximum (online) or by the given factor (offline)."""
    rng = _rng(160 + (tile or 7) + int(offline))
    heads, kv_heads, d = 4, 2, 32
    q8, k8, v8, tables, ctx, kd, vd, ps = _int8q_case(rng, [37, 0, 5, 96], heads, kv_heads, d)
    mask = (rng.standard_normal((4, 1, 96)) * 2).astype(np.float32)       # one row per sequence, empty ones counted
    got = oracle.paged_attention_int8q(q8, k8, v8, tables, ctx, kd, vd, 0.11, p_scale=ps if offline else None, tile=tile,
                                       mask=mask, mask_per_head=False, out_init=7.0)
    assert got.shape == (3, heads, d)
    row = 0
    for b, n in enumerate(ctx):
        if n == 0:
            continue
        for h in range(heads):
            g = h // (heads // kv_heads)
            s = []
            for t in range(n):
                blk, off = tables[b, t // 16], t % 16
                prod = sum(int(a) * int(c) for a, c in zip(q8[row, h], k8[blk, off, g]))
                s.append(np.float32(np.float32(np.float32(prod) * kd[h]) * np.float32(0.11)) + mask[b, 0, t])
            s = np.array(s, np.float64)
            step = n if tile is None else tile
            num, den, ref = np.zeros(d), 0.0, None
            for t0 in range(0, n, step):
                st = s[t0:t0 + step]
                new = st.max() if ref is None else max(ref, st.max())
                if ref is not None:
                    num, den = num * math.exp(ref - new), den * math.exp(ref - new)
                ref = new
                w = np.exp(st - ref).astype(np.float32)
                if offline:
                    p8, vs = np.rint((w * ps[h]).astype(np.float16)), float(vd[h])
                else:
                    p8 = np.rint((w / np.float32(w.max() / np.float32(127))).astype(np.float16))
                    vs = float(vd[h]) * float(w.max()) / 127
                for i, t in enumerate(range(t0, min(n, t0 + step))):
                    blk, off = tables[b, t // 16], t % 16
                    num += p8[i] * v8[blk, off, g].astype(np.float64) * vs
                den += float(w.astype(np.float64).sum())
            np.testing.assert_allclose(got[row, h], num / den, rtol=3e-5, atol=3e-6)
        row += 1


@pytest.mark.parametrize("offline", [False, True])
def test_int8q_pieces_start_from_scratch_and_merge_by_log_sum_exp(oracle, offline):
    """A context cut into pieces: every piece is the attention over its own tokens (computed here as a sequence of its
    own, from the block-table entries of its tokens), and the pieces are joined as out = sum_p exp(lse_p - L) out_p
    with lse_p = log sum exp(score) over the piece, in float64. piece_tiles with piece_unit and piece_cuts name the
    same cuts; online the cut moves nothing but rounding."""
    rng = _rng(180 + int(offline))
    heads, kv_heads, d, block, tile = 4, 2, 32, 16, 16
    q8, k8, v8, tables, ctx, kd, vd, ps = _int8q_case(rng, [300, 70, 5], heads, kv_heads, d, block)
    kw = dict(p_scale=ps if offline else None, tile=tile)
    # units of 64 tokens, at most 2 a piece: the 5 units of the first sequence become 2 + 2 + 1, the others stay whole
    same = oracle.paged_attention_int8q(q8, k8, v8, tables, ctx, kd, vd, 0.09, piece_tiles=2, piece_unit=64, **kw)
    assert np.array_equal(same, oracle.paged_attention_int8q(q8, k8, v8, tables, ctx, kd, vd, 0.09,
                                                             piece_cuts={0: [128, 256]}, **kw))
    cuts = {0: [128, 256], 1: [64]}
    got = oracle.paged_attention_int8q(q8, k8, v8, tables, ctx, kd, vd, 0.09, piece_cuts=cuts, **kw)
    assert np.array_equal(got[0], same[0]) and np.array_equal(got[2], same[2])
    uncut = oracle.paged_attention_int8q(q8, k8, v8, tables, ctx, kd, vd, 0.09, **kw)
    if not offline:
        np.testing.assert_allclose(got, uncut, rtol=2e-5, atol=2e-6)
    else:
        assert np.abs(got - uncut).max() > 1e-4          # the weights of a piece are taken against its own maximum
    group = heads // kv_heads
    for b, row in ((0, 0), (1, 1)):
        bounds = [0] + cuts[b] + [int(ctx[b])]
        outs, lses = [], []
        for lo, hi in zip(bounds[:-1], bounds[1:]):
            # the piece as a sequence of its own: its blocks, its length, the same query row
            piece = oracle.paged_attention_int8q(q8[row:row + 1], k8, v8, tables[b:b + 1, lo // block:], np.array([hi - lo]),
                                                 kd, vd, 0.09, **kw)[0]
            keys = np.concatenate([k8[tables[b, t // block], t % block][None] for t in range(lo, hi)]).astype(np.int64)
            lse = []
            for h in range(heads):
                prod = keys[:, h // group, :] @ q8[row, h].astype(np.int64)
                sc = (prod.astype(np.float32) * kd[h] * np.float32(0.09)).astype(np.float64)
                lse.append(sc.max() + math.log(np.exp(sc - sc.max()).sum()))
            outs.append(piece.astype(np.float64))
            lses.append(np.array(lse))
        lses = np.array(lses)                                   # [pieces, heads]
        total = lses.max(0) + np.log(np.exp(lses - lses.max(0)).sum(0))
        want = sum(np.exp(l - total)[:, None] * o for l, o in zip(lses, outs))
        np.testing.assert_allclose(got[row], want, rtol=2e-5, atol=2e-6)


def test_int8q_attention_limits_and_closed_forms(oracle):
    rng = _rng(170)
    heads, kv_heads, d = 4, 2, 64
    q8, k8, v8, tables, ctx, kd, vd, ps = _int8q_case(rng, [1, 64, 33], heads, kv_heads, d)
    got = oracle.paged_attention_int8q(q8, k8, v8, tables, ctx, kd, vd, 0.05, tile=16)
    group = heads // kv_heads
    # one token: its weight is 127 of 127, the output is its value row times the head's descale
    one = v8[tables[0, 0], 0][np.arange(heads) // group].astype(np.float32) * vd[:, None]
    np.testing.assert_allclose(got[0], one, rtol=1e-6)
    # 127 levels per tile: within about half a level of ordinary attention over the dequantised tensors
    plain = oracle.paged_attention(q8.astype(np.float32) * kd[None, :, None], k8.astype(np.float32), v8.astype(np.float32),
                                   tables, ctx, 0.05) * vd[None, :, None]
    assert 0 < np.abs(got - plain).max() <= 0.012 * np.abs(v8).max() * np.abs(vd).max() * 4
    # equal scores (a zero query): every weight is 127 whatever the tile, the output is the mean of the value rows;
    # offline with a factor f the weights are f and the value descale is taken as given, so the mean comes f-fold
    q0 = np.zeros_like(q8)
    for kwargs, fold in (({"tile": 16}, 1), ({"tile": None}, 1), ({"tile": 16, "p_scale": np.full(heads, 100, np.float32)}, 100)):
        flat = oracle.paged_attention_int8q(q0, k8, v8, tables, ctx, kd, vd, 0.05, **kwargs)
        rows = v8[tables[1, np.arange(64) // 16], np.arange(64) % 16].astype(np.float64)       # [64, G, d]
        np.testing.assert_allclose(flat[1], fold * rows.mean(0)[np.arange(heads) // group] * vd[:, None], rtol=1e-5,
                                   atol=1e-6)
    # one KV head, head size 512, no rotary part: the computation of the int8 MLA decode
    q8m = rng.integers(-5, 6, size=(3, 2, 512)).astype(np.int8)
    kvm = rng.integers(-5, 6, size=(k8.shape[0], 16, 1, 512)).astype(np.int8)
    qd, pd = np.abs(kd[:2]) + np.float32(0.01), vd[:2]
    zero_q, zero_k = np.zeros((3, 2, 64), np.float32), np.zeros((k8.shape[0], 16, 1, 64), np.float32)
    a = oracle.paged_attention_int8q(q8m, kvm, kvm, tables, ctx, qd, pd, 0.05, tile=16)
    b = oracle.mla_int8_decode(q8m, zero_q, kvm, zero_k, tables, ctx, qd, pd, 0.05, tile=16)
    np.testing.assert_allclose(a, b, rtol=1e-6, atol=1e-7)


def _prefill_case(rng, q_lens, kv_lens, heads, kv_heads):
    tq, tk = int(sum(q_lens)), int(sum(kv_lens))
    mk = lambda *shape: rng.standard_normal(shape).astype(np.float32)
    return mk(tq, heads, 128), mk(tq, heads, 64), mk(tk, kv_heads, 128), mk(tk, kv_heads, 64), mk(tk, kv_heads, 128)


@pytest.mark.parametrize("mask", ["none", "causal", "window"])
def test_mla_prefill_matches_torch_sdpa_per_sequence(oracle, mask):
    """Every sequence and head on its own through torch's scaled_dot_product_attention over the concatenated
    128 + 64 channels: no mask, is_causal, and an explicit boolean band for the window."""
    rng = _rng(130)
    lens = [37, 1, 0, 64, 130]
    heads, window = 3, 20
    qn, qr, kn, kr, v = _prefill_case(rng, lens, lens, heads, heads)
    got = oracle.mla_prefill(qn, qr, kn, kr, v, lens, lens, 0.11, mask=mask, window=window)
    assert got.shape == (sum(lens), heads, 128)
    pos = 0
    for n in lens:
        if n == 0:
            continue
        q = torch.from_numpy(np.concatenate([qn[pos:pos + n], qr[pos:pos + n]], -1)).permute(1, 0, 2).double()
        k = torch.from_numpy(np.concatenate([kn[pos:pos + n], kr[pos:pos + n]], -1)).permute(1, 0, 2).double()
        vv = torch.from_numpy(v[pos:pos + n]).permute(1, 0, 2).double()
        if mask == "none":
            want = torch.nn.functional.scaled_dot_product_attention(q, k, vv, scale=0.11)
        elif mask == "causal":
            want = torch.nn.functional.scaled_dot_product_attention(q, k, vv, is_causal=True, scale=0.11)
        else:
            i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
            want = torch.nn.functional.scaled_dot_product_attention(q, k, vv, attn_mask=(j <= i) & (j > i - window),
                                                                    scale=0.11)
        np.testing.assert_allclose(got[pos:pos + n], want.permute(1, 0, 2).numpy(), rtol=2e-5, atol=2e-5)
        pos += n


def test_mla_prefill_closed_forms_grouping_and_padded_keys(oracle):
    rng = _rng(131)
    lens = [5, 9]
    qn, qr, kn, kr, v = _prefill_case(rng, lens, lens, 4, 2)
    # a window of one key: every query sees only its own position
    one = oracle.mla_prefill(qn, qr, kn, kr, v, lens, lens, 0.3, mask="window", window=1)
    for h in range(4):
        np.testing.assert_allclose(one[:, h], v[:, h // 2], rtol=1e-6, atol=1e-6)
    # causal: the first query of a sequence sees one key; the last one sees them all, like an unmasked query
    causal = oracle.mla_prefill(qn, qr, kn, kr, v, lens, lens, 0.3, mask="causal")
    plain = oracle.mla_prefill(qn, qr, kn, kr, v, lens, lens, 0.3)
    np.testing.assert_allclose(causal[0, 3], v[0, 1], rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(causal[5, 0], v[5, 0], rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(causal[4], plain[4], rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(causal[13], plain[13], rtol=1e-6, atol=1e-6)
    # query head h reads KV head h // 2: the same as replicated KV heads
    rep = oracle.mla_prefill(qn, qr, np.repeat(kn, 2, 1), np.repeat(kr, 2, 1), np.repeat(v, 2, 1), lens, lens, 0.3,
                             mask="causal")
    assert np.array_equal(rep, causal)
    # a float64 loop over one (query, head): softmax over the visible keys of the 192 channels
    b0, i, h = 5, 6, 2
    sc = np.array([0.3 * (np.dot(qn[b0 + i, h].astype(np.float64), kn[b0 + j, 1]) +
                          np.dot(qr[b0 + i, h].astype(np.float64), kr[b0 + j, 1])) for j in range(i + 1)])
    w = np.exp(sc - sc.max())
    w /= w.sum()
    np.testing.assert_allclose(causal[b0 + i, h], (w[:, None] * v[b0:b0 + i + 1, 1]).sum(0), rtol=1e-5, atol=1e-5)
    # keys padded per sequence to 12 rows, garbage in the padding
    pad = lambda t: np.concatenate([np.concatenate([t[:5], np.full((7,) + t.shape[1:], np.nan, np.float32)]),
                                    np.concatenate([t[5:], np.full((3,) + t.shape[1:], np.nan, np.float32)])])
    padded = oracle.mla_prefill(qn, qr, pad(kn), pad(kr), pad(v), lens, lens, 0.3, mask="causal", kv_padded_rows=12)
    assert np.array_equal(padded, causal)
    # more keys than queries without a mask: every query sees them all
    qn2, qr2, kn2, kr2, v2 = _prefill_case(rng, [2], [7], 1, 1)
    cross = oracle.mla_prefill(qn2, qr2, kn2, kr2, v2, [2], [7], 1.0)
    sc = np.concatenate([qn2[1, 0], qr2[1, 0]]) @ np.concatenate([kn2[:, 0], kr2[:, 0]], -1).T
    w = np.exp(sc - sc.max())
    np.testing.assert_allclose(cross[1, 0], (w / w.sum()) @ v2[:, 0], rtol=1e-5, atol=1e-5)


def test_q_scale_rounds_in_query_dtype(oracle):
    rng = _rng(13)
    q, kc, vc, tables, ctx = _paged_case(rng)
    q = q.astype(np.float16).astype(np.float32)
    a = oracle.paged_attention(q, kc, vc, tables, ctx, 0.25, q_scale=0.3, q_dtype="float16")
    b = oracle.paged_attention((q * np.float32(0.3)).astype(np.float16).astype(np.float32), kc, vc, tables, ctx, 0.25)
    assert np.array_equal(a, b)
    for noop in (0.0, 1.0):
        assert np.array_equal(oracle.paged_attention(q, kc, vc, tables, ctx, 0.25, q_scale=noop),
                              oracle.paged_attention(q, kc, vc, tables, ctx, 0.25))


def test_split_kv_merge_equals_single_pass(oracle):
    rng = _rng(14)
    ctx = 53
    q = rng.standard_normal((6, 16)).astype(np.float32)
    keys = rng.standard_normal((ctx, 2, 16)).astype(np.float32) * 3
    values = rng.standard_normal((ctx, 2, 8)).astype(np.float32)
    full = oracle.attention_one(q, keys, values, 0.3)
    for cuts in ([0, 53], [0, 1, 53], [0, 20, 21, 40, 53], list(range(0, 54))):
        outs, lses = [], []
        for a, b in zip(cuts[:-1], cuts[1:]):
            o, l = oracle.partial_attention(q, keys[a:b], values[a:b], 0.3)
            outs.append(o)
            lses.append(l)
        # an empty split contributes nothing
        outs.append(np.full_like(outs[0], 7.0))
        lses.append(np.full_like(lses[0], -np.inf))
        np.testing.assert_allclose(oracle.merge_partials(outs, lses), full, rtol=2e-6, atol=2e-6)


def test_bf16_round(oracle):
    x = np.array([1.0, 1.00390625, 1.0 + 2 ** -8, 1.0 + 3 * 2 ** -8, -2.5, 3.0e38, 1e-40], dtype=np.float32)
    want = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    assert np.array_equal(oracle.bf16_round(x), want)
    big = _rng(15).standard_normal(10000).astype(np.float32) * 100
    assert np.array_equal(oracle.bf16_round(big), torch.from_numpy(big).to(torch.bfloat16).float().numpy())
