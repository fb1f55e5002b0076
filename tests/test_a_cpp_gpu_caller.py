"""The atb::Operation layer driven from C++ on the GPU: tests/cpp/atb_gpu_caller.cpp (CreateContext ->
SetExecuteStream -> CreateOperation -> Setup -> Execute -> synchronise, cache write then attention, as the
reference's own demos do) runs as a child process on inputs prepared here with numpy, and its results are
compared with the oracle: caches bit for bit, attention within rtol = atol = 1e-3 (fp16) / 2e-2 (bf16).

This file is collected before the other GPU tests on purpose: the child is started from a process
that has not touched the GPU itself (a program is never started from one that has)."""
import os
import struct
import subprocess
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB_DIR = os.path.join(ROOT, "ascend-transformer-boost_amd", "lib")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")


def _gpu_touched_in_this_process():
    torch = sys.modules.get("torch")
    if torch is not None and torch.cuda.is_initialized():
        return True
    pkg = sys.modules.get("ascend-transformer-boost_amd.binding")
    return pkg is not None and getattr(pkg, "_kernels", None) is not None


def _bf16_bits(x):
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def _from_bits(bits, dtype):
    if dtype == "float16":
        return bits.view(np.float16).astype(np.float32)
    return (bits.astype(np.uint32) << 16).view(np.float32)


@pytest.fixture(scope="module")
def caller(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("cpp") / "atb_gpu_caller")
    build = subprocess.run(
        ["g++", "-std=c++17", "-O1", "-Wall", "-Wextra", "-Werror", "-D__HIP_PLATFORM_AMD__",
         "-I" + os.path.join(ROOT, "include"), "-isystem", os.path.join(ROCM, "include"),
         os.path.join(HERE, "cpp", "atb_gpu_caller.cpp"), "-o", exe, "-L" + LIB_DIR, "-latb", "-latbmi_kernels",
         "-L" + os.path.join(ROCM, "lib"), "-lamdhip64", "-Wl,-rpath," + LIB_DIR + ":" + os.path.join(ROCM, "lib")],
        stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert build.returncode == 0, build.stdout
    return exe


# batch, heads, kvHeads, headSize, blockSize, contexts, dtype: the small benchmark configuration (fp16), a
# GQA step with rows cut by ranges (bf16), and one short sequence with fewer steps than a workgroup has waves
CASES = [
    (4, 8, 8, 128, 128, [64, 300, 512, 129], "float16"),
    (6, 32, 8, 128, 128, [1500, 33, 2048, 700, 1, 964], "bf16"),
    (1, 8, 1, 128, 128, [96], "float16"),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "b%d_h%d_g%d_%s" % (c[0], c[1], c[2], c[6]))
def test_cpp_caller_executes_a_decode_step_on_the_gpu(caller, oracle, tmp_path, case):
    if _gpu_touched_in_this_process():
        pytest.skip("a child program is only started from a process that has not initialised the GPU; "
                    "run this file first (pytest collects it first) or on its own")
    batch, heads, kv_heads, d, block, ctx, dtype = case
    rng = np.random.Generator(np.random.PCG64(77 + batch))
    ctx = np.asarray(ctx, dtype=np.int32)
    nblk = (ctx + block - 1) // block
    width = int(nblk.max())
    pool = int(nblk.sum()) + 3
    ids = rng.permutation(pool)
    tables = np.zeros((batch, width), dtype=np.int32)
    pos = 0
    for b in range(batch):
        tables[b, :nblk[b]] = ids[pos:pos + nblk[b]]
        tables[b, nblk[b]:] = ids[pos]
        pos += nblk[b]
    # the step's new token is the last one of every sequence
    slots = np.array([tables[b, (n - 1) // block] * block + (n - 1) % block for b, n in enumerate(ctx)], dtype=np.int32)

    def to_bits(x):
        return x.astype(np.float16).view(np.uint16) if dtype == "float16" else _bf16_bits(x)
    q = to_bits(rng.uniform(-1, 1, (batch, heads, d)))
    k_new = to_bits(rng.uniform(-1, 1, (batch, kv_heads, d)))
    v_new = to_bits(rng.uniform(-1, 1, (batch, kv_heads, d)))
    kc = to_bits(rng.uniform(-1, 1, (pool, block, kv_heads, d)))
    vc = to_bits(rng.uniform(-1, 1, (pool, block, kv_heads, d)))
    src, dst = str(tmp_path / "in.bin"), str(tmp_path / "out.bin")
    with open(src, "wb") as f:
        f.write(struct.pack("<9i", 0x41544231, batch, heads, kv_heads, d, block, pool, width, 1 if dtype == "float16" else 27))
        for a in (ctx, tables, slots, q, k_new, v_new, kc, vc):
            f.write(np.ascontiguousarray(a).tobytes())

    print("starting", caller, flush=True)
    run = subprocess.run([caller, src, dst], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=100)
    assert run.returncode == 0 and run.stdout.strip().startswith("ok"), run.stdout + run.stderr

    got = np.fromfile(dst, dtype=np.uint16)
    n_out, n_cache = batch * heads * d, kc.size
    assert got.size == n_out + 2 * n_cache
    got_out = got[:n_out].reshape(batch, heads, d)
    got_kc = got[n_out:n_out + n_cache].reshape(kc.shape)
    got_vc = got[n_out + n_cache:].reshape(vc.shape)

    want_kc, want_vc = oracle.reshape_and_cache(k_new.view(np.int16), v_new.view(np.int16), kc.view(np.int16),
                                                vc.view(np.int16), slots)
    assert np.array_equal(got_kc.view(np.int16), want_kc), "key cache differs"
    assert np.array_equal(got_vc.view(np.int16), want_vc), "value cache differs"
    want = oracle.paged_attention(_from_bits(q, dtype), _from_bits(want_kc.view(np.uint16), dtype),
                                  _from_bits(want_vc.view(np.uint16), dtype), tables, ctx, 1.0 / np.sqrt(d),
                                  q_dtype=dtype)
    tol = 1e-3 if dtype == "float16" else 2e-2
    err = np.abs(_from_bits(got_out, dtype) - want)
    assert (err <= tol + tol * np.abs(want)).all(), "attention differs: max err %g" % err.max()
