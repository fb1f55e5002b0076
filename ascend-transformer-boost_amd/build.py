"""Builds the two shared libraries of the package, in-tree:

  lib/libatbmi_kernels.so  HIP kernels + C ABI (hipcc, --offload-arch=gfx950)
  lib/libatb.so            atb::Operation layer + flat C view (g++), links the first

hipcc cross-compiles gfx950 code objects without a GPU, so this runs anywhere
the ROCm toolchain is installed. Usage: python3 build.py [--jobs N]
"""
import argparse
import concurrent.futures
import glob
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
HOST = os.path.join(PKG, "host")
LIB = os.path.join(PKG, "lib")
OBJ = os.path.join(PKG, "build")
INCLUDE = os.path.join(ROOT, "include")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
CXX = os.environ.get("CXX", "g++")

# -packed-fp32-ops off: the compiler must not form v_pk_*_f32 instructions.
HIP_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + INCLUDE, "-I" + CSRC,
]
CXX_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-I" + INCLUDE, "-I" + HOST]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature; harmless.
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_kernels(jobs):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIB, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    objects = [os.path.join(OBJ, os.path.basename(s) + ".o") for s in sources]
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        futures = [pool.submit(_run, [HIPCC] + HIP_FLAGS + ["-c", s, "-o", o]) for s, o in zip(sources, objects)]
        for f in futures:
            out = f.result()
            if out.strip():
                print(out)
    target = os.path.join(LIB, "libatbmi_kernels.so")
    _run([HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", target] + objects)
    return target


def build_host():
    os.makedirs(LIB, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(HOST, "*.cpp")))
    target = os.path.join(LIB, "libatb.so")
    out = _run([CXX] + CXX_FLAGS + ["-shared", "-o", target] + sources +
               ["-L" + LIB, "-latbmi_kernels", "-Wl,-rpath,$ORIGIN"])
    if out.strip():
        print(out)
    return target


def build_all(jobs=8):
    return [build_kernels(jobs), build_host()]


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=8)
    args = ap.parse_args()
    for path in build_all(args.jobs):
        print("built", path)
    sys.exit(0)
