"""Builds the two shared libraries of the package, in-tree:

  lib/libatbmi_kernels.so  HIP kernels + C ABI (hipcc, --offload-arch=gfx950)
  lib/libatb.so            atb::Operation layer + flat C view (g++), links the first

hipcc cross-compiles gfx950 code objects without a GPU, so this runs anywhere
the ROCm toolchain is installed. Usage: python3 build.py [--jobs N] [--sanitize]

--sanitize builds both libraries a second time into lib_sanitize/ with AddressSanitizer and
UndefinedBehaviorSanitizer on all HOST code (the operator layer, and the planner / launch code of the
kernel layer; device code is compiled as usual), the counterpart of the reference's USE_ASAN build
(reference CMakeLists.txt:33,59-61). Both are compiled with ROCm's clang so that they share one
sanitizer runtime; a process that loads them must have that runtime loaded first
(LD_PRELOAD = sanitizer_runtime()). tests/test_sanitized_host_layer.py runs the host-side tests that way.
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
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-Wall", "-Wno-unused-function", "-Wno-inline-asm",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + INCLUDE, "-I" + CSRC,
]
CXX_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-I" + INCLUDE, "-I" + HOST]

LIB_SANITIZE = os.path.join(PKG, "lib_sanitize")
OBJ_SANITIZE = os.path.join(PKG, "build", "sanitize")
CLANGXX = os.environ.get("ROCM_CLANGXX", "/opt/rocm/lib/llvm/bin/clang++")
SANITIZERS = ["-fsanitize=address", "-fsanitize=undefined"]


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


def build_tools():
    """The stand-alone HBM streaming benchmark (an executable, not part of the libraries)."""
    os.makedirs(LIB, exist_ok=True)
    target = os.path.join(LIB, "bench_hbm_stream")
    _run([HIPCC, "-O3", "-std=c++17", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang",
          "-packed-fp32-ops", os.path.join(PKG, "bench_hbm_stream.hip"), "-o", target])
    return target


def build_all(jobs=8):
    return [build_kernels(jobs), build_host(), build_tools()]


def sanitizer_runtime():
    """Path of the shared AddressSanitizer runtime of ROCm's clang (it carries the UBSan runtime as well)."""
    out = subprocess.run([CLANGXX, "-print-file-name=libclang_rt.asan-x86_64.so"], stdout=subprocess.PIPE, text=True)
    path = out.stdout.strip()
    if not os.path.isabs(path):  # older layouts keep it under lib/linux of the resource directory
        res = subprocess.run([CLANGXX, "-print-resource-dir"], stdout=subprocess.PIPE, text=True).stdout.strip()
        path = os.path.join(res, "lib", "linux", "libclang_rt.asan-x86_64.so")
    return path


def build_sanitized(jobs=8):
    """Both libraries with ASan + UBSan on host code, into lib_sanitize/."""
    os.makedirs(OBJ_SANITIZE, exist_ok=True)
    os.makedirs(LIB_SANITIZE, exist_ok=True)
    host_san = []
    for flag in SANITIZERS + ["-fno-omit-frame-pointer", "-fno-sanitize-recover=undefined"]:
        host_san += ["-Xarch_host", flag]
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    objects = [os.path.join(OBJ_SANITIZE, os.path.basename(s) + ".o") for s in sources]
    # (device code keeps -O3: the sanitizers see host code only, and the assembly kernels leave the register
    # allocator no room for the spills of an unoptimised build)
    flags = HIP_FLAGS + ["-Xarch_host", "-O1", "-Xarch_host", "-g"] + host_san
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        futures = [pool.submit(_run, [HIPCC] + flags + ["-c", s, "-o", o]) for s, o in zip(sources, objects)]
        for f in futures:
            f.result()
    kernels = os.path.join(LIB_SANITIZE, "libatbmi_kernels.so")
    _run([HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-shared-libsan"] + host_san + ["-o", kernels] + objects)
    host_sources = sorted(glob.glob(os.path.join(HOST, "*.cpp")))
    target = os.path.join(LIB_SANITIZE, "libatb.so")
    _run([CLANGXX] + [f for f in CXX_FLAGS if f != "-O2"] + ["-O1", "-g", "-fno-omit-frame-pointer", "-shared-libsan",
         "-fno-sanitize-recover=undefined"] + SANITIZERS + ["-shared", "-o", target] + host_sources +
         ["-L" + LIB_SANITIZE, "-latbmi_kernels", "-Wl,-rpath,$ORIGIN"])
    return [kernels, target]


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=8)
    ap.add_argument("--sanitize", action="store_true", help="also build lib_sanitize/ (ASan + UBSan on host code)")
    args = ap.parse_args()
    for path in build_all(args.jobs):
        print("built", path)
    if args.sanitize:
        for path in build_sanitized(args.jobs):
            print("built", path)
    sys.exit(0)
