"""The host layer under AddressSanitizer + UndefinedBehaviorSanitizer (the counterpart of the reference's
USE_ASAN build, reference CMakeLists.txt:33,59-61): build.py --sanitize compiles the operator layer and the
host code of the kernel layer (planner, argument checks, launch code) with both sanitizers, and the
host-side tests (the reference's CSV tables replayed, the Setup / Execute error paths, the C-ABI argument
checks) run against that build in a child process. No GPU is involved."""
import glob
import importlib
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
PKG = os.path.join(ROOT, "ascend-transformer-boost_amd")


def _newest(paths):
    return max(os.path.getmtime(p) for p in paths)


def test_host_api_tests_pass_under_asan_and_ubsan():
    build = importlib.import_module("ascend-transformer-boost_amd.build")
    libs = [os.path.join(build.LIB_SANITIZE, n) for n in ("libatbmi_kernels.so", "libatb.so")]
    sources = (glob.glob(os.path.join(PKG, "csrc", "*")) + glob.glob(os.path.join(PKG, "host", "*")) +
               glob.glob(os.path.join(ROOT, "include", "**", "*.h"), recursive=True) + [os.path.join(PKG, "build.py")])
    if not all(os.path.exists(p) for p in libs) or _newest(sources) > min(os.path.getmtime(p) for p in libs):
        build.build_sanitized()
    for lib in libs:  # both really carry the instrumentation
        syms = subprocess.run(["nm", "-D", lib], stdout=subprocess.PIPE, text=True).stdout
        assert "__asan_init" in syms and "__ubsan_handle" in syms, lib
    runtime = build.sanitizer_runtime()
    assert os.path.exists(runtime), runtime
    env = dict(os.environ)
    # the runtime has to come first among the loaded libraries; whatever is preloaded already stays
    env["LD_PRELOAD"] = runtime + (":" + env["LD_PRELOAD"] if env.get("LD_PRELOAD") else "")
    env["ASAN_OPTIONS"] = "detect_leaks=0"  # (the interpreter itself never frees everything)
    env["UBSAN_OPTIONS"] = "print_stacktrace=1"
    env["ATB_MI_LIB_DIR"] = build.LIB_SANITIZE
    run = subprocess.run(
        [sys.executable, "-m", "pytest", os.path.join(HERE, "test_host_api.py"), "-x", "-q", "-p", "no:cacheprovider",
         "-m", "not gpu",
         # left out: tests that link or inspect the ordinary build, and the torch binding (its import is no business of this run)
         "-k", "not torch_atb and not cpp_caller and not symbol"],
        stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env, cwd=ROOT, timeout=600)
    out = run.stdout
    assert run.returncode == 0, out[-4000:]
    assert "AddressSanitizer" not in out and "runtime error:" not in out, out[-4000:]
    passed = [line for line in out.splitlines() if " passed" in line]
    assert passed and int(passed[-1].split(" passed")[0].split()[-1]) >= 370, out[-500:]
