"""Builds libstrix_mi355.so (HIP kernels + C ABI) and libstrix_bench.so (measurement-only kernels) for
gfx950 with hipcc, in-tree.  Translation units compile in parallel, then link."""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libstrix_mi355.so")
BENCH_LIB = os.path.join(HERE, "libstrix_bench.so")
OBJ_DIR = os.path.join(HERE, "build")
SRC = sorted(glob.glob(os.path.join(HERE, "csrc", "*.hip")))
BENCH_SRC = sorted(glob.glob(os.path.join(HERE, "bench_csrc", "*.hip")))
HDR = sorted(glob.glob(os.path.join(HERE, "csrc", "*.h"))) + [os.path.join(HERE, "..", "include", "strix_mi355.h")]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed-fp32 instruction selection is switched off for all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-inline-asm",
]


def _run(cmd, what):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the device-only target feature and says so on every file
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"{what} failed:\n" + out)
    return out


def _compile(src, extra, incremental):
    obj = os.path.join(OBJ_DIR, os.path.basename(os.path.dirname(src)) + "_" + os.path.basename(src) + ".o")
    if incremental and os.path.exists(obj):
        newest = max(os.path.getmtime(f) for f in [src, *HDR])
        if os.path.getmtime(obj) > newest:
            return obj, ""
    return obj, _run([HIPCC, *FLAGS, *extra, "-c", src, "-o", obj], "hipcc " + os.path.basename(src))


def build(verbose=False, extra=(), incremental=False):
    """Compile every translation unit (all of them on every call unless `incremental`) and link."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    jobs = min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(jobs) as pool:
        res = list(pool.map(lambda s: _compile(s, list(extra), incremental), SRC + BENCH_SRC))
    objs = [o for o, _ in res]
    if verbose:
        for _, out in res:
            if out.strip():
                print(out)
    n = len(SRC)
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs[:n]], "link " + LIB)
    if BENCH_SRC:
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", BENCH_LIB, *objs[n:]], "link " + BENCH_LIB)
    build_selftest()
    return LIB


def build_selftest():
    """The C++ mirror of the accelerator trait and its driver program (host compiler only)."""
    host = os.path.join(HERE, "host")
    exe = os.path.join(host, "selftest")
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-Wextra", os.path.join(host, "selftest.cpp"), "-o", exe,
           "-L" + HERE, "-lstrix_mi355", "-Wl,-rpath," + HERE, "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib"]
    _run(cmd, "g++ host/selftest.cpp")
    return exe


if __name__ == "__main__":
    args = sys.argv[1:]
    inc = "--incremental" in args
    print(build(verbose=True, extra=[a for a in args if a != "--incremental"], incremental=inc))
