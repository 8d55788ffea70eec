"""Builds libstrix_mi355.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree."""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libstrix_mi355.so")
SRC = sorted(glob.glob(os.path.join(HERE, "csrc", "*.hip")))
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # packed-fp32 instruction selection is switched off for all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def build(verbose=False, extra=()):
    cmd = [HIPCC, *FLAGS, *extra, "-o", LIB, *SRC]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the device-only target feature and says so on every file
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    build_selftest()
    return LIB


def build_selftest():
    """The C++ mirror of the accelerator trait and its driver program (host compiler only)."""
    host = os.path.join(HERE, "host")
    exe = os.path.join(host, "selftest")
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-Wextra", os.path.join(host, "selftest.cpp"), "-o", exe,
           "-L" + HERE, "-lstrix_mi355", "-Wl,-rpath," + HERE, "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib"]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("g++ failed on host/selftest.cpp:\n" + proc.stdout)
    return exe


if __name__ == "__main__":
    print(build(verbose=True, extra=sys.argv[1:]))
