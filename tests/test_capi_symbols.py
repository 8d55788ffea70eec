"""The C-ABI library loads and exports every symbol include/strix_mi355.h declares.
No compute: without a GPU the only call made is smx_create, which must fail loudly."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "strix_mi355.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(smx_[a-z0-9_]+)\s*\(", text)))


def test_header_cites_the_reference_interface():
    text = open(HEADER).read()
    for cite in ("accel.rs:150", "accel.rs:391", "accel.rs:397", "accel.rs:213", "accel.rs:217",
                 "accel.rs:201-210", "accel.rs:311-321", "decode.rs:2491-2521", "decode.rs:3827-3898"):
        assert cite in text, cite


def test_library_exports_every_declared_symbol(pkg):
    lib = ctypes.CDLL(pkg.LIB_PATH)
    syms = declared_symbols()
    assert len(syms) >= 30
    for s in syms:
        assert hasattr(lib, s), f"{s} declared in the header but not exported"
    assert sorted(pkg.EXPORTS) == syms


def test_create_without_gpu_fails_loudly(pkg):
    if os.path.exists("/dev/kfd"):
        pytest.skip("a GPU is present")
    with pytest.raises(pkg.SmxError) as ei:
        pkg.Mi355WeightAccel(0)
    assert "no HIP device" in str(ei.value)
    L = pkg.load_library()
    assert L.smx_create(0, None) < 0           # null out pointer is an argument error, not a crash
    assert L.smx_resident_count(None) == 0
    assert L.smx_gemv(None, b"k", None, 0, None, 0) < 0


def test_missing_library_is_an_error_not_a_fallback(pkg, monkeypatch):
    monkeypatch.setattr(pkg, "_lib", None)
    monkeypatch.setattr(pkg, "LIB_PATH", os.path.join(ROOT, "does", "not", "exist.so"))
    with pytest.raises(FileNotFoundError):
        pkg.load_library()


def test_cpp_mirror_builds_and_declines_without_gpu():
    import subprocess
    if os.path.exists("/dev/kfd"):
        pytest.skip("a GPU is present")
    exe = os.path.join(ROOT, "strix.rs_amd", "host", "selftest")
    if not os.path.exists(exe):
        pytest.skip("host/selftest not built")
    r = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=60)
    assert r.returncode == 77 and "no HIP device" in r.stdout
