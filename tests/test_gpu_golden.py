"""GPU results against the committed golden fixtures (inputs + expected integers and outputs)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
UPLOAD = {2: "upload_q4_0", 8: "upload_q8_0", 14: "upload_q6_k"}


@pytest.mark.parametrize("name", ["q4_0_small.npz", "q8_0_small.npz", "q6_k_small.npz"])
def test_golden_case(accel, golden, relerr, name):
    g = golden(name)
    ty, N, K = int(g["ty"]), int(g["N"]), int(g["K"])
    assert getattr(accel, UPLOAD[ty])("t.golden", g["raw"], K, N)
    xq, xd, xs = accel.quantize(g["x"], K)
    assert np.array_equal(xq, g["xq"]) and np.array_equal(xd, g["xd"]) and np.array_equal(xs, g["xs16"])
    per = K // 16 if ty == 14 else K // 32
    for t in range(g["x"].shape[0]):
        assert np.array_equal(accel.gemv_block_dots("t.golden", g["x"][t], N, per), g["block_dots"][t])
        assert relerr(accel.gemv("t.golden", g["x"][t], N), g["y_q8"][t]) <= 1e-5
    if ty != 14:
        m = g["x"].shape[0]
        assert relerr(accel.prefill_q8_gemm("t.golden", g["x"], m, N), g["y_q8"]) <= 1e-5
        assert np.array_equal(accel.gemm_block_dots("t.golden", g["x"], m, N, K // 32), g["block_dots"])


def test_literal_blocks_through_the_device(accel, golden):
    """The reference's literal blocks (ggml_quant.rs:443-469, 497-514): with a one-hot activation the
    GEMV returns the dequantised weight element times the quantised 1.0 (= 127 * (1/127))."""
    g = golden("literal_blocks.npz")
    for name, ty, K in (("q8_0", 8, 32), ("q4_0", 2, 32), ("q6_k", 14, 256)):
        assert getattr(accel, UPLOAD[ty])("t.lit", g[name + "_raw"], K, 1)
        for i in (0, 1, 16, 17, K - 1):
            x = np.zeros(K, np.float32)
            x[i] = 1.0
            y = accel.gemv("t.lit", x, 1)[0]
            assert abs(y - g[name + "_out"][i]) <= 1e-5 * max(1.0, abs(g[name + "_out"][i]))


def test_cpp_mirror_of_the_trait_selftest():
    """host/selftest drives strix::Mi355WeightAccel (the C++ restatement of the WeightAccel trait)."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "strix.rs_amd", "host", "selftest")
    assert os.path.exists(exe), "build it with python strix.rs_amd/build.py"
    r = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=100)
    assert r.returncode == 0, r.stdout
    assert "selftest ok" in r.stdout
