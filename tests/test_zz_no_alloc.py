"""The allocation-free GEMV entry point (static device scratch) against the ordinary device entry
point, through the C ABI: where both run the same kernels the results must be identical bit for bit;
for 5..8 rows of a Q6_K weight the ordinary entry point takes the tiled GEMM (whose scratch grows with
the call) while this one keeps the GEMV, so there the two agree to the fp32 bar of every other test."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _run(accel, key, xs, N, fn):
    m, K = xs.shape
    xd, yd = accel.dev_alloc(xs.nbytes), accel.dev_alloc(m * N * 4)
    accel.h2d(xd, xs)
    accel.h2d(yd, np.full(m * N, np.nan, np.float32))
    assert fn(key, xd, m, yd) is True
    y = accel.d2h(np.empty((m, N), np.float32), yd).copy()
    accel.dev_free(xd)
    accel.dev_free(yd)
    return y


def test_noalloc_gemv_equals_gemv_dev_two_calls_in_a_row(accel, orc, synth, relerr, pkg):
    # first call: 8 rows of the longest row the static scratch takes; second call: fewer, shorter rows,
    # so the scratch still holds the first call's bytes beyond what the second one writes
    big = (8, 96, 16384, 8)       # (type, N, K, m)
    small = (2, 130, 2560, 3)
    raws = {}
    for ty, N, K, m in (big, small):
        raws[(ty, N, K)] = synth.make_weight(ty, N, K, seed=ty + N)
        up = {2: accel.upload_q4_0, 8: accel.upload_q8_0, 14: accel.upload_q6_k}[ty]
        assert up(f"t.na{ty}", raws[(ty, N, K)], K, N)
    for ty, N, K, m in (big, small):
        xs = synth.make_acts(m, K, seed=70 + m)
        got = _run(accel, f"t.na{ty}", xs, N, accel.gemv_noalloc_dev)
        want = _run(accel, f"t.na{ty}", xs, N, accel.gemv_dev)
        assert np.array_equal(got, want), (ty, N, K, m)
        assert relerr(got, orc.matmul_q8_from_f32(ty, raws[(ty, N, K)], K, N, xs)) <= 1e-5


@pytest.mark.parametrize("ty,N,K,m", [(14, 70, 3840, 7), (8, 37, 9728, 2), (2, 1000, 2592, 5), (2, 64, 256, 1)])
def test_noalloc_gemv_other_shapes(accel, orc, synth, relerr, ty, N, K, m):
    # Q6_K with more than four rows (two passes over the scratch), a row-per-wave shape, one fused row
    raw = synth.make_weight(ty, N, K, seed=3 * N + m)
    up = {2: accel.upload_q4_0, 8: accel.upload_q8_0, 14: accel.upload_q6_k}[ty]
    assert up("t.nb", raw, K, N)
    xs = synth.make_acts(m, K, seed=90 + m)
    got, want = _run(accel, "t.nb", xs, N, accel.gemv_noalloc_dev), _run(accel, "t.nb", xs, N, accel.gemv_dev)
    if ty == 14 and m > 4:   # different kernels: same integers, another fp32 summation order
        assert relerr(got, want) <= 1e-5
    else:
        assert np.array_equal(got, want)
    assert relerr(got, orc.matmul_q8_from_f32(ty, raw, K, N, xs)) <= 1e-5


def test_noalloc_gemv_limits_and_declines(accel, synth, pkg):
    raw = synth.make_weight(2, 4, 16384 + 32, seed=1)
    assert accel.upload_q4_0("t.nc", raw, 16384 + 32, 4)
    xd, yd = accel.dev_alloc(9 * (16384 + 32) * 4), accel.dev_alloc(9 * 4 * 4)
    with pytest.raises(pkg.SmxError) as ei:
        accel.gemv_noalloc_dev("t.nc", xd, 1, yd)         # rows longer than the static scratch takes
    assert ei.value.code == -3 and "static scratch" in str(ei.value)
    raw = synth.make_weight(2, 4, 64, seed=2)
    assert accel.upload_q4_0("t.nd", raw, 64, 4)
    with pytest.raises(pkg.SmxError) as ei:
        accel.gemv_noalloc_dev("t.nd", xd, 9, yd)         # more rows than it takes
    assert ei.value.code == -3
    assert accel.gemv_noalloc_dev("t.absent", xd, 1, yd) is False
    accel.dev_free(xd)
    accel.dev_free(yd)
