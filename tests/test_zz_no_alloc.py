"""The allocation-free GEMV entry point (static device scratch) against the ordinary device entry
point, through the C ABI: both run the same kernels (the dot4 GEMV up to 4 rows, the small-batch kernel
on the matrix cores for 5..8), so the results must be identical bit for bit; and under graph capture,
where any growth of the context's scratch is refused, so a call that allocated would fail."""
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
    # Q6_K with more than four rows (the small-batch kernel, its fragment-ordered quants in the array), a row-per-wave shape, one fused row
    raw = synth.make_weight(ty, N, K, seed=3 * N + m)
    up = {2: accel.upload_q4_0, 8: accel.upload_q8_0, 14: accel.upload_q6_k}[ty]
    assert up("t.nb", raw, K, N)
    xs = synth.make_acts(m, K, seed=90 + m)
    got, want = _run(accel, "t.nb", xs, N, accel.gemv_noalloc_dev), _run(accel, "t.nb", xs, N, accel.gemv_dev)
    assert np.array_equal(got, want)
    assert relerr(got, orc.matmul_q8_from_f32(ty, raw, K, N, xs)) <= 1e-5


def test_noalloc_gemv_limits_and_declines(accel, synth, pkg):
    raw = synth.make_weight(2, 4, 16384 + 32, seed=1)
    assert accel.upload_q4_0("t.nc", raw, 16384 + 32, 4)
    xd, yd = accel.dev_alloc(9 * (16384 + 32) * 4), accel.dev_alloc(9 * 4 * 4)
    with pytest.raises(pkg.SmxError) as ei:
        accel.gemv_noalloc_dev("t.nc", xd, 2, yd)         # two rows longer than the static scratch takes
    assert ei.value.code == -3 and "static scratch" in str(ei.value)
    assert accel.gemv_noalloc_dev("t.nc", xd, 1, yd) is True   # one row does not use the scratch: any length the GEMV serves
    raw = synth.make_weight(2, 4, 64, seed=2)
    assert accel.upload_q4_0("t.nd", raw, 64, 4)
    with pytest.raises(pkg.SmxError) as ei:
        accel.gemv_noalloc_dev("t.nd", xd, 9, yd)         # more rows than it takes
    assert ei.value.code == -3
    assert accel.gemv_noalloc_dev("t.absent", xd, 1, yd) is False
    accel.dev_free(xd)
    accel.dev_free(yd)


def test_noalloc_gemv_under_graph_capture_on_a_fresh_context(pkg, orc, synth, relerr):
    """The stated use: a caller under HIP graph capture.  A fresh context has no scratch at all and refuses to grow any
    while it captures, so a captured call that needed an allocation would fail.  Rows 2 (quantised inside the GEMV), 5 and
    8 (the small-batch kernel, quantiser launch + matmul launch on the static array), captured together, replayed twice
    with the activations changed in between, against smx_gemv_dev on another context."""
    N, K = 384, 2560
    raw = synth.make_weight(8, N, K, seed=5)
    ref_acc, acc = pkg.Mi355WeightAccel(0), pkg.Mi355WeightAccel(0)
    try:
        assert ref_acc.upload_q8_0("t.ng", raw, K, N) and acc.upload_q8_0("t.ng", raw, K, N)
        ms = (2, 5, 8)
        xds = {m: acc.dev_alloc(m * K * 4) for m in ms}
        yds = {m: acc.dev_alloc(m * N * 4) for m in ms}
        for m in ms:   # one eager call per kernel first: the first launch of a kernel raises its LDS limit, which is not capturable
            acc.h2d(xds[m], synth.make_acts(m, K, seed=m))
            assert acc.gemv_noalloc_dev("t.ng", xds[m], m, yds[m])
        acc.sync()
        acc.graph_begin()
        for m in ms:
            assert acc.gemv_noalloc_dev("t.ng", xds[m], m, yds[m])
        with pytest.raises(pkg.SmxError):
            acc.gemv_dev("t.ng", xds[8], 8, yds[8])      # the ordinary entry point needs scratch: refused while capturing
        g = acc.graph_end()
        for rep in range(2):
            xs = {m: synth.make_acts(m, K, seed=100 * rep + m) for m in ms}
            for m in ms:
                acc.h2d(xds[m], xs[m])
                acc.h2d(yds[m], np.full(m * N, np.nan, np.float32))
            acc.graph_launch(g)
            acc.sync()
            for m in ms:
                got = acc.d2h(np.empty((m, N), np.float32), yds[m])
                want = _run(ref_acc, "t.ng", xs[m], N, ref_acc.gemv_dev)
                assert np.array_equal(got, want), (rep, m)
                assert relerr(got, orc.matmul_q8_from_f32(8, raw, K, N, xs[m])) <= 1e-5
        acc.graph_destroy(g)
    finally:
        acc.close()
        ref_acc.close()
