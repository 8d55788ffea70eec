"""GPU parity of the decode GEMV path against the Q8 oracle, through the C ABI.

Bar: per-block i32 dots bit-exact; fp32 outputs within 1e-5 (max|d|/max|ref|) of the oracle.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
TOL = 1e-5
UPLOAD = {2: "upload_q4_0", 8: "upload_q8_0", 14: "upload_q6_k"}


def _up(accel, ty, key, raw, K, N):
    assert getattr(accel, UPLOAD[ty])(key, raw, K, N) is True


@pytest.mark.parametrize("m,K", [(1, 32), (1, 2560), (3, 256), (2, 9728), (5, 96)])
def test_quantiser_bit_exact(accel, orc, synth, m, K):
    x = synth.make_acts(m, K, seed=100 + K)
    x[0, :32] = 0.0                      # an all-zero block: d = 0, q = 0
    if K >= 64:
        x[-1, 32:64] *= 1e-30            # tiny magnitudes
    xq, xd, xs = accel.quantize(x, K)
    rq, rd, rs = orc.actquant(x, K)
    assert np.array_equal(xq, rq)
    assert np.array_equal(xd.view(np.uint32), rd.view(np.uint32))
    assert np.array_equal(xs, rs)


# (type, N, K): ragged row counts, single-block rows, rows longer than one pass, odd block counts
SHAPES = [
    (2, 1, 32), (2, 7, 96), (2, 96, 256), (2, 130, 2560), (2, 64, 4128), (2, 33, 15360),
    (8, 1, 32), (8, 7, 96), (8, 96, 256), (8, 130, 2560), (8, 40, 9728),
    (14, 1, 256), (14, 9, 512), (14, 70, 3840), (14, 33, 4352),
]


@pytest.mark.parametrize("ty,N,K", SHAPES)
def test_gemv_block_dots_bit_exact(accel, orc, synth, ty, N, K):
    raw = synth.make_weight(ty, N, K, seed=7 * N + K)
    x = synth.make_acts(1, K, seed=N + 3 * K)
    _up(accel, ty, "t.bd", raw, K, N)
    per = K // 16 if ty == 14 else K // 32
    got = accel.gemv_block_dots("t.bd", x, N, per)
    xq, _, _ = orc.actquant(x, K)
    ref = orc.block_dots(ty, raw, K, N, xq[0])
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("ty,N,K", SHAPES)
def test_gemv_matches_q8_oracle(accel, orc, synth, relerr, ty, N, K):
    raw = synth.make_weight(ty, N, K, seed=11 * N + K)
    x = synth.make_acts(1, K, seed=5 * N + K)
    _up(accel, ty, "t.gemv", raw, K, N)
    y = accel.gemv("t.gemv", x, N)
    ref = orc.matmul_q8_from_f32(ty, raw, K, N, x)[0]
    assert relerr(y, ref) <= TOL
    # the f32 oracle (what strix-backend-cpu computes) differs only by activation rounding: single rows
    # of a few blocks cancel badly, everything longer stays within 2e-2
    f32 = orc.matmul_f32(ty, raw, K, N, x, order=1)[0]
    assert relerr(y, f32) <= (5e-2 if N * K <= 4096 else 2e-2)


# Small single-row GEMVs have two forms: rows dealt to waves (any shape) and the flat form (rows that are
# a whole number of 8- or 16-unit groups).  Shapes on both sides of every condition: group size 16 and 8,
# ragged row counts, fewer rows than workgroups, one and several rounds of loads, rows too long or too
# odd for the flat form.
FORM_SHAPES = [(2, 130, 2560), (2, 9, 96 * 32), (2, 2500, 2560), (2, 3, 4096 + 256), (2, 1, 512), (2, 300, 256),
               (2, 700, 8192), (2, 40, 16384), (2, 24, 16384 + 512), (2, 50, 32 * 129),
               (8, 130, 2560), (8, 37, 9728), (8, 5, 32 * 68), (8, 1000, 1024), (8, 77, 128), (8, 60, 32 * 67),
               (14, 70, 3840), (14, 9, 4352), (14, 1500, 256), (14, 33, 2048), (14, 5, 16384), (14, 3, 16640)]


@pytest.mark.parametrize("ty,N,K", FORM_SHAPES)
def test_gemv_forms_agree_with_oracle(accel, orc, synth, relerr, ty, N, K):
    raw = synth.make_weight(ty, N, K, seed=13 * N + K)
    x = synth.make_acts(1, K, seed=N + 7 * K)
    _up(accel, ty, "t.form", raw, K, N)
    y = accel.gemv("t.form", x, N)
    # the integers behind y, dumped by the same kernel form the call above ran (flat or row-per-wave)
    xq, _, _ = orc.actquant(x, K)
    per = K // 16 if ty == 14 else K // 32
    assert np.array_equal(accel.gemv_block_dots("t.form", x, N, per), orc.block_dots(ty, raw, K, N, xq[0]))
    # a group of two jobs with different row counts shares one launch geometry
    raw2 = synth.make_weight(ty, N + 5, K, seed=17 * N + K)
    _up(accel, ty, "t.form2", raw2, K, N + 5)
    pair = accel.gemv_batch([("t.form", x), ("t.form2", x)], [N, N + 5])
    ref = orc.matmul_q8_from_f32(ty, raw, K, N, x)[0]
    assert relerr(y, ref) <= TOL
    assert relerr(pair[0], ref) <= TOL
    assert relerr(pair[1], orc.matmul_q8_from_f32(ty, raw2, K, N + 5, x)[0]) <= TOL
    accel.evict("t.form")
    accel.evict("t.form2")


def test_gemv_group_of_very_different_row_counts(accel, orc, synth, relerr):
    # the launch geometry follows the largest job: most workgroups of the 2-row job have no rows at all
    K = 2560
    for ty in (2, 8, 14):
        raws = {n: synth.make_weight(ty, n, K, seed=ty * 100 + n) for n in (2, 3000)}
        for n, raw in raws.items():
            _up(accel, ty, f"t.n{n}", raw, K, n)
        x = synth.make_acts(1, K, seed=ty)[0]
        out = accel.gemv_batch([("t.n2", x), ("t.n3000", x)], [2, 3000])
        for o, n in zip(out, (2, 3000)):
            assert relerr(o, orc.matmul_q8_from_f32(ty, raws[n], K, n, x)[0]) <= TOL
            accel.evict(f"t.n{n}")


def test_gemv_group_with_more_workgroups_than_cus(accel, orc, synth, relerr):
    # eight jobs share the chip: a job's share of 30000 x 80 units per CU exceeds what a workgroup of the
    # flat form indexes, so each job runs as two rounds of workgroups
    N, K = 30000, 2560
    raw = synth.make_weight(2, N, K, seed=99)
    _up(accel, 2, "t.big", raw, K, N)
    xs = [synth.make_acts(1, K, seed=300 + i)[0] for i in range(8)]
    out = accel.gemv_batch([("t.big", x) for x in xs], [N] * 8)
    for i in (0, 3, 7):
        assert relerr(out[i], orc.matmul_q8_from_f32(2, raw, K, N, xs[i])[0]) <= TOL
    accel.evict("t.big")


@pytest.mark.parametrize("ty", [2, 8])
@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 6, 7, 8])
def test_gemv_rows_batched(accel, orc, synth, relerr, ty, m):
    N, K = 200, 2560
    raw = synth.make_weight(ty, N, K, seed=31 + m)
    xs = synth.make_acts(m, K, seed=77 + m)
    _up(accel, ty, "t.rows", raw, K, N)
    y = accel.gemv_rows("t.rows", xs, N)
    ref = orc.matmul_q8_from_f32(ty, raw, K, N, xs)
    assert y.shape == ref.shape and relerr(y, ref) <= TOL
    # row t of the batch equals the single-row call on xs[t] bit for bit (same kernel arithmetic)
    y0 = accel.gemv("t.rows", xs[m - 1], N)
    assert relerr(y[m - 1], y0) <= TOL


@pytest.mark.parametrize("m", [2, 4, 5, 8, 20, 32])
def test_gemv_rows_q6k(accel, orc, synth, relerr, m):
    # Q6_K: up to 4 rows in the dot4 GEMV, more in the tiled GEMM (whose sparse tiles share their row tiles
    # out over the waves); the lm_head argmax entry point takes the same route
    N, K = 300, 2560
    raw = synth.make_weight(14, N, K, seed=40 + m)
    xs = synth.make_acts(m, K, seed=50 + m)
    _up(accel, 14, "t.q6rows", raw, K, N)
    y = accel.gemv_rows("t.q6rows", xs, N)
    ref = orc.matmul_q8_from_f32(14, raw, K, N, xs)
    assert y.shape == ref.shape and relerr(y, ref) <= TOL
    assert [int(v) for v in accel.lm_head_argmax_rows("t.q6rows", xs, m)] == [int(np.argmax(r)) for r in y]
    accel.evict("t.q6rows")


@pytest.mark.parametrize("ty,N,K", [(2, 130, 256), (8, 96, 4096), (14, 200, 4096), (2, 64, 4128), (8, 300, 8192), (14, 40, 8192), (2, 9728, 2560),
                                    (8, 2560, 9728), (2, 77, 16384), (14, 33, 10240), (8, 50, 8224), (2, 40, 16416), (8, 90, 12288),
                                    (2, 70, 12320), (14, 35, 12288), (8, 64, 10240)])
def test_gemv_rows_quantised_in_kernel(accel, orc, synth, relerr, ty, N, K):
    # 2..4 fp32 rows of at most 49152 values in all (counting 4 rows for 3) are quantised by the GEMV kernel itself, one to
    # three half blocks per thread; longer ones by a quantiser launch of their own: both sides of the bound (12288 / 12320
    # elements per row at 4 rows, 16384 / 16416 at 2), one, two and three items per thread (4096, 8192, 9728..12288 elements
    # at 4 rows), a row of eight blocks, three rows in the four-row variant (its fourth row is staged as zeros)
    raw = synth.make_weight(ty, N, K, seed=N + K)
    _up(accel, ty, "t.rq", raw, K, N)
    for m in (2, 3, 4):
        xs = synth.make_acts(m, K, seed=m + K)
        xs[m - 1, 32:64] = 0.0                # an all-zero block: d = 0
        y = accel.gemv_rows("t.rq", xs, N)
        ref = orc.matmul_q8_from_f32(ty, raw, K, N, xs)
        assert y.shape == ref.shape and relerr(y, ref) <= TOL, m
        for t in range(m):                    # the single-row kernel quantises with the same arithmetic
            assert relerr(y[t], accel.gemv("t.rq", xs[t], N)) <= TOL, (m, t)
    accel.evict("t.rq")


def test_gemv_rows_long_k_batched(accel, orc, synth, relerr):
    # the batched verify shape: Q8_0 2560 x 9728, M = 8 (large LDS staging, 16-wave groups)
    N, K, m = 2560, 9728, 8
    raw = synth.make_weight(8, N, K, seed=5)
    xs = synth.make_acts(m, K, seed=6)
    _up(accel, 8, "t.long", raw, K, N)
    y = accel.gemv_rows("t.long", xs, N)
    ref = orc.matmul_q8_from_f32(8, raw, K, N, xs)
    assert relerr(y, ref) <= TOL
    accel.evict("t.long")


def test_gemv_batch_and_declines(accel, orc, synth, relerr, pkg):
    K, N = 256, 64
    raws = [synth.make_weight(ty, N, K, seed=ty) for ty in (2, 8, 14)]
    for ty, raw in zip((2, 8, 14), raws):
        _up(accel, ty, f"t.b{ty}", raw, K, N)
    xs = [synth.make_acts(1, K, seed=40 + i)[0] for i in range(4)]
    calls = [("t.b2", xs[0]), ("t.nope", xs[1]), ("t.b8", xs[2]), ("t.b14", xs[3])]
    out = accel.gemv_batch(calls, [N] * 4)
    assert out[1] is None                                   # not resident -> None (accel.rs:396)
    for i, ty in ((0, 2), (2, 8), (3, 14)):
        ref = orc.matmul_q8_from_f32(ty, raws[(2, 8, 14).index(ty)], K, N, xs[i])[0]
        assert relerr(out[i], ref) <= TOL
    assert accel.gemv("t.nope", xs[0], N) is None
    with pytest.raises(pkg.SmxError):                        # wrong activation length is an error, not a CPU fallback
        accel.gemv("t.b2", xs[0][:128], N)


def test_upload_rejects_bad_shapes(accel, synth, pkg):
    raw = synth.make_weight(2, 4, 64, seed=1)
    with pytest.raises(pkg.SmxError):
        accel.upload_q4_0("bad", raw, 48, 4)                # in_dim not a multiple of 32 (decode.rs:2492)
    with pytest.raises(pkg.SmxError):
        accel.upload_q4_0("bad", raw[:-1], 64, 4)           # byte length mismatch (decode.rs:2497)
    with pytest.raises(pkg.SmxError):
        accel.upload_q6_k("bad", raw, 64, 4)                # Q6_K needs multiples of 256 (decode.rs:2630)
    assert accel.gemv("bad", np.zeros(64, np.float32), 4) is None
    n0 = accel.resident_count()
    assert accel.upload_q4_0("tmp.count", raw, 64, 4) and accel.resident_count() == n0 + 1
    assert accel.evict("tmp.count") and accel.resident_count() == n0
    assert "gfx950" in accel.name()


def test_lm_head_argmax_rows(accel, orc, synth):
    N, K, m = 3000, 256, 5
    for ty in (8, 2, 14):
        raw = synth.make_weight(ty, N, K, seed=90 + ty)
        xs = synth.make_acts(m, K, seed=91 + ty)
        _up(accel, ty, "t.head", raw, K, N)
        got = accel.lm_head_argmax_rows("t.head", xs, m)
        ref = orc.matmul_q8_from_f32(ty, raw, K, N, xs)
        # compare through values: a near-tie may legitimately resolve differently under fp32 reassociation
        for t in range(m):
            assert ref[t, got[t]] >= ref[t].max() - 1e-5 * np.abs(ref[t]).max()


def test_lm_head_argmax_ties_take_the_lowest_index(accel, synth):
    """Identical weight rows give bit-identical logits: the strict '>' scan of the reference (decode.rs:3677-3683)
    keeps the first of them.  The winning row is copied to places in other chunks of the two-stage argmax."""
    N, K, m = 9000, 256, 3
    raw = synth.make_weight(8, N, K, seed=5).reshape(N, -1).copy()
    xs = synth.make_acts(m, K, seed=6)
    assert accel.upload_q8_0("t.tie", raw.reshape(-1), K, N)
    y = accel.gemv_rows("t.tie", xs, N)
    top = [int(np.argmax(r)) for r in y]
    dup = raw.copy()
    for t in top:                       # every row's winner also sits later in its own chunk and in later chunks
        for pos in (t + 1, 2048 + 7, 4096 + 300, N - 1):
            if pos != t and pos < N and pos not in top:
                dup[pos] = raw[t]
    assert accel.upload_q8_0("t.tie", dup.reshape(-1), K, N)
    y2 = accel.gemv_rows("t.tie", xs, N)
    got = [int(v) for v in accel.lm_head_argmax_rows("t.tie", xs, m)]
    assert got == [int(np.argmax(r)) for r in y2]     # numpy's argmax also returns the first maximum
    for t, g in zip(range(m), got):
        assert (y2[t] == y2[t, g]).sum() >= 2 or g == top[t]
    accel.evict("t.tie")


def _reference_device_test_data(orc, in_dim=15360, out_dim=3840):
    """The data of the reference's own device test (strix-backend-rocm/src/lib.rs:135-153): LCG
    0xA5A5_1234, per block one draw for the scale 0.03 + (r % 32) * 0.003 (made f16 by truncating the
    mantissa, lib.rs:110-119) and four draws for the nibble words; x = 0.5 sin(0.017 i)."""
    nblk = in_dim // 32
    total = nblk * out_dim
    draws, _ = orc.lcg(0xA5A51234, total * 5)
    draws = draws.reshape(total, 5)
    sc = (np.float32(0.03) + (draws[:, 0] % 32).astype(np.float32) * np.float32(0.003)).astype(np.float32)
    bits = sc.view(np.uint32)
    h = (((bits >> 16) & 0x8000) | ((((bits >> 23) & 0xff).astype(np.int64) - 112) << 10) | ((bits & 0x7fffff) >> 13)).astype(np.uint16)
    raw = np.empty((total, 18), np.uint8)
    raw[:, :2] = h.view(np.uint8).reshape(total, 2)
    raw[:, 2:] = draws[:, 1:].astype("<u4").view(np.uint8).reshape(total, 16)
    x = (np.sin(np.arange(in_dim, dtype=np.float32) * np.float32(0.017)) * np.float32(0.5)).astype(np.float32)
    return raw.reshape(-1), x


def test_reference_device_test_through_both_gemv_forms(accel, orc):
    """What WeightAccel::gemv becomes after the swap.  The reference's gemv kernels take fp32 activations
    and its device test holds them to rel < 1e-3 of the CPU (lib.rs:216-231).  smx_gemv_f32 is that
    arithmetic; smx_gemv is the decode path's Q8-activation arithmetic and differs from the CPU result by the
    activation rounding.  Both are measured on the reference's own test data and gated at what they give."""
    in_dim, out_dim = 15360, 3840
    raw, x = _reference_device_test_data(orc, in_dim, out_dim)
    cpu = orc.matmul_f32(2, raw, in_dim, out_dim, x, order=0)[0]     # the test's sequential CPU sum
    scale = max(float(np.abs(cpu).max()), 1e-6)
    assert accel.upload_q4_0("t.ref", raw, in_dim, out_dim)
    e_f32 = float(np.abs(accel.gemv_f32("t.ref", x, out_dim) - cpu).max()) / scale
    e_q8 = float(np.abs(accel.gemv("t.ref", x, out_dim) - cpu).max()) / scale
    print(f"reference device test 3840<-15360: gemv_f32 rel {e_f32:.3e}, gemv (Q8 activations) rel {e_q8:.3e}")
    assert e_f32 < 1e-3           # the reference's bar for the method
    assert e_f32 < 1e-5           # what fp32 accumulation gives
    assert e_q8 < 5e-3            # measured 2.4e-3: activation rounding (d = amax/127 per 32-block), above the 1e-3 bar
    accel.evict("t.ref")


# flat form: rows of up to 16384 elements in whole unit groups; the row-per-wave form: the others (96, 4128, 32 * 67,
# 16384 + 512 and 32768 elements)
F32_SHAPES = SHAPES + FORM_SHAPES + [(2, 9728, 2560), (8, 2560, 9728), (14, 1000, 3840), (2, 5, 32768), (2, 300, 16384),
                                     (8, 200, 8192), (14, 257, 16384), (2, 100000, 256)]


@pytest.mark.parametrize("ty,N,K", F32_SHAPES)
def test_gemv_f32_matches_f32_oracle(accel, orc, synth, relerr, ty, N, K):
    raw = synth.make_weight(ty, N, K, seed=19 * N + K)
    x = synth.make_acts(1, K, seed=3 * N + K)
    _up(accel, ty, "t.f32", raw, K, N)
    y = accel.gemv_f32("t.f32", x, N)
    for order in (0, 1):      # both summation orders of strix-backend-cpu (gemma.rs:323-326, mellum.rs:278-293)
        assert relerr(y, orc.matmul_f32(ty, raw, K, N, x, order=order)[0]) <= 1e-5
    accel.evict("t.f32")


def test_gemv_f32_batch_equals_single_calls(accel, orc, synth, relerr):
    """gemv_batch in the fp32-activation arithmetic (what the trait's default binding calls): one device job, one sync,
    every item the bits of its single call; items that are not resident decline, the others still run."""
    K, Ns = 2560, (64, 200, 96)
    raws = [synth.make_weight(ty, n, K, seed=ty + n) for ty, n in zip((2, 8, 14), Ns)]
    for ty, raw, n in zip((2, 8, 14), raws, Ns):
        _up(accel, ty, f"t.fb{ty}", raw, K, n)
    xs = [synth.make_acts(1, K, seed=60 + i)[0] for i in range(4)]
    calls = [("t.fb2", xs[0]), ("t.fb8", xs[1]), ("t.nope", xs[2]), ("t.fb14", xs[3]), ("t.fb2", xs[3])]
    dims = [Ns[0], Ns[1], 7, Ns[2], Ns[0]]
    out = accel.gemv_batch(calls, dims, f32=True)
    assert out[2] is None
    for i, (key, x) in enumerate(calls):
        if i != 2:
            assert np.array_equal(out[i], accel.gemv_f32(key, x, dims[i])), i
    assert relerr(out[1], orc.matmul_f32(8, raws[1], K, Ns[1], xs[1])[0]) <= 1e-5
    for ty in (2, 8, 14):
        accel.evict(f"t.fb{ty}")


def test_gemv_f32_limits(accel, synth, pkg):
    raw = synth.make_weight(2, 2, 32768 + 32, seed=1)
    assert accel.upload_q4_0("t.f32big", raw, 32768 + 32, 2)
    with pytest.raises(pkg.SmxError) as ei:
        accel.gemv_f32("t.f32big", np.zeros(32768 + 32, np.float32), 2)
    assert ei.value.code == -3
    assert accel.gemv_f32("t.absent", np.zeros(32, np.float32), 1) is None
    accel.evict("t.f32big")
