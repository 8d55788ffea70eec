"""GPU parity of the int8 MFMA prefill GEMM against the Q8 oracle, through the C ABI."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
TOL = 1e-5
UPLOAD = {2: "upload_q4_0", 8: "upload_q8_0", 14: "upload_q6_k"}

# (type, M, N, K): tile multiples, ragged edges (N=96, M=37), K not a multiple of the 4-block stage,
# long K that triggers split-K, single token
SHAPES = [
    (8, 128, 128, 128), (2, 128, 128, 128), (8, 37, 96, 256), (2, 37, 96, 256), (8, 1, 300, 32),
    # at most 32 live tokens in a tile (every wave one row tile): ragged rows, K of 1, 2, 3 and many stages, a 160-token M whose last tile holds 32
    (8, 32, 13000, 2560), (8, 9, 12500, 9728), (8, 17, 300, 96), (8, 30, 257, 288), (8, 160, 200, 2560),
    (2, 200, 130, 160), (8, 256, 384, 2560), (2, 130, 257, 3840), (8, 64, 128, 15360), (2, 96, 256, 15360),
    # Q6_K (16-element sub-block scales, two K = 16 MFMAs per 32-block): one superblock, ragged, long K with split-K
    (14, 128, 128, 256), (14, 37, 96, 512), (14, 9, 300, 256), (14, 200, 130, 2560), (14, 96, 256, 15360),
]


@pytest.mark.parametrize("ty,M,N,K", SHAPES)
def test_gemm_matches_q8_oracle(accel, orc, synth, relerr, ty, M, N, K):
    raw = synth.make_weight(ty, N, K, seed=M + 3 * N + K)
    xs = synth.make_acts(M, K, seed=M * 7 + K)
    assert getattr(accel, UPLOAD[ty])("t.gemm", raw, K, N)
    y = accel.prefill_q8_gemm("t.gemm", xs, M, N)
    ref = orc.matmul_q8_from_f32(ty, raw, K, N, xs)
    assert y.shape == ref.shape
    assert relerr(y, ref) <= TOL


@pytest.mark.parametrize("ty,M,N,K", [(8, 37, 96, 256), (2, 37, 96, 256), (8, 130, 40, 160), (2, 64, 130, 2560),
                                      (8, 20, 13000, 160), (8, 5, 12400, 96),   # tiles of at most 32 live tokens: one row tile per wave

                                      (14, 37, 96, 256), (14, 130, 40, 768), (14, 64, 130, 2560)])
def test_gemm_block_dots_bit_exact(accel, orc, synth, ty, M, N, K):
    raw = synth.make_weight(ty, N, K, seed=M + N + K)
    xs = synth.make_acts(M, K, seed=M * 5 + K)
    assert getattr(accel, UPLOAD[ty])("t.gbd", raw, K, N)
    got = accel.gemm_block_dots("t.gbd", xs, M, N, K // (16 if ty == 14 else 32))
    xq, _, _ = orc.actquant(xs, K)
    for t in range(M):
        assert np.array_equal(got[t], orc.block_dots(ty, raw, K, N, xq[t])), f"token {t}"


@pytest.mark.parametrize("ty", [8, 14])
def test_gemm_row_equals_gemv(accel, synth, relerr, ty):
    # row t of the GEMM is the GEMV of xs[t]: same integers, fp32 association may differ
    M, N, K = 40, 200, 2560
    raw = synth.make_weight(ty, N, K, seed=3)
    xs = synth.make_acts(M, K, seed=4)
    assert getattr(accel, UPLOAD[ty])("t.rg", raw, K, N)
    y = accel.prefill_q8_gemm("t.rg", xs, M, N)
    for t in (0, 17, 39):
        assert relerr(y[t], accel.gemv("t.rg", xs[t], N)) <= TOL


@pytest.mark.parametrize("ty,M,N,K", [(8, 96, 2560, 2560), (2, 128, 300, 1280), (8, 65, 130, 288), (8, 100, 257, 96), (14, 70, 130, 512)])
def test_gemm_64_token_tiles(accel, orc, synth, relerr, ty, M, N, K):
    """65..128 tokens of a Q8_0 / Q4_0 weight run as two rows of 64-token tiles; the knob forces either tiling on any
    shape.  Same integers, same fp32 association per output: the two tilings agree bit for bit."""
    raw = synth.make_weight(ty, N, K, seed=M + N)
    assert getattr(accel, UPLOAD[ty])("t.t64", raw, K, N)
    xs = synth.make_acts(M + 150, K, seed=M)
    ref = orc.matmul_q8_from_f32(ty, raw, K, N, xs)
    for m in (M, M + 150):      # the second size has three or four 64-token rows, the last one ragged
        ys = {}
        for tile in (0, 64, 128):
            accel.tune("gemm_tile_m", tile)
            ys[tile] = accel.prefill_q8_gemm("t.t64", xs[:m], m, N)
            assert relerr(ys[tile], ref[:m]) <= TOL, (m, tile)
        accel.tune("gemm_tile_m", 64)
        xq, _, _ = orc.actquant(xs[:m], K)
        dots = accel.gemm_block_dots("t.t64", xs[:m], m, N, K // (16 if ty == 14 else 32))
        for t in (0, 63, 64, m - 1):
            assert np.array_equal(dots[t], orc.block_dots(ty, raw, K, N, xq[t])), (m, t)
        accel.tune("gemm_tile_m", 0)
        if K <= 1280:   # at most 10 stages: never split over K, identical association
            assert np.array_equal(ys[64], ys[128]) and np.array_equal(ys[0], ys[64])
    accel.evict("t.t64")


@pytest.mark.parametrize("ty,M,N,K", [(8, 200, 416, 512), (2, 130, 1000, 640), (14, 150, 330, 512), (8, 129, 96, 256), (8, 300, 100, 96)])
def test_gemm_96_row_strips(accel, orc, synth, relerr, ty, M, N, K):
    """A launch whose last round of workgroups would be partly filled cuts the first weight strips at 96 rows; the knob
    forces any number of them on any shape (N a whole number of strips or ragged, one strip only, more asked for than fit).
    Same integers, same fp32 association per output: bit-equal to the plain tiling."""
    raw = synth.make_weight(ty, N, K, seed=M + N)
    assert getattr(accel, UPLOAD[ty])("t.n96", raw, K, N)
    xs = synth.make_acts(M, K, seed=N)
    ref = orc.matmul_q8_from_f32(ty, raw, K, N, xs)
    accel.tune("gemm_splitk", 1)
    accel.tune("gemm_narrow", 1)
    plain = accel.prefill_q8_gemm("t.n96", xs, M, N)
    assert relerr(plain, ref) <= TOL
    for n in (1, 2, 3, 1000):
        accel.tune("gemm_narrow", 1 + n)
        assert np.array_equal(accel.prefill_q8_gemm("t.n96", xs, M, N), plain), n
    accel.tune("gemm_narrow", 0)
    accel.tune("gemm_splitk", 0)
    accel.evict("t.n96")


def test_gemm_declines_and_errors(accel, synth, pkg):
    assert accel.prefill_q8_gemm("t.absent", np.zeros((2, 64), np.float32), 2, 8) is None
    raw = synth.make_weight(8, 8, 256, seed=1)
    assert accel.upload_q8_0("t.e", raw, 256, 8)
    with pytest.raises(pkg.SmxError):   # wrong activation length
        accel.prefill_q8_gemm("t.e", np.zeros((16, 128), np.float32), 16, 8)


# The small-batch kernel on the matrix cores serves 5..64 rows of a Q8_0 / Q4_0 weight (17..64 rows up to 32768 weight
# rows) and 5..16 rows of a Q6_K weight (kernels.rs:830-857, 1016-1045, 1605-1632).  (type, N, K): one and two K slices
# per row group (two when the row groups alone would leave CUs idle and K has at least 64 blocks), K not a multiple of
# the 4-block piece, ragged row counts, fewer pieces than waves, row groups of fewer than 32 rows (whole rounds of
# CUs), the two decode shapes of the benchmark, a weight taller than 32768 rows, Q6_K from one superblock to a long row.
SMALL_BATCH = [(8, 96, 256), (8, 130, 2560), (8, 37, 9728), (2, 130, 2560), (2, 33, 4128), (8, 64, 2592), (2, 1000, 160),
               (8, 300, 128), (2, 7, 15360), (8, 2560, 9728), (2, 9728, 2560), (8, 12288, 512), (8, 40000, 256), (2, 9000, 320),
               (14, 96, 256), (14, 130, 2560), (14, 37, 9728), (14, 1000, 512), (14, 300, 768), (14, 9000, 1024)]


@pytest.mark.parametrize("ty,N,K", SMALL_BATCH)
def test_small_batch_matches_oracle(accel, orc, synth, relerr, ty, N, K):
    raw = synth.make_weight(ty, N, K, seed=N + K)
    assert getattr(accel, UPLOAD[ty])("t.sb", raw, K, N)
    for m in (5, 6, 7, 8, 9, 16, 17, 32, 33, 47, 64):          # 33..64: two token tiles per weight piece (Q8_0 / Q4_0)
        xs = synth.make_acts(m, K, seed=m + N)
        ref = orc.matmul_q8_from_f32(ty, raw, K, N, xs)
        y = accel.prefill_q8_gemm("t.sb", xs, m, N)               # WeightAccel::prefill_q8_gemm with a short chunk
        assert y.shape == ref.shape and relerr(y, ref) <= TOL, m
        if m <= 32:
            assert np.array_equal(accel.gemv_rows("t.sb", xs, N), y)  # the verify-step entry point runs the same kernel
        assert np.array_equal(accel.prefill_q8_gemm("t.sb", xs, m, N), y)   # two K slices add in either order: same bits
        if N * K <= 400000:   # the integers behind it, dumped by the same kernel
            xq, _, _ = orc.actquant(xs, K)
            dots = accel.gemm_block_dots("t.sb", xs, m, N, K // (16 if ty == 14 else 32))
            for t in range(m):
                assert np.array_equal(dots[t], orc.block_dots(ty, raw, K, N, xq[t])), (m, t)
    accel.evict("t.sb")


@pytest.mark.parametrize("ty", [8, 2])
def test_small_batch_ignores_stale_scales_past_k(accel, orc, synth, relerr, ty):
    """The activation scales of a call's last 4-block piece have slots past K when K is not a multiple of 128.  An earlier
    call leaves its own scales there (here: infinite ones, from infinite activations on a longer row); the next call's
    outputs must not see them (0 * inf would be NaN in every output)."""
    N = 64
    for m in (5, 12, 20):
        k_long, k_short = 2688, 2592          # 21 whole pieces / 20 pieces + 1 block
        raw_long = synth.make_weight(ty, N, k_long, seed=1)
        raw = synth.make_weight(ty, N, k_short, seed=2)
        assert getattr(accel, UPLOAD[ty])("t.stale.a", raw_long, k_long, N)
        assert getattr(accel, UPLOAD[ty])("t.stale.b", raw, k_short, N)
        accel.gemv_rows("t.stale.a", np.full((m, k_long), np.inf, np.float32), N)
        xs = synth.make_acts(m, k_short, seed=m)
        y = accel.gemv_rows("t.stale.b", xs, N)
        assert np.isfinite(y).all()
        assert relerr(y, orc.matmul_q8_from_f32(ty, raw, k_short, N, xs)) <= TOL
    accel.evict("t.stale.a")
    accel.evict("t.stale.b")


def test_small_batch_rows_equal_single_rows(accel, synth, relerr):
    # row t of a 20-row call is the GEMV of xs[t] (same integers; fp32 association differs), for both kernels' ranges
    N, K = 520, 4096
    for ty in (8, 2):
        raw = synth.make_weight(ty, N, K, seed=ty)
        xs = synth.make_acts(20, K, seed=5)
        assert getattr(accel, UPLOAD[ty])("t.sbr", raw, K, N)
        y = accel.gemv_rows("t.sbr", xs, N)
        y4 = accel.gemv_rows("t.sbr", xs[:4], N)                    # 4 rows: the dot4 GEMV
        assert relerr(y[:4], y4) <= TOL
        for t in (0, 9, 19):
            assert relerr(y[t], accel.gemv("t.sbr", xs[t], N)) <= TOL
    with pytest.raises(Exception):
        accel.gemv_rows("t.sbr", synth.make_acts(33, K, seed=1), N)   # gemv_rows takes up to 32 rows
    accel.evict("t.sbr")
