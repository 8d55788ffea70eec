"""GPU parity of the activation producers fused into the GEMV (norm / SwiGLU / GeGLU + quantiser + GEMV in
one launch) against the oracle's producer followed by its quantiser and Q8 matmul."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
TOL = 1e-5
UP = {2: "upload_q4_0", 8: "upload_q8_0", 14: "upload_q6_k"}


def _inputs(synth, K, seed):
    a = synth.make_acts(1, K, seed=seed)[0] * 1.7
    b = synth.make_acts(1, K, seed=seed + 1)[0] * 0.5 + 1.0
    return a, b


@pytest.mark.parametrize("ty", [2, 8, 14])
@pytest.mark.parametrize("act", [1, 2, 3])
@pytest.mark.parametrize("N,K", [(96, 256), (1024, 2560), (300, 9728)])
def test_fused_producer_matches_oracle(accel, orc, synth, relerr, ty, act, N, K):
    if ty == 14 and K % 256:
        pytest.skip("Q6_K rows are whole superblocks")
    raw = synth.make_weight(ty, N, K, seed=ty + act)
    assert getattr(accel, UP[ty])("t.fused", raw, K, N)
    a, b = _inputs(synth, K, seed=40 + act)
    eps = 1e-6 if act == 1 else 0.0
    y = accel.gemv_fused("t.fused", act, a, b, N, eps)
    x = orc.act_produce(act, a, b, eps)
    assert relerr(y, orc.matmul_q8_from_f32(ty, raw, K, N, x)[0]) <= TOL
    # the unfused route through the same library (producer on the host) gives the same integers
    assert relerr(y, accel.gemv("t.fused", x, N)) <= TOL


def test_rmsnorm_without_weight_and_plain(accel, orc, synth, relerr):
    N, K = 512, 2560
    raw = synth.make_weight(2, N, K, seed=5)
    assert accel.upload_q4_0("t.fused2", raw, K, N)
    a, _ = _inputs(synth, K, seed=60)
    y = accel.gemv_fused("t.fused2", 1, a, None, N, 1e-5)
    assert relerr(y, orc.matmul_q8_from_f32(2, raw, K, N, orc.act_produce(1, a, None, 1e-5))[0]) <= TOL
    # producer 0 is the plain fused-quantiser GEMV, bit for bit
    assert np.array_equal(accel.gemv_fused("t.fused2", 0, a, None, N), accel.gemv("t.fused2", a, N))


def test_rmsnorm_zero_row_and_extremes(accel, orc, synth, relerr):
    N, K = 64, 256
    raw = synth.make_weight(8, N, K, seed=6)
    assert accel.upload_q8_0("t.fused3", raw, K, N)
    z = np.zeros(K, np.float32)
    assert np.array_equal(accel.gemv_fused("t.fused3", 1, z, None, N, 1e-6), np.zeros(N, np.float32))
    g = np.linspace(-60, 60, K).astype(np.float32)   # saturated tanh / exp on both ends
    u = np.ones(K, np.float32)
    for act in (2, 3):
        y = accel.gemv_fused("t.fused3", act, g, u, N)
        assert relerr(y, orc.matmul_q8_from_f32(8, raw, K, N, orc.act_produce(act, g, u))[0]) <= TOL


def test_fused_group_launch_and_errors(accel, orc, synth, relerr, pkg):
    """rmsnorm -> q/k/v: three weights, one launch, one read of the activation."""
    K, Ns = 2560, [4096, 1024, 130]
    raws = [synth.make_weight(2, n, K, seed=80 + i) for i, n in enumerate(Ns)]
    for i, (n, r) in enumerate(zip(Ns, raws)):
        assert accel.upload_q4_0(f"t.fq{i}", r, K, n)
    a, w = _inputs(synth, K, seed=70)
    ad, wd = accel.dev_alloc(K * 4), accel.dev_alloc(K * 4)
    accel.h2d(ad, a)
    accel.h2d(wd, w)
    yds = [accel.dev_alloc(n * 4) for n in Ns]
    assert accel.gemv_fused_dev([f"t.fq{i}" for i in range(3)], 1, ad, wd, yds, 1e-6)
    x = orc.act_produce(1, a, w, 1e-6)
    for i, n in enumerate(Ns):
        y = accel.d2h(np.empty(n, np.float32), yds[i])
        assert relerr(y, orc.matmul_q8_from_f32(2, raws[i], K, n, x)[0]) <= TOL
    assert accel.gemv_fused_dev(["t.fq0", "t.absent"], 1, ad, wd, yds[:2]) is False
    with pytest.raises(pkg.SmxError):
        accel.gemv_fused_dev(["t.fq0"], 2, ad, None, yds[:1])      # silu_mul needs its second operand
    with pytest.raises(pkg.SmxError):
        accel.gemv_fused_dev(["t.fq0"], 7, ad, wd, yds[:1])        # unknown producer
    with pytest.raises(pkg.SmxError):
        accel.gemv_fused("t.fq0", 1, a[:64], None, Ns[0])           # wrong length
    assert accel.gemv_fused("t.absent", 1, a, None, 8) is None
    for p in [ad, wd] + yds:
        accel.dev_free(p)


@pytest.mark.parametrize("ty", [2, 8, 14])
@pytest.mark.parametrize("act", [1, 2, 3])
def test_prefill_rows_through_a_producer(accel, orc, synth, relerr, ty, act):
    """smx_gemm_fused_dev: m rows, producer inside the quantiser launch, then the int8 GEMM; row t equals
    the oracle's producer + quantiser + Q8 matmul of row t (kernels.rs:1174-1187 silu_quant_rows)."""
    M, N, K = 70, 200, 1280
    raw = synth.make_weight(ty, N, K, seed=ty + 10 * act)
    assert getattr(accel, UP[ty])("t.pf", raw, K, N)
    a = synth.make_acts(M, K, seed=80 + act) * 1.7
    a[3] = 0.0                                                   # an all-zero row: scale 0, quants 0
    b = (synth.make_acts(1, K, seed=90)[0] * 0.1 + 1.0) if act == 1 else (synth.make_acts(M, K, seed=91) * 0.5 + 1.0)
    eps = 1e-6 if act == 1 else 0.0
    ad, bd, yd = accel.dev_alloc(a.nbytes), accel.dev_alloc(b.nbytes), accel.dev_alloc(M * N * 4)
    accel.h2d(ad, a)
    accel.h2d(bd, b)
    assert accel.gemm_fused_dev("t.pf", act, ad, bd, M, yd, eps)
    y = accel.d2h(np.empty((M, N), np.float32), yd)
    x = np.stack([orc.act_produce(act, a[t], b if act == 1 else b[t], eps) for t in range(M)])
    assert relerr(y, orc.matmul_q8_from_f32(ty, raw, K, N, x)) <= TOL
    # the decode form of the same producer gives the same row
    for t in (0, 3, M - 1):
        assert relerr(y[t], accel.gemv_fused("t.pf", act, a[t], b if act == 1 else b[t], N, eps)) <= TOL
    assert accel.gemm_fused_dev("t.absent", act, ad, bd, M, yd, eps) is False
    for p in (ad, bd, yd):
        accel.dev_free(p)


@pytest.mark.parametrize("ty,N,K", [(2, 9728, 2560), (8, 300, 1024), (14, 130, 2560), (2, 96, 256), (8, 77, 96), (2, 40, 16384 + 512)])
@pytest.mark.parametrize("act", [2, 3])
@pytest.mark.parametrize("norm", [False, True])
def test_ffn_gate_up_with_the_product_in_the_tail(accel, orc, synth, relerr, ty, N, K, act, norm):
    """smx_ffn_gate_up_dev: gate and up in one launch, h = act(g) * u from the kernel's tail (shapes of the flat form), or
    the pair launch followed by the product (rows of 96 and 16896 elements).  Each dot has the bits of
    smx_gemv_fused_dev, the product those of the oracle's producer on them."""
    if ty == 14 and K % 256:
        pytest.skip("Q6_K rows are whole superblocks")
    rg, ru = synth.make_weight(ty, N, K, seed=N + act), synth.make_weight(ty, N, K, seed=N + act + 7)
    assert getattr(accel, UP[ty])("t.g", rg, K, N) and getattr(accel, UP[ty])("t.u", ru, K, N)
    x, w = _inputs(synth, K, seed=70 + act)
    eps = 1e-6
    xd, wd = accel.dev_alloc(K * 4), accel.dev_alloc(K * 4)
    gd, ud, hd = (accel.dev_alloc(N * 4) for _ in range(3))
    accel.h2d(xd, x); accel.h2d(wd, w)
    assert accel.ffn_gate_up_dev("t.g", "t.u", act, xd, hd, norm=norm, norm_w_dev=wd if norm else None, eps=eps)
    h = accel.d2h(np.empty(N, np.float32), hd)
    # the two dots through the existing pair launch
    assert accel.gemv_fused_dev(["t.g", "t.u"], 1 if norm else 0, xd, wd if norm else None, [gd, ud], eps if norm else 0.0)
    g, u = accel.d2h(np.empty(N, np.float32), gd), accel.d2h(np.empty(N, np.float32), ud)
    assert np.array_equal(h, orc.act_produce(act, g, u, 0.0))
    # and against the oracle end to end
    xn = orc.act_produce(1, x, w, eps) if norm else x
    g_ref = orc.matmul_q8_from_f32(ty, rg, K, N, xn)[0]
    u_ref = orc.matmul_q8_from_f32(ty, ru, K, N, xn)[0]
    assert relerr(g, g_ref) <= TOL and relerr(u, u_ref) <= TOL
    assert relerr(h, orc.act_produce(act, g_ref, u_ref, 0.0)) <= 2e-5    # the product of two 1e-5 quantities
    for p in (xd, wd, gd, ud, hd):
        accel.dev_free(p)
    accel.evict("t.g"); accel.evict("t.u")


def test_ffn_gate_up_errors(accel, synth, pkg):
    raw = synth.make_weight(2, 64, 256, seed=1)
    assert accel.upload_q4_0("t.g", raw, 256, 64) and accel.upload_q4_0("t.u2", synth.make_weight(2, 32, 256, seed=2), 256, 32)
    xd, hd = accel.dev_alloc(256 * 4), accel.dev_alloc(64 * 4)
    assert accel.ffn_gate_up_dev("t.g", "t.absent", 2, xd, hd) is False     # declines: not resident
    with pytest.raises(pkg.SmxError):   # shapes differ
        accel.ffn_gate_up_dev("t.g", "t.u2", 2, xd, hd)
    with pytest.raises(pkg.SmxError):   # not an activation product
        accel.ffn_gate_up_dev("t.g", "t.g", 1, xd, hd)
    accel.dev_free(xd); accel.dev_free(hd)
    accel.evict("t.g"); accel.evict("t.u2")
