"""Device-resident entry points, graph capture, tuning knobs, timing, copy kernel."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_dev_entry_points_match_host_ones(accel, synth):
    N, K, m = 640, 2560, 5
    raw = synth.make_weight(8, N, K, seed=1)
    assert accel.upload_q8_0("t.dev", raw, K, N)
    xs = synth.make_acts(m, K, seed=2)
    xd, yd = accel.dev_alloc(xs.nbytes), accel.dev_alloc(m * N * 4)
    accel.h2d(xd, xs)
    assert accel.gemv_dev("t.dev", xd, m, yd)
    got = accel.d2h(np.empty((m, N), np.float32), yd)
    assert np.array_equal(got, accel.gemv_rows("t.dev", xs, N))
    assert accel.gemm_dev("t.dev", xd, m, yd)
    got = accel.d2h(np.empty((m, N), np.float32), yd)
    assert np.array_equal(got, accel.prefill_q8_gemm("t.dev", xs, m, N))
    assert accel.gemv_dev("t.absent", xd, 1, yd) is False
    accel.dev_free(xd)
    accel.dev_free(yd)


def test_graph_replays_equal_eager(accel, synth):
    """A captured chain of GEMV, GEMM and MoE-decode launches, replayed several times with eager work and
    synchronisations in between, must reproduce the eager results every time."""
    N, K = 512, 1024
    raw4, raw8 = synth.make_weight(2, N, K, seed=3), synth.make_weight(8, K, N, seed=4)
    assert accel.upload_q4_0("t.g4", raw4, K, N) and accel.upload_q8_0("t.g8", raw8, N, K)
    gate, up, down = synth.make_moe_q8(8, K, 96, seed=5)
    assert accel.upload_moe_q8(31, gate, up, down, K, 96, 8)
    ids, w = synth.zipf_routing(1, 8, 2, seed=6)
    x = synth.make_acts(4, K, seed=7)
    xd = accel.dev_alloc(x.nbytes)
    h1, h2, h3, h4 = (accel.dev_alloc(4 * max(N, K) * 4) for _ in range(4))
    accel.h2d(xd, x)

    def chain():
        accel.gemv_dev("t.g4", xd, 1, h1)          # K -> N
        accel.gemv_dev("t.g8", h1, 1, h2)          # N -> K  (dependent)
        accel.moe_ffn_dev(31, ids[0], w[0], h2, h3)
        accel.gemm_dev("t.g4", xd, 4, h4)

    def read():
        return [accel.d2h(np.empty(n, np.float32), p) for p, n in ((h1, N), (h2, K), (h3, K), (h4, 4 * N))]

    chain()
    eager = read()
    accel.graph_begin()
    chain()
    g = accel.graph_end()
    for rep in range(4):
        for p in (h1, h2, h3, h4):
            accel.h2d(p, np.zeros(4 * max(N, K), np.float32))     # eager work between replays
        accel.gemv_dev("t.g8", xd, 1, h1)                         # an unrelated eager launch
        accel.sync()
        accel.graph_launch(g)
        accel.sync()
        for a, b in zip(read(), eager):
            assert np.array_equal(a, b), f"replay {rep}"
    accel.graph_destroy(g)
    for p in (xd, h1, h2, h3, h4):
        accel.dev_free(p)


def test_graph_survives_later_scratch_growth(pkg, synth):
    """A graph captured with small scratch buffers must keep working after a larger eager call made
    the context reallocate them (the captured buffers are retired, not freed)."""
    acc = pkg.Mi355WeightAccel(0)                    # a fresh context: its scratch starts at the minimum size
    N, K, m = 256, 4096, 48
    raw = synth.make_weight(8, N, K, seed=41)
    assert acc.upload_q8_0("t.sg", raw, K, N)
    xs = synth.make_acts(m, K, seed=42)
    xd, yd = acc.dev_alloc(xs.nbytes), acc.dev_alloc(m * N * 4)
    acc.h2d(xd, xs)
    acc.gemm_dev("t.sg", xd, m, yd)                  # quantiser scratch + split-K partials
    want = acc.d2h(np.empty((m, N), np.float32), yd)
    acc.graph_begin()
    acc.gemm_dev("t.sg", xd, m, yd)
    g = acc.graph_end()
    big = synth.make_acts(3000, K, seed=43)          # 12 MB of int8 rows, 3 MB of partials: every scratch buffer grows
    bd, by = acc.dev_alloc(big.nbytes), acc.dev_alloc(3000 * N * 4)
    acc.h2d(bd, big)
    acc.gemm_dev("t.sg", bd, 3000, by)
    acc.sync()
    for rep in range(3):
        acc.h2d(yd, np.zeros((m, N), np.float32))
        acc.graph_launch(g)
        acc.sync()
        assert np.array_equal(acc.d2h(np.empty((m, N), np.float32), yd), want), f"replay {rep}"
    acc.graph_destroy(g)
    for p in (xd, yd, bd, by):
        acc.dev_free(p)
    acc.close()


def test_capture_refuses_scratch_growth(accel, synth, pkg):
    raw = synth.make_weight(8, 128, 4096, seed=8)
    assert accel.upload_q8_0("t.grow", raw, 4096, 128)
    m = 40000                                     # 164 MB of int8 rows: larger than any scratch grown so far
    xd, yd = accel.dev_alloc(m * 4096 * 4), accel.dev_alloc(m * 128 * 4)
    accel.graph_begin()
    with pytest.raises(pkg.SmxError):
        accel.gemm_dev("t.grow", xd, m, yd)
    g = accel.graph_end()
    accel.graph_destroy(g)
    accel.dev_free(xd)
    accel.dev_free(yd)


def test_tuning_knobs_keep_results(accel, orc, synth, relerr, pkg):
    # the GEMV knobs shape the row-per-wavefront kernel: rows that are not a whole number of unit groups
    # (81 blocks) or longer than 16384 elements (Q6_K rows are always whole groups)
    for ty, up, N, K in ((2, accel.upload_q4_0, 1000, 2592), (8, accel.upload_q8_0, 1000, 2592), (14, accel.upload_q6_k, 300, 16640)):
        raw = synth.make_weight(ty, N, K, seed=ty)
        x = synth.make_acts(1, K, seed=9)
        assert up("t.tune", raw, K, N)
        ref = orc.matmul_q8_from_f32(ty, raw, K, N, x)[0]
        for knobs in ({"gemv_lpr": 16}, {"gemv_lpr": 32, "gemv_rpw": 2}, {"gemv_lpr": 64, "gemv_rpw": 4},
                      {"gemv_lpr": 64, "gemv_ks": 2}, {"gemv_lpr": 64, "gemv_ks": 4}, {"gemv_wpc": 2}):
            for k, v in knobs.items():
                accel.tune(k, v)
            assert relerr(accel.gemv("t.tune", x, N), ref) <= 1e-5, knobs
            for k in knobs:
                accel.tune(k, 0)
    raw = synth.make_weight(8, 256, 4096, seed=11)
    xs = synth.make_acts(96, 4096, seed=12)             # 96 rows: the tiled GEMM (up to 64 run in the small-batch kernel)
    assert accel.upload_q8_0("t.tune", raw, 4096, 256)
    ref = orc.matmul_q8_from_f32(8, raw, 4096, 256, xs)
    for sk in (1, 2, 4, 8, 16):
        accel.tune("gemm_splitk", sk)
        assert relerr(accel.prefill_q8_gemm("t.tune", xs, 96, 256), ref) <= 1e-5
        assert relerr(accel.prefill_q8_gemm("t.tune", xs[:40], 40, 256), ref[:40]) <= 1e-5   # small-batch kernel: one or two K slices
    accel.tune("gemm_splitk", 0)
    # the GEMM's tile walk only renumbers tiles: every grouping of the token tiles gives the same bits
    raw = synth.make_weight(2, 1000, 512, seed=13)
    xs = synth.make_acts(1100, 512, seed=14)            # 9 token tiles x 8 weight strips
    assert accel.upload_q4_0("t.tune", raw, 512, 1000)
    base = accel.prefill_q8_gemm("t.tune", xs, 1100, 1000)
    assert relerr(base, orc.matmul_q8_from_f32(2, raw, 512, 1000, xs)) <= 1e-5
    for walk in (1, 2, 3, 9, 64):
        accel.tune("gemm_walk", walk)
        assert np.array_equal(accel.prefill_q8_gemm("t.tune", xs, 1100, 1000), base), walk
    accel.tune("gemm_walk", 0)
    # host-pointer calls: the kernels working on the pinned buffers themselves, or copy commands in front and behind: same bits
    raw6 = synth.make_weight(14, 300, 2560, seed=15)
    assert accel.upload_q6_k("t.tune6", raw6, 2560, 300)
    x1, x3 = synth.make_acts(1, 512, seed=16)[0], synth.make_acts(3, 512, seed=17)
    x6 = synth.make_acts(1, 2560, seed=18)[0]
    want = None
    for mode in (0, 1, 2):
        accel.tune("host_io", mode)
        got = (accel.gemv("t.tune", x1, 1000), accel.gemv_rows("t.tune", x3, 1000), accel.gemv_f32("t.tune", x1, 1000),
               accel.gemv("t.tune6", x6, 300), accel.gemv_f32("t.tune6", x6, 300),
               accel.gemv_fused("t.tune", 1, x1, None, 1000, eps=1e-6),
               *accel.gemv_batch([("t.tune", x1), ("t.tune6", x6), ("t.tune", x3[1])], [1000, 300, 1000]))
        if want is None:
            want = [np.array(g).copy() for g in got]
            assert relerr(want[0], orc.matmul_q8_from_f32(2, raw, 512, 1000, x1.reshape(1, -1))[0]) <= 1e-5
        for g, w_ in zip(got, want):
            assert np.array_equal(np.array(g), w_), mode
    accel.tune("host_io", 0)
    accel.evict("t.tune6")
    with pytest.raises(pkg.SmxError):
        accel.tune("gemv_flat", 1)          # no knob re-routes a shape to another kernel
    with pytest.raises(pkg.SmxError):
        accel.tune("no_such_knob", 1)
    with pytest.raises(pkg.SmxError):
        accel.tune("gemv_lpr", 48)


def test_copy_kernel_and_profiling(accel, synth):
    a = np.random.default_rng(0).integers(0, 255, 1 << 20, dtype=np.uint8)
    s, d = accel.dev_alloc(a.nbytes), accel.dev_alloc(a.nbytes)
    accel.h2d(s, a)
    accel.prof_reset()
    accel.prof_enable(True)
    accel.timer_begin()
    accel.dev_copy(d, s, a.nbytes)
    ms = accel.timer_end()
    accel.prof_enable(False)
    assert np.array_equal(accel.d2h(np.empty_like(a), d), a)
    tot, n = accel.prof_read("copy")
    assert n == 1 and 0 < tot <= ms * 1.5 + 0.1 and "copy" in accel.prof_names()
    accel.prof_reset()
    assert accel.prof_read("copy")[1] == 0
    accel.dev_free(s)
    accel.dev_free(d)


def test_grouped_gemv_launch(accel, orc, synth, relerr):
    """gemv_batch puts items of one format and row length in one launch (q/k/v: same K, different N)."""
    K = 2560
    for ty, up in ((2, accel.upload_q4_0), (8, accel.upload_q8_0), (14, accel.upload_q6_k)):
        Ns = [4096, 1024, 1024, 9728, 130]
        raws = [synth.make_weight(ty, n, K, seed=ty * 10 + i) for i, n in enumerate(Ns)]
        for i, (n, r) in enumerate(zip(Ns, raws)):
            assert up(f"t.grp{i}", r, K, n)
        xs = [synth.make_acts(1, K, seed=70 + i)[0] for i in range(len(Ns))]
        out = accel.gemv_batch([(f"t.grp{i}", xs[i]) for i in range(len(Ns))], Ns)
        for i, n in enumerate(Ns):
            assert relerr(out[i], orc.matmul_q8_from_f32(ty, raws[i], K, n, xs[i])[0]) <= 1e-5
            assert np.array_equal(out[i], accel.gemv(f"t.grp{i}", xs[i], n)) or relerr(out[i], accel.gemv(f"t.grp{i}", xs[i], n)) <= 1e-5
    # device-pointer form: gate + up share the activation
    xd = accel.dev_alloc(K * 4)
    accel.h2d(xd, xs[0])
    y0, y1 = accel.dev_alloc(4096 * 4), accel.dev_alloc(9728 * 4)
    assert accel.gemv_batch_dev(["t.grp0", "t.grp3"], [xd, xd], [y0, y1])
    a = accel.d2h(np.empty(4096, np.float32), y0)
    b = accel.d2h(np.empty(9728, np.float32), y1)
    assert relerr(a, accel.gemv("t.grp0", xs[0], 4096)) <= 1e-5 and relerr(b, accel.gemv("t.grp3", xs[0], 9728)) <= 1e-5
    assert accel.gemv_batch_dev(["t.grp0", "t.absent"], [xd, xd], [y0, y1]) is False
    for p in (xd, y0, y1):
        accel.dev_free(p)


@pytest.mark.parametrize("act", [2, 3])
def test_ffn_block_two_launches_in_a_graph(accel, orc, synth, relerr, act):
    """A dense FFN decode step as two launches (norm + quantiser + gate/up; SwiGLU or GeGLU + quantiser
    + down), captured in a graph and replayed: equal to the eager run every time and to the oracle chain."""
    H, F = 1024, 2560
    rg, ru, rd = synth.make_weight(2, F, H, seed=21), synth.make_weight(2, F, H, seed=22), synth.make_weight(2, H, F, seed=23)
    assert accel.upload_q4_0("t.ffn.gate", rg, H, F) and accel.upload_q4_0("t.ffn.up", ru, H, F)
    assert accel.upload_q4_0("t.ffn.down", rd, F, H)
    x = synth.make_acts(1, H, seed=24)[0] * 2.0
    nw = synth.make_acts(1, H, seed=25)[0] * 0.1 + 1.0
    xd, wd, gd, ud, yd = (accel.dev_alloc(n * 4) for n in (H, H, F, F, H))
    accel.h2d(xd, x)
    accel.h2d(wd, nw)

    def block():
        accel.gemv_fused_dev(["t.ffn.gate", "t.ffn.up"], 1, xd, wd, [gd, ud], 1e-6)
        accel.gemv_fused_dev(["t.ffn.down"], act, gd, ud, [yd])

    block()
    eager = accel.d2h(np.empty(H, np.float32), yd)
    xn = orc.act_produce(1, x, nw, 1e-6)
    g = orc.matmul_q8_from_f32(2, rg, H, F, xn)[0]
    u = orc.matmul_q8_from_f32(2, ru, H, F, xn)[0]
    gdev, udev = accel.d2h(np.empty(F, np.float32), gd), accel.d2h(np.empty(F, np.float32), ud)
    assert relerr(gdev, g) <= 1e-5 and relerr(udev, u) <= 1e-5
    # the second stage is checked on the device's own g/u (a rounding flip in g would move a quant)
    assert relerr(eager, orc.matmul_q8_from_f32(2, rd, F, H, orc.act_produce(act, gdev, udev))[0]) <= 1e-5
    accel.graph_begin()
    block()
    graph = accel.graph_end()
    for rep in range(3):
        accel.h2d(yd, np.zeros(H, np.float32))
        accel.gemv_dev("t.ffn.gate", xd, 1, gd)      # eager work between replays, clobbers g
        accel.sync()
        accel.graph_launch(graph)
        accel.sync()
        assert np.array_equal(accel.d2h(np.empty(H, np.float32), yd), eager), f"replay {rep}"
    accel.graph_destroy(graph)
    for p in (xd, wd, gd, ud, yd):
        accel.dev_free(p)


@pytest.mark.parametrize("act", [2, 3])
def test_ffn_block_with_the_product_in_the_first_launch_in_a_graph(accel, orc, synth, relerr, act):
    """The same step as smx_ffn_gate_up_dev (norm + quantiser + gate/up + activation product) and a plain GEMV on the
    product: its quantised input has the bits of the three-launch form's, so the two forms give identical outputs;
    captured and replayed with the activation changed between replays."""
    H, F = 1024, 2560
    rg, ru, rd = synth.make_weight(2, F, H, seed=31), synth.make_weight(2, F, H, seed=32), synth.make_weight(2, H, F, seed=33)
    assert accel.upload_q4_0("t.ffn.gate", rg, H, F) and accel.upload_q4_0("t.ffn.up", ru, H, F)
    assert accel.upload_q4_0("t.ffn.down", rd, F, H)
    xs = synth.make_acts(3, H, seed=34) * 2.0
    nw = synth.make_acts(1, H, seed=35)[0] * 0.1 + 1.0
    xd, wd, gd, ud, hd, yd = (accel.dev_alloc(n * 4) for n in (H, H, F, F, F, H))
    accel.h2d(wd, nw)

    def three(out):
        accel.gemv_fused_dev(["t.ffn.gate", "t.ffn.up"], 1, xd, wd, [gd, ud], 1e-6)
        accel.gemv_fused_dev(["t.ffn.down"], act, gd, ud, [out])

    def two(out):
        accel.ffn_gate_up_dev("t.ffn.gate", "t.ffn.up", act, xd, hd, norm=True, norm_w_dev=wd, eps=1e-6)
        accel.gemv_dev("t.ffn.down", hd, 1, out)

    accel.h2d(xd, xs[0])
    two(yd)
    accel.graph_begin()
    two(yd)
    graph = accel.graph_end()
    for rep in range(3):
        accel.h2d(xd, xs[rep])
        three(yd)
        ref = accel.d2h(np.empty(H, np.float32), yd)
        accel.h2d(yd, np.zeros(H, np.float32))
        accel.graph_launch(graph)
        accel.sync()
        assert np.array_equal(accel.d2h(np.empty(H, np.float32), yd), ref), f"replay {rep}"
    accel.graph_destroy(graph)
    for p in (xd, wd, gd, ud, hd, yd):
        accel.dev_free(p)
    for k in ("gate", "up", "down"):
        accel.evict("t.ffn." + k)


def test_evict_and_reupload_keep_a_live_graph_valid(pkg, synth):
    """A captured graph holds the plane pointers of the weights it uses.  While it is alive, evicting or
    replacing such a weight must not free the device memory under it: replays keep giving the result
    they were captured with."""
    acc = pkg.Mi355WeightAccel(0)
    N, K = 384, 1024
    raw_a, raw_b = synth.make_weight(8, N, K, seed=61), synth.make_weight(8, N, K, seed=62)
    gate, up, down = synth.make_moe_q8(4, K, 64, seed=63)
    gate2, up2, down2 = synth.make_moe_q8(4, K, 64, seed=64)
    assert acc.upload_q8_0("t.live", raw_a, K, N) and acc.upload_moe_q8(5, gate, up, down, K, 64, 4)
    assert acc.weight_dims("t.live") == (K, N) and acc.weight_dims("t.none") is None
    x = synth.make_acts(1, K, seed=65)
    ids, w = synth.zipf_routing(1, 4, 2, seed=66)
    xd, yd, zd = acc.dev_alloc(x.nbytes), acc.dev_alloc(N * 4), acc.dev_alloc(K * 4)
    acc.h2d(xd, x)

    def chain():
        acc.gemv_dev("t.live", xd, 1, yd)
        acc.moe_ffn_dev(5, ids[0], w[0], xd, zd)

    def read():
        return acc.d2h(np.empty(N, np.float32), yd).copy(), acc.d2h(np.empty(K, np.float32), zd).copy()

    chain()
    want = read()
    acc.graph_begin()
    chain()
    g = acc.graph_end()
    assert acc.upload_q8_0("t.live", raw_b, K, N)                    # replaces the weight the graph reads
    assert acc.upload_moe_q8(5, gate2, up2, down2, K, 64, 4)         # and the expert layer
    junk = [acc.dev_alloc(raw_a.size) for _ in range(4)]             # allocations that would reuse freed memory
    for p in junk:
        acc.h2d(p, np.full(raw_a.size, 0x55, np.uint8))
    for rep in range(2):
        acc.h2d(yd, np.zeros(N, np.float32))
        acc.h2d(zd, np.zeros(K, np.float32))
        acc.graph_launch(g)
        acc.sync()
        got = read()
        assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1]), f"replay {rep}"
    assert acc.evict("t.live") and acc.weight_dims("t.live") is None
    acc.graph_launch(g)                                              # still reads memory the context keeps
    acc.sync()
    assert np.array_equal(read()[0], want[0])
    chain_new = acc.gemv_dev("t.live", xd, 1, yd)                    # eager calls see the eviction
    assert chain_new is False
    acc.graph_destroy(g)
    for p in junk + [xd, yd, zd]:
        acc.dev_free(p)
    acc.close()
