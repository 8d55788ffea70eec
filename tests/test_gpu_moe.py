"""GPU parity of the MoE decode / prefill paths against the Q8 oracle, stage by stage."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
TOL = 1e-5


def _layer(accel, synth, layer, ne, hidden, eff, seed):
    gate, up, down = synth.make_moe_q8(ne, hidden, eff, seed)
    assert accel.upload_moe_q8(layer, gate, up, down, hidden, eff, ne)
    return gate, up, down


# k = 12: the 24 gate/up GEMVs exceed one grouped launch; eff = 416: down-projection units with a ragged tail;
# eff = 32, 96, 416, 224 / 64 / 128 / 768: unit groups of 2 / 4 / 8 / 16 lanes in the flat down kernel;
# (8, 1024, 2560): k * eff too large for it (the row-per-wave down kernel); hidden 2592 / 2336: gate and up
# rows that are not a whole number of unit groups (the row-per-wave GEMV).
@pytest.mark.parametrize("ne,hidden,eff,k", [(4, 64, 32, 2), (8, 256, 96, 3), (64, 2048, 768, 8), (16, 320, 416, 12),
                                             (8, 96, 224, 4), (8, 192, 128, 4), (8, 128, 64, 2), (8, 1024, 2560, 8),
                                             (4, 2592, 96, 2), (4, 2336, 64, 3)])
def test_moe_ffn_stagewise(accel, orc, synth, relerr, ne, hidden, eff, k):
    gate, up, down = _layer(accel, synth, 3, ne, hidden, eff, seed=ne + hidden)
    ids, w = synth.zipf_routing(1, ne, k, seed=5)
    x = synth.make_acts(1, hidden, seed=6)[0]
    _moe_stagewise(accel, orc, relerr, gate, up, down, ne, hidden, eff, k, ids, w, x)


def _moe_stagewise(accel, orc, relerr, gate, up, down, ne, hidden, eff, k, ids, w, x):
    y, gu, aq, ad = accel.moe_ffn_stages(3, ids[0], w[0], x, eff)
    ry, rgu, raq, rad = orc.moe_ffn_q8(gate, up, down, hidden, eff, ne, ids[0], w[0], x)
    # stage 1: gate/up GEMVs
    assert relerr(gu, rgu) <= TOL
    # stage 2: silu(g)*u + quantiser, bit-exact on the device's own g/u
    a = np.array([[orc.silu(g) * u for g, u in zip(gu[kk, 0], gu[kk, 1])] for kk in range(k)], np.float32)
    q2, d2, _ = orc.actquant(a, eff)
    assert np.array_equal(aq, q2)
    assert np.array_equal(ad.view(np.uint32), d2.view(np.uint32))
    # stage 3: down GEMVs + weighted sum, fed with the device's quantised activations
    ry2, _, _, _ = orc.moe_ffn_q8(gate, up, down, hidden, eff, ne, ids[0], w[0], x, aq_in=aq, ad_in=ad)
    assert relerr(y, ry2) <= TOL
    # end to end the two chains differ only where a quant sits on a rounding boundary
    assert relerr(y, ry) <= 2e-2
    assert np.array_equal(accel.moe_ffn(3, ids[0], w[0], x), y)


@pytest.mark.parametrize("ne,hidden,eff,k", [(4, 256, 256, 2), (8, 512, 768, 3), (16, 2048, 768, 8), (32, 256, 512, 20)])
def test_moe_ffn_q6k_experts_stagewise(accel, orc, synth, relerr, pkg, ne, hidden, eff, k):
    """Q6_K expert layers (upload_moe_q6, decode.rs:2793-2852): same stages, Q6_K integer sub-block dots."""
    gate, up, down = synth.make_moe_q6(ne, hidden, eff, seed=ne + eff)
    assert accel.upload_moe_q6(7, gate, up, down, hidden, eff, ne)
    ids, w = synth.zipf_routing(1, ne, k, seed=11)
    x = synth.make_acts(1, hidden, seed=12)[0]
    y, gu, aq, ad = accel.moe_ffn_stages(7, ids[0], w[0], x, eff)
    ry, rgu, raq, rad = orc.moe_ffn_q8(gate, up, down, hidden, eff, ne, ids[0], w[0], x, ty=14)
    assert relerr(gu, rgu) <= TOL
    a = np.array([[orc.silu(g) * u for g, u in zip(gu[kk, 0], gu[kk, 1])] for kk in range(k)], np.float32)
    q2, d2, _ = orc.actquant(a, eff)
    assert np.array_equal(aq, q2)
    assert np.array_equal(ad.view(np.uint32), d2.view(np.uint32))
    ry2, _, _, _ = orc.moe_ffn_q8(gate, up, down, hidden, eff, ne, ids[0], w[0], x, aq_in=aq, ad_in=ad, ty=14)
    assert relerr(y, ry2) <= TOL
    assert relerr(y, ry) <= 2e-2
    assert np.array_equal(accel.moe_ffn(7, ids[0], w[0], x), y)
    with pytest.raises(pkg.SmxError):
        accel.upload_moe_q6(8, gate[:-1], up, down, hidden, eff, ne)


def test_moe_ffn_declines_and_errors(accel, synth, pkg):
    x = np.zeros(64, np.float32)
    assert accel.moe_ffn(999, [0], [1.0], x) is None
    _layer(accel, synth, 4, 4, 64, 32, seed=1)
    with pytest.raises(pkg.SmxError):
        accel.moe_ffn(4, [7], [1.0], x)          # expert id out of range
    with pytest.raises(pkg.SmxError):
        accel.moe_ffn(4, [0], [1.0], x[:32])     # wrong hidden
    assert accel.moe_ffn(4, [0], [1.0], x, sgate=0.5) is None   # no shared expert resident: declines (decode.rs:2865)


@pytest.mark.parametrize("ty,hidden,sff", [(8, 256, 512), (2, 256, 4608), (14, 512, 256)])
def test_moe_ffn_shared_expert(accel, orc, synth, relerr, ty, hidden, sff):
    """moe_ffn with a shared-expert gate (decode.rs:1820-1855 queue_shexp, kernels.rs:1747-1751):
    y = routed + sgate * down_s(silu(gate_s x) * (up_s x)), checked stage by stage on the device's own g, u."""
    ne, eff, k, layer, sgate = 4, 256, 2, 23, 0.37
    gate, up, down = synth.make_moe_q8(ne, hidden, eff, seed=50)
    assert accel.upload_moe_q8(layer, gate, up, down, hidden, eff, ne)
    upl = {2: accel.upload_q4_0, 8: accel.upload_q8_0, 14: accel.upload_q6_k}[ty]
    sg, su, sd = synth.make_weight(ty, sff, hidden, seed=51), synth.make_weight(ty, sff, hidden, seed=52), synth.make_weight(ty, hidden, sff, seed=53)
    names = [f"blk.{layer}.ffn_{p}_shexp.weight" for p in ("gate", "up", "down")]
    assert upl(names[0], sg, hidden, sff) and upl(names[1], su, hidden, sff)
    ids, w = synth.zipf_routing(1, ne, k, seed=54)
    x = synth.make_acts(1, hidden, seed=55)[0]
    assert accel.moe_ffn(layer, ids[0], w[0], x, sgate=sgate) is None      # down weight still missing
    assert upl(names[2], sd, sff, hidden)
    routed = accel.moe_ffn(layer, ids[0], w[0], x)
    y = accel.moe_ffn(layer, ids[0], w[0], x, sgate=sgate)
    g, u = accel.gemv(names[0], x, sff), accel.gemv(names[1], x, sff)
    assert relerr(g, orc.matmul_q8_from_f32(ty, sg, hidden, sff, x)[0]) <= TOL
    shared = orc.matmul_q8_from_f32(ty, sd, sff, hidden, orc.act_produce(2, g, u))[0]
    assert relerr(y, routed + np.float32(sgate) * shared) <= TOL
    # device-resident form: routed part, then the shared expert on top
    xd, yd = accel.dev_alloc(x.nbytes), accel.dev_alloc(x.nbytes)
    accel.h2d(xd, x)
    assert accel.moe_ffn_dev(layer, ids[0], w[0], xd, yd) and accel.moe_shexp_dev(layer, sgate, xd, yd)
    assert np.array_equal(accel.d2h(np.empty(hidden, np.float32), yd), y)
    accel.dev_free(xd)
    accel.dev_free(yd)
    for n in names:
        accel.evict(n)


def _moe_layer_oracle(orc, gate, up, down, hidden, eff, ne, xs, ids, w, ty=8):
    """Per token: the decode oracle with experts in ascending slot (= ascending expert) order."""
    m = xs.shape[0]
    out = np.zeros((m, hidden), np.float32)
    for t in range(m):
        order = np.argsort(ids[t], kind="stable")
        out[t], _, _, _ = orc.moe_ffn_q8(gate, up, down, hidden, eff, ne, ids[t][order], w[t][order], xs[t], ty=ty)
    return out


# (16, 512, 256, 4, 300): expert groups that span several 128-token tiles with ragged tails;
# (8, 256, 160, 3, 37): weight-row tiles with a ragged tail (eff 160, hidden 256); (4, 64, 32, 2, 5): one tiny tile each
@pytest.mark.parametrize("ne,hidden,eff,k,m", [(4, 64, 32, 2, 5), (8, 256, 160, 3, 37), (16, 512, 256, 4, 300), (3, 384, 416, 2, 700)])
def test_moe_layer_stagewise(accel, orc, synth, moe_stagewise, ne, hidden, eff, k, m):
    """The grouped prefill path (decode.rs:1608-1739: gather -> per-expert GEMMs -> silu_quant_rows ->
    per-expert GEMMs -> weighted scatter) held to the decode path's bar at every stage."""
    gate, up, down = _layer(accel, synth, 7, ne, hidden, eff, seed=hidden + m)
    ids, w = synth.zipf_routing(m, ne, k, seed=9)
    xs = synth.make_acts(m, hidden, seed=10)
    plan, slot_tok, wslot = synth.group_by_expert(ids, w, ne)
    y, worst = moe_stagewise(accel, orc, 7, 8, gate, up, down, ne, hidden, eff, xs, plan, slot_tok, wslot)
    assert np.array_equal(y, accel.moe_layer_q8_dev(7, xs, m, plan, slot_tok, wslot))   # the plain call is the same computation


@pytest.mark.parametrize("ne,hidden,eff,k,m", [(4, 256, 256, 2, 5), (8, 512, 256, 3, 37), (16, 512, 768, 4, 300)])
def test_moe_layer_q6k_stagewise(accel, orc, synth, moe_stagewise, ne, hidden, eff, k, m):
    """The same for Q6_K expert layers (q6_gemm_moe, kernels.rs:1688-1735): two K = 16 MFMAs per 32-block."""
    gate, up, down = synth.make_moe_q6(ne, hidden, eff, seed=hidden + m)
    assert accel.upload_moe_q6(17, gate, up, down, hidden, eff, ne)
    ids, w = synth.zipf_routing(m, ne, k, seed=19)
    xs = synth.make_acts(m, hidden, seed=20)
    plan, slot_tok, wslot = synth.group_by_expert(ids, w, ne)
    y, worst = moe_stagewise(accel, orc, 17, 14, gate, up, down, ne, hidden, eff, xs, plan, slot_tok, wslot)
    assert np.array_equal(y, accel.moe_layer_q8_dev(17, xs, m, plan, slot_tok, wslot))


@pytest.mark.parametrize("ne,hidden,eff,k,m", [(4, 64, 32, 2, 5), (8, 256, 160, 3, 37), (16, 512, 256, 4, 300)])
def test_moe_layer_matches_decode_path(accel, orc, synth, relerr, ne, hidden, eff, k, m):
    gate, up, down = _layer(accel, synth, 7, ne, hidden, eff, seed=hidden + m)
    ids, w = synth.zipf_routing(m, ne, k, seed=9)
    xs = synth.make_acts(m, hidden, seed=10)
    plan, slot_tok, wslot = synth.group_by_expert(ids, w, ne)
    y = accel.moe_layer_q8_dev(7, xs, m, plan, slot_tok, wslot)
    assert y.shape == (m, hidden)
    ref = _moe_layer_oracle(orc, gate, up, down, hidden, eff, ne, xs, ids, w)
    # the intermediate quantisation makes the chains diverge where a quant sits on a rounding
    # boundary; the stage-exact check is against the device's own decode path below
    assert relerr(y, ref) <= 2e-2
    for t in (0, m // 2, m - 1):
        order = np.argsort(ids[t], kind="stable")
        yt = accel.moe_ffn(7, ids[t][order], w[t][order], xs[t])
        assert relerr(y[t], yt) <= 2e-2


@pytest.mark.parametrize("ne,hidden,eff,k,m", [(4, 256, 256, 2, 5), (8, 512, 256, 3, 37), (16, 512, 768, 4, 300)])
def test_moe_layer_q6k_experts(accel, orc, synth, relerr, ne, hidden, eff, k, m):
    """Grouped prefill over Q6_K expert layers (q6_gemm_moe, kernels.rs:1688-1735; moe_layer_ffn,
    decode.rs:3552-3629): the table-driven GEMM with Q6_K sub-block scales."""
    gate, up, down = synth.make_moe_q6(ne, hidden, eff, seed=hidden + m)
    assert accel.upload_moe_q6(17, gate, up, down, hidden, eff, ne)
    ids, w = synth.zipf_routing(m, ne, k, seed=19)
    xs = synth.make_acts(m, hidden, seed=20)
    plan, slot_tok, wslot = synth.group_by_expert(ids, w, ne)
    y = accel.moe_layer_q8_dev(17, xs, m, plan, slot_tok, wslot)
    assert y.shape == (m, hidden)
    ref = _moe_layer_oracle(orc, gate, up, down, hidden, eff, ne, xs, ids, w, ty=14)
    assert relerr(y, ref) <= 2e-2     # re-quantised intermediate, as for Q8_0 experts above
    for t in (0, m // 2, m - 1):
        order = np.argsort(ids[t], kind="stable")
        yt = accel.moe_ffn(17, ids[t][order], w[t][order], xs[t])
        assert relerr(y[t], yt) <= 2e-2


@pytest.mark.parametrize("ty", [8, 14])
def test_moe_layer_ffn_and_expert_ffn(accel, orc, synth, relerr, pkg, ty):
    """moe_layer_ffn (expert-major rows in, unweighted expert outputs out; decode.rs:3552-3629) and
    moe_expert_ffn: each output row is that expert's FFN of its input row."""
    ne, hidden, eff, layer = 8, 512, 256, 27
    gate, up, down = (synth.make_moe_q8 if ty == 8 else synth.make_moe_q6)(ne, hidden, eff, seed=70)
    assert (accel.upload_moe_q8 if ty == 8 else accel.upload_moe_q6)(layer, gate, up, down, hidden, eff, ne)
    plan = [(5, 3), (0, 140), (7, 1), (2, 33)]          # an expert may come in any order; one group spans two tiles
    rows = sum(n for _, n in plan)
    xs = synth.make_acts(rows, hidden, seed=71)
    dy = accel.moe_layer_ffn(layer, plan, xs, rows)
    assert dy.shape == (rows, hidden)
    r = 0
    for e, n in plan:
        for t in (r, r + n - 1):
            one = np.array([1.0], np.float32)
            yd, gu, aq, ad = accel.moe_ffn_stages(layer, [e], one, xs[t], eff)      # the decode path, weight 1
            ref, _, _, _ = orc.moe_ffn_q8(gate, up, down, hidden, eff, ne, np.array([e], np.int32), one, xs[t], aq_in=aq, ad_in=ad, ty=ty)
            assert relerr(yd, ref) <= TOL
            assert relerr(dy[t], yd) <= 2e-2            # chains differ only at quantiser rounding boundaries
        r += n
    ye = accel.moe_expert_ffn(layer, 2, xs[-33:], 33)
    assert np.array_equal(ye, dy[-33:])
    assert accel.moe_layer_ffn(999, plan, xs, rows) is None
    with pytest.raises(pkg.SmxError):
        accel.moe_layer_ffn(layer, [(8, 3)], xs[:3], 3)             # expert out of range
    with pytest.raises(pkg.SmxError):
        accel.moe_layer_ffn(layer, [(1, 3)], xs[:4], 4)             # groups do not cover the rows


def test_moe_layer_resident_equals_host_call(accel, synth, pkg):
    ne, hidden, eff, k, m = 8, 256, 96, 3, 70
    _layer(accel, synth, 9, ne, hidden, eff, seed=33)
    ids, w = synth.zipf_routing(m, ne, k, seed=34)
    plan, slot_tok, wslot = synth.group_by_expert(ids, w, ne)
    xs = synth.make_acts(m, hidden, seed=35)
    want = accel.moe_layer_q8_dev(9, xs, m, plan, slot_tok, wslot)
    xd, yd = accel.dev_alloc(xs.nbytes), accel.dev_alloc(xs.nbytes)
    accel.h2d(xd, xs)
    assert accel.moe_layer_resident(9, xd, m, plan, slot_tok, wslot, yd)
    assert np.array_equal(accel.d2h(np.empty_like(xs), yd), want)
    accel.graph_begin()
    with pytest.raises(pkg.SmxError):
        accel.moe_layer_resident(9, xd, m, plan, slot_tok, wslot, yd)   # host tables: not capturable
    accel.graph_destroy(accel.graph_end())
    assert accel.moe_layer_resident(99, xd, m, plan, slot_tok, wslot, yd) is False
    accel.dev_free(xd)
    accel.dev_free(yd)


def test_moe_layer_rejects_bad_plan(accel, synth, pkg):
    _layer(accel, synth, 8, 4, 64, 32, seed=2)
    xs = synth.make_acts(2, 64, seed=1)
    with pytest.raises(pkg.SmxError):   # plan does not cover the slots
        accel.moe_layer_q8_dev(8, xs, 2, [(0, 0, 1)], [0, 1], [0.5, 0.5])
    with pytest.raises(pkg.SmxError):   # token index out of range
        accel.moe_layer_q8_dev(8, xs, 2, [(0, 0, 2)], [0, 5], [0.5, 0.5])
    assert accel.moe_layer_q8_dev(12345, xs, 2, [(0, 0, 2)], [0, 1], [0.5, 0.5]) is None


@pytest.mark.parametrize("ne,k", [(8, 2), (64, 8), (128, 16), (300, 5), (1024, 64), (5, 5), (64, 1)])
def test_device_router_matches_oracle(accel, orc, ne, k):
    """topk_router (kernels.rs:1846-1872) against the CPU routing of mellum.rs:1178-1192: same experts in the
    same order, weights to fp32 rounding; equal logits keep ascending index order."""
    rng = np.random.default_rng(ne * 100 + k)
    for case in range(4):
        logits = rng.standard_normal(ne).astype(np.float32) * np.float32(2.0)
        if case == 1:
            logits = np.round(logits * 2) / 2          # many exact ties
        if case == 2:
            logits[:] = np.float32(0.75)                 # all equal: experts 0 .. k - 1 in order
        if case == 3:
            logits = logits * np.float32(6.0)            # a peaked distribution (probabilities down to e-40 are told apart)
        ids, w = accel.moe_route(logits, k)
        rids, rw = orc.route_topk(logits, k)
        assert np.array_equal(ids, rids), (case, ids, rids)
        assert np.abs(w - rw).max() <= 2e-6 * max(float(rw.max()), 1e-30)
        assert abs(float(w.sum()) - 1.0) < 1e-5


@pytest.mark.parametrize("ty", [8, 14])
def test_moe_decode_graph_serves_each_tokens_own_routing(accel, orc, synth, ty):
    """Router and expert FFN of a decode token captured once (decode.rs:3053-3203): the replays read the
    routing the router wrote for THAT token, so each equals the eager host-routed call for its token."""
    ne, hidden, eff, k, layer = 16, 512, 256, 4, 41
    gate, up, down = (synth.make_moe_q8 if ty == 8 else synth.make_moe_q6)(ne, hidden, eff, seed=80)
    assert (accel.upload_moe_q8 if ty == 8 else accel.upload_moe_q6)(layer, gate, up, down, hidden, eff, ne)
    rng = np.random.default_rng(81)
    toks = [(rng.standard_normal(ne).astype(np.float32) * 3, synth.make_acts(1, hidden, seed=82 + t)[0]) for t in range(4)]
    want = []
    for logits, x in toks:
        ids, w = accel.moe_route(logits, k)
        assert np.array_equal(ids, orc.route_topk(logits, k)[0])
        want.append(accel.moe_ffn(layer, ids, w, x))
    assert len({tuple(accel.moe_route(l, k)[0]) for l, _ in toks}) > 1           # the tokens do route differently
    ld, xd, yd = accel.dev_alloc(ne * 4), accel.dev_alloc(hidden * 4), accel.dev_alloc(hidden * 4)
    idd, wd = accel.dev_alloc(k * 4), accel.dev_alloc(k * 4)

    def step():
        assert accel.moe_route_dev(ld, ne, k, idd, wd)
        assert accel.moe_ffn_routed_dev(layer, idd, wd, k, xd, yd)

    accel.h2d(ld, toks[0][0])
    accel.h2d(xd, toks[0][1])
    step()                                                                        # scratch sized outside capture
    assert np.array_equal(accel.d2h(np.empty(hidden, np.float32), yd), want[0])   # eager device-routed == host-routed
    accel.graph_begin()
    step()
    g = accel.graph_end()
    for t in (1, 2, 3, 0, 2):
        accel.h2d(ld, toks[t][0])
        accel.h2d(xd, toks[t][1])
        accel.h2d(yd, np.zeros(hidden, np.float32))
        accel.graph_launch(g)
        accel.sync()
        assert np.array_equal(accel.d2h(np.empty(hidden, np.float32), yd), want[t]), f"token {t}"
    accel.graph_destroy(g)
    for p in (ld, xd, yd, idd, wd):
        accel.dev_free(p)
    assert accel.moe_ffn_routed_dev(999, idd, wd, k, xd, yd) is False


@pytest.mark.parametrize("ty,ne,hidden,eff,k", [(8, 64, 2048, 768, 8), (8, 16, 512, 256, 4), (14, 16, 512, 256, 4), (8, 64, 512, 256, 12),
                                                (8, 128, 256, 128, 6), (8, 8, 256, 96, 2), (8, 5, 256, 64, 5)])
def test_moe_ffn_from_router_logits(accel, orc, synth, ty, ne, hidden, eff, k):
    """smx_moe_ffn_logits_dev: the routing of a decode token computed in the prologue of the experts' gate/up launch (up to 64
    experts, k <= 8, paired flat-form expert rows), or by a routing launch in front of it (the other shapes here: 12 routed
    experts, 128 experts, expert rows of 96 elements): the routing and the output have the bits of smx_moe_route_dev +
    smx_moe_ffn_routed_dev, the experts are those the oracle routes; captured once and replayed with other logits."""
    layer = 45
    gate, up, down = (synth.make_moe_q8 if ty == 8 else synth.make_moe_q6)(ne, hidden, eff, seed=ne + eff)
    assert (accel.upload_moe_q8 if ty == 8 else accel.upload_moe_q6)(layer, gate, up, down, hidden, eff, ne)
    rng = np.random.default_rng(ne + k)
    ld, xd, yd, y2 = accel.dev_alloc(ne * 4), accel.dev_alloc(hidden * 4), accel.dev_alloc(hidden * 4), accel.dev_alloc(hidden * 4)
    idd, wd, id2, w2 = (accel.dev_alloc(k * 4) for _ in range(4))
    toks = []
    for t in range(4):
        logits = (rng.standard_normal(ne) * 2.5).astype(np.float32)
        if t == 2:
            logits = np.round(logits)                      # exact ties: the lowest index first
        toks.append((logits, synth.make_acts(1, hidden, seed=200 + t)[0]))
    want = []
    for logits, x in toks:
        accel.h2d(ld, logits)
        accel.h2d(xd, x)
        assert accel.moe_route_dev(ld, ne, k, id2, w2) and accel.moe_ffn_routed_dev(layer, id2, w2, k, xd, y2)
        assert accel.moe_ffn_logits_dev(layer, ld, k, xd, yd, idd, wd)
        ids = accel.d2h(np.empty(k, np.int32), idd).copy()
        assert np.array_equal(ids, accel.d2h(np.empty(k, np.int32), id2)) and np.array_equal(ids, orc.route_topk(logits, k)[0])
        assert np.array_equal(accel.d2h(np.empty(k, np.float32), wd), accel.d2h(np.empty(k, np.float32), w2))
        y = accel.d2h(np.empty(hidden, np.float32), yd).copy()
        assert np.array_equal(y, accel.d2h(np.empty(hidden, np.float32), y2))
        want.append(y)
    accel.graph_begin()
    assert accel.moe_ffn_logits_dev(layer, ld, k, xd, yd, idd, wd)
    g = accel.graph_end()
    for t in (1, 3, 0, 2):
        accel.h2d(ld, toks[t][0])
        accel.h2d(xd, toks[t][1])
        accel.h2d(yd, np.zeros(hidden, np.float32))
        accel.h2d(idd, np.full(k, -1, np.int32))
        accel.graph_launch(g)
        accel.sync()
        assert np.array_equal(accel.d2h(np.empty(hidden, np.float32), yd), want[t]), f"token {t}"
    accel.graph_destroy(g)
    assert accel.moe_ffn_logits_dev(998, ld, k, xd, yd, idd, wd) is False
    for p in (ld, xd, yd, y2, idd, wd, id2, w2):
        accel.dev_free(p)
