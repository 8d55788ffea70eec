"""The decode chain that bench.py times (strix.rs_amd/chain.py: per layer rmsnorm + gate/up + SwiGLU product, down GEMV,
router logits, routed expert FFN with the routing in its gate/up launch; the reference's captured token, decode.rs:3053-3203) against the oracle, stage by stage,
eager and as a replayed graph, and the router call on its own."""
import importlib.util
import os
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
TOL = 1e-5
PKG_DIR = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "strix.rs_amd")


@pytest.fixture(scope="module")
def chain_mod():
    name = "strix_rs_amd_chain"
    if name not in sys.modules:
        spec = importlib.util.spec_from_file_location(name, os.path.join(PKG_DIR, "chain.py"))
        sys.modules[name] = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(sys.modules[name])
    return sys.modules[name]


def _router_weight(synth, ty, ne, K, seed, factor):
    """A synthetic weight with its block scales multiplied by `factor`: router logits of a real model spread over a few
    units, and experts more than 87 below the largest logit are outside what the router tells apart (their probability
    is below 2e-38 on the device and on the CPU alike)."""
    raw = synth.make_weight(ty, ne, K, seed=seed).copy()
    if ty == 14:
        d = raw.reshape(-1, 210)[:, 208:210].copy().view(np.float16)
        raw.reshape(-1, 210)[:, 208:210] = (d.astype(np.float32) * np.float32(factor)).astype(np.float16).view(np.uint8)
    else:
        bb = 18 if ty == 2 else 34
        d = raw.reshape(-1, bb)[:, 0:2].copy().view(np.float16)
        raw.reshape(-1, bb)[:, 0:2] = (d.astype(np.float32) * np.float32(factor)).astype(np.float16).view(np.uint8)
    return raw


def _read(accel, ptr, n, dtype=np.float32):
    return accel.d2h(np.empty(n, dtype), ptr).copy()


@pytest.mark.parametrize("ty,ne,K,k", [(8, 64, 2048, 8), (8, 16, 512, 4), (2, 64, 1024, 8), (14, 64, 2048, 6), (8, 200, 512, 5),
                                       (8, 300, 256, 3), (8, 33, 4128, 4), (8, 64, 32768, 2)])
def test_router_call_equals_gemv_then_route(accel, orc, synth, relerr, ty, ne, K, k):
    """smx_moe_router_dev: logits with the bits of smx_gemv_dev, routing with the bits of smx_moe_route_dev on them, experts
    as the oracle routes the oracle-checked logits; all three formats, 16..300 experts, flat-form and other row lengths."""
    raw = _router_weight(synth, ty, ne, K, ne + K, 0.05 if ty != 14 else 0.1)
    assert {2: accel.upload_q4_0, 8: accel.upload_q8_0, 14: accel.upload_q6_k}[ty]("t.router", raw, K, ne)
    xd, ld, l2 = accel.dev_alloc(K * 4), accel.dev_alloc(ne * 4), accel.dev_alloc(ne * 4)
    idd, wd, id2, w2 = (accel.dev_alloc(k * 4) for _ in range(4))
    for t in range(3):
        x = synth.make_acts(1, K, seed=50 + t)[0]
        accel.h2d(xd, x)
        assert accel.moe_router_dev("t.router", xd, k, idd, wd, ld)
        assert accel.gemv_dev("t.router", xd, 1, l2) and accel.moe_route_dev(l2, ne, k, id2, w2)
        logits = _read(accel, ld, ne)
        assert np.array_equal(logits, _read(accel, l2, ne))
        ids, w = _read(accel, idd, k, np.int32), _read(accel, wd, k)
        assert np.array_equal(ids, _read(accel, id2, k, np.int32)) and np.array_equal(w, _read(accel, w2, k))
        assert relerr(logits, orc.matmul_q8_from_f32(ty, raw, K, ne, x)[0]) <= TOL
        assert float(logits.max() - logits.min()) < 80.0
        rids, rw = orc.route_topk(logits, k)
        assert np.array_equal(ids, rids) and np.abs(w - rw).max() <= 2e-6 * float(rw.max())
        assert accel.moe_router_dev("t.router", xd, k, idd, wd)          # without a logits buffer
        assert np.array_equal(_read(accel, idd, k, np.int32), ids)
    assert accel.moe_router_dev("t.absent", xd, k, idd, wd) is False
    for p in (xd, ld, l2, idd, wd, id2, w2):
        accel.dev_free(p)
    accel.evict("t.router")


@pytest.mark.parametrize("ety", [8, 14])
def test_decode_chain_stage_by_stage_eager_and_replayed(accel, orc, synth, relerr, chain_mod, ety):
    """Two layers of the benchmarked chain at small dimensions.  Every stage of every layer against the oracle on the
    device's own input to that stage (a rounding flip upstream would move a quant downstream): SwiGLU product and down
    GEMV <= 1e-5, router logits <= 1e-5 and expert ids identical to the oracle's routing of them, the routed expert FFN
    bit-identical to the host-routed call (itself checked stage-wise against the oracle).  Then the same chain captured
    once and replayed on three other tokens: every replay equals the eager run on that token, bit for bit."""
    layers, H, F, ne, eff, k, base = 2, 512, 1536, 16, 256, 4, 60
    rng = np.random.default_rng(5)
    W = []
    for l in range(layers):
        rg, ru = synth.make_weight(2, F, H, seed=100 + l), synth.make_weight(2, F, H, seed=110 + l)
        rd, rr = synth.make_weight(2, H, F, seed=120 + l), _router_weight(synth, 8, ne, H, 130 + l, 0.05)
        assert accel.upload_q4_0(f"t.ch.g{l}", rg, H, F) and accel.upload_q4_0(f"t.ch.u{l}", ru, H, F)
        assert accel.upload_q4_0(f"t.ch.d{l}", rd, F, H) and accel.upload_q8_0(f"t.ch.r{l}", rr, H, ne)
        experts = (synth.make_moe_q8 if ety == 8 else synth.make_moe_q6)(ne, H, eff, seed=140 + l)
        assert (accel.upload_moe_q8 if ety == 8 else accel.upload_moe_q6)(base + l, *experts, H, eff, ne)
        W.append((rg, ru, rd, rr, experts))
    nw = (rng.standard_normal(H) * 0.1 + 1.0).astype(np.float32)
    nwd, xd = accel.dev_alloc(H * 4), accel.dev_alloc(H * 4)
    accel.h2d(nwd, nw)
    ch = chain_mod.FfnMoeChain(accel, layers, H, F, ne, k, lambda l: tuple(f"t.ch.{t}{l}" for t in "gudr"), lambda l: base + l,
                               nwd, eps=1e-6, keep_stages=True)
    assert ch.launches_per_token() == 10
    toks = synth.make_acts(4, H, seed=77) * np.float32(1.5)

    def run_eager(x):
        accel.h2d(xd, x)
        out = ch.enqueue(xd)
        accel.sync()
        return _read(accel, out, H)

    y_last = run_eager(toks[0])
    x_in = toks[0]
    for l in range(layers):
        rg, ru, rd, rr, (gate, up, down) = W[l]
        b, yptr = ch.buffers(l)
        xn = orc.act_produce(1, x_in, nw, 1e-6)
        g, u = orc.matmul_q8_from_f32(2, rg, H, F, xn)[0], orc.matmul_q8_from_f32(2, ru, H, F, xn)[0]
        h = _read(accel, b["h"], F)
        assert relerr(h, orc.act_produce(2, g, u)) <= 2 * TOL, f"layer {l}: SwiGLU product"   # two dots at 1e-5 each
        d = _read(accel, b["d"], H)
        assert relerr(d, orc.matmul_q8_from_f32(2, rd, F, H, h)[0]) <= TOL, f"layer {l}: down"
        logits = _read(accel, b["logits"], ne)
        assert relerr(logits, orc.matmul_q8_from_f32(8, rr, H, ne, d)[0]) <= TOL, f"layer {l}: router logits"
        ids, w = _read(accel, b["ids"], k, np.int32), _read(accel, b["w"], k)
        assert float(logits.max() - logits.min()) < 80.0
        rids, rw = orc.route_topk(logits, k)
        assert np.array_equal(ids, rids) and np.abs(w - rw).max() <= 2e-6 * float(rw.max()), f"layer {l}: routing"
        y = _read(accel, yptr, H)
        ys, gu, aq, ad = accel.moe_ffn_stages(base + l, ids, w, d, eff)
        assert np.array_equal(y, ys), f"layer {l}: device-routed expert FFN differs from the host-routed call"
        _, rgu, _, _ = orc.moe_ffn_q8(gate, up, down, H, eff, ne, ids, w, d, ty=ety)
        assert relerr(gu, rgu) <= TOL
        a = orc.act_produce(2, gu[:, 0].reshape(-1), gu[:, 1].reshape(-1)).reshape(k, eff)
        q2, d2, _ = orc.actquant(a, eff)
        assert np.array_equal(aq, q2) and np.array_equal(ad.view(np.uint32), d2.view(np.uint32))
        ry, _, _, _ = orc.moe_ffn_q8(gate, up, down, H, eff, ne, ids, w, d, aq_in=aq, ad_in=ad, ty=ety)
        assert relerr(y, ry) <= TOL, f"layer {l}: expert FFN"
        x_in = y
    assert np.array_equal(y_last, x_in)

    want = [run_eager(t) for t in toks]
    assert len({w_.tobytes() for w_ in want}) == 4
    accel.h2d(xd, toks[0])
    accel.graph_begin()
    out = ch.enqueue(xd)
    g = accel.graph_end()
    for t in (1, 2, 3, 0, 2):
        accel.h2d(xd, toks[t])
        accel.h2d(out, np.zeros(H, np.float32))
        accel.gemv_dev("t.ch.r0", xd, 1, ch.buffers(0)[0]["logits"])      # eager work between replays, clobbers a stage buffer
        accel.sync()
        accel.graph_launch(g)
        accel.sync()
        assert np.array_equal(_read(accel, out, H), want[t]), f"replay of token {t}"
    accel.graph_destroy(g)

    # the chain with the routing as a launch of its own (router call, or GEMV + routing) gives the same bits
    for route in ("call", "launches"):
        ch2 = chain_mod.FfnMoeChain(accel, layers, H, F, ne, k, lambda l: tuple(f"t.ch.{t}{l}" for t in "gudr"), lambda l: base + l,
                                    nwd, eps=1e-6, route=route)
        assert ch2.launches_per_token() == 12
        accel.h2d(xd, toks[3])
        out2 = ch2.enqueue(xd)
        accel.sync()
        assert np.array_equal(_read(accel, out2, H), want[3]), route
        ch2.close()
    ch.close()
    accel.dev_free(nwd)
    accel.dev_free(xd)
    for l in range(layers):
        for t in "gudr":
            accel.evict(f"t.ch.{t}{l}")
