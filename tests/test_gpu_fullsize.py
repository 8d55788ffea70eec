"""Parity at the benchmark's full sizes.  The decode GEMVs are compared with the oracle outright; the
2048-token GEMMs are too large for the CPU oracle in seconds, so they are checked on row/column
samples (the oracle on a subset of weight rows) and through the GEMM-row == GEMV identity."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
TOL = 1e-5
UPLOAD = {2: "upload_q4_0", 8: "upload_q8_0", 14: "upload_q6_k"}
BB = {2: 18, 8: 34, 14: 210}
BE = {2: 32, 8: 32, 14: 256}


@pytest.mark.parametrize("ty,N,K", [(2, 9728, 2560), (8, 2560, 9728), (14, 15360, 3840)])
def test_decode_gemv_full_size(accel, orc, synth, relerr, ty, N, K):
    raw = synth.make_weight(ty, N, K, seed=ty)
    x = synth.make_acts(1, K, seed=50 + ty)
    assert getattr(accel, UPLOAD[ty])("t.full", raw, K, N)
    y = accel.gemv("t.full", x, N)
    assert relerr(y, orc.matmul_q8_from_f32(ty, raw, K, N, x)[0]) <= TOL
    per = K // 16 if ty == 14 else K // 32
    xq, _, _ = orc.actquant(x, K)
    assert np.array_equal(accel.gemv_block_dots("t.full", x, N, per), orc.block_dots(ty, raw, K, N, xq[0]))
    if ty != 14:   # batched verify rows, M = 1..8
        xs = synth.make_acts(8, K, seed=60 + ty)
        ref = orc.matmul_q8_from_f32(ty, raw, K, N, xs)
        for m in (2, 3, 8):
            assert relerr(accel.gemv_rows("t.full", xs[:m], N), ref[:m]) <= TOL
    # the fp32-activation form of the same weight against the f32 oracle
    assert relerr(accel.gemv_f32("t.full", x, N), orc.matmul_f32(ty, raw, K, N, x, order=0)[0]) <= TOL
    accel.evict("t.full")


def test_lm_head_q6k_sampled(accel, orc, synth, relerr):
    # 262144 x 3840 Q6_K head: 826 MB of weights; oracle on sampled rows, argmax against the device's own logits
    N, K = 262144, 3840
    raw = synth.make_q6_k(N, K, seed=3)
    x = synth.make_acts(1, K, seed=4)
    assert accel.upload_q6_k("t.head", raw, K, N)
    y = accel.gemv("t.head", x, N)
    rows = np.unique(np.concatenate([np.arange(0, 64), np.arange(N - 64, N), np.random.default_rng(1).integers(0, N, 400)]))
    sub = raw.reshape(N, -1)[rows].reshape(-1)
    ref = orc.matmul_q8_from_f32(14, sub, K, rows.size, x)[0]
    assert np.abs(y[rows] - ref).max() / np.abs(y).max() <= TOL
    assert int(accel.lm_head_argmax_rows("t.head", x, 1)[0]) == int(np.argmax(y))
    # three rows per weight pass (the verify step of speculative decoding): the group sums of a CU's
    # 1024 rows x 4 rows of activations no longer fit LDS, so the launch takes two rounds of workgroups
    xs = synth.make_acts(3, K, seed=5)
    ys = accel.gemv_rows("t.head", xs, N)
    refs = orc.matmul_q8_from_f32(14, sub, K, rows.size, xs)
    assert np.abs(ys[:, rows] - refs).max() / np.abs(ys).max() <= TOL
    assert [int(v) for v in accel.lm_head_argmax_rows("t.head", xs, 3)] == [int(np.argmax(r)) for r in ys]
    # fp32 activations: a CU's share is 1024 rows x 60 units, just inside the flat form's 16-bit unit index
    yf = accel.gemv_f32("t.head", x, N)
    reff = orc.matmul_f32(14, sub, K, rows.size, x, order=0)[0]
    assert np.abs(yf[rows] - reff).max() / np.abs(yf).max() <= TOL
    accel.evict("t.head")


def test_gemv_f32_two_rounds_of_workgroups(accel, orc, synth):
    # 33000 rows of 512 units: a CU's share (129 rows) no longer fits the flat form's 16-bit unit index, so the launch
    # takes two rounds of workgroups; oracle on sampled rows
    ty, N, K = 8, 33000, 8192
    raw = synth.make_weight(ty, N, K, seed=77)
    x = synth.make_acts(1, K, seed=78)
    assert accel.upload_q8_0("t.rounds", raw, K, N)
    y = accel.gemv_f32("t.rounds", x, N)
    rows = np.unique(np.concatenate([np.arange(0, 140), np.arange(N - 140, N), np.random.default_rng(2).integers(0, N, 600)]))
    sub = raw.reshape(N, -1)[rows].reshape(-1)
    ref = orc.matmul_f32(ty, sub, K, rows.size, x, order=0)[0]
    assert np.abs(y[rows] - ref).max() / np.abs(y).max() <= TOL
    # and the int8-activation form of the same launch geometry
    yq = accel.gemv("t.rounds", x, N)
    refq = orc.matmul_q8_from_f32(ty, sub, K, rows.size, x)[0]
    assert np.abs(yq[rows] - refq).max() / np.abs(yq).max() <= TOL
    accel.evict("t.rounds")


@pytest.mark.parametrize("ty,M,N,K", [(8, 2048, 15360, 3840), (2, 2048, 15360, 3840), (8, 2048, 3840, 15360), (2, 2048, 3840, 15360),
                                      (14, 2048, 15360, 3840), (14, 1000, 3840, 15360)])
def test_prefill_gemm_full_size_sampled(accel, orc, synth, relerr, ty, M, N, K):
    raw = synth.make_weight(ty, N, K, seed=10 + ty)
    xs = synth.make_acts(M, K, seed=20 + ty)
    assert getattr(accel, UPLOAD[ty])("t.fg", raw, K, N)
    y = accel.prefill_q8_gemm("t.fg", xs, M, N)
    assert y.shape == (M, N) and np.isfinite(y).all()
    scale = np.abs(y).max()
    # oracle on 96 sampled weight rows (all tokens): covers every token tile and the edges of the row tiles
    rows = np.unique(np.concatenate([[0, 1, 31, 32, 127, 128, N - 129, N - 128, N - 1], np.random.default_rng(2).integers(0, N, 87)]))
    sub = raw.reshape(N, -1)[rows].reshape(-1)
    ref = orc.matmul_q8_from_f32(ty, sub, K, rows.size, xs)
    assert np.abs(y[:, rows] - ref).max() / scale <= TOL
    # a GEMM row is the GEMV of that token (same integers; fp32 association differs)
    for t in (0, 777, M - 1):
        assert np.abs(y[t] - accel.gemv("t.fg", xs[t], N)).max() / scale <= TOL
    # determinism: split-K partials are reduced in a fixed order
    assert np.array_equal(y, accel.prefill_q8_gemm("t.fg", xs, M, N))
    accel.evict("t.fg")


@pytest.mark.parametrize("ty", [8, 14])
def test_moe_full_size_prefill_stagewise(accel, orc, synth, moe_stagewise, ty):
    """cfg5 prefill (64 experts, hidden 2048, eff 768, top-8, 512 tokens = 4096 slots): every stage of the
    grouped path against the oracle at 1e-5 / bit-exact quants; the gate/up and down GEMMs on a sample of the
    expert groups (the largest, the smallest and six others), the combine on every token."""
    ne, hidden, eff, k, m = 64, 2048, 768, 8, 512
    gate, up, down = (synth.make_moe_q8 if ty == 8 else synth.make_moe_q6)(ne, hidden, eff, seed=30)
    assert (accel.upload_moe_q8 if ty == 8 else accel.upload_moe_q6)(22, gate, up, down, hidden, eff, ne)
    ids, w = synth.zipf_routing(m, ne, k, seed=31)
    xs = synth.make_acts(m, hidden, seed=32)
    plan, slot_tok, wslot = synth.group_by_expert(ids, w, ne)
    assert slot_tok.size == 4096
    by_size = np.argsort(plan[:, 2])
    groups = sorted(set([int(by_size[0]), int(by_size[-1])] + [int(g) for g in np.random.default_rng(3).choice(len(plan), 6, replace=False)]))
    moe_stagewise(accel, orc, 22, ty, gate, up, down, ne, hidden, eff, xs, plan, slot_tok, wslot, groups=groups)


@pytest.mark.parametrize("ty", [8, 14])
def test_moe_full_size_decode_and_prefill(accel, orc, synth, relerr, ty):
    ne, hidden, eff, k, m = 64, 2048, 768, 8, 512
    gate, up, down = (synth.make_moe_q8 if ty == 8 else synth.make_moe_q6)(ne, hidden, eff, seed=30)
    assert (accel.upload_moe_q8 if ty == 8 else accel.upload_moe_q6)(21, gate, up, down, hidden, eff, ne)
    ids, w = synth.zipf_routing(m, ne, k, seed=31)
    xs = synth.make_acts(m, hidden, seed=32)
    plan, slot_tok, wslot = synth.group_by_expert(ids, w, ne)
    assert slot_tok.size == 4096
    y = accel.moe_layer_q8_dev(21, xs, m, plan, slot_tok, wslot)
    assert np.array_equal(y, accel.moe_layer_q8_dev(21, xs, m, plan, slot_tok, wslot))   # no atomics: repeatable
    for t in (0, 255, 511):
        order = np.argsort(ids[t], kind="stable")
        yd, gu, aq, ad = accel.moe_ffn_stages(21, ids[t][order], w[t][order], xs[t], eff)
        ref, _, _, _ = orc.moe_ffn_q8(gate, up, down, hidden, eff, ne, ids[t][order], w[t][order], xs[t], aq_in=aq, ad_in=ad, ty=ty)
        assert relerr(yd, ref) <= TOL
        assert relerr(y[t], yd) <= 2e-2      # prefill and decode chains differ only at quantiser rounding boundaries
