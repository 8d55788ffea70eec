"""Host-side logic that needs no GPU: synthetic generators, expert grouping, golden fixtures."""
import numpy as np
import pytest


def test_generators_follow_the_benchmark_distributions(synth, orc):
    raw = synth.make_q4_0(16, 256, seed=1).reshape(-1, 18)
    d = raw[:, :2].copy().view(np.float16).astype(np.float32)
    assert raw.shape[0] == 16 * 8 and d.min() >= 0.00099 and d.max() <= 0.0201
    nib = np.concatenate([raw[:, 2:] & 15, raw[:, 2:] >> 4]).ravel()
    assert nib.min() == 0 and nib.max() == 15
    r8 = synth.make_q8_0(16, 256, seed=2).reshape(-1, 34)
    q = r8[:, 2:].copy().view(np.int8)
    assert q.min() == -127 and q.max() == 127
    r6 = synth.make_q6_k(8, 512, seed=3).reshape(-1, 210)
    sc = r6[:, 192:208].copy().view(np.int8)
    d6 = r6[:, 208:].copy().view(np.float16).astype(np.float32)
    assert sc.min() >= -64 and sc.max() <= 63 and d6.min() >= 0.99e-4 and d6.max() <= 2.01e-3
    assert np.array_equal(synth.make_q4_0(4, 64, 9), synth.make_q4_0(4, 64, 9))       # seeded
    x = synth.make_acts(64, 2560, seed=4)
    assert abs(x.mean()) < 0.02 and abs(x.std() - 1) < 0.02
    for ty in (2, 8, 14):
        assert synth.make_weight(ty, 4, 256, 1).size == 4 * (256 // synth.BLOCK_ELEMS[ty]) * synth.BLOCK_BYTES[ty]
        assert synth.BLOCK_BYTES[ty] == orc.BLOCK_BYTES[ty]


def test_zipf_routing_and_grouping(synth):
    m, ne, k = 512, 64, 8
    ids, w = synth.zipf_routing(m, ne, k, seed=5)
    assert ids.shape == (m, k) and all(len(set(r)) == k for r in ids)
    assert np.allclose(w.sum(1), 1, atol=1e-5)
    counts = np.bincount(ids.ravel(), minlength=ne)
    assert counts.max() > 6 * np.median(counts)                     # skewed popularity
    plan, slot_tok, wslot = synth.group_by_expert(ids, w, ne)
    assert slot_tok.size == m * k == wslot.size                     # 4096 slots
    assert plan[:, 2].sum() == m * k and np.array_equal(plan[:, 1], np.concatenate([[0], np.cumsum(plan[:, 2])[:-1]]))
    assert np.all(np.diff(plan[:, 0]) > 0)                          # expert-major, ascending
    for e, off, cnt in plan:
        toks = slot_tok[off:off + cnt]
        assert np.all(np.diff(toks) > 0)                            # token-major within an expert
        for s, t in enumerate(toks):
            j = list(ids[t]).index(e)
            assert wslot[off + s] == w[t, j]


@pytest.mark.parametrize("name", ["q4_0_small.npz", "q8_0_small.npz", "q6_k_small.npz"])
def test_oracle_reproduces_golden_fixtures(orc, golden, name):
    g = golden(name)
    ty, N, K = int(g["ty"]), int(g["N"]), int(g["K"])
    xq, xd, xs = orc.actquant(g["x"], K)
    assert np.array_equal(xq, g["xq"]) and np.array_equal(xd, g["xd"]) and np.array_equal(xs, g["xs16"])
    for t in range(g["x"].shape[0]):
        assert np.array_equal(orc.block_dots(ty, g["raw"], K, N, xq[t]), g["block_dots"][t])
    assert np.array_equal(orc.matmul_q8(ty, g["raw"], K, N, xq, xd), g["y_q8"])
    assert np.array_equal(orc.matmul_f32(ty, g["raw"], K, N, g["x"], 1), g["y_f32"])
    # hand check of one stored block dot from the stored bytes alone
    raw = g["raw"]
    if ty == 8:
        q = raw[:34][2:].view(np.int8).astype(np.int64)
        assert int((q * g["xq"][0, :32].astype(np.int64)).sum()) == int(g["block_dots"][0, 0, 0])
    if ty == 2:
        b = raw[2:18].astype(np.int64)
        q = np.concatenate([b & 15, b >> 4]) - 8
        assert int((q * g["xq"][0, :32].astype(np.int64)).sum()) == int(g["block_dots"][0, 0, 0])


def test_multiply_high_division_used_by_the_flat_kernels_is_exact():
    """The flat GEMV and the flat MoE down kernel find a unit's row with one multiply-high:
    floor(f * ceil(2^32 / U) / 2^32) must equal f // U for every unit index a workgroup can hold
    (f < 2^16) and every row length the launchers admit (U < 2^16)."""
    import numpy as np
    f = np.arange(1 << 16, dtype=np.uint64)
    for U in list(range(1, 2049)) + [3040, 4095, 4096, 6144, 12288, 32767, 32768, 65535]:
        magic = np.uint64(((1 << 32) + U - 1) // U)
        assert np.array_equal((f * magic) >> np.uint64(32), f // np.uint64(U)), U
