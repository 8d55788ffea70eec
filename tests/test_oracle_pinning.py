"""Pins the CPU oracle before anything is compared with it.

* block layout + dequant: the reference's own literal-value tests
  (crates/strix-models/src/ggml_quant.rs:443-469, 497-514, 562-565);
* f32 matmul: the reference's seeded device-test data
  (crates/strix-backend-rocm/src/lib.rs:135-180) against an independent float64 computation;
* integer path (no reference test exists for it): brute-force int64 dots over integers recovered
  through the pinned dequantiser, algebraic identities, quantiser invariants.
"""
import numpy as np
import pytest

Q4_0, Q8_0, Q6_K = 2, 8, 14


def f16_bytes(orc, v):
    h = orc.f32_to_f16(v)
    return [h & 0xff, h >> 8]


# ---------------------------------------------------------------- half precision

def test_f16_exact_against_numpy(orc):
    hs = np.arange(0, 65536, dtype=np.uint16)
    ref = hs.view(np.float16).astype(np.float32)
    got = np.array([orc.f16_to_f32(int(h)) for h in hs], np.float32)
    ok = ~np.isnan(ref)
    assert np.array_equal(got[ok].view(np.uint32), ref[ok].view(np.uint32))
    # subnormal case the reference's device decode handles by hand (kernels.rs:9-15)
    assert orc.f16_to_f32(0x0001) == 2.0 ** -24
    rng = np.random.default_rng(0)
    fs = np.concatenate([rng.standard_normal(2000).astype(np.float32) * 10.0 ** rng.integers(-8, 5, 2000),
                         np.array([0.0, -0.0, 65504.0, 65520.0, 1e-8, 6e-8, 6.1e-5], np.float32)]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = fs.astype(np.float16).view(np.uint16)
    got = np.array([orc.f32_to_f16(float(f)) for f in fs], np.uint16)
    assert np.array_equal(got, want)


# ---------------------------------------------------------------- reference literal vectors

def test_q8_0_scales_each_int(orc):          # ggml_quant.rs:443-453
    qs = np.arange(32, dtype=np.int32) - 4
    raw = np.array(f16_bytes(orc, 0.5) + [int(q) & 0xff for q in qs], np.uint8)
    y = orc.dequantize(Q8_0, raw, 32)
    assert np.abs(y - 0.5 * (np.arange(32) - 4.0)).max() < 1e-3


def test_q4_0_nibble_layout_and_bias(orc):   # ggml_quant.rs:456-469
    qs = [0] * 16
    qs[0], qs[1] = 0x80, 0xF1
    raw = np.array(f16_bytes(orc, 2.0) + qs, np.uint8)
    y = orc.dequantize(Q4_0, raw, 32)
    assert (y[0], y[16], y[1], y[17]) == (-16.0, 0.0, -14.0, 14.0)


def test_q6_k_decodes_known_values(orc):     # ggml_quant.rs:497-514
    blk = np.zeros(210, np.uint8)
    blk[0] = 0x05
    blk[128] = 0x01
    blk[192:208] = 1
    blk[208:210] = f16_bytes(orc, 1.0)
    y = orc.dequantize(Q6_K, blk, 256)
    assert y[0] == -11.0 and y[1] == -32.0 and y[32] == -32.0 and y.size == 256


def test_q4_k_with_zero_min_decodes_to_scaled_nibbles(orc):   # ggml_quant.rs:472-494
    blk = np.zeros(144, np.uint8)
    blk[0:2] = f16_bytes(orc, 1.0)
    blk[4] = 1                                   # sub-block 0: scale 1
    blk[16:48] = np.arange(32) % 16              # low nibbles of the first 32 quant bytes
    y = orc.dequantize(12, blk, 256)
    assert y.size == 256 and np.abs(y[:32] - np.arange(32) % 16).max() < 1e-4


def test_q5_k_first_value_uses_high_bit(orc):                 # ggml_quant.rs:525-541
    blk = np.zeros(176, np.uint8)
    blk[0:2] = f16_bytes(orc, 1.0)
    blk[4] = 1
    blk[16] = 0b00000001
    blk[48] = 0x0F
    y = orc.dequantize(13, blk, 256)
    assert y.size == 256 and abs(y[0] - 31.0) < 1e-3 and y[32] == 0.0


def test_unimplemented_quant_errors(orc):                     # ggml_quant.rs:517-521
    with pytest.raises(ValueError):
        orc.dequantize(10, np.zeros(84, np.uint8), 256)


def test_rejects_bad_sizes(orc):             # ggml_quant.rs:562-565
    with pytest.raises(ValueError):
        orc.dequantize(Q8_0, np.zeros(34, np.uint8), 16)
    with pytest.raises(ValueError):
        orc.dequantize(Q4_0, np.zeros(4, np.uint8), 32)


def test_golden_literal_fixture(orc, golden):
    g = golden("literal_blocks.npz")
    for name, ty in (("q8_0", Q8_0), ("q4_0", Q4_0), ("q6_k", Q6_K)):
        y = orc.dequantize(ty, g[name + "_raw"], g[name + "_out"].size)
        assert np.array_equal(y, g[name + "_out"])


# ---------------------------------------------------------------- independent decoders (numpy)

def np_q4_ints(raw, N, K):
    b = raw.reshape(N, K // 32, 18)
    d = b[:, :, :2].copy().view(np.float16).astype(np.float64)[:, :, 0]
    qs = b[:, :, 2:].astype(np.int64)
    q = np.concatenate([qs & 15, qs >> 4], axis=2) - 8          # elems 0..15 low nibbles, 16..31 high
    return d, q


def np_q8_ints(raw, N, K):
    b = raw.reshape(N, K // 32, 34)
    d = b[:, :, :2].copy().view(np.float16).astype(np.float64)[:, :, 0]
    q = b[:, :, 2:].copy().view(np.int8).astype(np.int64)
    return d, q


@pytest.mark.parametrize("ty", [Q4_0, Q8_0])
def test_dequant_matches_independent_numpy(orc, synth, ty):
    N, K = 5, 160
    raw = synth.make_weight(ty, N, K, seed=3)
    d, q = (np_q4_ints if ty == Q4_0 else np_q8_ints)(raw, N, K)
    want = (d[:, :, None].astype(np.float32) * q.astype(np.float32)).reshape(N, K)
    assert np.array_equal(orc.dequantize(ty, raw, N * K).reshape(N, K), want)


def _f16(b):
    return np.ascontiguousarray(b).view(np.float16).astype(np.float32)[..., 0]


def _np_q4_1_q5(ty, raw, n):
    """Q4_1 / Q5_0 / Q5_1 as the published GGML block layouts describe them (vectorised, no loops):
    value i = nibble (low halves first) | bit i of the 32-bit field << 4."""
    bb = {3: 20, 6: 22, 7: 24}[ty]
    b = raw.reshape(-1, bb)
    d = _f16(b[:, 0:2])
    pos = 2
    m = np.zeros_like(d)
    if ty in (3, 7):
        m = _f16(b[:, 2:4])
        pos = 4
    hi = np.zeros((b.shape[0], 32), np.int64)
    if ty in (6, 7):
        bits = b[:, pos:pos + 4].copy().view("<u4")[:, 0].astype(np.int64)
        hi = (bits[:, None] >> np.arange(32)[None, :]) & 1
        pos += 4
    qs = b[:, pos:pos + 16].astype(np.int64)
    q = np.concatenate([qs & 15, qs >> 4], axis=1) | (hi << 4)
    if ty == 6:
        return ((q - 16).astype(np.float32) * d[:, None]).reshape(-1)[:n]
    return (q.astype(np.float32) * d[:, None] + m[:, None]).reshape(-1)[:n]


def _np_q45_k(ty, raw, n):
    """Q4_K / Q5_K: scales and mins are 6-bit fields packed in 12 bytes (llama.cpp get_scale_min_k4)."""
    bb = 144 if ty == 12 else 176
    b = raw.reshape(-1, bb)
    nb = b.shape[0]
    d, dmin = _f16(b[:, 0:2]), _f16(b[:, 2:4])
    p = b[:, 4:16].astype(np.int64)
    sc = np.empty((nb, 8), np.int64)
    mn = np.empty((nb, 8), np.int64)
    sc[:, :4], mn[:, :4] = p[:, 0:4] & 63, p[:, 4:8] & 63
    sc[:, 4:] = (p[:, 8:12] & 15) | ((p[:, 0:4] >> 6) << 4)
    mn[:, 4:] = (p[:, 8:12] >> 4) | ((p[:, 4:8] >> 6) << 4)
    qs = b[:, bb - 128:].astype(np.int64).reshape(nb, 4, 32)
    q = np.stack([qs & 15, qs >> 4], axis=2).reshape(nb, 8, 32)          # sub-block 2c: low, 2c+1: high
    if ty == 13:
        hb = b[:, 16:48].astype(np.int64)
        q = q + (((hb[:, None, :] >> np.arange(8)[None, :, None]) & 1) << 4)
    ds = d[:, None] * sc.astype(np.float32)
    ms = dmin[:, None] * mn.astype(np.float32)
    return (ds[:, :, None] * q.astype(np.float32) - ms[:, :, None]).reshape(-1)[:n]


@pytest.mark.parametrize("ty", [3, 6, 7, 12, 13])
def test_requantisation_sources_match_independent_numpy(orc, ty):
    """Q4_1, Q5_0, Q5_1, Q4_K, Q5_K (ggml_quant.rs:265-400) only ever feed the host requantisers; the
    reference tests pin one literal block of Q4_K and Q5_K (above), the rest is pinned here against a
    vectorised decoder written from the format description."""
    be, bb = {3: (32, 20), 6: (32, 22), 7: (32, 24), 12: (256, 144), 13: (256, 176)}[ty]
    rng = np.random.default_rng(ty)
    raw = rng.integers(0, 256, (40, bb), dtype=np.uint8)
    sc = rng.uniform(-0.1, 0.1, (40, 2)).astype(np.float16)
    raw[:, 0:2] = sc[:, 0:1].view(np.uint8)
    if ty != 6:
        raw[:, 2:4] = sc[:, 1:2].view(np.uint8)      # m / dmin; for Q5_0 these bytes belong to the bit field
    raw = raw.reshape(-1)
    want = (_np_q4_1_q5 if ty in (3, 6, 7) else _np_q45_k)(ty, raw, 40 * be)
    got = orc.dequantize(ty, raw, 40 * be)
    assert np.array_equal(got, want)


def test_f32_oracle_on_reference_seeded_data(orc):
    """lib.rs:135-153: LCG 0xA5A5_1234, scales 0.03+(r%32)*0.003 as f16, x = 0.5 sin(0.017 i);
    (rows cut from 3840 to 64 to keep the float64 check quick; same generator stream)."""
    in_dim, out_dim = 15360, 64
    nblk = in_dim // 32
    total = nblk * out_dim
    draws, _ = orc.lcg(0xA5A51234, total * 5)
    draws = draws.reshape(total, 5)
    sc = (np.float32(0.03) + (draws[:, 0] % 32).astype(np.float32) * np.float32(0.003)).astype(np.float32)
    # the reference truncates toward zero in its test helper; both conversions of these values
    # agree with numpy's to within one f16 ulp, and the test's claim is on the decoded value
    sch = sc.astype(np.float16)
    raw = np.empty((total, 18), np.uint8)
    raw[:, :2] = sch.view(np.uint8).reshape(total, 2)
    raw[:, 2:] = draws[:, 1:].astype("<u4").view(np.uint8).reshape(total, 16)
    x = (np.sin(np.arange(in_dim, dtype=np.float32) * np.float32(0.017)) * np.float32(0.5)).astype(np.float32)
    d, q = np_q4_ints(raw.reshape(-1), out_dim, in_dim)
    want = (d[:, :, None] * q).reshape(out_dim, in_dim) @ x.astype(np.float64)
    for order in (0, 1):
        y = orc.matmul_f32(Q4_0, raw.reshape(-1), in_dim, out_dim, x, order)[0]
        rel = np.abs(y - want).max() / np.abs(want).max()
        assert rel < 1e-3          # the reference's own bar (lib.rs:231)
        assert rel < 2e-5          # and what fp32 accumulation over 15360 terms actually gives


def test_two_reference_summation_orders_differ_only_by_rounding(orc, synth):
    raw = synth.make_weight(Q8_0, 8, 2560, seed=1)
    x = synth.make_acts(1, 2560, seed=2)
    a = orc.matmul_f32(Q8_0, raw, 2560, 8, x, 0)
    b = orc.matmul_f32(Q8_0, raw, 2560, 8, x, 1)
    assert np.abs(a - b).max() / np.abs(a).max() < 1e-5


# ---------------------------------------------------------------- quantiser

def test_actquant_invariants_and_brute_force(orc, synth):
    K = 256
    x = synth.make_acts(4, K, seed=11)
    x[0, :32] = 0.0
    x[1, 32:64] = np.float32(3.5)                     # constant block: every q = 127
    xq, xd, xs = orc.actquant(x, K)
    xb, qb = x.reshape(4, K // 32, 32), xq.reshape(4, K // 32, 32).astype(np.int32)
    amax = np.abs(xb).max(axis=2)
    assert np.array_equal(xd, (amax / np.float32(127.0)).astype(np.float32))
    assert np.all(np.abs(qb).max(axis=2)[amax > 0] == 127)
    assert np.all(qb[0, 0] == 0) and xd[0, 0] == 0.0
    assert np.all(qb[1, 1] == 127)
    assert np.all(np.abs(xb - qb * xd[:, :, None]) <= xd[:, :, None] * 0.5000001 + 1e-12)
    assert np.array_equal(xs.reshape(4, K // 32, 2).astype(np.int32),
                          np.stack([qb[:, :, :16].sum(2), qb[:, :, 16:].sum(2)], axis=2))
    # elementwise definition, rint = ties to even (kernels.rs:86-88)
    inv = np.where(xd > 0, np.float32(1.0) / np.where(xd > 0, xd, 1), 0).astype(np.float32)
    want = np.clip(np.rint((xb * inv[:, :, None]).astype(np.float32)), -127, 127).astype(np.int8)
    assert np.array_equal(xq.reshape(4, K // 32, 32), want)
    # a value that lands exactly on .5 rounds to even, not away (unlike ggml_quant.rs:203)
    x2 = np.zeros((1, 32), np.float32)
    x2[0, 0], x2[0, 1] = 127.0, 2.5
    assert orc.actquant(x2, 32)[0][0, 1] == 2


# ---------------------------------------------------------------- integer block dots

@pytest.mark.parametrize("ty", [Q4_0, Q8_0])
def test_block_dots_brute_force(orc, synth, ty):
    N, K = 6, 192
    raw = synth.make_weight(ty, N, K, seed=21)
    x = synth.make_acts(1, K, seed=22)
    xq, xd, xs = orc.actquant(x, K)
    _, q = (np_q4_ints if ty == Q4_0 else np_q8_ints)(raw, N, K)
    xi = xq[0].astype(np.int64).reshape(K // 32, 32)
    want = np.einsum("nbk,bk->nb", q, xi)
    got = orc.block_dots(ty, raw, K, N, xq[0])
    assert np.array_equal(got.astype(np.int64), want)
    if ty == Q4_0:   # sum((q-8)x) = sum(qx) - 8 sum(x)  (kernels.rs:250)
        s32 = xs[0].astype(np.int64).reshape(-1, 2).sum(1)
        assert np.array_equal(want, np.einsum("nbk,bk->nb", q + 8, xi) - 8 * s32[None, :])


def test_block_dots_extremes(orc):
    # all-max magnitudes: |isum| = 32*127*127 for Q8_0, 32*8*127 for Q4_0 (q=0 -> -8)
    K = 32
    x = np.full((1, K), 5.0, np.float32)
    xq, _, _ = orc.actquant(x, K)
    assert np.all(xq == 127)
    raw8 = np.array([0, 0x3c] + [0x81] * 32, np.uint8)     # d = 1.0, q = -127
    assert orc.block_dots(Q8_0, raw8, K, 1, xq[0])[0, 0] == -32 * 127 * 127
    raw4 = np.array([0, 0x3c] + [0x00] * 16, np.uint8)
    assert orc.block_dots(Q4_0, raw4, K, 1, xq[0])[0, 0] == -8 * 32 * 127


def test_q6k_block_dots_via_pinned_dequant(orc, synth):
    """With d = 1 and every sub-scale 1 the (reference-pinned) dequantiser returns q-32 itself."""
    N, K = 3, 512
    raw = synth.make_q6_k(N, K, seed=31).reshape(-1, 210).copy()
    raw[:, 192:208] = 1
    raw[:, 208:210] = [0x00, 0x3c]
    raw = raw.reshape(-1)
    qi = orc.dequantize(Q6_K, raw, N * K).reshape(N, K).astype(np.int64)
    assert qi.min() >= -32 and qi.max() <= 31
    x = synth.make_acts(1, K, seed=32)
    xq, _, _ = orc.actquant(x, K)
    want = (qi * xq[0].astype(np.int64)[None, :]).reshape(N, K // 16, 16).sum(2)
    assert np.array_equal(orc.block_dots(Q6_K, raw, K, N, xq[0]).astype(np.int64), want)


# ---------------------------------------------------------------- fp32 combine

@pytest.mark.parametrize("ty,K", [(Q4_0, 2560), (Q8_0, 2560), (Q6_K, 2560 + 256 * 2)])
def test_q8_matmul_against_float64(orc, synth, ty, K):
    """Exact value of the quantised product: sum over elements of w_dequant * (xq * xd), in float64."""
    N, m = 12, 3
    raw = synth.make_weight(ty, N, K, seed=41)
    x = synth.make_acts(m, K, seed=42)
    xq, xd, _ = orc.actquant(x, K)
    wd = orc.dequantize(ty, raw, N * K).reshape(N, K).astype(np.float64)
    xdeq = xq.astype(np.float64) * np.repeat(xd.astype(np.float64), 32, axis=1)
    want = xdeq @ wd.T
    got = orc.matmul_q8(ty, raw, K, N, xq, xd)
    assert np.abs(got - want).max() / np.abs(want).max() < 2e-6
    # and it sits within activation-rounding distance of the f32 oracle
    f32 = orc.matmul_f32(ty, raw, K, N, x, 1)
    assert np.abs(got - f32).max() / np.abs(f32).max() < 3e-2


def test_q8_matmul_block_order_is_sequential(orc, synth):
    """acc += (dw*dx)*float(isum), b ascending: replay in numpy float32."""
    N, K = 4, 320
    raw = synth.make_weight(Q8_0, N, K, seed=51)
    x = synth.make_acts(1, K, seed=52)
    xq, xd, _ = orc.actquant(x, K)
    d, _ = np_q8_ints(raw, N, K)
    isum = orc.block_dots(Q8_0, raw, K, N, xq[0])
    acc = np.zeros(N, np.float32)
    for b in range(K // 32):
        acc = (acc + (d[:, b].astype(np.float32) * xd[0, b]) * isum[:, b].astype(np.float32)).astype(np.float32)
    assert np.array_equal(orc.matmul_q8(Q8_0, raw, K, N, xq, xd)[0], acc)


def test_gemm_rows_equal_gemv(orc, synth):
    # mellum.rs:239-243: a batch row is bit-identical to the single-token result
    raw = synth.make_weight(Q4_0, 10, 256, seed=61)
    xs = synth.make_acts(4, 256, seed=62)
    full = orc.matmul_q8_from_f32(Q4_0, raw, 256, 10, xs)
    for t in range(4):
        assert np.array_equal(full[t], orc.matmul_q8_from_f32(Q4_0, raw, 256, 10, xs[t])[0])


# ---------------------------------------------------------------- GGUF-side quantisers

def test_cpu_quantisers_roundtrip(orc, synth):
    x = synth.make_acts(1, 256, seed=71)[0]
    r8 = orc.quantize_q8_0(x)
    y8 = orc.dequantize(Q8_0, r8, 256)
    assert np.abs(y8 - x).max() <= np.abs(x).max() / 127 * 0.51 + 1e-3
    r4 = orc.quantize_q4_0(x)
    y4 = orc.dequantize(Q4_0, r4, 256)
    assert np.abs(y4 - x).max() <= np.abs(x).max() / 8 * 1.01
    # ggml_quant.rs:203 rounds ties away from zero
    t = np.zeros(32, np.float32)
    t[0], t[1] = 127.0, 2.5
    assert orc.quantize_q8_0(t).view(np.int8)[2 + 1] == 3


# ---------------------------------------------------------------- MoE

def test_expf_and_silu_accuracy(orc):
    xs = np.linspace(-30, 30, 4001, dtype=np.float32)
    got = np.array([orc.expf(float(v)) for v in xs], np.float64)
    want = np.exp(xs.astype(np.float64))
    assert np.abs(got / want - 1).max() < 3e-7
    assert orc.silu(0.0) == 0.0
    g = np.array([orc.silu(float(v)) for v in xs], np.float64)
    assert np.abs(g - xs / (1 + np.exp(-xs.astype(np.float64)))).max() < 3e-6


def test_activation_producers_known_values(orc):
    """The reference's own literal checks: ops.rs:204-232 (rmsnorm), 260-276 (silu, swiglu), 287-294 (gelu_tanh)."""
    out = orc.act_produce(orc.ACT_RMSNORM, [1.0, 2.0, 3.0, 4.0], [1.0] * 4, 0.0)
    assert abs(out[0] - 0.365148) <= 1e-5 and abs(out[3] - 1.460593) <= 1e-5
    out = orc.act_produce(orc.ACT_RMSNORM, [2.0, 2.0], [3.0, 0.5], 0.0)
    assert abs(out[0] - 3.0) <= 1e-6 and abs(out[1] - 0.5) <= 1e-6
    assert np.array_equal(orc.act_produce(orc.ACT_RMSNORM, [2.0, 2.0], None, 0.0), np.ones(2, np.float32))
    assert abs(orc.silu(1.0) - 0.731059) <= 1e-5 and abs(orc.silu(20.0) - 20.0) <= 1e-3
    out = orc.act_produce(orc.ACT_SILU_MUL, [0.0, 1.0], [5.0, 2.0])
    assert abs(out[0]) <= 1e-6 and abs(out[1] - 0.731059 * 2.0) <= 1e-5
    assert abs(orc.gelu_tanh(0.0)) <= 1e-7 and abs(orc.gelu_tanh(1.0) - 0.8412) <= 1e-3
    assert abs(orc.gelu_tanh(10.0) - 10.0) <= 1e-3 and abs(orc.gelu_tanh(-10.0)) < 1e-3
    out = orc.act_produce(orc.ACT_GEGLU, [1.0, -10.0], [2.0, 3.0])
    assert abs(out[0] - 2 * 0.8412) <= 2e-3 and abs(out[1]) < 3e-3


def test_activation_producers_against_float64(orc):
    """What the literals leave open: the whole range against numpy float64 formulas, and rmsnorm's
    independence of the summation order (the double-precision mean is rounded once)."""
    rng = np.random.default_rng(3)
    g = np.concatenate([rng.normal(0, 3, 4000), np.linspace(-30, 30, 601), [88.0, -88.0, 1e-8, -1e-8]]).astype(np.float32)
    u = rng.normal(0, 1, g.size).astype(np.float32)
    g64, u64 = g.astype(np.float64), u.astype(np.float64)
    ref_gelu = 0.5 * g64 * (1 + np.tanh(np.float64(np.float32(0.7978845608)) * (g64 + 0.044715 * g64 ** 3)))
    got = orc.act_produce(orc.ACT_GEGLU, g, u).astype(np.float64)
    assert np.max(np.abs(got - ref_gelu * u64) / (1 + np.abs(ref_gelu * u64))) <= 2e-6
    got = orc.act_produce(orc.ACT_SILU_MUL, g, u).astype(np.float64)
    ref = g64 / (1 + np.exp(-g64)) * u64
    assert np.max(np.abs(got - ref) / (1 + np.abs(ref))) <= 1e-6
    x = rng.normal(0, 2, 2560).astype(np.float32)
    w = rng.normal(1, 0.1, 2560).astype(np.float32)
    for eps in (0.0, 1e-6, 1e-5):
        got = orc.act_produce(orc.ACT_RMSNORM, x, w, eps)
        scale = np.float32(1.0 / np.sqrt(np.mean(x.astype(np.float64) ** 2) + np.float64(np.float32(eps))))
        assert np.array_equal(got, (x * scale) * w)
        perm = rng.permutation(x.size)   # summing the squares in another order changes nothing
        assert np.array_equal(orc.act_produce(orc.ACT_RMSNORM, x[perm], w[perm], eps), got[perm])
    assert np.array_equal(orc.act_produce(orc.ACT_NONE, x), x)


def test_route_topk_ties_lowest_index(orc):
    ids, w = orc.route_topk(np.array([0.5, 2.0, 2.0, -1.0, 2.0], np.float32), 2)
    assert list(ids) == [1, 2] and abs(w.sum() - 1) < 1e-6 and abs(w[0] - 0.5) < 1e-6
    logits = np.random.default_rng(3).standard_normal(64).astype(np.float32)
    ids, w = orc.route_topk(logits, 8)
    assert list(ids) == list(np.argsort(-logits, kind="stable")[:8])
    p = np.exp(logits - logits.max())
    p /= p.sum()
    assert np.allclose(w, p[ids] / p[ids].sum(), rtol=1e-5)


@pytest.mark.parametrize("TY", [Q8_0, Q6_K])
def test_moe_ffn_equals_sum_of_dense_experts(orc, synth, TY):
    """mellum.rs:1623-1669: y = sum_k w_k * down_k(silu(gate_k x) * up_k x), routed order; Q8_0 and
    Q6_K expert tensors (decode.rs:2717-2831)."""
    ne, hidden, eff, k = (6, 128, 64, 3) if TY == Q8_0 else (5, 256, 512, 3)
    gate, up, down = (synth.make_moe_q8 if TY == Q8_0 else synth.make_moe_q6)(ne, hidden, eff, seed=81)
    ids, w = synth.zipf_routing(1, ne, k, seed=82)
    x = synth.make_acts(1, hidden, seed=83)[0]
    y, gu, aq, ad = orc.moe_ffn_q8(gate, up, down, hidden, eff, ne, ids[0], w[0], x, ty=TY)
    be, bb = (32, 34) if TY == Q8_0 else (256, 210)
    geb, deb = (hidden // be) * bb * eff, (eff // be) * bb * hidden
    acc = np.zeros(hidden, np.float32)
    for kk, e in enumerate(ids[0]):
        g = orc.matmul_q8_from_f32(TY, gate[e * geb:(e + 1) * geb], hidden, eff, x)[0]
        u = orc.matmul_q8_from_f32(TY, up[e * geb:(e + 1) * geb], hidden, eff, x)[0]
        assert np.array_equal(gu[kk, 0], g) and np.array_equal(gu[kk, 1], u)
        a = np.array([orc.silu(float(a_)) for a_ in g], np.float32) * u
        dy = orc.matmul_q8_from_f32(TY, down[e * deb:(e + 1) * deb], eff, hidden, a)[0]
        acc = (acc + w[0][kk] * dy).astype(np.float32)
    assert np.array_equal(y, acc)
    # against the f32 path end to end: only quantisation noise
    accf = np.zeros(hidden, np.float64)
    for kk, e in enumerate(ids[0]):
        g = orc.matmul_f32(TY, gate[e * geb:(e + 1) * geb], hidden, eff, x, 1)[0].astype(np.float64)
        u = orc.matmul_f32(TY, up[e * geb:(e + 1) * geb], hidden, eff, x, 1)[0].astype(np.float64)
        a = (g / (1 + np.exp(-g)) * u).astype(np.float32)
        accf += w[0][kk] * orc.matmul_f32(TY, down[e * deb:(e + 1) * deb], eff, hidden, a, 1)[0]
    assert np.abs(y - accf).max() / np.abs(accf).max() < 5e-2


def q4_0_literal_blocks():
    """Two Q4_0 blocks worked out by hand from ggml_quant.rs:212-237 (d = vmax / -8 with vmax the signed
    value of largest magnitude, q = clamp(trunc(x / d + 8.5), 0, 15), byte j = q[j] | q[j + 16] << 4).
    A: vmax = +8 -> d = -1 (f16 0xBC00): 8 -> 0, -4 -> 12, 1 -> 7, 0.4 -> 8, 0 -> 8, 3 -> 5, -7 -> 15, 7.9 -> 0.
    B: vmax = -4 -> d = +0.5 (f16 0x3800): -4 -> 0, 2 -> 12, -1 -> 6, 3.9 -> 16 clamped to 15, 0.26 -> 9, -0.24 -> 8."""
    a = np.zeros(32, np.float32)
    a[[0, 1, 2, 3, 16, 17, 31]] = [8.0, -4.0, 1.0, 0.4, 3.0, -7.0, 7.9]
    a_bytes = bytes([0x00, 0xBC, 0x50, 0xFC, 0x87, 0x88] + [0x88] * 11 + [0x08])
    b = np.zeros(32, np.float32)
    b[[5, 0, 1, 2, 20, 21]] = [-4.0, 2.0, -1.0, 3.9, 0.26, -0.24]
    b_bytes = bytes([0x00, 0x38, 0x8C, 0x86, 0x8F, 0x88, 0x98, 0x80] + [0x88] * 10)
    return (a, a_bytes), (b, b_bytes)


def test_quantize_q4_0_literal_blocks(orc):
    """Pins the sign convention (the value of largest magnitude maps to nibble 0, the scale takes its
    negated sign) and the +8.5 truncation, which a round-trip bound cannot tell from their mirror images."""
    for x, want in q4_0_literal_blocks():
        got = orc.quantize_q4_0(x)
        assert bytes(got) == want, (bytes(got).hex(), want.hex())
    both = np.concatenate([q4_0_literal_blocks()[0][0], q4_0_literal_blocks()[1][0]])
    assert bytes(orc.quantize_q4_0(both)) == q4_0_literal_blocks()[0][1] + q4_0_literal_blocks()[1][1]
    # the decoded values land where the encoding says: (q - 8) * d
    y = orc.dequantize(Q4_0, np.frombuffer(q4_0_literal_blocks()[0][1], np.uint8), 32)
    assert y[0] == 8.0 and y[1] == -4.0 and y[17] == -7.0 and y[31] == 8.0
