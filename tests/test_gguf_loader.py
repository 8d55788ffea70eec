"""GGUF loader (host side of the upload pipeline): parsing, error handling and the host quantisers,
checked against the reference's own fixture (crates/strix-models/src/gguf.rs:381-452) and the oracle."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import gguf_writer as gw  # noqa: E402


def test_reference_fixture_metadata_and_f16_tensor(pkg, tmp_path):
    """gguf.rs:381-441: architecture "test", test.block_count = 7, one F16 tensor [1.5, -0.5]."""
    f16 = np.array([1.5, -0.5], np.float16).view(np.uint8)
    p = gw.write_gguf(tmp_path / "a.gguf", [("general.architecture", gw.T_STR, "test"), ("test.block_count", gw.T_U32, 7)],
                      [("w", 1, [2], f16)])
    g = pkg.GgufFile(p)
    assert g.meta_str("general.architecture") == "test"
    assert g.meta_u64("test.block_count") == 7 and g.meta_f32("test.block_count") == 7.0
    assert g.meta_u64("missing") is None
    with pytest.raises(TypeError):
        g.meta_u64("general.architecture")
    assert len(g) == 1
    name, ty, dims, raw = g.tensor(0)
    assert (name, ty, dims) == ("w", 1, [2])
    assert list(pkg.host_dequantize(1, raw, 2)) == [1.5, -0.5]
    assert g.find("w") == 0 and g.find("nope") is None


def test_bad_files_are_errors(pkg, tmp_path):
    """gguf.rs:443-452 (bad magic) and the parse errors of :119-176."""
    (tmp_path / "zero.gguf").write_bytes(bytes(64))
    with pytest.raises(pkg.SmxError, match="magic"):
        pkg.GgufFile(tmp_path / "zero.gguf")
    with pytest.raises(pkg.SmxError):
        pkg.GgufFile(tmp_path / "does_not_exist.gguf")
    raw = np.zeros(34, np.uint8)
    p = gw.write_gguf(tmp_path / "v9.gguf", [], [("w", 8, [32], raw)], version=9)
    with pytest.raises(pkg.SmxError, match="version"):
        pkg.GgufFile(p)
    p = gw.write_gguf(tmp_path / "ok.gguf", [("k", gw.T_STR, "v")], [("w", 8, [32], raw)])
    data = p.read_bytes()
    for cut in (10, 30, 60, len(data) - 40):     # inside the header, the metadata, the index, the data
        (tmp_path / "cut.gguf").write_bytes(data[:cut])
        with pytest.raises(pkg.SmxError):
            pkg.GgufFile(tmp_path / "cut.gguf")
    p = gw.write_gguf(tmp_path / "ty.gguf", [], [("w", 99, [32], raw)])
    with pytest.raises(pkg.SmxError, match="encoding"):
        pkg.GgufFile(p)


def test_all_metadata_kinds_alignment_and_v2(pkg, synth, tmp_path):
    meta = [("a.u8", gw.T_U8, 200), ("a.i8", gw.T_I8, -3), ("a.u16", gw.T_U16, 65535), ("a.i16", gw.T_I16, 12),
            ("a.i32", gw.T_I32, -70000), ("a.f32", gw.T_F32, 1e-6), ("a.bool", gw.T_BOOL, 1), ("a.u64", gw.T_U64, 1 << 40),
            ("a.i64", gw.T_I64, 5), ("a.f64", gw.T_F64, 0.25), ("a.arr", gw.T_ARR, (gw.T_U32, [1, 2, 3])),
            ("tok.list", gw.T_ARR, (gw.T_STR, ["<s>", "</s>", "hello"]))]
    q4, q6 = synth.make_weight(2, 8, 64, seed=1), synth.make_weight(14, 4, 256, seed=2)
    for version, alignment in ((3, None), (3, 64), (2, 256)):
        p = gw.write_gguf(tmp_path / f"m{version}_{alignment}.gguf", meta, [("blk.0.attn_q.weight", 2, [64, 8], q4),
                                                                              ("output.weight", 14, [256, 4], q6)],
                          version=version, alignment=alignment)
        g = pkg.GgufFile(p)
        assert g.meta_u64("a.u8") == 200 and g.meta_u64("a.u16") == 65535 and g.meta_u64("a.u64") == 1 << 40
        assert g.meta_u64("a.i16") == 12 and g.meta_u64("a.i64") == 5
        for neg in ("a.i8", "a.i32"):                 # as_u64 refuses negative values (gguf.rs:43-56)
            with pytest.raises(TypeError):
                g.meta_u64(neg)
        assert abs(g.meta_f32("a.f32") - 1e-6) < 1e-12 and g.meta_f32("a.f64") == 0.25 and g.meta_f32("a.u8") == 200.0
        with pytest.raises(TypeError):
            g.meta_str("a.u8")
        t = g.tensors()
        assert t["blk.0.attn_q.weight"][1:3] == (2, [64, 8]) and np.array_equal(t["blk.0.attn_q.weight"][3], q4)
        assert t["output.weight"][1:3] == (14, [256, 4]) and np.array_equal(t["output.weight"][3], q6)


def test_host_quantisers_match_the_oracle(pkg, orc, synth):
    """quantize_q8_0 / quantize_q4_0 (ggml_quant.rs:193-237) and the dequantisers: bit for bit the oracle's,
    which is pinned to the reference's literal blocks."""
    rng = np.random.default_rng(5)
    x = np.concatenate([rng.normal(0, 1, 32 * 50), np.zeros(32), rng.normal(0, 1e-6, 32), [0.5, -0.5] * 16,
                        rng.normal(0, 300, 64)]).astype(np.float32)
    assert np.array_equal(pkg.host_quantize_q8_0(x), orc.quantize_q8_0(x))
    assert np.array_equal(pkg.host_quantize_q4_0(x), orc.quantize_q4_0(x))
    # and against blocks worked out by hand from ggml_quant.rs:212-237 (sign of d, +8.5 truncation, clamping)
    a = np.zeros(32, np.float32)
    a[[0, 1, 2, 3, 16, 17, 31]] = [8.0, -4.0, 1.0, 0.4, 3.0, -7.0, 7.9]
    assert bytes(pkg.host_quantize_q4_0(a)) == bytes([0x00, 0xBC, 0x50, 0xFC, 0x87, 0x88] + [0x88] * 11 + [0x08])
    b = np.zeros(32, np.float32)
    b[[5, 0, 1, 2, 20, 21]] = [-4.0, 2.0, -1.0, 3.9, 0.26, -0.24]
    assert bytes(pkg.host_quantize_q4_0(b)) == bytes([0x00, 0x38, 0x8C, 0x86, 0x8F, 0x88, 0x98, 0x80] + [0x88] * 10)
    for ty, n_rows, K in ((2, 16, 256), (8, 16, 256), (14, 8, 512)):
        raw = synth.make_weight(ty, n_rows, K, seed=ty)
        assert np.array_equal(pkg.host_dequantize(ty, raw, n_rows * K), orc.dequantize(ty, raw, n_rows * K))
    # every f16 bit pattern converts exactly; every finite f16 survives f32 -> f16 through the Q8_0 scale
    h = np.arange(65536, dtype=np.uint16)
    f = pkg.host_dequantize(1, h.view(np.uint8), 65536)
    assert np.array_equal(f.view(np.uint32), h.view(np.float16).astype(np.float32).view(np.uint32))
    # the encodings that only feed the requantisers (Q4_1, Q5_0, Q5_1, Q4_K, Q5_K), random bytes with sane scales
    for ty, be, bb in ((3, 32, 20), (6, 32, 22), (7, 32, 24), (12, 256, 144), (13, 256, 176)):
        raw = rng.integers(0, 256, (64, bb), dtype=np.uint8)
        raw[:, 0:2] = rng.uniform(-0.1, 0.1, (64, 1)).astype(np.float16).view(np.uint8)
        if ty != 6:
            raw[:, 2:4] = rng.uniform(-0.1, 0.1, (64, 1)).astype(np.float16).view(np.uint8)
        got, want = pkg.host_dequantize(ty, raw, 64 * be), orc.dequantize(ty, raw, 64 * be)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), ty
    with pytest.raises(ValueError):
        pkg.host_dequantize(10, np.zeros(84, np.uint8), 256)    # Q2_K has no dequantiser (ggml_quant.rs:517-521)
    with pytest.raises(ValueError):
        pkg.host_quantize_q8_0(np.zeros(33, np.float32))


def test_f32_to_f16_rounding_through_q8_scale(pkg):
    """The block scale written by quantize_q8_0 is f16(amax/127): compare with numpy's IEEE conversion over
    magnitudes that hit normals, subnormals, ties, overflow and underflow."""
    rng = np.random.default_rng(6)
    mags = np.concatenate([10.0 ** rng.uniform(-9, 7, 4000), [65504 * 127, 65520 * 127, 6e-8 * 127, 2.98e-8 * 127, 0.0],
                           (np.arange(1, 2049, dtype=np.float64) + 0.5) * 2.0 ** -24 * 127]).astype(np.float32)
    x = np.zeros((mags.size, 32), np.float32)
    x[:, 0] = mags
    got = pkg.host_quantize_q8_0(x).reshape(-1, 34)[:, :2].copy().view(np.uint16).reshape(-1)
    with np.errstate(over="ignore"):
        want = (mags / np.float32(127.0)).astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)


@pytest.mark.gpu
def test_attach_uploads_matrices_and_expert_layers(accel, pkg, orc, synth, relerr, tmp_path):
    """attach_accel (mellum.rs:460-535): served matrices under their GGUF names, expert triples by layer;
    F32 norms, 1-D tensors and unserved encodings stay with the caller."""
    H, F, NE, EFF = 256, 512, 4, 256
    q = synth.make_weight(2, F, H, seed=1)
    o = synth.make_weight(14, 96, H, seed=2)
    d8 = synth.make_weight(8, H, F, seed=3)
    g8, u8, dn8 = synth.make_moe_q8(NE, H, EFF, seed=4)
    g6, u6, dn6 = synth.make_moe_q6(NE, H, EFF, seed=5)
    tensors = [
        ("token_embd.weight", 12, [H, 8], np.zeros(8 * H // 256 * 144, np.uint8)),   # Q4_K: not served
        ("blk.0.attn_norm.weight", 0, [H], np.ones(H, np.float32).view(np.uint8)),   # 1-D F32
        ("blk.0.ffn_up.weight", 2, [H, F], q),
        ("blk.0.ffn_down.weight", 8, [F, H], d8),
        ("output.weight", 14, [H, 96], o),
        ("blk.0.ffn_gate_exps.weight", 8, [H, EFF, NE], g8), ("blk.0.ffn_up_exps.weight", 8, [H, EFF, NE], u8),
        ("blk.0.ffn_down_exps.weight", 8, [EFF, H, NE], dn8),
        ("blk.1.ffn_gate_exps.weight", 14, [H, EFF, NE], g6), ("blk.1.ffn_up_exps.weight", 14, [H, EFF, NE], u6),
        ("blk.1.ffn_down_exps.weight", 14, [EFF, H, NE], dn6),
        ("blk.2.ffn_gate_exps.weight", 8, [H, EFF, NE], g8),                          # no siblings: skipped
    ]
    p = gw.write_gguf(tmp_path / "model.gguf", [("general.architecture", gw.T_STR, "test")], tensors)
    g = pkg.GgufFile(p)
    before = accel.resident_count()
    assert accel.attach_gguf(g) == (3, 2)
    assert accel.resident_count() >= before + 3
    g.close()                                   # uploads are copies: the mapping may go away
    x = synth.make_acts(1, H, seed=7)[0]
    assert relerr(accel.gemv("blk.0.ffn_up.weight", x, F), orc.matmul_q8_from_f32(2, q, H, F, x)[0]) <= 1e-5
    assert relerr(accel.gemv("output.weight", x, 96), orc.matmul_q8_from_f32(14, o, H, 96, x)[0]) <= 1e-5
    xf = synth.make_acts(1, F, seed=8)[0]
    assert relerr(accel.gemv("blk.0.ffn_down.weight", xf, H), orc.matmul_q8_from_f32(8, d8, F, H, xf)[0]) <= 1e-5
    assert accel.gemv("token_embd.weight", x, 8) is None
    ids, w = synth.zipf_routing(1, NE, 2, seed=9)
    y8, _, aq, ad = accel.moe_ffn_stages(0, ids[0], w[0], x, EFF)
    assert relerr(y8, orc.moe_ffn_q8(g8, u8, dn8, H, EFF, NE, ids[0], w[0], x, aq_in=aq, ad_in=ad)[0]) <= 1e-5
    y6, _, aq, ad = accel.moe_ffn_stages(1, ids[0], w[0], x, EFF)
    assert relerr(y6, orc.moe_ffn_q8(g6, u6, dn6, H, EFF, NE, ids[0], w[0], x, aq_in=aq, ad_in=ad, ty=14)[0]) <= 1e-5
    assert accel.moe_ffn(2, ids[0], w[0], x) is None
    # a tensor that is not in a served format: dequantise + requantise on the host, then upload (gemma3n.rs:464)
    f = pkg.host_dequantize(14, o, 96 * H)
    assert accel.upload_q8_0("output.q8", pkg.host_quantize_q8_0(f), H, 96)
    assert relerr(accel.gemv("output.q8", x, 96), orc.matmul_q8_from_f32(8, orc.quantize_q8_0(f), H, 96, x)[0]) <= 1e-5


@pytest.mark.gpu
def test_upload_as_requantises_unserved_encodings(accel, pkg, orc, synth, relerr, tmp_path):
    """gemma3n.rs:455-470 (Q4_K token_embd -> Q8_0 lm_head) and qwen35.rs:741-760 (Q8_0 -> Q4_0) in one call."""
    H, V = 512, 300
    rng = np.random.default_rng(3)
    k4 = rng.integers(0, 256, (V * H // 256, 144), dtype=np.uint8)
    k4[:, 0:2] = rng.uniform(0.001, 0.02, (k4.shape[0], 1)).astype(np.float16).view(np.uint8)
    k4[:, 2:4] = rng.uniform(0.001, 0.02, (k4.shape[0], 1)).astype(np.float16).view(np.uint8)
    k4 = k4.reshape(-1)
    d8 = synth.make_weight(8, 64, H, seed=3)
    p = gw.write_gguf(tmp_path / "m.gguf", [], [("token_embd.weight", 12, [H, V], k4), ("blk.0.attn_q.weight", 8, [H, 64], d8),
                                                 ("blk.0.attn_norm.weight", 0, [H], np.ones(H, np.float32).view(np.uint8))])
    g = pkg.GgufFile(p)
    x = synth.make_acts(1, H, seed=4)[0]
    assert accel.upload_as(g, "token_embd.weight", 8, key="lm_head.q8")
    want8 = orc.quantize_q8_0(orc.dequantize(12, k4, V * H))
    assert relerr(accel.gemv("lm_head.q8", x, V), orc.matmul_q8_from_f32(8, want8, H, V, x)[0]) <= 1e-5
    assert accel.upload_as(g, "blk.0.attn_q.weight", 2)                 # under its own name, lighter
    want4 = orc.quantize_q4_0(orc.dequantize(8, d8, 64 * H))
    assert relerr(accel.gemv("blk.0.attn_q.weight", x, 64), orc.matmul_q8_from_f32(2, want4, H, 64, x)[0]) <= 1e-5
    assert accel.upload_as(g, "blk.0.attn_q.weight", 8, key="q.same")   # already in the target encoding: plain upload
    assert relerr(accel.gemv("q.same", x, 64), orc.matmul_q8_from_f32(8, d8, H, 64, x)[0]) <= 1e-5
    assert accel.upload_as(g, "no.such.tensor", 8) is False
    with pytest.raises(pkg.SmxError):
        accel.upload_as(g, "blk.0.attn_norm.weight", 8)                 # not a matrix
    with pytest.raises(pkg.SmxError):
        accel.upload_as(g, "token_embd.weight", 14)                     # no host quantiser for Q6_K
    g.close()
