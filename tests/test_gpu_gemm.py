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


def test_gemm_declines_and_errors(accel, synth, pkg):
    assert accel.prefill_q8_gemm("t.absent", np.zeros((2, 64), np.float32), 2, 8) is None
    raw = synth.make_weight(8, 8, 256, seed=1)
    assert accel.upload_q8_0("t.e", raw, 256, 8)
    with pytest.raises(pkg.SmxError):   # wrong activation length
        accel.prefill_q8_gemm("t.e", np.zeros((16, 128), np.float32), 16, 8)
