"""ctypes/numpy wrapper around libstrix_oracle.so (the CPU oracle).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
CPU-baseline leg of the benchmark.  The product package never imports it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libstrix_oracle.so")

Q4_0, Q8_0, Q6_K = 2, 8, 14
BLOCK_ELEMS = {Q4_0: 32, Q8_0: 32, Q6_K: 256}
BLOCK_BYTES = {Q4_0: 18, Q8_0: 34, Q6_K: 210}


def build(force=False):
    """Compile the oracle with gcc (strict IEEE, no FMA contraction)."""
    srcs = [os.path.join(_HERE, f) for f in ("strix_oracle.c", "strix_oracle.h", "Makefile")]
    stale = not os.path.exists(_LIB_PATH) or any(os.path.getmtime(f) > os.path.getmtime(_LIB_PATH) for f in srcs)
    if force or stale:
        subprocess.check_call(["make", "-C", _HERE, "-B", "libstrix_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        vp, i, sz = C.c_void_p, C.c_int, C.c_size_t
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [C.c_float]
        L.orc_dequantize.argtypes = [i, vp, sz, vp, sz]
        L.orc_quantize_q8_0.argtypes = [vp, sz, vp]
        L.orc_quantize_q4_0.argtypes = [vp, sz, vp]
        L.orc_matmul_f32.argtypes = [i, vp, i, i, vp, i, vp, i, i]
        L.orc_actquant.argtypes = [vp, i, i, vp, vp, vp]
        L.orc_block_dots.argtypes = [i, vp, i, i, vp, vp]
        L.orc_matmul_q8.argtypes = [i, vp, i, i, vp, vp, i, vp, i]
        L.orc_expf.restype = C.c_float
        L.orc_expf.argtypes = [C.c_float]
        L.orc_silu.restype = C.c_float
        L.orc_silu.argtypes = [C.c_float]
        L.orc_gelu_tanh.restype = C.c_float
        L.orc_gelu_tanh.argtypes = [C.c_float]
        L.orc_tanhf.restype = C.c_float
        L.orc_tanhf.argtypes = [C.c_float]
        L.orc_act_produce.argtypes = [i, vp, vp, i, C.c_float, vp]
        L.orc_moe_ffn_q8.argtypes = [vp, vp, vp, i, i, i, vp, vp, i, vp, vp, vp, vp, vp, vp, vp]
        L.orc_moe_ffn.argtypes = [i, vp, vp, vp, i, i, i, vp, vp, i, vp, vp, vp, vp, vp, vp, vp]
        L.orc_route_topk.argtypes = [vp, i, i, vp, vp]
        L.orc_lcg_fill.argtypes = [vp, vp, sz]
        _lib = L
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


def f16_to_f32(h):
    return float(lib().orc_f16_to_f32(int(h)))


def f32_to_f16(f):
    return int(lib().orc_f32_to_f16(float(f)))


def dequantize(ty, raw, n):
    raw = _c(raw, np.uint8)
    out = np.empty(n, np.float32)
    rc = lib().orc_dequantize(ty, _p(raw), raw.size, _p(out), n)
    if rc != 0:
        raise ValueError("dequantize: bad element count or too few bytes")
    return out


def quantize_q8_0(x):
    x = _c(x, np.float32)
    out = np.empty(x.size // 32 * 34, np.uint8)
    lib().orc_quantize_q8_0(_p(x), x.size, _p(out))
    return out


def quantize_q4_0(x):
    x = _c(x, np.float32)
    out = np.empty(x.size // 32 * 18, np.uint8)
    lib().orc_quantize_q4_0(_p(x), x.size, _p(out))
    return out


def matmul_f32(ty, raw, K, N, x, order=0, nthreads=None):
    """f32 oracle: y[m][N] = dequant(W) . x, reference summation order 0|1."""
    raw = _c(raw, np.uint8)
    x = _c(x, np.float32).reshape(-1, K)
    y = np.empty((x.shape[0], N), np.float32)
    rc = lib().orc_matmul_f32(ty, _p(raw), K, N, _p(x), x.shape[0], _p(y), order,
                              nthreads or os.cpu_count())
    if rc != 0:
        raise ValueError("matmul_f32 failed")
    return y


def actquant(x, K):
    """Device activation quantiser: returns (xq[m][K] i8, xd[m][K/32] f32, xs16[m][K/16] i16)."""
    x = _c(x, np.float32).reshape(-1, K)
    m = x.shape[0]
    xq = np.empty((m, K), np.int8)
    xd = np.empty((m, K // 32), np.float32)
    xs = np.empty((m, K // 16), np.int16)
    lib().orc_actquant(_p(x), m, K, _p(xq), _p(xd), _p(xs))
    return xq, xd, xs


def block_dots(ty, raw, K, N, xq_row):
    """Exact i32 block dots of one quantised row: [N][K/32] (Q6_K: [N][K/16])."""
    raw = _c(raw, np.uint8)
    xq_row = _c(xq_row, np.int8).reshape(K)
    per = K // 16 if ty == Q6_K else K // 32
    out = np.empty((N, per), np.int32)
    rc = lib().orc_block_dots(ty, _p(raw), K, N, _p(xq_row), _p(out))
    if rc != 0:
        raise ValueError("block_dots failed")
    return out


def matmul_q8(ty, raw, K, N, xq, xd, nthreads=None):
    """Q8 oracle: integer block dots + fp32 combine in ascending block order."""
    raw = _c(raw, np.uint8)
    xq = _c(xq, np.int8).reshape(-1, K)
    xd = _c(xd, np.float32).reshape(-1, K // 32)
    y = np.empty((xq.shape[0], N), np.float32)
    rc = lib().orc_matmul_q8(ty, _p(raw), K, N, _p(xq), _p(xd), xq.shape[0], _p(y),
                             nthreads or os.cpu_count())
    if rc != 0:
        raise ValueError("matmul_q8 failed")
    return y


def matmul_q8_from_f32(ty, raw, K, N, x, nthreads=None):
    xq, xd, _ = actquant(x, K)
    return matmul_q8(ty, raw, K, N, xq, xd, nthreads)


def expf(x):
    return float(lib().orc_expf(float(x)))


def silu(x):
    return float(lib().orc_silu(float(x)))


def gelu_tanh(x):
    return float(lib().orc_gelu_tanh(float(x)))


ACT_NONE, ACT_RMSNORM, ACT_SILU_MUL, ACT_GEGLU = 0, 1, 2, 3


def act_produce(act, a, b=None, eps=0.0):
    """The fp32 activation a GEMV's quantiser sees: rmsnorm(a)*b, silu(a)*b or gelu_tanh(a)*b."""
    a = _c(a, np.float32)
    if b is not None:
        b = _c(b, np.float32)
    out = np.empty_like(a)
    rc = lib().orc_act_produce(int(act), _p(a), _p(b), a.size, float(eps), _p(out))
    if rc != 0:
        raise ValueError("act_produce failed")
    return out


def moe_ffn_q8(gate, up, down, hidden, eff, ne, ids, wexp, x, aq_in=None, ad_in=None, ty=Q8_0):
    """Returns (y[hidden], gu[k][2][eff], aq[k][eff], ad[k][eff/32]).  ty: Q8_0 or Q6_K expert tensors."""
    gate, up, down = _c(gate, np.uint8), _c(up, np.uint8), _c(down, np.uint8)
    ids = _c(ids, np.int32)
    wexp = _c(wexp, np.float32)
    x = _c(x, np.float32)
    k = ids.size
    y = np.empty(hidden, np.float32)
    gu = np.empty((k, 2, eff), np.float32)
    aq = np.empty((k, eff), np.int8)
    ad = np.empty((k, eff // 32), np.float32)
    if aq_in is not None:
        aq_in, ad_in = _c(aq_in, np.int8), _c(ad_in, np.float32)
    rc = lib().orc_moe_ffn(ty, _p(gate), _p(up), _p(down), hidden, eff, ne, _p(ids), _p(wexp), k,
                           _p(x), _p(y), _p(gu), _p(aq), _p(ad), _p(aq_in), _p(ad_in))
    if rc != 0:
        raise ValueError("moe_ffn_q8 failed")
    return y, gu, aq, ad


def route_topk(logits, k):
    logits = _c(logits, np.float32)
    ids = np.empty(k, np.int32)
    w = np.empty(k, np.float32)
    lib().orc_route_topk(_p(logits), logits.size, k, _p(ids), _p(w))
    return ids, w


def lcg(seed, n):
    """n draws of the reference tests' LCG; returns (u32 array, new seed)."""
    s = C.c_uint64(seed)
    out = np.empty(n, np.uint32)
    lib().orc_lcg_fill(C.byref(s), _p(out), n)
    return out, s.value
