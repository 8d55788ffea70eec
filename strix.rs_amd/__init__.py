"""Python binding of libstrix_mi355.so (ctypes over the C ABI in include/strix_mi355.h).

`Mi355WeightAccel` mirrors the method names, argument meaning and decline
behaviour of the reference's `WeightAccel` trait
(crates/strix-core/src/accel.rs:147-405): `upload_*` return True/False, `gemv`
and friends return a numpy array or None when the key is not resident.  Errors
the reference would swallow into a decline (bad shapes, HIP failures) raise
`SmxError` instead, since this backend has no CPU fallback to decline to.

The directory name contains a dot, so load this package by path, e.g.
    importlib.util.spec_from_file_location("strix_rs_amd", ".../strix.rs_amd/__init__.py",
                                           submodule_search_locations=[".../strix.rs_amd"])
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libstrix_mi355.so")

SMX_OK, SMX_NOT_RESIDENT = 1, 0
GEMV_MAX_M = 8

EXPORTS = [
    "smx_create", "smx_destroy", "smx_last_error", "smx_name", "smx_resident_count",
    "smx_resident_bytes", "smx_upload_q4_0", "smx_upload_q8_0", "smx_upload_q6_k",
    "smx_upload_moe_q8", "smx_evict", "smx_gemv", "smx_gemv_rows", "smx_gemv_batch", "smx_gemm",
    "smx_lm_head_argmax_rows", "smx_moe_ffn", "smx_moe_layer", "smx_dev_alloc", "smx_dev_free",
    "smx_h2d", "smx_d2h", "smx_sync", "smx_gemv_dev", "smx_gemm_dev", "smx_moe_ffn_dev", "smx_moe_shexp_dev", "smx_gemm_fused_dev", "smx_moe_layer_ffn", "smx_moe_expert_ffn",
    "smx_prof_enable", "smx_prof_reset", "smx_prof_read", "smx_prof_names", "smx_timer_begin",
    "smx_timer_end", "smx_quantize", "smx_gemv_block_dots", "smx_gemm_block_dots",
    "smx_moe_ffn_stages", "smx_tune", "smx_graph_begin", "smx_graph_end", "smx_graph_launch",
    "smx_graph_destroy", "smx_dev_copy", "smx_gemv_batch_dev", "smx_gemv_fused_dev", "smx_gemv_fused", "smx_ffn_gate_up_dev",
    "smx_upload_moe_q6", "smx_gguf_open", "smx_gguf_close", "smx_gguf_tensor_count", "smx_gguf_tensor",
    "smx_gguf_find", "smx_gguf_meta_u64", "smx_gguf_meta_f32", "smx_gguf_meta_str", "smx_gguf_attach", "smx_gguf_upload_as",
    "smx_host_quantize_q8_0", "smx_host_quantize_q4_0", "smx_host_dequantize", "smx_moe_layer_dev",
    "smx_weight_dims", "smx_moe_layer_stages", "smx_gemv_noalloc_dev",
    "smx_gemv_f32", "smx_gemv_f32_dev", "smx_gemv_f32_batch", "smx_moe_route_dev", "smx_moe_route", "smx_moe_ffn_routed_dev", "smx_moe_router_dev", "smx_moe_ffn_logits_dev",
]
ACT_NONE, ACT_RMSNORM, ACT_SILU_MUL, ACT_GEGLU = 0, 1, 2, 3


class SmxError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"smx error {code}: {msg}")
        self.code = code


_lib = None


def load_library():
    """Load the built library; fails loudly if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FileNotFoundError(
            f"{LIB_PATH} is missing: build it with `python strix.rs_amd/build.py` "
            "(there is no CPU fallback)")
    L = C.CDLL(LIB_PATH)
    vp, sz, i, cp = C.c_void_p, C.c_size_t, C.c_int, C.c_char_p
    L.smx_create.argtypes = [i, C.POINTER(vp)]
    L.smx_destroy.argtypes = [vp]
    L.smx_destroy.restype = None
    L.smx_last_error.argtypes = [vp]
    L.smx_last_error.restype = cp
    L.smx_name.argtypes = [vp]
    L.smx_name.restype = cp
    L.smx_resident_count.argtypes = [vp]
    L.smx_resident_count.restype = sz
    L.smx_resident_bytes.argtypes = [vp]
    L.smx_resident_bytes.restype = sz
    for n in ("smx_upload_q4_0", "smx_upload_q8_0", "smx_upload_q6_k"):
        getattr(L, n).argtypes = [vp, cp, vp, sz, sz, sz]
    L.smx_upload_moe_q8.argtypes = [vp, sz, vp, sz, vp, sz, vp, sz, sz, sz, sz]
    L.smx_upload_moe_q6.argtypes = [vp, sz, vp, sz, vp, sz, vp, sz, sz, sz, sz]
    L.smx_evict.argtypes = [vp, cp]
    L.smx_gemv.argtypes = [vp, cp, vp, sz, vp, sz]
    L.smx_gemv_f32.argtypes = [vp, cp, vp, sz, vp, sz]
    L.smx_gemv_f32_dev.argtypes = [vp, cp, vp, vp]
    L.smx_gemv_rows.argtypes = [vp, cp, vp, sz, sz, vp, sz]
    L.smx_gemv_batch.argtypes = [vp, sz, vp, vp, vp, vp, vp, vp]
    L.smx_gemv_f32_batch.argtypes = [vp, sz, vp, vp, vp, vp, vp, vp]
    L.smx_gemm.argtypes = [vp, cp, vp, sz, sz, vp, sz]
    L.smx_lm_head_argmax_rows.argtypes = [vp, cp, vp, sz, sz, vp]
    L.smx_moe_ffn.argtypes = [vp, sz, vp, vp, sz, vp, sz, C.c_float, vp, sz]
    L.smx_moe_layer.argtypes = [vp, sz, vp, sz, vp, sz, vp, vp, sz, vp, sz]
    L.smx_moe_layer_dev.argtypes = [vp, sz, vp, sz, vp, sz, vp, vp, sz, vp]
    L.smx_moe_layer_stages.argtypes = [vp, sz, vp, sz, vp, sz, vp, vp, sz, vp, sz, vp, vp, vp, vp]
    L.smx_weight_dims.argtypes = [vp, cp, C.POINTER(sz), C.POINTER(sz)]
    L.smx_dev_alloc.argtypes = [vp, sz, C.POINTER(vp)]
    L.smx_dev_free.argtypes = [vp, vp]
    L.smx_h2d.argtypes = [vp, vp, vp, sz]
    L.smx_d2h.argtypes = [vp, vp, vp, sz]
    L.smx_sync.argtypes = [vp]
    L.smx_dev_copy.argtypes = [vp, vp, vp, sz]
    L.smx_gemv_dev.argtypes = [vp, cp, vp, sz, vp]
    L.smx_gemm_dev.argtypes = [vp, cp, vp, sz, vp]
    L.smx_gemv_noalloc_dev.argtypes = [vp, cp, vp, sz, vp]
    L.smx_gemv_batch_dev.argtypes = [vp, sz, vp, vp, vp]
    L.smx_gemv_fused_dev.argtypes = [vp, sz, vp, i, vp, vp, C.c_float, vp]
    L.smx_ffn_gate_up_dev.argtypes = [vp, C.c_char_p, C.c_char_p, i, vp, i, vp, C.c_float, vp]
    L.smx_gemv_fused.argtypes = [vp, cp, i, vp, vp, sz, C.c_float, vp, sz]
    L.smx_moe_ffn_dev.argtypes = [vp, sz, vp, vp, sz, vp, vp]
    L.smx_moe_shexp_dev.argtypes = [vp, sz, C.c_float, vp, vp]
    L.smx_moe_route_dev.argtypes = [vp, vp, sz, sz, vp, vp]
    L.smx_moe_route.argtypes = [vp, vp, sz, sz, vp, vp]
    L.smx_moe_router_dev.argtypes = [vp, cp, vp, sz, vp, vp, vp]
    L.smx_moe_ffn_logits_dev.argtypes = [vp, sz, vp, sz, vp, vp, vp, vp]
    L.smx_moe_ffn_routed_dev.argtypes = [vp, sz, vp, vp, sz, vp, vp]
    L.smx_gemm_fused_dev.argtypes = [vp, cp, i, vp, vp, sz, C.c_float, vp]
    L.smx_moe_layer_ffn.argtypes = [vp, sz, vp, sz, vp, sz, vp, sz]
    L.smx_moe_expert_ffn.argtypes = [vp, sz, sz, vp, sz, vp, sz]
    L.smx_prof_enable.argtypes = [vp, i]
    L.smx_prof_reset.argtypes = [vp]
    L.smx_prof_read.argtypes = [vp, cp, C.POINTER(C.c_double), C.POINTER(sz)]
    L.smx_prof_names.argtypes = [vp]
    L.smx_prof_names.restype = cp
    L.smx_timer_begin.argtypes = [vp]
    L.smx_timer_end.argtypes = [vp, C.POINTER(C.c_float)]
    L.smx_quantize.argtypes = [vp, vp, sz, sz, vp, vp, vp]
    L.smx_gemv_block_dots.argtypes = [vp, cp, vp, sz, vp, sz]
    L.smx_gemm_block_dots.argtypes = [vp, cp, vp, sz, sz, vp, sz]
    L.smx_moe_ffn_stages.argtypes = [vp, sz, vp, vp, sz, vp, sz, vp, vp, vp, vp]
    L.smx_tune.argtypes = [vp, cp, i]
    L.smx_graph_begin.argtypes = [vp]
    L.smx_graph_end.argtypes = [vp, C.POINTER(vp)]
    L.smx_graph_launch.argtypes = [vp, vp]
    L.smx_graph_destroy.argtypes = [vp, vp]
    L.smx_graph_destroy.restype = None
    L.smx_gguf_open.argtypes = [cp, C.POINTER(vp), cp, sz]
    L.smx_gguf_close.argtypes = [vp]
    L.smx_gguf_close.restype = None
    L.smx_gguf_tensor_count.argtypes = [vp]
    L.smx_gguf_tensor_count.restype = sz
    L.smx_gguf_tensor.argtypes = [vp, sz, C.POINTER(cp), C.POINTER(i), C.POINTER(sz), C.POINTER(sz), sz, C.POINTER(vp),
                                  C.POINTER(sz)]
    L.smx_gguf_find.argtypes = [vp, cp, C.POINTER(sz)]
    L.smx_gguf_meta_u64.argtypes = [vp, cp, C.POINTER(C.c_uint64)]
    L.smx_gguf_meta_f32.argtypes = [vp, cp, C.POINTER(C.c_float)]
    L.smx_gguf_meta_str.argtypes = [vp, cp, C.POINTER(cp)]
    L.smx_gguf_attach.argtypes = [vp, vp, C.POINTER(sz), C.POINTER(sz)]
    L.smx_host_quantize_q8_0.argtypes = [vp, sz, vp]
    L.smx_host_quantize_q4_0.argtypes = [vp, sz, vp]
    L.smx_host_dequantize.argtypes = [i, vp, sz, vp]
    L.smx_gguf_upload_as.argtypes = [vp, vp, C.c_char_p, C.c_char_p, i]
    _lib = L
    return L


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dt):
    return np.ascontiguousarray(a, dtype=dt)


class GgufFile:
    """A memory-mapped GGUF file: metadata and tensor index (crates/strix-models/src/gguf.rs:104-238).
    Needs no GPU."""

    def __init__(self, path):
        self._L = load_library()
        h = C.c_void_p()
        err = C.create_string_buffer(512)
        rc = self._L.smx_gguf_open(str(path).encode(), C.byref(h), err, len(err))
        if rc != SMX_OK:
            raise SmxError(rc, err.value.decode())
        self._h = h

    def close(self):
        if getattr(self, "_h", None):
            self._L.smx_gguf_close(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def __len__(self):
        return self._L.smx_gguf_tensor_count(self._h)

    def tensor(self, index):
        """(name, ggml_type, dims, bytes) of tensor `index`; bytes is a copy of its raw data."""
        name, ty, nd, nb, data = C.c_char_p(), C.c_int(), C.c_size_t(), C.c_size_t(), C.c_void_p()
        dims = (C.c_size_t * 8)()
        rc = self._L.smx_gguf_tensor(self._h, index, C.byref(name), C.byref(ty), C.byref(nd), dims, 8, C.byref(data),
                                     C.byref(nb))
        if rc != SMX_OK:
            raise IndexError(index)
        raw = np.ctypeslib.as_array((C.c_uint8 * nb.value).from_address(data.value)).copy() if nb.value else np.empty(0, np.uint8)
        return name.value.decode(), ty.value, [dims[d] for d in range(nd.value)], raw

    def find(self, name):
        idx = C.c_size_t()
        return idx.value if self._L.smx_gguf_find(self._h, name.encode(), C.byref(idx)) == SMX_OK else None

    def tensors(self):
        return {t[0]: t for t in (self.tensor(i) for i in range(len(self)))}

    def _meta(self, fn, key, out, what):
        rc = fn(self._h, key.encode(), C.byref(out))
        if rc == 0:
            return None
        if rc < 0:
            raise TypeError(f"GGUF metadata {key!r} is not {what}")
        return out.value

    def meta_u64(self, key):
        return self._meta(self._L.smx_gguf_meta_u64, key, C.c_uint64(), "an unsigned integer")

    def meta_f32(self, key):
        return self._meta(self._L.smx_gguf_meta_f32, key, C.c_float(), "a number")

    def meta_str(self, key):
        v = self._meta(self._L.smx_gguf_meta_str, key, C.c_char_p(), "a string")
        return None if v is None else v.decode()


def host_quantize_q8_0(x):
    """f32 -> GGUF Q8_0 bytes (crates/strix-models/src/ggml_quant.rs:193-207)."""
    x = _c(x, np.float32).reshape(-1)
    out = np.empty(x.size // 32 * 34, np.uint8)
    if load_library().smx_host_quantize_q8_0(_p(x), x.size, _p(out)) != SMX_OK:
        raise ValueError("length must be a multiple of 32")
    return out


def host_quantize_q4_0(x):
    """f32 -> GGUF Q4_0 bytes (ggml_quant.rs:212-237)."""
    x = _c(x, np.float32).reshape(-1)
    out = np.empty(x.size // 32 * 18, np.uint8)
    if load_library().smx_host_quantize_q4_0(_p(x), x.size, _p(out)) != SMX_OK:
        raise ValueError("length must be a multiple of 32")
    return out


def host_dequantize(ggml_type, raw, n):
    """GGUF bytes -> f32 for F32, F16, Q4_0, Q8_0, Q6_K (ggml_quant.rs:239-262, 401-430)."""
    raw = _c(raw, np.uint8)
    out = np.empty(n, np.float32)
    rc = load_library().smx_host_dequantize(int(ggml_type), _p(raw), n, _p(out))
    if rc != SMX_OK:
        raise ValueError(f"cannot dequantise ggml type {ggml_type} with {n} elements")
    return out


class Mi355WeightAccel:
    """One device, one stream, resident quantized weights (WeightAccel, accel.rs:147)."""

    def __init__(self, device=0):
        self._L = load_library()
        h = C.c_void_p()
        rc = self._L.smx_create(device, C.byref(h))
        if rc != SMX_OK:
            raise SmxError(rc, self._L.smx_last_error(None).decode())
        self._h = h

    def close(self):
        if getattr(self, "_h", None):
            self._L.smx_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    # -- helpers
    def _check(self, rc):
        """1 -> True, 0 -> False (not resident), <0 -> raise."""
        if rc < 0:
            raise SmxError(rc, self._L.smx_last_error(self._h).decode())
        return rc == SMX_OK

    def last_error(self):
        return self._L.smx_last_error(self._h).decode()

    # -- WeightAccel surface
    def name(self):
        return self._L.smx_name(self._h).decode()

    def resident_count(self):
        return int(self._L.smx_resident_count(self._h))

    def resident_bytes(self):
        return int(self._L.smx_resident_bytes(self._h))

    def _upload(self, fn, key, raw, in_dim, out_dim):
        raw = _c(raw, np.uint8)
        return self._check(fn(self._h, key.encode(), _p(raw), raw.size, in_dim, out_dim))

    def upload_q4_0(self, key, raw, in_dim, out_dim):
        return self._upload(self._L.smx_upload_q4_0, key, raw, in_dim, out_dim)

    def upload_q8_0(self, key, raw, in_dim, out_dim):
        return self._upload(self._L.smx_upload_q8_0, key, raw, in_dim, out_dim)

    def upload_q6_k(self, key, raw, in_dim, out_dim):
        return self._upload(self._L.smx_upload_q6_k, key, raw, in_dim, out_dim)

    def upload_moe_q8(self, layer, gate, up, down, hidden, eff, ne):
        gate, up, down = _c(gate, np.uint8), _c(up, np.uint8), _c(down, np.uint8)
        return self._check(self._L.smx_upload_moe_q8(self._h, layer, _p(gate), gate.size, _p(up), up.size,
                                                     _p(down), down.size, hidden, eff, ne))

    def upload_moe_q6(self, layer, gate, up, down, hidden, eff, ne):
        gate, up, down = _c(gate, np.uint8), _c(up, np.uint8), _c(down, np.uint8)
        return self._check(self._L.smx_upload_moe_q6(self._h, layer, _p(gate), gate.size, _p(up), up.size,
                                                     _p(down), down.size, hidden, eff, ne))

    def attach_gguf(self, gguf):
        """The upload loop of the models' attach_accel (mellum.rs:460-535): returns (matrices, expert layers)."""
        nw, nl = C.c_size_t(), C.c_size_t()
        self._check(self._L.smx_gguf_attach(self._h, gguf._h, C.byref(nw), C.byref(nl)))
        return nw.value, nl.value

    def upload_as(self, gguf, tensor, target_type, key=None):
        """One matrix of the file re-encoded as Q8_0 (8) or Q4_0 (2) on the host and uploaded
        (gemma3n.rs:455-470, qwen35.rs:741-760)."""
        return self._check(self._L.smx_gguf_upload_as(self._h, gguf._h, tensor.encode(),
                                                      key.encode() if key else None, int(target_type)))

    def evict(self, key):
        return self._check(self._L.smx_evict(self._h, key.encode()))

    def weight_dims(self, key):
        """(in_dim, out_dim) of a resident weight, or None."""
        i, o = C.c_size_t(), C.c_size_t()
        ok = self._check(self._L.smx_weight_dims(self._h, key.encode(), C.byref(i), C.byref(o)))
        return (i.value, o.value) if ok else None

    def gemv(self, key, x, out_dim):
        x = _c(x, np.float32).reshape(-1)
        y = np.empty(out_dim, np.float32)
        ok = self._check(self._L.smx_gemv(self._h, key.encode(), _p(x), x.size, _p(y), y.size))
        return y if ok else None

    def gemv_f32(self, key, x, out_dim):
        """gemv with fp32 activations (the arithmetic of the reference's per-weight gemv and of its CPU path)."""
        x = _c(x, np.float32).reshape(-1)
        y = np.empty(out_dim, np.float32)
        ok = self._check(self._L.smx_gemv_f32(self._h, key.encode(), _p(x), x.size, _p(y), y.size))
        return y if ok else None

    def gemv_f32_dev(self, key, x_dev, y_dev):
        return self._check(self._L.smx_gemv_f32_dev(self._h, key.encode(), x_dev, y_dev))

    def gemv_fused(self, key, act, a, b, out_dim, eps=0.0):
        """GEMV of producer(a, b): rmsnorm(a)*b, silu(a)*b or gelu_tanh(a)*b (kernels.rs:101-226), one launch."""
        a = _c(a, np.float32).reshape(-1)
        b = None if b is None else _c(b, np.float32).reshape(-1)
        y = np.empty(out_dim, np.float32)
        ok = self._check(self._L.smx_gemv_fused(self._h, key.encode(), int(act), _p(a), _p(b), a.size, float(eps),
                                                _p(y), y.size))
        return y if ok else None

    def gemv_rows(self, key, xs, out_dim):
        xs = _c(xs, np.float32)
        m, k = xs.shape
        y = np.empty((m, out_dim), np.float32)
        ok = self._check(self._L.smx_gemv_rows(self._h, key.encode(), _p(xs), m, k, _p(y), y.size))
        return y if ok else None

    def gemv_batch(self, calls, out_dims, f32=False):
        """calls: [(key, x)], out_dims: [out_dim]; returns [array | None] (accel.rs:397).  f32: the arithmetic of gemv_f32."""
        n = len(calls)
        xs = [_c(x, np.float32).reshape(-1) for _, x in calls]
        ys = [np.empty(d, np.float32) for d in out_dims]
        keys = (C.c_char_p * n)(*[k.encode() for k, _ in calls])
        xp = (C.c_void_p * n)(*[x.ctypes.data for x in xs])
        yp = (C.c_void_p * n)(*[y.ctypes.data for y in ys])
        il = (C.c_size_t * n)(*[x.size for x in xs])
        oc = (C.c_size_t * n)(*[y.size for y in ys])
        st = (C.c_int * n)()
        fn = self._L.smx_gemv_f32_batch if f32 else self._L.smx_gemv_batch
        self._check(fn(self._h, n, keys, xp, il, yp, oc, st))
        out = []
        for i in range(n):
            if st[i] < 0:
                raise SmxError(st[i], self.last_error())
            out.append(ys[i] if st[i] == SMX_OK else None)
        return out

    def prefill_q8_gemm(self, key, xs, m, out_dim):
        """y[m][out_dim] token-major (accel.rs:213)."""
        xs = _c(xs, np.float32).reshape(m, -1)
        y = np.empty((m, out_dim), np.float32)
        ok = self._check(self._L.smx_gemm(self._h, key.encode(), _p(xs), m, xs.shape[1], _p(y), y.size))
        return y if ok else None

    def lm_head_argmax_rows(self, key, xs, m):
        xs = _c(xs, np.float32).reshape(m, -1)
        out = np.empty(m, np.uint32)
        ok = self._check(self._L.smx_lm_head_argmax_rows(self._h, key.encode(), _p(xs), m, xs.shape[1], _p(out)))
        return out if ok else None

    def moe_ffn(self, layer, ids, wexp, x, sgate=0.0):
        ids, wexp, x = _c(ids, np.int32), _c(wexp, np.float32), _c(x, np.float32).reshape(-1)
        y = np.empty(x.size, np.float32)
        ok = self._check(self._L.smx_moe_ffn(self._h, layer, _p(ids), _p(wexp), ids.size, _p(x), x.size,
                                             sgate, _p(y), y.size))
        return y if ok else None

    def moe_layer_q8_dev(self, layer, xs, m, plan, slot_tok, wslot):
        xs = _c(xs, np.float32).reshape(m, -1)
        plan = _c(plan, np.uint64).reshape(-1, 3)
        slot_tok, wslot = _c(slot_tok, np.int32), _c(wslot, np.float32)
        y = np.empty_like(xs)
        ok = self._check(self._L.smx_moe_layer(self._h, layer, _p(xs), m, _p(plan), plan.shape[0],
                                               _p(slot_tok), _p(wslot), slot_tok.size, _p(y), y.size))
        return y if ok else None

    def moe_layer_ffn(self, layer, plan, xs, rows):
        """plan: (expert, rows) pairs; xs[rows][hidden] expert-major; returns dy[rows][hidden] (accel.rs:238-246)."""
        plan = _c(plan, np.int32).reshape(-1, 2)
        xs = _c(xs, np.float32).reshape(rows, -1)
        dy = np.empty_like(xs)
        ok = self._check(self._L.smx_moe_layer_ffn(self._h, layer, _p(plan), plan.shape[0], _p(xs), rows, _p(dy), dy.size))
        return dy if ok else None

    def moe_expert_ffn(self, layer, expert, xs, m):
        xs = _c(xs, np.float32).reshape(m, -1)
        y = np.empty_like(xs)
        ok = self._check(self._L.smx_moe_expert_ffn(self._h, layer, expert, _p(xs), m, _p(y), y.size))
        return y if ok else None

    def moe_layer_resident(self, layer, xs_dev, m, plan, slot_tok, wslot, y_dev):
        """moe_layer_q8_dev with activations and result already on the device (enqueue only)."""
        plan = _c(plan, np.uint64).reshape(-1, 3)
        slot_tok, wslot = _c(slot_tok, np.int32), _c(wslot, np.float32)
        return self._check(self._L.smx_moe_layer_dev(self._h, layer, xs_dev, m, _p(plan), plan.shape[0],
                                                     _p(slot_tok), _p(wslot), slot_tok.size, y_dev))

    # -- parity instrumentation
    def quantize(self, x, k):
        x = _c(x, np.float32).reshape(-1, k)
        m = x.shape[0]
        xq = np.empty((m, k), np.int8)
        xd = np.empty((m, k // 32), np.float32)
        xs = np.empty((m, k // 16), np.int16)
        self._check(self._L.smx_quantize(self._h, _p(x), m, k, _p(xq), _p(xd), _p(xs)))
        return xq, xd, xs

    def gemv_block_dots(self, key, x, out_dim, per_row):
        x = _c(x, np.float32).reshape(-1)
        out = np.empty((out_dim, per_row), np.int32)
        ok = self._check(self._L.smx_gemv_block_dots(self._h, key.encode(), _p(x), x.size, _p(out), out.size))
        return out if ok else None

    def gemm_block_dots(self, key, xs, m, out_dim, nb):
        xs = _c(xs, np.float32).reshape(m, -1)
        out = np.empty((m, out_dim, nb), np.int32)
        ok = self._check(self._L.smx_gemm_block_dots(self._h, key.encode(), _p(xs), m, xs.shape[1], _p(out), out.size))
        return out if ok else None

    def moe_ffn_stages(self, layer, ids, wexp, x, eff):
        ids, wexp, x = _c(ids, np.int32), _c(wexp, np.float32), _c(x, np.float32).reshape(-1)
        k = ids.size
        y = np.empty(x.size, np.float32)
        gu = np.empty((k, 2, eff), np.float32)
        aq = np.empty((k, eff), np.int8)
        ad = np.empty((k, eff // 32), np.float32)
        ok = self._check(self._L.smx_moe_ffn_stages(self._h, layer, _p(ids), _p(wexp), k, _p(x), x.size,
                                                    _p(y), _p(gu), _p(aq), _p(ad)))
        return (y, gu, aq, ad) if ok else None

    def moe_layer_stages(self, layer, xs, m, plan, slot_tok, wslot, eff):
        """moe_layer_q8_dev with the per-slot stages: (y, gu[slots][2][eff], aq, ad, dy[slots][hidden])."""
        xs = _c(xs, np.float32).reshape(m, -1)
        hidden = xs.shape[1]
        plan = _c(plan, np.uint64).reshape(-1, 3)
        slot_tok, wslot = _c(slot_tok, np.int32), _c(wslot, np.float32)
        slots = slot_tok.size
        y = np.empty_like(xs)
        gu = np.empty((slots, 2, eff), np.float32)
        aq = np.empty((slots, eff), np.int8)
        ad = np.empty((slots, eff // 32), np.float32)
        dy = np.empty((slots, hidden), np.float32)
        ok = self._check(self._L.smx_moe_layer_stages(self._h, layer, _p(xs), m, _p(plan), plan.shape[0], _p(slot_tok),
                                                      _p(wslot), slots, _p(y), y.size, _p(gu), _p(aq), _p(ad), _p(dy)))
        return (y, gu, aq, ad, dy) if ok else None

    # -- device-resident + timing (used by the benchmark)
    def dev_alloc(self, nbytes):
        d = C.c_void_p()
        self._check(self._L.smx_dev_alloc(self._h, nbytes, C.byref(d)))
        return d.value

    def dev_free(self, dptr):
        self._check(self._L.smx_dev_free(self._h, dptr))

    def h2d(self, dptr, arr):
        arr = np.ascontiguousarray(arr)
        self._check(self._L.smx_h2d(self._h, dptr, _p(arr), arr.nbytes))

    def d2h(self, arr, dptr):
        self._check(self._L.smx_d2h(self._h, _p(arr), dptr, arr.nbytes))
        return arr

    def dev_copy(self, dst, src, nbytes):
        self._check(self._L.smx_dev_copy(self._h, dst, src, nbytes))

    def sync(self):
        self._check(self._L.smx_sync(self._h))

    def gemv_dev(self, key, xs_dev, m, y_dev):
        return self._check(self._L.smx_gemv_dev(self._h, key.encode(), xs_dev, m, y_dev))

    def gemv_noalloc_dev(self, key, xs_dev, m, y_dev):
        """gemv_dev that allocates nothing (static device scratch; m <= 8, in_dim <= 16384)."""
        return self._check(self._L.smx_gemv_noalloc_dev(self._h, key.encode(), xs_dev, m, y_dev))

    def gemv_batch_dev(self, keys, xs_dev, ys_dev):
        n = len(keys)
        k = (C.c_char_p * n)(*[s.encode() for s in keys])
        xp = (C.c_void_p * n)(*xs_dev)
        yp = (C.c_void_p * n)(*ys_dev)
        return self._check(self._L.smx_gemv_batch_dev(self._h, n, k, xp, yp))

    def gemv_fused_dev(self, keys, act, a_dev, b_dev, ys_dev, eps=0.0):
        n = len(keys)
        k = (C.c_char_p * n)(*[s.encode() for s in keys])
        yp = (C.c_void_p * n)(*ys_dev)
        return self._check(self._L.smx_gemv_fused_dev(self._h, n, k, int(act), a_dev, b_dev, float(eps), yp))

    def ffn_gate_up_dev(self, gate_key, up_key, act, x_dev, h_dev, norm=False, norm_w_dev=None, eps=0.0):
        """h = act(gate . x') * (up . x') in one launch, x' = x or rmsnorm(x) * norm_w (see smx_ffn_gate_up_dev)."""
        return self._check(self._L.smx_ffn_gate_up_dev(self._h, gate_key.encode(), up_key.encode(), int(act), x_dev,
                                                       1 if norm else 0, norm_w_dev, float(eps), h_dev))

    def gemm_fused_dev(self, key, act, a_dev, b_dev, m, y_dev, eps=0.0):
        """Prefill rows through a producer + quantiser + int8 GEMM (see smx_gemm_fused_dev)."""
        return self._check(self._L.smx_gemm_fused_dev(self._h, key.encode(), int(act), a_dev, b_dev, m, float(eps), y_dev))

    def gemm_dev(self, key, xs_dev, m, y_dev):
        return self._check(self._L.smx_gemm_dev(self._h, key.encode(), xs_dev, m, y_dev))

    def moe_ffn_dev(self, layer, ids, wexp, x_dev, y_dev):
        ids, wexp = _c(ids, np.int32), _c(wexp, np.float32)
        return self._check(self._L.smx_moe_ffn_dev(self._h, layer, _p(ids), _p(wexp), ids.size, x_dev, y_dev))

    def moe_route(self, logits, k):
        """Router on the device (topk_router, kernels.rs:1846-1872): (ids[k] i32, w[k] f32)."""
        logits = _c(logits, np.float32).reshape(-1)
        ids, w = np.empty(k, np.int32), np.empty(k, np.float32)
        self._check(self._L.smx_moe_route(self._h, _p(logits), logits.size, k, _p(ids), _p(w)))
        return ids, w

    def moe_route_dev(self, logits_dev, ne, k, ids_dev, w_dev):
        return self._check(self._L.smx_moe_route_dev(self._h, logits_dev, ne, k, ids_dev, w_dev))

    def moe_router_dev(self, key, x_dev, k, ids_dev, w_dev, logits_dev=None):
        """Router logits (GEMV of the resident router weight) + softmax + top-k in one call."""
        return self._check(self._L.smx_moe_router_dev(self._h, key.encode(), x_dev, k, ids_dev, w_dev, logits_dev))

    def moe_ffn_logits_dev(self, layer, logits_dev, k, x_dev, y_dev, ids_dev, w_dev):
        """Routed expert FFN of a decode token from the router logits (routing inside the gate/up launch where it serves)."""
        return self._check(self._L.smx_moe_ffn_logits_dev(self._h, layer, logits_dev, k, x_dev, y_dev, ids_dev, w_dev))

    def moe_ffn_routed_dev(self, layer, ids_dev, w_dev, k, x_dev, y_dev):
        """moe_ffn_dev reading the routing from device memory at run time (capturable with new routing)."""
        return self._check(self._L.smx_moe_ffn_routed_dev(self._h, layer, ids_dev, w_dev, k, x_dev, y_dev))

    def moe_shexp_dev(self, layer, sgate, x_dev, y_dev):
        """y_dev += sgate * shared_expert(x_dev) (decode.rs:1820-1855)."""
        return self._check(self._L.smx_moe_shexp_dev(self._h, layer, float(sgate), x_dev, y_dev))

    def graph_begin(self):
        self._check(self._L.smx_graph_begin(self._h))

    def graph_end(self):
        g = C.c_void_p()
        self._check(self._L.smx_graph_end(self._h, C.byref(g)))
        return g

    def graph_launch(self, g):
        self._check(self._L.smx_graph_launch(self._h, g))

    def graph_destroy(self, g):
        self._L.smx_graph_destroy(self._h, g)

    def tune(self, knob, value):
        self._check(self._L.smx_tune(self._h, knob.encode(), int(value)))

    def prof_enable(self, on=True):
        self._check(self._L.smx_prof_enable(self._h, 1 if on else 0))

    def prof_reset(self):
        self._check(self._L.smx_prof_reset(self._h))

    def prof_read(self, prefix):
        ms, n = C.c_double(), C.c_size_t()
        self._check(self._L.smx_prof_read(self._h, prefix.encode(), C.byref(ms), C.byref(n)))
        return ms.value, n.value

    def prof_names(self):
        s = self._L.smx_prof_names(self._h).decode()
        return s.split(",") if s else []

    def timer_begin(self):
        self._check(self._L.smx_timer_begin(self._h))

    def timer_end(self):
        ms = C.c_float()
        self._check(self._L.smx_timer_end(self._h, C.byref(ms)))
        return ms.value
