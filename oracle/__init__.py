"""CPU checker for the HIP path (test infrastructure only).

Thin ctypes/numpy wrappers over ``libksearch_oracle.so`` (built by
``oracle/Makefile`` from ``ksearch_oracle.c``).  Only ``tests/``, the smoke
check and the benchmark's ``cpu_baseline`` leg may import this package; the
shipped library never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libksearch_oracle.so")

F32, F16, Q4K, Q5K, Q6K, Q40, BF16 = range(7)
BLOCK = {Q40: (32, 18), Q4K: (256, 144), Q5K: (256, 176), Q6K: (256, 210)}


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (always when ``force``; else only if absent)."""
    if force or not os.path.exists(LIB_PATH):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE])
    return LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(LIB_PATH)
        vp, sz, i32, u32, f32 = C.c_void_p, C.c_size_t, C.c_int, C.c_uint32, C.c_float
        sig = {
            "ko_bf16_to_f32": (f32, [C.c_uint16]),
            "ko_f32_to_bf16": (C.c_uint16, [f32]),
            "ko_f16_to_f32": (f32, [C.c_uint16]),
            "ko_f32_to_f16": (C.c_uint16, [f32]),
            "ko_f32_to_f16_rne": (C.c_uint16, [f32]),
            "ko_get_scale_min_k4": (None, [i32, vp, vp, vp]),
            "ko_row_bytes": (sz, [i32, sz]),
            "ko_dequant": (i32, [i32, vp, sz, vp]),
            "ko_quantize_q4k": (None, [vp, sz, vp]),
            "ko_quantize_q6k": (None, [vp, sz, vp]),
            "ko_pack_q40": (None, [vp, sz, vp, i32]),
            "ko_matvec": (i32, [i32, vp, sz, sz, vp, vp, i32]),
            "ko_matmul": (i32, [i32, vp, sz, sz, vp, sz, vp, i32]),
            "ko_matvec_f64": (i32, [i32, vp, sz, sz, vp, vp, i32]),
            "ko_max_threads": (i32, []),
            "ko_sdpa_online": (None, [vp, vp, vp, i32, i32, i32, i32, i32, f32, vp]),
            "ko_sdpa_mwg": (None, [vp, vp, vp, i32, i32, i32, i32, i32, f32, i32, vp]),
            "ko_sdpa_f64": (None, [vp, vp, vp, i32, i32, i32, i32, i32, f32, vp]),
            "ko_softcap_argmax": (u32, [vp, sz, f32]),
            "ko_rmsnorm": (None, [vp, vp, vp, f32, f32, i32, sz, vp]),
            "ko_rmsnorm_add_then_rmsnorm": (None, [vp, vp, vp, vp, f32, sz, vp, vp]),
            "ko_rope_table": (None, [i32, i32, f32, i32, vp]),
            "ko_rmsnorm_per_head_qkv_q40": (None, [vp, vp, vp, vp, vp, vp, i32, i32, i32, f32, vp, vp, vp]),
            "ko_gelu_mul": (f32, [f32, f32]),
            "ko_copy_scale_indexed": (i32, [i32, vp, u32, sz, f32, vp]),
            "ko_gemma_create": (vp, [vp, vp, vp, vp]),
            "ko_gemma_destroy": (None, [vp]),
            "ko_gemma_reset": (None, [vp]),
            "ko_gemma_forward": (u32, [vp, u32, i32, vp, i32]),
            "ko_gemma_pos": (i32, [vp]),
            "ko_gemma_kv": (vp, [vp, i32, i32]),
            "ko_gemma_hidden": (vp, [vp]),
            "ko_gemma_set_row_sync": (None, [vp, vp]),
            "ko_gemma4_set_row_sync": (None, [vp, vp]),
            "ko_sample_softcap_min_p": (u32, [vp, sz, f32, f32, f32, u32]),
            "ko_rmsnorm_per_head": (None, [vp, vp, vp, i32, i32, f32, vp]),
            "ko_add_scale": (None, [vp, vp, f32, sz, vp]),
            "ko_matvec_gelu_mul": (i32, [i32, vp, sz, sz, vp, vp, vp, i32]),
            "ko_gemma4_create": (vp, [vp, vp, vp]),
            "ko_gemma4_destroy": (None, [vp]),
            "ko_gemma4_reset": (None, [vp]),
            "ko_gemma4_forward": (u32, [vp, u32, i32, vp, i32]),
            "ko_gemma4_pos": (i32, [vp]),
            "ko_gemma4_kv_source": (i32, [vp, i32]),
            "ko_gemma4_kv": (vp, [vp, i32, i32]),
            "ko_gemma4_hidden": (vp, [vp]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def _p(a: np.ndarray) -> int:
    return a.ctypes.data


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.uint8)


def row_bytes(dtype: int, cols: int) -> int:
    return lib().ko_row_bytes(dtype, cols)


def f16_to_f32(bits) -> np.ndarray:
    bits = np.asarray(bits, dtype=np.uint16).ravel()
    L = lib()
    return np.array([L.ko_f16_to_f32(int(b)) for b in bits], dtype=np.float32)


def f32_to_f16(vals, rne: bool = False) -> np.ndarray:
    fn = lib().ko_f32_to_f16_rne if rne else lib().ko_f32_to_f16
    return np.array([fn(float(v)) for v in np.asarray(vals, dtype=np.float32).ravel()], dtype=np.uint16)


def get_scale_min_k4(j: int, q12) -> tuple[int, int]:
    q = _u8(q12)
    d, m = C.c_uint8(), C.c_uint8()
    lib().ko_get_scale_min_k4(j, _p(q), C.addressof(d), C.addressof(m))
    return d.value, m.value


def dequant(dtype: int, data, n_elems: int) -> np.ndarray:
    data = _u8(data)
    out = np.empty(n_elems, dtype=np.float32)
    if lib().ko_dequant(dtype, _p(data), n_elems, _p(out)):
        raise ValueError("unsupported dtype")
    return out


def quantize_q4k(x) -> np.ndarray:
    x = _f32(x).ravel()
    out = np.empty(x.size // 256 * 144, dtype=np.uint8)
    lib().ko_quantize_q4k(_p(x), x.size, _p(out))
    return out


def quantize_q6k(x) -> np.ndarray:
    x = _f32(x).ravel()
    out = np.empty(x.size // 256 * 210, dtype=np.uint8)
    lib().ko_quantize_q6k(_p(x), x.size, _p(out))
    return out


def pack_q40(x, half_roundtrip: bool = True) -> np.ndarray:
    x = _f32(x).ravel()
    out = np.empty(x.size // 32 * 18, dtype=np.uint8)
    lib().ko_pack_q40(_p(x), x.size, _p(out), int(half_roundtrip))
    return out


def matvec(dtype: int, w, rows: int, cols: int, x, threads: int = 0) -> np.ndarray:
    w, x = _u8(w), _f32(x)
    y = np.empty(rows, dtype=np.float32)
    if lib().ko_matvec(dtype, _p(w), rows, cols, _p(x), _p(y), threads):
        raise ValueError("bad matvec shape/dtype")
    return y


def matvec_f64(dtype: int, w, rows: int, cols: int, x, threads: int = 0) -> np.ndarray:
    w, x = _u8(w), _f32(x)
    y = np.empty(rows, dtype=np.float64)
    if lib().ko_matvec_f64(dtype, _p(w), rows, cols, _p(x), _p(y), threads):
        raise ValueError("bad matvec shape/dtype")
    return y


def matmul(dtype: int, w, rows: int, cols: int, x, batch: int, threads: int = 0) -> np.ndarray:
    w, x = _u8(w), _f32(x)
    y = np.empty((batch, rows), dtype=np.float32)
    if lib().ko_matmul(dtype, _p(w), rows, cols, _p(x), batch, _p(y), threads):
        raise ValueError("bad matmul shape/dtype")
    return y


def max_threads() -> int:
    return lib().ko_max_threads()


def sdpa(q, k, v, n_q, n_kv, hd, tlen, start=0, scale=1.0, nwg: int | None = None, f64=False):
    q, k, v = _f32(q), _u8(k), _u8(v)
    L = lib()
    if f64:
        out = np.empty(n_q * hd, dtype=np.float64)
        L.ko_sdpa_f64(_p(q), _p(k), _p(v), n_q, n_kv, hd, tlen, start, scale, _p(out))
        return out
    out = np.empty(n_q * hd, dtype=np.float32)
    if nwg is None:
        L.ko_sdpa_online(_p(q), _p(k), _p(v), n_q, n_kv, hd, tlen, start, scale, _p(out))
    else:
        L.ko_sdpa_mwg(_p(q), _p(k), _p(v), n_q, n_kv, hd, tlen, start, scale, nwg, _p(out))
    return out


def sdpa_hybrid(q, k, v, n_q, n_kv, hd, tlen, start=0, scale=1.0):
    """sdpa_hybrid_kv: online below 128 rows, 16-way split from 128 on
    (ksearch_kernels/src/lib.rs:1114-1178)."""
    return sdpa(q, k, v, n_q, n_kv, hd, tlen, start, scale, nwg=16 if tlen >= 128 else None)


def softcap_argmax(x, cap: float) -> int:
    x = _f32(x)
    return lib().ko_softcap_argmax(_p(x), x.size, cap)


def rmsnorm(x, w, eps, res=None, scale=None) -> np.ndarray:
    x, w = _f32(x), _f32(w)
    out = np.empty_like(x)
    r = _f32(res) if res is not None else None
    lib().ko_rmsnorm(_p(x), _p(w), _p(r) if r is not None else None, eps,
                     scale if scale is not None else 0.0, int(scale is not None), x.size, _p(out))
    return out


def rmsnorm_add_then_rmsnorm(y, w_post, res, w_ffn, eps):
    y, w_post, res, w_ffn = _f32(y), _f32(w_post), _f32(res), _f32(w_ffn)
    ox, ox2 = np.empty_like(y), np.empty_like(y)
    lib().ko_rmsnorm_add_then_rmsnorm(_p(y), _p(w_post), _p(res), _p(w_ffn), eps, y.size, _p(ox), _p(ox2))
    return ox, ox2


def rope_table(max_seq, hd, theta, rope_angles=None) -> np.ndarray:
    out = np.empty((max_seq, hd), dtype=np.float32)
    lib().ko_rope_table(max_seq, hd, theta, hd // 2 if rope_angles is None else rope_angles, _p(out))
    return out


def rmsnorm_per_head_qkv_q40(q, qw, rope_row, k, kw, v, n_q, n_kv, hd, eps):
    q, qw, rope_row, k, kw, v = map(_f32, (q, qw, rope_row, k, kw, v))
    qo = np.empty(n_q * hd, dtype=np.float32)
    ko = np.empty(n_kv * hd // 32 * 18, dtype=np.uint8)
    vo = np.empty_like(ko)
    lib().ko_rmsnorm_per_head_qkv_q40(_p(q), _p(qw), _p(rope_row), _p(k), _p(kw), _p(v),
                                      n_q, n_kv, hd, eps, _p(qo), _p(ko), _p(vo))
    return qo, ko, vo


def gelu_mul(g, u) -> np.ndarray:
    g, u = _f32(g).ravel(), _f32(u).ravel()
    L = lib()
    return np.array([L.ko_gelu_mul(float(a), float(b)) for a, b in zip(g, u)], dtype=np.float32)


def copy_scale_indexed(dtype, src, idx, n, scale) -> np.ndarray:
    src = _u8(src)
    out = np.empty(n, dtype=np.float32)
    if lib().ko_copy_scale_indexed(dtype, _p(src), idx, n, scale, _p(out)):
        raise ValueError("bad dtype")
    return out


class RowSync(C.Structure):
    _fields_ = [("rows", C.c_void_p), ("row_stride", C.c_size_t), ("diff_bytes", C.c_void_p), ("max_step", C.c_void_p)]


class _RowAdoption:
    """Shared by the two decode loops: `forward(..., adopt_rows=a)` makes every cache-appending layer pack its
    own Q4_0 K / V rows, measure how the rows in `a` ([n_layers, 2, row_bytes] uint8, another implementation's
    rows for this position) differ from them, and continue with those.  Afterwards `row_diff_bytes` and
    `row_max_step` ([n_layers, 2]; a step of 1.0 is one code of the own block) describe the differences."""

    _set_sync = None

    def _forward_adopting(self, fwd, n_layers, adopt_rows):
        if adopt_rows is None:
            return fwd()
        rows = np.ascontiguousarray(adopt_rows, dtype=np.uint8)
        assert rows.ndim == 3 and rows.shape[:2] == (n_layers, 2), rows.shape
        self.row_diff_bytes = np.zeros((n_layers, 2), dtype=np.int32)
        self.row_max_step = np.zeros((n_layers, 2), dtype=np.float32)
        s = RowSync(_p(rows), rows.shape[2], _p(self.row_diff_bytes), _p(self.row_max_step))
        getattr(lib(), self._set_sync)(self.h, C.byref(s))
        try:
            return fwd()
        finally:
            getattr(lib(), self._set_sync)(self.h, None)


class GemmaCfg(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("n_layers", "hidden", "ffn", "n_q", "n_kv", "hd", "vocab", "max_seq")] + \
               [(n, C.c_float) for n in ("eps", "softcap", "rope_theta", "attn_scale")]


class GemmaLayer(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in (
        "wq", "wk", "wv", "wo", "wgate", "wup", "wdown",
        "attn_norm", "q_norm", "k_norm", "post_attn_norm", "ffn_norm", "post_ffw_norm")]


class Gemma(_RowAdoption):
    """CPU greedy decoder over the same packed weights the HIP path uses.

    ``weights`` is the dict produced by ``ksearch_amd.synth.gemma_weights``:
    per-layer arrays under ``layers[i][name]`` plus ``token_embd`` and
    ``output_norm``.  Arrays are kept alive for the oracle's lifetime.
    """

    def __init__(self, cfg: dict, weights: dict):
        self._keep = weights
        self.cfg = GemmaCfg(**cfg)
        n = cfg["n_layers"]
        arr = (GemmaLayer * n)()
        for i, lw in enumerate(weights["layers"]):
            for name, _ in GemmaLayer._fields_:
                setattr(arr[i], name, _p(lw[name]))
        self._layers = arr
        self.h = lib().ko_gemma_create(C.byref(self.cfg), arr, _p(weights["token_embd"]),
                                       _p(weights["output_norm"]))
        self.vocab = cfg["vocab"]

    def reset(self):
        lib().ko_gemma_reset(self.h)

    @property
    def pos(self) -> int:
        return lib().ko_gemma_pos(self.h)

    _set_sync = "ko_gemma_set_row_sync"

    def forward(self, token: int, want_logits: bool = True, return_logits: bool = False, threads: int = 0,
                adopt_rows=None):
        logits = np.empty(self.vocab, dtype=np.float32) if return_logits else None
        nxt = self._forward_adopting(
            lambda: lib().ko_gemma_forward(self.h, int(token), int(want_logits),
                                           _p(logits) if logits is not None else None, threads),
            self.cfg.n_layers, adopt_rows)
        return (nxt, logits) if return_logits else nxt

    def kv(self, layer: int, which: int, nbytes: int) -> np.ndarray:
        ptr = lib().ko_gemma_kv(self.h, layer, which)
        return np.ctypeslib.as_array(C.cast(ptr, C.POINTER(C.c_uint8)), shape=(nbytes,)).copy()

    def hidden(self) -> np.ndarray:
        ptr = lib().ko_gemma_hidden(self.h)
        return np.ctypeslib.as_array(C.cast(ptr, C.POINTER(C.c_float)), shape=(self.cfg.hidden,)).copy()

    def close(self):
        if self.h:
            lib().ko_gemma_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def rmsnorm_per_head(x, w, n_heads, hd, eps, rope_row=None) -> np.ndarray:
    x, w = _f32(x), _f32(w)
    r = _f32(rope_row) if rope_row is not None else None
    out = np.empty(n_heads * hd, dtype=np.float32)
    lib().ko_rmsnorm_per_head(_p(x), _p(w), _p(r) if r is not None else None, n_heads, hd, eps, _p(out))
    return out


def add_scale(a, b, scale) -> np.ndarray:
    a, b = _f32(a), _f32(b)
    out = np.empty_like(a)
    lib().ko_add_scale(_p(a), _p(b), scale, a.size, _p(out))
    return out


def matvec_gelu_mul(dtype, w, rows, cols, x, ctx, threads=0) -> np.ndarray:
    w, x, ctx = _u8(w), _f32(x), _f32(ctx)
    y = np.empty(rows, dtype=np.float32)
    if lib().ko_matvec_gelu_mul(dtype, _p(w), rows, cols, _p(x), _p(ctx), _p(y), threads):
        raise ValueError("bad dtype/shape")
    return y


G4_CFG_INTS = ("n_layers", "hidden", "n_q", "n_kv", "vocab", "max_seq", "hd_swa", "hd_full", "sliding_window",
               "shared_kv_layers", "ple_dim")
G4_CFG_FLOATS = ("eps", "softcap", "rope_theta_swa", "rope_theta_full", "partial_rotary", "attn_scale")
G4_DTYPES = ("dt_q", "dt_k", "dt_v", "dt_o", "dt_gate", "dt_up", "dt_down", "dt_inp_gate", "dt_proj")
G4_WEIGHTS = ("wq", "wk", "wv", "wo", "wgate", "wup", "wdown", "inp_gate", "proj")
G4_NORMS = ("attn_norm", "q_norm", "k_norm", "post_attn_norm", "ffn_norm", "post_ffw_norm", "post_norm")


class Gemma4Cfg(C.Structure):
    _fields_ = [(n, C.c_int) for n in G4_CFG_INTS] + [(n, C.c_float) for n in G4_CFG_FLOATS]


class Gemma4Layer(C.Structure):
    _fields_ = [("is_swa", C.c_int), ("ffn", C.c_int)] + [(n, C.c_int) for n in G4_DTYPES] + \
               [(n, C.c_void_p) for n in G4_WEIGHTS + G4_NORMS] + [("layer_scale", C.c_float)]


class Gemma4Globals(C.Structure):
    _fields_ = [("token_embd", C.c_void_p), ("dt_embd", C.c_int), ("output_norm", C.c_void_p),
                ("ple_embd", C.c_void_p), ("dt_ple", C.c_int), ("ple_model_proj", C.c_void_p),
                ("dt_ple_proj", C.c_int), ("ple_proj_norm", C.c_void_p)]


class Gemma4(_RowAdoption):
    """CPU greedy decoder with the real checkpoints' layer features, over the
    same packed host arrays the HIP path uploads (``cfg`` / ``weights`` as for
    ``ksearch_amd.hip.Gemma4``; dtype codes are the shared 0..6 numbering)."""

    def __init__(self, cfg: dict, weights: dict):
        self._keep = weights
        self.cfg = Gemma4Cfg(**{k: cfg[k] for k in G4_CFG_INTS + G4_CFG_FLOATS})
        n = cfg["n_layers"]
        arr = (Gemma4Layer * n)()
        for i, lw in enumerate(weights["layers"]):
            arr[i].is_swa, arr[i].ffn = int(lw["is_swa"]), int(lw["ffn"])
            arr[i].layer_scale = float(lw.get("layer_scale", 1.0))
            for name in G4_DTYPES:
                setattr(arr[i], name, int(lw.get(name, Q4K)))
            for name in G4_WEIGHTS + G4_NORMS:
                a = lw.get(name)
                setattr(arr[i], name, _p(a) if a is not None else None)
        self._layers = arr
        g, gw = Gemma4Globals(), weights["globals"]
        for name in ("token_embd", "output_norm", "ple_embd", "ple_model_proj", "ple_proj_norm"):
            a = gw.get(name)
            setattr(g, name, _p(a) if a is not None else None)
        for name in ("dt_embd", "dt_ple", "dt_ple_proj"):
            setattr(g, name, int(gw.get(name, Q4K)))
        self._globals = g
        self.h = lib().ko_gemma4_create(C.byref(self.cfg), arr, C.byref(g))
        self.vocab = cfg["vocab"]

    def reset(self):
        lib().ko_gemma4_reset(self.h)

    @property
    def pos(self) -> int:
        return lib().ko_gemma4_pos(self.h)

    def kv_source(self, layer: int) -> int:
        return lib().ko_gemma4_kv_source(self.h, layer)

    _set_sync = "ko_gemma4_set_row_sync"

    def forward(self, token: int, want_logits: bool = True, return_logits: bool = False, threads: int = 0,
                adopt_rows=None):
        logits = np.empty(self.vocab, dtype=np.float32) if return_logits else None
        nxt = self._forward_adopting(
            lambda: lib().ko_gemma4_forward(self.h, int(token), int(want_logits),
                                            _p(logits) if logits is not None else None, threads),
            self.cfg.n_layers, adopt_rows)
        return (nxt, logits) if return_logits else nxt

    def kv(self, layer: int, which: int, nbytes: int) -> np.ndarray:
        ptr = lib().ko_gemma4_kv(self.h, layer, which)
        return np.ctypeslib.as_array(C.cast(ptr, C.POINTER(C.c_uint8)), shape=(nbytes,)).copy()

    def hidden(self) -> np.ndarray:
        ptr = lib().ko_gemma4_hidden(self.h)
        return np.ctypeslib.as_array(C.cast(ptr, C.POINTER(C.c_float)), shape=(self.cfg.hidden,)).copy()

    def close(self):
        if self.h:
            lib().ko_gemma4_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def sample_softcap_min_p(logits, cap, temperature, min_p=0.05, seed=1) -> int:
    x = _f32(logits)
    return lib().ko_sample_softcap_min_p(_p(x), x.size, cap, temperature, min_p, seed)
