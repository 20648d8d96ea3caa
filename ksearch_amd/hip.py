"""ctypes binding of libksearch_hip.so (include/ksearch_hip.h).

``Context`` carries the method names of ksearch's ``MetalContext``
(crates/ksearch_metal/src/lib.rs) and ``Eng`` those of
``ksearch_kernels::Eng`` (crates/ksearch_kernels/src/lib.rs), so code and
tests written against the reference's runtime read the same here.  This
module never computes anything itself: if the shared library is missing, or
no gfx950 GPU is usable, it raises.
"""
from __future__ import annotations

import ctypes as C
import enum
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libksearch_hip.so")


class KshError(RuntimeError):
    pass


class DType(enum.IntEnum):          # crates/ksearch_ir/src/lib.rs:17-27
    F32 = 0
    F16 = 1
    Q4K = 2
    Q5K = 3
    Q6K = 4
    Q40 = 5
    BF16 = 6
    Q6K_ROWS = 7                    # Q6_K regrouped by field inside every row (ksearch_hip.h)


class Kind(enum.IntEnum):           # enum ksh_kind
    MATVEC = 1
    MATVEC_BATCH = 2
    MATVEC_QKV = 3
    MATVEC_GATE_UP_GELU = 4
    SDPA_NAIVE = 5
    SDPA_MWG_PART = 6
    SDPA_MWG_REDUCE = 7
    SDPA_SLOTS = 8
    QUANTIZE_Q40 = 9
    RMSNORM = 10
    RMSNORM_ADD_THEN_RMSNORM = 11
    RMSNORM_PER_HEAD_QKV_Q40 = 12
    COPY_SCALE_INDEXED = 13
    GELU_MUL = 14
    COPY_SLICE = 15
    SOFTCAP_ARGMAX = 16
    DEQUANT = 17
    QUANTIZE_K = 18
    RMSNORM_MATVEC = 19
    RMSNORM_MATVEC_QKV = 20
    RMSNORM_MATVEC_GATE_UP_GELU = 21
    ATTEND_DECODE = 22
    ATTN_MERGE_MATVEC = 23
    REPACK_ROWS = 24
    RMSNORM_PER_HEAD = 25
    ADD_SCALE = 26
    MATVEC_GELU_MUL = 27
    READ_FLOOR = 28
    SDPA_BATCH = 29
    ROUND_PREP = 30
    MATVEC_ROUND = 31


class Sched(C.Structure):           # ksh_sched: OptSchedule retargeted to gfx950
    _fields_ = [("tg", C.c_uint64), ("vec", C.c_uint32), ("unroll", C.c_uint32), ("nsg", C.c_uint32),
                ("nr0", C.c_uint32), ("k_split", C.c_uint32), ("lds_tile", C.c_uint32)]

    def as_dict(self) -> dict:
        return {n: int(getattr(self, n)) for n, _ in self._fields_}


class KernelDesc(C.Structure):
    _fields_ = [("kind", C.c_int32), ("dtypes", C.c_int32 * 4), ("dims", C.c_int64 * 8),
                ("params", C.c_float * 4), ("sched", Sched)]


class KernelInfo(C.Structure):
    _fields_ = [("n_inputs", C.c_int32), ("n_outputs", C.c_int32), ("grid", C.c_uint32 * 3),
                ("block", C.c_uint32 * 3), ("lds_bytes", C.c_uint32), ("sched", Sched), ("name", C.c_char * 64)]


class GemmaCfg(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n_layers", "hidden", "ffn", "n_q", "n_kv", "hd", "vocab", "max_seq")] + \
               [(n, C.c_float) for n in ("eps", "softcap", "rope_theta", "attn_scale")]


GEMMA_LAYER_FIELDS = ("wq", "wk", "wv", "wo", "wgate", "wup", "wdown",
                      "attn_norm", "q_norm", "k_norm", "post_attn_norm", "ffn_norm", "post_ffw_norm")


class GemmaLayer(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in GEMMA_LAYER_FIELDS]


GEMMA4_CFG_INTS = ("n_layers", "hidden", "n_q", "n_kv", "vocab", "max_seq", "hd_swa", "hd_full", "sliding_window",
                   "shared_kv_layers", "ple_dim")
GEMMA4_CFG_FLOATS = ("eps", "softcap", "rope_theta_swa", "rope_theta_full", "partial_rotary", "attn_scale")
GEMMA4_WEIGHTS = ("wq", "wk", "wv", "wo", "wgate", "wup", "wdown", "inp_gate", "proj")
GEMMA4_NORMS = ("attn_norm", "q_norm", "k_norm", "post_attn_norm", "ffn_norm", "post_ffw_norm", "post_norm")
GEMMA4_DTYPES = ("dt_q", "dt_k", "dt_v", "dt_o", "dt_gate", "dt_up", "dt_down", "dt_inp_gate", "dt_proj")


class Gemma4Cfg(C.Structure):
    _fields_ = [(n, C.c_int32) for n in GEMMA4_CFG_INTS] + [(n, C.c_float) for n in GEMMA4_CFG_FLOATS]


class Gemma4Layer(C.Structure):
    _fields_ = [("is_swa", C.c_int32), ("ffn", C.c_int32)] + [(n, C.c_int32) for n in GEMMA4_DTYPES] + \
               [(n, C.c_void_p) for n in GEMMA4_WEIGHTS + GEMMA4_NORMS] + [("layer_scale", C.c_float)]


class Gemma4Globals(C.Structure):
    _fields_ = [("token_embd", C.c_void_p), ("dt_embd", C.c_int32), ("output_norm", C.c_void_p),
                ("ple_embd", C.c_void_p), ("dt_ple", C.c_int32), ("ple_model_proj", C.c_void_p),
                ("dt_ple_proj", C.c_int32), ("ple_proj_norm", C.c_void_p)]


SERVE_STOP_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_uint64, C.c_uint32)


class ServeCfg(C.Structure):
    _fields_ = [("slots", C.c_int32), ("prefill_chunk", C.c_int32), ("prefill_tokens_per_tick", C.c_int32),
                ("eos", C.c_uint32 * 2), ("use_graph", C.c_int32), ("batched_decode", C.c_int32), ("stop", SERVE_STOP_FN),
                ("stop_user", C.c_void_p)]


class ServeEvent(C.Structure):
    _fields_ = [("request", C.c_uint64), ("kind", C.c_int32), ("token", C.c_uint32), ("reason", C.c_int32),
                ("prompt_tokens", C.c_uint32), ("completion_tokens", C.c_uint32)]


# every symbol include/ksearch_hip.h declares: name -> (restype, argtypes)
_vp, _sz, _i, _u64p, _dp = C.c_void_p, C.c_size_t, C.c_int, C.POINTER(C.c_uint64), C.POINTER(C.c_double)
_vpp = C.POINTER(C.c_void_p)
_i64p = C.POINTER(C.c_int64)
SYMBOLS = {
    "ksh_last_error": (C.c_char_p, []),
    "ksh_ctx_create": (_i, [_vpp]),
    "ksh_ctx_destroy": (None, [_vp]),
    "ksh_device_name": (_i, [_vp, C.c_char_p, _sz]),
    "ksh_stream": (_vp, [_vp]),
    "ksh_buffer_alloc": (_i, [_vp, _sz, _vp, _vpp]),
    "ksh_buffer_retain": (None, [_vp]),
    "ksh_buffer_release": (None, [_vp]),
    "ksh_buffer_size": (_sz, [_vp]),
    "ksh_buffer_device_ptr": (_vp, [_vp]),
    "ksh_buffer_write": (_i, [_vp, _vp, _sz, _vp, _sz, _i]),
    "ksh_buffer_read": (_i, [_vp, _vp, _sz, _vp, _sz, _i]),
    "ksh_buffer_fill_zero": (_i, [_vp, _vp]),
    "ksh_kernel_get": (_i, [_vp, C.POINTER(KernelDesc), _vpp]),
    "ksh_kernel_info_get": (_i, [_vp, C.POINTER(KernelInfo)]),
    "ksh_encode": (_i, [_vp, _vp, _vpp, _u64p, _i, _vpp, _u64p, _i]),
    "ksh_softcap_argmax_static": (_i, [_vp, _vp, C.c_uint64, C.c_int64, C.c_float, _vp, C.c_uint64]),
    "ksh_run_timed": (_i, [_vp, _vp, _vpp, _u64p, _i, _vpp, _u64p, _i, _i, _dp]),
    "ksh_beam_search_chain": (_i, [_vp, C.POINTER(KernelDesc), _i, _vpp, _i, _vpp, _i, _i, _i, C.POINTER(Sched), _dp, C.POINTER(C.c_int)]),
    "ksh_flush_async": (_i, [_vp]),
    "ksh_wait_inflight_at_most": (_i, [_vp, _i]),
    "ksh_barrier": (_i, [_vp]),
    "ksh_synchronize": (_i, [_vp]),
    "ksh_has_gpu_work": (_i, [_vp]),
    "ksh_graph_begin": (_i, [_vp]),
    "ksh_graph_end": (_i, [_vp, _vpp]),
    "ksh_graph_launch": (_i, [_vp, _vp]),
    "ksh_graph_destroy": (None, [_vp]),
    "ksh_plan_key": (_i, [C.c_char_p, _i64p, _i, C.c_char_p, C.c_char_p, _sz]),
    "ksh_plan_save": (_i, [C.c_char_p, _i64p, _i, C.c_char_p, C.POINTER(Sched), C.c_double]),
    "ksh_plan_load": (_i, [C.c_char_p, _i64p, _i, C.c_char_p, C.POINTER(Sched), _dp]),
    "ksh_plan_kind": (C.c_char_p, [C.POINTER(KernelDesc)]),
    "ksh_beam_candidates": (_i, [C.POINTER(KernelDesc), C.POINTER(Sched), _i]),
    "ksh_beam_search": (_i, [_vp, C.POINTER(KernelDesc), _vpp, _i, _vpp, _i, _i, _i, C.POINTER(Sched), _dp,
                             C.POINTER(C.c_int)]),
    "ksh_gemma_create": (_i, [_vp, C.POINTER(GemmaCfg), C.POINTER(GemmaLayer), _vp, _vp, _vpp]),
    "ksh_gemma_destroy": (None, [_vp]),
    "ksh_gemma_reset": (_i, [_vp]),
    "ksh_gemma_forward_token": (_i, [_vp, C.c_uint32, _i, C.POINTER(C.c_uint32)]),
    "ksh_gemma_prefill_chunk": (_i, [_vp, C.POINTER(C.c_uint32), _i]),
    "ksh_gemma_generate": (_i, [_vp, C.POINTER(C.c_uint32), _i, _i, _i, C.POINTER(C.c_uint32), _dp, _dp]),
    "ksh_gemma_logits": (_vp, [_vp]),
    "ksh_gemma_hidden": (_vp, [_vp]),
    "ksh_gemma_kv": (_vp, [_vp, _i, _i]),
    "ksh_gemma_pos": (_i, [_vp]),
    "ksh_gemma_launches_per_token": (_i, [_vp]),
    "ksh_gemma4_create": (_i, [_vp, C.POINTER(Gemma4Cfg), C.POINTER(Gemma4Layer), C.POINTER(Gemma4Globals), _vpp]),
    "ksh_gemma4_destroy": (None, [_vp]),
    "ksh_gemma4_reset": (_i, [_vp]),
    "ksh_gemma4_forward_token": (_i, [_vp, C.c_uint32, _i, _i, C.POINTER(C.c_uint32)]),
    "ksh_gemma4_generate": (_i, [_vp, C.POINTER(C.c_uint32), _i, _i, _i, C.POINTER(C.c_uint32), _dp, _dp]),
    "ksh_gemma4_generate_until": (_i, [_vp, C.POINTER(C.c_uint32), _i, _i, C.POINTER(C.c_uint32), _i, _i, C.POINTER(C.c_uint32),
                                       C.POINTER(C.c_int), _dp, _dp]),
    "ksh_gemma4_logits": (_vp, [_vp]),
    "ksh_gemma4_hidden": (_vp, [_vp]),
    "ksh_gemma4_kv_source": (_i, [_vp, _i]),
    "ksh_gemma4_kv": (_vp, [_vp, _i, _i]),
    "ksh_gemma4_pos": (_i, [_vp]),
    "ksh_gemma4_launches_per_token": (_i, [_vp]),
    "ksh_gemma4_config": (_i, [_vp, C.POINTER(Gemma4Cfg)]),
    "ksh_kvpool_create": (_i, [_vp, _i, _i, _i, _i, _i, _vpp]),
    "ksh_kvpool_destroy": (None, [_vp]),
    "ksh_kvpool_alloc": (_i, [_vp, C.POINTER(C.c_int)]),
    "ksh_kvpool_free": (_i, [_vp, _i]),
    "ksh_kvpool_clear_slot": (_i, [_vp, _i]),
    "ksh_kvpool_seq_len": (_i, [_vp, _i]),
    "ksh_kvpool_occupied": (_i, [_vp, _i]),
    "ksh_kvpool_bump_len_by": (_i, [_vp, _i, _i, C.POINTER(C.c_int)]),
    "ksh_kvpool_active_batch": (_i, [_vp, C.POINTER(C.c_int), _i]),
    "ksh_kvpool_k": (_vp, [_vp, _i, _i]),
    "ksh_kvpool_v": (_vp, [_vp, _i, _i]),
    "ksh_kvpool_layer_k": (_vp, [_vp, _i]),
    "ksh_kvpool_layer_v": (_vp, [_vp, _i]),
    "ksh_kvpool_dims": (_i, [_vp] + [C.POINTER(C.c_int)] * 5),
    "ksh_gemma4_bind_slot": (_i, [_vp, _vp, _i]),
    "ksh_gemma4_decode_token_sampled": (_i, [_vp, C.c_uint32, C.c_float, C.c_float, C.c_uint32, _i, C.POINTER(C.c_uint32)]),
    "ksh_gemma4_prefill_chunk": (_i, [_vp, C.POINTER(C.c_uint32), _i, _i]),
    "ksh_gemma4_decode_round": (_i, [_vp, _vp, C.POINTER(C.c_int32), C.POINTER(C.c_uint32), _i, C.POINTER(C.c_float), C.POINTER(C.c_float),
                                     C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]),
    "ksh_gemma4_round_logits": (_vp, [_vp]),
    "ksh_serve_default_cfg": (_i, [C.POINTER(ServeCfg)]),
    "ksh_serve_create": (_i, [_vp, _vp, C.POINTER(ServeCfg), _vpp]),
    "ksh_serve_destroy": (None, [_vp]),
    "ksh_serve_submit": (_i, [_vp, C.POINTER(C.c_uint32), _sz, _sz, C.c_float, C.c_float, C.c_uint32, _u64p]),
    "ksh_serve_cancel": (_i, [_vp, C.c_uint64]),
    "ksh_serve_tick": (_i, [_vp]),
    "ksh_serve_poll": (_sz, [_vp, C.POINTER(ServeEvent), _sz]),
    "ksh_serve_error_text": (C.c_char_p, [_vp]),
    "ksh_serve_pending": (_i, [_vp, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "ksh_sample_softcap_min_p": (_i, [_vp, _sz, C.c_float, C.c_float, C.c_float, C.c_uint32, C.POINTER(C.c_uint32)]),
    "ksh_gguf_open": (_i, [C.c_char_p, _vpp]),
    "ksh_gguf_close": (None, [_vp]),
    "ksh_gguf_version": (_i, [_vp]),
    "ksh_gguf_n_tensors": (C.c_int64, [_vp]),
    "ksh_gguf_tensor_name": (_i, [_vp, C.c_int64, C.c_char_p, _sz]),
    "ksh_gguf_has_tensor": (_i, [_vp, C.c_char_p]),
    "ksh_gguf_tensor": (_i, [_vp, C.c_char_p, C.POINTER(C.c_int32), _i64p, C.POINTER(C.c_int32), _vpp, C.POINTER(_sz)]),
    "ksh_gguf_get_u32": (_i, [_vp, C.c_char_p, C.POINTER(C.c_uint32)]),
    "ksh_gguf_get_f32": (_i, [_vp, C.c_char_p, C.POINTER(C.c_float)]),
    "ksh_gguf_get_str": (_i, [_vp, C.c_char_p, C.c_char_p, _sz]),
    "ksh_gguf_get_arr_u32": (_i, [_vp, C.c_char_p, C.POINTER(C.c_uint32), _i, C.POINTER(C.c_int)]),
    "ksh_gguf_arr_is_bool": (_i, [_vp, C.c_char_p]),
    "ksh_gguf_dequant_host": (_i, [C.c_int32, _vp, _sz, _vp]),
    "ksh_gemma4_config_from_gguf": (_i, [_vp, _i, C.POINTER(Gemma4Cfg), C.POINTER(C.c_int32), C.POINTER(C.c_int32), _i]),
    "ksh_gemma4_load_gguf": (_i, [_vp, _vp, _i, _i, _vpp]),
}

_lib = None


def lib() -> C.CDLL:
    """Loads the prebuilt library; never builds and never falls back."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise KshError(f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'`")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def _check(rc: int) -> None:
    if rc:
        raise KshError(lib().ksh_last_error().decode(errors="replace"))


def make_desc(kind: int, dims=(), dtypes=(), params=(), sched: Sched | dict | None = None) -> KernelDesc:
    d = KernelDesc()
    d.kind = int(kind)
    for i, v in enumerate(dims):
        d.dims[i] = int(v)
    for i, v in enumerate(dtypes):
        d.dtypes[i] = int(v)
    for i, v in enumerate(params):
        d.params[i] = float(v)
    if isinstance(sched, dict):
        sched = Sched(**sched)
    if sched is not None:
        d.sched = sched
    return d


def plan_kind(desc: KernelDesc) -> str | None:
    r = lib().ksh_plan_kind(C.byref(desc))
    return r.decode() if r else None


def plan_key(kind: str, dims, chip: str) -> str:
    arr = (C.c_int64 * len(dims))(*dims)
    buf = C.create_string_buffer(256)
    _check(lib().ksh_plan_key(kind.encode(), arr, len(dims), chip.encode(), buf, 256))
    return buf.value.decode()


def plan_save(kind: str, dims, chip: str, sched: Sched, ms: float) -> None:
    arr = (C.c_int64 * len(dims))(*dims)
    _check(lib().ksh_plan_save(kind.encode(), arr, len(dims), chip.encode(), C.byref(sched), ms))


def plan_load(kind: str, dims, chip: str):
    arr = (C.c_int64 * len(dims))(*dims)
    s, ms = Sched(), C.c_double()
    rc = lib().ksh_plan_load(kind.encode(), arr, len(dims), chip.encode(), C.byref(s), C.byref(ms))
    return (s, ms.value) if rc == 0 else None


def beam_candidates(desc: KernelDesc, cap: int = 128) -> list[Sched]:
    arr = (Sched * cap)()
    n = lib().ksh_beam_candidates(C.byref(desc), arr, cap)
    return [arr[i] for i in range(n)]


class Buffer:
    """A device allocation (the reference's metal::Buffer)."""

    def __init__(self, ctx: "Context", handle: int, owned: bool = True):
        self.ctx, self.h, self._owned = ctx, handle, owned

    @property
    def nbytes(self) -> int:
        return lib().ksh_buffer_size(self.h)

    @property
    def device_ptr(self) -> int:
        return lib().ksh_buffer_device_ptr(self.h)

    def release(self) -> None:
        if self.h and self._owned:
            lib().ksh_buffer_release(self.h)
        self.h = None

    def __del__(self):
        try:
            self.release()
        except Exception:
            pass


class Kernel:
    def __init__(self, handle: int):
        self.h = handle
        info = KernelInfo()
        _check(lib().ksh_kernel_info_get(handle, C.byref(info)))
        self.info = info

    @property
    def name(self) -> str:
        return self.info.name.decode()

    @property
    def grid(self):
        return tuple(self.info.grid)

    @property
    def block(self):
        return tuple(self.info.block)


def _bufs(bufs):
    arr = (C.c_void_p * max(1, len(bufs)))(*[b.h for b in bufs])
    return arr


def _offs(offs, n):
    if offs is None:
        return None
    return (C.c_uint64 * max(1, n))(*[int(o) for o in offs])


class Context:
    """MetalContext for one MI355X: device 0, one in-order HIP stream."""

    def __init__(self):
        h = C.c_void_p()
        _check(lib().ksh_ctx_create(C.byref(h)))
        self.h = h

    # -- lifetime -----------------------------------------------------------
    def close(self) -> None:
        if self.h:
            lib().ksh_ctx_destroy(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    def device_name(self) -> str:
        buf = C.create_string_buffer(128)
        _check(lib().ksh_device_name(self.h, buf, 128))
        return buf.value.decode()

    @property
    def stream(self) -> int:
        return lib().ksh_stream(self.h)

    # -- buffers (crates/ksearch_metal/src/lib.rs:63-135) -------------------
    def _alloc(self, nbytes: int, init) -> Buffer:
        h = C.c_void_p()
        _check(lib().ksh_buffer_alloc(self.h, nbytes, init, C.byref(h)))
        return Buffer(self, h.value)

    def buffer_bytes(self, data) -> Buffer:
        a = np.ascontiguousarray(data)
        return self._alloc(a.nbytes, a.ctypes.data)

    def buffer_f32(self, data) -> Buffer:
        return self.buffer_bytes(np.ascontiguousarray(data, dtype=np.float32))

    def buffer_empty_bytes(self, n: int) -> Buffer:
        return self._alloc(int(n), None)

    def buffer_empty_f32(self, n: int) -> Buffer:
        return self._alloc(int(n) * 4, None)

    def buffer_empty_f16(self, n: int) -> Buffer:
        return self._alloc(int(n) * 2, None)

    def _read(self, buf: Buffer, dtype, n: int, off: int, sync: bool) -> np.ndarray:
        out = np.empty(n, dtype=dtype)
        _check(lib().ksh_buffer_read(self.h, buf.h, off, out.ctypes.data, out.nbytes, int(sync)))
        return out

    def read_f32(self, buf: Buffer, n: int, off: int = 0) -> np.ndarray:
        return self._read(buf, np.float32, n, off, True)

    def read_f32_nosync(self, buf: Buffer, n: int, off: int = 0) -> np.ndarray:
        return self._read(buf, np.float32, n, off, False)

    def read_u16(self, buf: Buffer, n: int, off: int = 0) -> np.ndarray:
        return self._read(buf, np.uint16, n, off, True)

    def read_bytes(self, buf: Buffer, n: int, off: int = 0) -> np.ndarray:
        return self._read(buf, np.uint8, n, off, True)

    def _write(self, buf: Buffer, data, off: int, sync: bool) -> None:
        a = np.ascontiguousarray(data)
        _check(lib().ksh_buffer_write(self.h, buf.h, off, a.ctypes.data, a.nbytes, int(sync)))

    def write_buffer(self, buf: Buffer, data, off: int = 0) -> None:
        self._write(buf, np.ascontiguousarray(data, dtype=np.float32), off, True)

    def write_buffer_nosync(self, buf: Buffer, data, off: int = 0) -> None:
        self._write(buf, np.ascontiguousarray(data, dtype=np.float32), off, False)

    def write_u16s(self, buf: Buffer, data, off: int = 0) -> None:
        self._write(buf, np.ascontiguousarray(data, dtype=np.uint16), off, True)

    def write_bytes(self, buf: Buffer, data, off: int = 0, sync: bool = True) -> None:
        self._write(buf, data, off, sync)

    def fill_zero(self, buf: Buffer) -> None:
        _check(lib().ksh_buffer_fill_zero(self.h, buf.h))

    # -- kernels ------------------------------------------------------------
    def compile(self, desc: KernelDesc) -> Kernel:
        h = C.c_void_p()
        _check(lib().ksh_kernel_get(self.h, C.byref(desc), C.byref(h)))
        return Kernel(h.value)

    def encode_offsets_multi(self, kernel: Kernel, inputs, in_offs, outputs, out_offs) -> None:
        _check(lib().ksh_encode(self.h, kernel.h, _bufs(inputs), _offs(in_offs, len(inputs)), len(inputs),
                                _bufs(outputs), _offs(out_offs, len(outputs)), len(outputs)))

    def encode_multi(self, kernel: Kernel, inputs, outputs) -> None:
        self.encode_offsets_multi(kernel, inputs, None, outputs, None)

    def encode(self, kernel: Kernel, inputs, output) -> None:
        self.encode_offsets_multi(kernel, inputs, None, [output], None)

    def run(self, kernel: Kernel, inputs, outputs, iters: int = 1, in_offs=None, out_offs=None) -> float:
        """Timed launches with HIP events on the context's stream; ms per launch."""
        if isinstance(outputs, Buffer):
            outputs = [outputs]
        ms = C.c_double()
        _check(lib().ksh_run_timed(self.h, kernel.h, _bufs(inputs), _offs(in_offs, len(inputs)), len(inputs),
                                   _bufs(outputs), _offs(out_offs, len(outputs)), len(outputs), iters,
                                   C.byref(ms)))
        return ms.value

    def flush_async(self) -> None:
        _check(lib().ksh_flush_async(self.h))

    def wait_inflight_at_most(self, n: int) -> None:
        _check(lib().ksh_wait_inflight_at_most(self.h, n))

    def encoder_barrier(self) -> None:
        _check(lib().ksh_barrier(self.h))

    def synchronize(self) -> None:
        _check(lib().ksh_synchronize(self.h))

    def has_gpu_work(self) -> bool:
        return bool(lib().ksh_has_gpu_work(self.h))

    # -- graphs -------------------------------------------------------------
    def graph_begin(self) -> None:
        _check(lib().ksh_graph_begin(self.h))

    def graph_end(self) -> int:
        g = C.c_void_p()
        _check(lib().ksh_graph_end(self.h, C.byref(g)))
        return g.value

    def graph_launch(self, g: int) -> None:
        _check(lib().ksh_graph_launch(self.h, g))

    def graph_destroy(self, g: int) -> None:
        lib().ksh_graph_destroy(g)

    # -- BEAM ---------------------------------------------------------------
    def beam_search(self, desc: KernelDesc, inputs, outputs, iters: int = 3, force: bool = False):
        best, ms, cached = Sched(), C.c_double(), C.c_int()
        _check(lib().ksh_beam_search(self.h, C.byref(desc), _bufs(inputs), len(inputs), _bufs(outputs),
                                     len(outputs), iters, int(force), C.byref(best), C.byref(ms), C.byref(cached)))
        return best, ms.value, bool(cached.value)

    def beam_search_chain(self, desc: KernelDesc, input_sets, output_sets, iters: int = 3, force: bool = False):
        """Every candidate timed as one graph of len(input_sets) dependent launches, launch i over set i."""
        n_sets, n_in, n_out = len(input_sets), len(input_sets[0]), len(output_sets[0])
        assert len(output_sets) == n_sets and all(len(s) == n_in for s in input_sets) and all(len(s) == n_out for s in output_sets)
        best, ms, cached = Sched(), C.c_double(), C.c_int()
        _check(lib().ksh_beam_search_chain(self.h, C.byref(desc), n_sets, _bufs([b for s in input_sets for b in s]), n_in,
                                           _bufs([b for s in output_sets for b in s]), n_out, iters, int(force),
                                           C.byref(best), C.byref(ms), C.byref(cached)))
        return best, ms.value, bool(cached.value)


class Eng:
    """One method per op, named as in ksearch_kernels::Eng.  Each call looks up
    (or binds) the kernel for its shape and appends one launch to the stream."""

    SDPA_MWG_NWG = 16           # crates/ksearch_kernels/src/lib.rs:1114
    SDPA_MWG_THRESHOLD = 128    # :1115

    def __init__(self):
        self.cache: dict = {}

    def _k(self, ctx: Context, kind, dims=(), dtypes=(), params=(), sched=None) -> Kernel:
        key = (int(kind), tuple(dims), tuple(int(d) for d in dtypes), tuple(params),
               tuple(sorted(sched.items())) if isinstance(sched, dict) else None)
        k = self.cache.get(key)
        if k is None:
            k = ctx.compile(make_desc(kind, dims, dtypes, params, sched))
            self.cache[key] = k
        return k

    # :137-160
    def matvec_wd(self, ctx, rows, cols, wdt, w, x, y, sched=None):
        self.matvec_wd_at(ctx, rows, cols, wdt, w, x, 0, y, 0, sched)

    def matvec_wd_at(self, ctx, rows, cols, wdt, w, x, x_off, y, y_off, sched=None):
        k = self._k(ctx, Kind.MATVEC, (rows, cols), (wdt, DType.F32), (), sched)
        ctx.encode_offsets_multi(k, [w, x], [0, x_off * 4], [y], [y_off * 4])

    # :227-261
    def matvec_qkv_wds(self, ctx, q_rows, kv_rows, cols, wdt, wq, wk, wv, x, q, k_out, v_out, sched=None):
        k = self._k(ctx, Kind.MATVEC_QKV, (q_rows, kv_rows, cols), (wdt, DType.F32), (), sched)
        ctx.encode_multi(k, [wq, wk, wv, x], [q, k_out, v_out])

    # :953-975
    def matvec_gate_up_gelu_wd(self, ctx, rows, cols, wdt, wg, wu, x, out, sched=None):
        k = self._k(ctx, Kind.MATVEC_GATE_UP_GELU, (rows, cols), (wdt, DType.F32), (), sched)
        ctx.encode_multi(k, [wg, wu, x], [out])

    # rmsnorm_matvec_wd / rmsnorm_matvec_qkv_w / rmsnorm_matvec_gate_up_gelu_w (:1233-1236, gemma_prim.rs:948-961,
    # 1121-1130).  With res/w_post given, the residual add of the previous block is folded in as well
    # and the new residual stream comes back in x_new (which must not alias res).
    def rmsnorm_matvec_wd(self, ctx, rows, cols, eps, wdt, x, w_norm, w, y, w_post=None, res=None, x_new=None, sched=None):
        has_res = res is not None
        k = self._k(ctx, Kind.RMSNORM_MATVEC, (rows, cols, int(has_res)), (wdt, DType.F32), (eps,), sched)
        ctx.encode_multi(k, [w, x, w_norm] + ([w_post, res] if has_res else []), [y] + ([x_new] if has_res else []))

    def rmsnorm_matvec_qkv_w(self, ctx, q_rows, kv_rows, cols, eps, wdt, x, w_norm, wq, wk, wv, q, k_out, v_out,
                             w_post=None, res=None, x_new=None, sched=None):
        has_res = res is not None
        k = self._k(ctx, Kind.RMSNORM_MATVEC_QKV, (q_rows, kv_rows, cols, int(has_res)), (wdt, DType.F32), (eps,), sched)
        ctx.encode_multi(k, [wq, wk, wv, x, w_norm] + ([w_post, res] if has_res else []),
                         [q, k_out, v_out] + ([x_new] if has_res else []))

    def rmsnorm_matvec_gate_up_gelu_w(self, ctx, rows, cols, eps, wdt, x, w_norm, wg, wu, out,
                                      w_post=None, res=None, x_new=None, sched=None):
        has_res = res is not None
        k = self._k(ctx, Kind.RMSNORM_MATVEC_GATE_UP_GELU, (rows, cols, int(has_res)), (wdt, DType.F32), (eps,), sched)
        ctx.encode_multi(k, [wg, wu, x, w_norm] + ([w_post, res] if has_res else []), [out] + ([x_new] if has_res else []))

    # the decode step's RmsNormPerHeadQkvQ40 -> SdpaMwgPart -> SdpaMwgReduce (gemma_prim.rs:984-1060) as one launch
    def attend_decode(self, ctx, n_q, n_kv, hd, max_seq, eps, scale, q, q_norm, rope, k, k_norm, v, meta, k_cache, v_cache,
                      tmp, out, nwg=0, sched=None):
        kk = self._k(ctx, Kind.ATTEND_DECODE, (n_q, n_kv, hd, max_seq, nwg), (DType.Q40, DType.F32), (eps, scale), sched)
        ctx.encode_multi(kk, [q, q_norm, rope, k, k_norm, v, meta], [k_cache, v_cache, tmp, out])
        return kk

    # the same without the merge: `parts` = o f32[n_q, nwg, hd] then (m, l) f32[n_q, nwg, 2], for attn_merge_matvec_wd
    def attend_decode_parts(self, ctx, n_q, n_kv, hd, max_seq, eps, scale, q, q_norm, rope, k, k_norm, v, meta, k_cache,
                            v_cache, parts, nwg, sched=None):
        kk = self._k(ctx, Kind.ATTEND_DECODE, (n_q, n_kv, hd, max_seq, nwg, 1), (DType.Q40, DType.F32), (eps, scale), sched)
        ctx.encode_multi(kk, [q, q_norm, rope, k, k_norm, v, meta], [k_cache, v_cache, parts])
        return kk

    # Q6_K -> Q6K_ROWS (a byte permutation inside every row)
    def repack_rows(self, ctx, rows, cols, src, dst):
        k = self._k(ctx, Kind.REPACK_ROWS, (rows, cols), (DType.Q6K, DType.Q6K_ROWS), ())
        ctx.encode_multi(k, [src], [dst])

    # SdpaMwgReduce (lower.rs:5897-6087) folded into the GEMV that consumes the attention output
    def attn_merge_matvec_wd(self, ctx, rows, n_q, hd, nwg, wdt, w, parts, y, sched=None):
        k = self._k(ctx, Kind.ATTN_MERGE_MATVEC, (rows, n_q, hd, nwg), (wdt, DType.F32), (), sched)
        ctx.encode_multi(k, [w, parts], [y])
        return k

    # :1414-1444
    def matvec_batch(self, ctx, rows, cols, batch, wdt, w, x, y, sched=None):
        k = self._k(ctx, Kind.MATVEC_BATCH, (rows, cols, batch), (wdt, DType.BF16, DType.F32), (), sched)
        ctx.encode_multi(k, [w, x], [y])

    # :468-490
    def rmsnorm(self, ctx, n, eps, x, w, out):
        k = self._k(ctx, Kind.RMSNORM, (n, 0, 0), (), (eps, 0.0))
        ctx.encode_multi(k, [x, w], [out])

    def rmsnorm_add(self, ctx, n, eps, x, w, res, out):
        k = self._k(ctx, Kind.RMSNORM, (n, 1, 0), (), (eps, 0.0))
        ctx.encode_multi(k, [x, w, res], [out])

    def rmsnorm_add_scale(self, ctx, n, eps, scale, x, w, res, out):
        k = self._k(ctx, Kind.RMSNORM, (n, 1, 1), (), (eps, scale))
        ctx.encode_multi(k, [x, w, res], [out])

    # :539-562
    def rmsnorm_add_then_rmsnorm(self, ctx, n, eps, y, w_post, res, w_ffn, out_x, out_x2):
        k = self._k(ctx, Kind.RMSNORM_ADD_THEN_RMSNORM, (n,), (), (eps,))
        ctx.encode_multi(k, [y, w_post, res, w_ffn], [out_x, out_x2])

    # :1257-1297
    def rmsnorm_per_head_qkv_q40_off(self, ctx, n_q, n_kv, hd, eps, q, qw, rope, rope_off, k, kw, v,
                                     q_out, k_out, v_out, kv_byte_off):
        kk = self._k(ctx, Kind.RMSNORM_PER_HEAD_QKV_Q40, (n_q, n_kv, hd), (), (eps,))
        ctx.encode_offsets_multi(kk, [q, qw, rope, k, kw, v], [0, 0, rope_off * 4, 0, 0, 0],
                                 [q_out, k_out, v_out], [0, kv_byte_off, kv_byte_off])

    # :564-583
    def rmsnorm_per_head(self, ctx, n_heads, hd, eps, x, w, y):
        k = self._k(ctx, Kind.RMSNORM_PER_HEAD, (n_heads, hd, 0), (), (eps,))
        ctx.encode_multi(k, [x, w], [y])

    # :601-632 (offsets in f32 elements)
    def rmsnorm_per_head_rope_off(self, ctx, n_heads, hd, eps, x, w, cos_sin, cos_sin_off, y, y_off=0):
        k = self._k(ctx, Kind.RMSNORM_PER_HEAD, (n_heads, hd, 1), (), (eps,))
        ctx.encode_offsets_multi(k, [x, w, cos_sin], [0, 0, cos_sin_off * 4], [y], [y_off * 4])

    # :918-937
    def add_scale(self, ctx, n, scale, a, b, y):
        k = self._k(ctx, Kind.ADD_SCALE, (n,), (), (scale,))
        ctx.encode_multi(k, [a, b], [y])

    # :791-822
    def matvec_gelu_mul_at(self, ctx, rows, cols, wdt, w, x, ctx_buf, ctx_off, y):
        k = self._k(ctx, Kind.MATVEC_GELU_MUL, (rows, cols), (wdt, DType.F32), ())
        ctx.encode_offsets_multi(k, [w, x, ctx_buf], [0, 0, ctx_off * 4], [y], [0])

    # :897-916: the projection, then rmsnorm_add_scale, as two launches like the reference's
    def matvec_rmsnorm_add_scale(self, ctx, rows, cols, eps, scale, wdt, w, x, w_norm, residual, y, scratch):
        self.matvec_wd(ctx, rows, cols, wdt, w, x, scratch)
        self.rmsnorm_add_scale(ctx, rows, eps, scale, scratch, w_norm, residual, y)

    # :1181-1197
    def quantize_q40(self, ctx, n, src, dst, dst_byte_off=0):
        k = self._k(ctx, Kind.QUANTIZE_Q40, (n,))
        ctx.encode_offsets_multi(k, [src], [0], [dst], [dst_byte_off])

    # :1086-1111
    def sdpa_naive_kv(self, ctx, n_q, n_kv, hd, max_t, kv_dtype, q, k, v, meta, out, scale=1.0):
        kk = self._k(ctx, Kind.SDPA_NAIVE, (n_q, n_kv, hd, max_t), (kv_dtype, DType.F32), (scale,))
        ctx.encode_multi(kk, [q, k, v, meta], [out])

    # :1118-1154
    def sdpa_mwg_kv(self, ctx, n_q, n_kv, hd, max_t, kv_dtype, q, k, v, meta, tmp, out, scale=1.0, nwg=None):
        nwg = nwg or self.SDPA_MWG_NWG
        part = self._k(ctx, Kind.SDPA_MWG_PART, (n_q, n_kv, hd, max_t, nwg), (kv_dtype, DType.F32), (scale,))
        red = self._k(ctx, Kind.SDPA_MWG_REDUCE, (n_q, hd, nwg))
        ctx.encode_multi(part, [q, k, v, meta], [tmp])
        ctx.encoder_barrier()
        ctx.encode_multi(red, [tmp], [out])

    # :1157-1178
    def sdpa_hybrid_kv(self, ctx, n_q, n_kv, hd, max_t, attn_t, kv_dtype, q, k, v, meta, tmp, out, scale=1.0):
        if attn_t >= self.SDPA_MWG_THRESHOLD:
            self.sdpa_mwg_kv(ctx, n_q, n_kv, hd, max_t, kv_dtype, q, k, v, meta, tmp, out, scale)
        else:
            self.sdpa_naive_kv(ctx, n_q, n_kv, hd, max_t, kv_dtype, q, k, v, meta, out, scale)

    def sdpa_slots(self, ctx, n_q, n_kv, hd, max_t, n_slots, q, k_pool, v_pool, meta, tmp, out, scale=1.0,
                   nwg=0, sched=None):
        kk = self._k(ctx, Kind.SDPA_SLOTS, (n_q, n_kv, hd, max_t, n_slots, nwg), (DType.Q40, DType.F32),
                     (scale,), sched)
        ctx.encode_multi(kk, [q, k_pool, v_pool, meta], [tmp, out])
        return kk

    # :1364-1384
    def copy_scale_indexed_wd(self, ctx, n, scale, src_dtype, src, idx, out, n_rows):
        k = self._k(ctx, Kind.COPY_SCALE_INDEXED, (n, n_rows), (src_dtype,), (scale,))
        ctx.encode_multi(k, [src, idx], [out])

    def gelu_mul(self, ctx, n, g, u, out):
        ctx.encode_multi(self._k(ctx, Kind.GELU_MUL, (n,)), [g, u], [out])

    def copy_slice(self, ctx, n, src, src_off, dst, dst_off):
        ctx.encode_offsets_multi(self._k(ctx, Kind.COPY_SLICE, (n,)), [src], [src_off * 4], [dst], [dst_off * 4])

    # :1966-1982
    def softcap_argmax(self, ctx, n, cap, x, out):
        ctx.encode_multi(self._k(ctx, Kind.SOFTCAP_ARGMAX, (n,), (), (cap,)), [x], [out])

    def softcap_argmax_static(self, ctx, n, cap, x, out, x_off=0, out_off=0):
        """The same op through the entry point that allocates nothing (no kernel handle, partial results in a fixed
        array of the device image); no counterpart in the reference."""
        _check(lib().ksh_softcap_argmax_static(ctx.h, x.h, x_off, n, cap, out.h, out_off))

    def dequant(self, ctx, dtype, n, src, dst):
        ctx.encode_multi(self._k(ctx, Kind.DEQUANT, (n,), (dtype,)), [src], [dst])

    def quantize_k(self, ctx, dtype, n, src, dst):
        ctx.encode_multi(self._k(ctx, Kind.QUANTIZE_K, (n,), (dtype,)), [src], [dst])

    # :1985-2043
    def beam_matvec(self, ctx, rows, cols, wdt, w, x, y, iters=3, force=False):
        return ctx.beam_search(make_desc(Kind.MATVEC, (rows, cols), (wdt, DType.F32)), [w, x], [y], iters, force)


def device_quantizers(ctx: Context, eng: Eng):
    """(quantize_q4k, quantize_q6k) for synth.gemma_weights: host f32 arrays go
    up, are packed by the device kernels and stay on the device as Buffers.
    The Q6_K one takes the embedding table as a list of row chunks."""

    def q4k(x: np.ndarray) -> Buffer:
        src = ctx.buffer_f32(x)
        dst = ctx.buffer_empty_bytes(x.size // 256 * 144)
        eng.quantize_k(ctx, DType.Q4K, x.size, src, dst)
        ctx.synchronize()
        src.release()
        return dst

    def q6k(parts) -> Buffer:
        total = sum(p.size for p in parts)
        dst = ctx.buffer_empty_bytes(total // 256 * 210)
        off = 0
        for p_ in parts:
            src = ctx.buffer_f32(p_)
            k = eng._k(ctx, Kind.QUANTIZE_K, (p_.size,), (DType.Q6K,))
            ctx.encode_offsets_multi(k, [src], [0], [dst], [off])
            ctx.synchronize()
            src.release()
            off += p_.size // 256 * 210
        return dst

    return q4k, q6k


class Gemma:
    """GemmaPrimModel for the synthetic Gemma-4-E2B shape
    (crates/ksearch_gemma/src/gemma_prim.rs:76-132, 881-1275, 1658-1768):
    weights packed on the host side are uploaded once; `generate` keeps token
    ids on the device between steps."""

    def __init__(self, ctx: Context, cfg: dict, weights: dict):
        self.ctx, self.cfg = ctx, dict(cfg)
        self._bufs = []

        def up(a):
            b = a if isinstance(a, Buffer) else ctx.buffer_bytes(a)
            self._bufs.append(b)
            return b

        n = cfg["n_layers"]
        arr = (GemmaLayer * n)()
        for i, lw in enumerate(weights["layers"]):
            for name in GEMMA_LAYER_FIELDS:
                setattr(arr[i], name, up(lw[name]).h)
        self._layers = arr
        self._embd, self._onorm = up(weights["token_embd"]), up(weights["output_norm"])
        c = GemmaCfg(**cfg)
        h = C.c_void_p()
        _check(lib().ksh_gemma_create(ctx.h, C.byref(c), arr, self._embd.h, self._onorm.h, C.byref(h)))
        self.h = h

    def close(self):
        if self.h:
            lib().ksh_gemma_destroy(self.h)
            self.h = None
        for b in self._bufs:
            b.release()
        self._bufs = []

    def reset(self):
        _check(lib().ksh_gemma_reset(self.h))

    @property
    def pos(self) -> int:
        return lib().ksh_gemma_pos(self.h)

    @property
    def launches_per_token(self) -> int:
        return lib().ksh_gemma_launches_per_token(self.h)

    def forward_token(self, token: int, use_graph: bool = False, read_next: bool = True):
        nxt = C.c_uint32()
        _check(lib().ksh_gemma_forward_token(self.h, int(token), int(use_graph), C.byref(nxt) if read_next else None))
        return nxt.value if read_next else None

    def prefill_chunk(self, tokens) -> None:
        """prefill_chunk: the tokens at the current position, no logits; batched per layer in chunks of 256."""
        p = (C.c_uint32 * max(1, len(tokens)))(*[int(t) for t in tokens])
        _check(lib().ksh_gemma_prefill_chunk(self.h, p, len(tokens)))

    def generate(self, prompt, n_new: int, use_graph: bool = True, serial_prefill: bool = False):
        p = (C.c_uint32 * len(prompt))(*[int(t) for t in prompt])
        out = (C.c_uint32 * max(1, n_new))()
        pre, dec = C.c_double(), C.c_double()
        flags = int(bool(use_graph)) | (2 if serial_prefill else 0)
        _check(lib().ksh_gemma_generate(self.h, p, len(prompt), n_new, flags, out, C.byref(pre), C.byref(dec)))
        return list(out[:n_new]), pre.value, dec.value

    def logits(self) -> np.ndarray:
        b = Buffer(self.ctx, lib().ksh_gemma_logits(self.h), owned=False)
        return self.ctx.read_f32(b, self.cfg["vocab"])

    def hidden(self) -> np.ndarray:
        b = Buffer(self.ctx, lib().ksh_gemma_hidden(self.h), owned=False)
        return self.ctx.read_f32(b, self.cfg["hidden"])

    def kv(self, layer: int, which: int, nbytes: int) -> np.ndarray:
        b = Buffer(self.ctx, lib().ksh_gemma_kv(self.h, layer, which), owned=False)
        return self.ctx.read_bytes(b, nbytes)


class GgmlType(enum.IntEnum):
    F32 = 0
    F16 = 1
    Q4_0 = 2
    Q4_1 = 3
    Q5_1 = 7
    Q8_0 = 8
    Q4_K = 12
    Q5_K = 13
    Q6_K = 14
    BF16 = 30


LOAD_KEEP_Q6K = 1


class Gguf:
    """A memory-mapped GGUF file (Gguf::open, crates/ksearch_gguf/src/gguf_impl.rs:217-420).  Needs no GPU."""

    def __init__(self, path: str):
        h = C.c_void_p()
        _check(lib().ksh_gguf_open(os.fsencode(path), C.byref(h)))
        self.h = h

    def close(self):
        if self.h:
            lib().ksh_gguf_close(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    @property
    def version(self) -> int:
        return lib().ksh_gguf_version(self.h)

    def tensor_names(self) -> list:
        buf = C.create_string_buffer(512)
        out = []
        for i in range(lib().ksh_gguf_n_tensors(self.h)):
            _check(lib().ksh_gguf_tensor_name(self.h, i, buf, 512))
            out.append(buf.value.decode(errors="replace"))   # (gguf_impl.rs:170-173 reads strings lossily)
        return out

    def has_tensor(self, name: str) -> bool:
        return bool(lib().ksh_gguf_has_tensor(self.h, name.encode()))

    def tensor(self, name: str):
        """(ggml type, dims as stored (dims[0] = columns), raw bytes as a numpy view into the mapping)."""
        ty, nd, dims = C.c_int32(), C.c_int32(), (C.c_int64 * 4)()
        data, nbytes = C.c_void_p(), C.c_size_t()
        _check(lib().ksh_gguf_tensor(self.h, name.encode(), C.byref(ty), dims, C.byref(nd), C.byref(data), C.byref(nbytes)))
        raw = np.ctypeslib.as_array(C.cast(data, C.POINTER(C.c_uint8)), shape=(nbytes.value,)) if nbytes.value else np.empty(0, np.uint8)
        return ty.value, tuple(dims[i] for i in range(nd.value)), raw

    def get_u32(self, key: str):
        v = C.c_uint32()
        return None if lib().ksh_gguf_get_u32(self.h, key.encode(), C.byref(v)) else v.value

    def get_f32(self, key: str):
        v = C.c_float()
        return None if lib().ksh_gguf_get_f32(self.h, key.encode(), C.byref(v)) else v.value

    def get_str(self, key: str):
        buf = C.create_string_buffer(4096)
        return None if lib().ksh_gguf_get_str(self.h, key.encode(), buf, 4096) else buf.value.decode(errors="replace")

    def get_list(self, key: str):
        n = C.c_int()
        if lib().ksh_gguf_get_arr_u32(self.h, key.encode(), None, 0, C.byref(n)):
            return None
        arr = (C.c_uint32 * max(1, n.value))()
        lib().ksh_gguf_get_arr_u32(self.h, key.encode(), arr, n.value, C.byref(n))
        vals = list(arr[:n.value])
        return [bool(v) for v in vals] if lib().ksh_gguf_arr_is_bool(self.h, key.encode()) else vals

    def gemma4_config(self, max_seq: int):
        """GemmaConfig::from_gguf: (cfg dict, ffn per layer, is_swa per layer)."""
        c = Gemma4Cfg()
        ffn, swa = (C.c_int32 * 4096)(), (C.c_int32 * 4096)()
        _check(lib().ksh_gemma4_config_from_gguf(self.h, max_seq, C.byref(c), ffn, swa, 4096))
        cfg = {k: getattr(c, k) for k in GEMMA4_CFG_INTS + GEMMA4_CFG_FLOATS}
        return cfg, list(ffn[:c.n_layers]), [bool(v) for v in swa[:c.n_layers]]


def sample_softcap_min_p(logits: np.ndarray, cap: float, temperature: float, min_p: float = 0.05, seed: int = 1) -> int:
    """crates/ksearch_gemma/src/sample.rs:9-77 on f32 logits (host)."""
    x = np.ascontiguousarray(logits, dtype=np.float32)
    out = C.c_uint32()
    _check(lib().ksh_sample_softcap_min_p(x.ctypes.data, x.size, cap, temperature, min_p, seed, C.byref(out)))
    return out.value


def gguf_dequant_host(ggml_type: int, raw: np.ndarray, n: int) -> np.ndarray:
    raw = np.ascontiguousarray(raw, dtype=np.uint8)
    out = np.empty(n, dtype=np.float32)
    _check(lib().ksh_gguf_dequant_host(int(ggml_type), raw.ctypes.data, n, out.ctypes.data))
    return out


class KvPool:
    """KvPool, Q4_0 form (crates/ksearch_gemma/src/kv_pool.rs)."""

    def __init__(self, ctx: Context, max_batch: int, max_seq: int, n_kv_layers: int, hd: int, n_kv: int):
        self.ctx = ctx
        h = C.c_void_p()
        _check(lib().ksh_kvpool_create(ctx.h, max_batch, max_seq, n_kv_layers, hd, n_kv, C.byref(h)))
        self.h, self.max_batch = h, max_batch

    def close(self):
        if self.h:
            lib().ksh_kvpool_destroy(self.h)
            self.h = None

    def alloc(self) -> int:
        s = C.c_int()
        _check(lib().ksh_kvpool_alloc(self.h, C.byref(s)))
        return s.value

    def free(self, slot: int):
        _check(lib().ksh_kvpool_free(self.h, slot))

    def clear_slot(self, slot: int):
        _check(lib().ksh_kvpool_clear_slot(self.h, slot))

    def seq_len(self, slot: int) -> int:
        return lib().ksh_kvpool_seq_len(self.h, slot)

    def bump_len(self, slot: int, n: int = 1) -> int:
        out = C.c_int()
        _check(lib().ksh_kvpool_bump_len_by(self.h, slot, n, C.byref(out)))
        return out.value

    def active_batch(self) -> list:
        arr = (C.c_int * self.max_batch)()
        n = lib().ksh_kvpool_active_batch(self.h, arr, self.max_batch)
        return list(arr[:n])

    def k_buf(self, slot: int, layer: int) -> Buffer:
        return Buffer(self.ctx, lib().ksh_kvpool_k(self.h, slot, layer), owned=False)

    def v_buf(self, slot: int, layer: int) -> Buffer:
        return Buffer(self.ctx, lib().ksh_kvpool_v(self.h, slot, layer), owned=False)

    def layer_bufs(self, layer: int):
        """The layer's K and V caches of all slots, [max_batch][max_seq * n_kv * (hd / 32) * 18] each."""
        return (Buffer(self.ctx, lib().ksh_kvpool_layer_k(self.h, layer), owned=False),
                Buffer(self.ctx, lib().ksh_kvpool_layer_v(self.h, layer), owned=False))


FINISH_REASONS = ("stop", "length", "cancelled", "error")


class Serve:
    """The decode-before-prefill slot scheduler (crates/ksearch_cli/src/scheduler.rs:78-349) as a tick the caller
    drives.  Events come back as tuples: ("token", request, id), ("done", request, reason, prompt_tokens,
    completion_tokens), ("error", request, text)."""

    def __init__(self, model, pool, slots: int = 4, prefill_chunk: int = 256, prefill_tokens_per_tick: int = 2048,
                 eos=(1, 106), use_graph: bool = True, stop=None, batched_decode: int = 3):
        cfg = ServeCfg()
        _check(lib().ksh_serve_default_cfg(C.byref(cfg)))
        cfg.batched_decode = int(batched_decode)      # joint decode steps from this many decoding requests on; 0: never
        cfg.slots, cfg.prefill_chunk, cfg.prefill_tokens_per_tick = slots, prefill_chunk, prefill_tokens_per_tick
        cfg.eos[0], cfg.eos[1] = int(eos[0]), int(eos[1])
        cfg.use_graph = int(use_graph)
        # the callback object must live as long as the scheduler
        self._stop = SERVE_STOP_FN(lambda user, req, tok: int(bool(stop(req, tok)))) if stop else SERVE_STOP_FN()
        cfg.stop = self._stop
        self.model, self.pool = model, pool
        h = C.c_void_p()
        _check(lib().ksh_serve_create(model.h, pool.h, C.byref(cfg), C.byref(h)))
        self.h = h

    def close(self):
        if self.h:
            lib().ksh_serve_destroy(self.h)
            self.h = None

    def submit(self, prompt, max_tokens: int, temperature: float = 0.0, min_p: float = 0.0, seed: int = 1) -> int:
        p = (C.c_uint32 * max(1, len(prompt)))(*[int(t) for t in prompt])
        rid = C.c_uint64()
        _check(lib().ksh_serve_submit(self.h, p, len(prompt), max_tokens, temperature, min_p, seed & 0xFFFFFFFF, C.byref(rid)))
        return rid.value

    def cancel(self, request: int):
        _check(lib().ksh_serve_cancel(self.h, request))

    def tick(self) -> list:
        _check(lib().ksh_serve_tick(self.h))
        return self.poll()

    def poll(self) -> list:
        out, buf = [], (ServeEvent * 64)()
        while True:
            n = lib().ksh_serve_poll(self.h, buf, 64)
            for e in buf[:n]:
                if e.kind == 0:
                    out.append(("token", e.request, e.token))
                elif e.kind == 1:
                    out.append(("done", e.request, FINISH_REASONS[e.reason], e.prompt_tokens, e.completion_tokens))
                else:
                    out.append(("error", e.request, (lib().ksh_serve_error_text(self.h) or b"").decode()))
            if n < 64:
                return out

    def pending(self):
        w, a = C.c_int(), C.c_int()
        _check(lib().ksh_serve_pending(self.h, C.byref(w), C.byref(a)))
        return w.value, a.value

    def run(self, max_ticks: int = 100000) -> list:
        """Ticks until nothing is waiting or running."""
        out = []
        for _ in range(max_ticks):
            out += self.tick()
            if self.pending() == (0, 0):
                return out
        raise KshError("Serve.run: still busy after max_ticks")


class Gemma4:
    """GemmaPrimModel with the layer features of the real Gemma-4 checkpoints
    (crates/ksearch_gemma/src/gemma_prim.rs:881-1275; crates/ksearch_gemma/src/lib.rs:39-167).

    ``cfg``: the fields of ksh_gemma4_cfg.  ``weights``: ``layers`` (one dict per
    layer: ``is_swa``, ``ffn``, ``layer_scale``, the weight tensors with their
    ``dt_*`` codes, the f32 norm vectors) and ``globals`` (``token_embd``,
    ``dt_embd``, ``output_norm`` and, with per-layer embeddings, ``ple_embd``,
    ``dt_ple``, ``ple_model_proj``, ``dt_ple_proj``, ``ple_proj_norm``).
    Tensors are host arrays (uploaded here) or device Buffers."""

    def __init__(self, ctx: Context, cfg: dict, weights: dict):
        self.ctx, self.cfg = ctx, dict(cfg)
        self._bufs = []

        def up(a):
            if a is None:
                return None
            b = a if isinstance(a, Buffer) else ctx.buffer_bytes(a)
            self._bufs.append(b)
            return b.h

        n = cfg["n_layers"]
        arr = (Gemma4Layer * n)()
        for i, lw in enumerate(weights["layers"]):
            arr[i].is_swa, arr[i].ffn = int(lw["is_swa"]), int(lw["ffn"])
            arr[i].layer_scale = float(lw.get("layer_scale", 1.0))
            for name in GEMMA4_DTYPES:
                setattr(arr[i], name, int(lw.get(name, DType.Q4K)))
            for name in GEMMA4_WEIGHTS + GEMMA4_NORMS:
                setattr(arr[i], name, up(lw.get(name)))
        self._layers = arr
        g, gw = Gemma4Globals(), weights["globals"]
        for name in ("token_embd", "output_norm", "ple_embd", "ple_model_proj", "ple_proj_norm"):
            setattr(g, name, up(gw.get(name)))
        for name in ("dt_embd", "dt_ple", "dt_ple_proj"):
            setattr(g, name, int(gw.get(name, DType.Q4K)))
        self._globals = g
        c = Gemma4Cfg(**{k: cfg[k] for k in GEMMA4_CFG_INTS + GEMMA4_CFG_FLOATS})
        h = C.c_void_p()
        _check(lib().ksh_gemma4_create(ctx.h, C.byref(c), arr, C.byref(g), C.byref(h)))
        self.h = h

    @classmethod
    def from_gguf(cls, ctx: Context, gguf: "Gguf", max_seq: int, keep_q6k: bool = False) -> "Gemma4":
        """GemmaPrimModel's load path: every tensor of the file onto the device, in the forms the loop takes."""
        self = cls.__new__(cls)
        self.ctx, self._bufs = ctx, []
        h = C.c_void_p()
        _check(lib().ksh_gemma4_load_gguf(ctx.h, gguf.h, max_seq, LOAD_KEEP_Q6K if keep_q6k else 0, C.byref(h)))
        self.h = h
        c = Gemma4Cfg()
        _check(lib().ksh_gemma4_config(h, C.byref(c)))
        self.cfg = {k: getattr(c, k) for k in GEMMA4_CFG_INTS + GEMMA4_CFG_FLOATS}
        return self

    def close(self):
        if self.h:
            lib().ksh_gemma4_destroy(self.h)
            self.h = None
        for b in self._bufs:
            b.release()
        self._bufs = []

    def reset(self):
        _check(lib().ksh_gemma4_reset(self.h))

    @property
    def pos(self) -> int:
        return lib().ksh_gemma4_pos(self.h)

    @property
    def launches_per_token(self) -> int:
        return lib().ksh_gemma4_launches_per_token(self.h)

    def kv_source(self, layer: int) -> int:
        return lib().ksh_gemma4_kv_source(self.h, layer)

    def forward_token(self, token: int, want_logits: bool = True, use_graph: bool = False, read_next: bool = True):
        nxt = C.c_uint32()
        _check(lib().ksh_gemma4_forward_token(self.h, int(token), int(want_logits), int(use_graph),
                                              C.byref(nxt) if read_next and want_logits else None))
        return nxt.value if read_next and want_logits else None

    def generate(self, prompt, n_new: int, use_graph: bool = True, serial_prefill: bool = False):
        p = (C.c_uint32 * len(prompt))(*[int(t) for t in prompt])
        out = (C.c_uint32 * max(1, n_new))()
        pre, dec = C.c_double(), C.c_double()
        flags = int(bool(use_graph)) | (2 if serial_prefill else 0)
        _check(lib().ksh_gemma4_generate(self.h, p, len(prompt), n_new, flags, out, C.byref(pre), C.byref(dec)))
        return list(out[:n_new]), pre.value, dec.value

    def decode_token_sampled(self, token: int, temperature: float, min_p: float, seed: int, use_graph: bool = False) -> int:
        """GemmaPrimModel::decode_token_sampled (gemma_prim.rs:1614-1635)."""
        nxt = C.c_uint32()
        _check(lib().ksh_gemma4_decode_token_sampled(self.h, int(token), temperature, min_p, seed & 0xFFFFFFFF, int(use_graph),
                                                     C.byref(nxt)))
        return nxt.value

    def prefill_chunk(self, tokens, use_graph: bool = False, serial: bool = False):
        """GemmaPrimModel::prefill_chunk (gemma_prim.rs:1305-1315): chunks of up to 256 tokens as one batched pass
        per layer; `serial` feeds every token through the decode step instead."""
        t = (C.c_uint32 * max(1, len(tokens)))(*[int(x) for x in tokens])
        _check(lib().ksh_gemma4_prefill_chunk(self.h, t, len(tokens), int(bool(use_graph)) | (2 if serial else 0)))

    def decode_round(self, pool, slots, tokens, temperature=None, min_p=None, seeds=None):
        """One decode step for several sequences as one pass over the weights (the scheduler's decode round,
        crates/ksearch_cli/src/scheduler.rs:163-231): row i feeds tokens[i] to the sequence in pool slot slots[i].
        Returns the next ids; the caller bumps the slots' lengths."""
        n = len(slots)
        sl = (C.c_int32 * n)(*[int(x) for x in slots])
        tk = (C.c_uint32 * n)(*[int(x) for x in tokens])
        out = (C.c_uint32 * n)()
        if temperature is None:
            te = mp = sd = None
        else:
            te = (C.c_float * n)(*[float(x) for x in temperature])
            mp = (C.c_float * n)(*[float(x) for x in min_p])
            sd = (C.c_uint32 * n)(*[int(x) & 0xFFFFFFFF for x in seeds])
        _check(lib().ksh_gemma4_decode_round(self.h, pool.h, sl, tk, n, te, mp, sd, out))
        return list(out)

    def round_logits(self, n: int) -> np.ndarray:
        buf = Buffer(self.ctx, lib().ksh_gemma4_round_logits(self.h), owned=False)
        v = self.cfg["vocab"]
        return self.ctx.read_f32(buf, n * v).reshape(n, v)

    def bind_slot(self, pool, slot: int):
        """GemmaPrimModel::bind_slot; pool=None goes back to the model's own caches at position `slot`."""
        _check(lib().ksh_gemma4_bind_slot(self.h, pool.h if pool is not None else None, slot))

    def generate_until(self, prompt, n_new: int, eos=(1, 106), use_graph: bool = True):
        """generate_timed with its stop rule: ends after the first id from `eos` (which is the last one returned)."""
        p = (C.c_uint32 * len(prompt))(*[int(t) for t in prompt])
        e = (C.c_uint32 * max(1, len(eos)))(*[int(t) for t in eos])
        out = (C.c_uint32 * max(1, n_new))()
        n, pre, dec = C.c_int(), C.c_double(), C.c_double()
        _check(lib().ksh_gemma4_generate_until(self.h, p, len(prompt), n_new, e, len(eos), int(use_graph), out, C.byref(n),
                                               C.byref(pre), C.byref(dec)))
        return list(out[:n.value]), pre.value, dec.value

    def logits(self) -> np.ndarray:
        b = Buffer(self.ctx, lib().ksh_gemma4_logits(self.h), owned=False)
        return self.ctx.read_f32(b, self.cfg["vocab"])

    def hidden(self) -> np.ndarray:
        b = Buffer(self.ctx, lib().ksh_gemma4_hidden(self.h), owned=False)
        return self.ctx.read_f32(b, self.cfg["hidden"])

    def kv(self, layer: int, which: int, nbytes: int) -> np.ndarray:
        b = Buffer(self.ctx, lib().ksh_gemma4_kv(self.h, layer, which), owned=False)
        return self.ctx.read_bytes(b, nbytes)
