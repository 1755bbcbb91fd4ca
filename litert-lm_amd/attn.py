"""ctypes binding of libmi355_attn.so, the C ABI declared in include/mi355_attn.h.

Thin by design: it turns tensors into pointers and status codes into
exceptions. There is no fallback of any kind: if the library is missing or no
gfx950 device is usable the calls raise.
"""
from __future__ import annotations

import ctypes
import os

import numpy as np

F32, F16, BF16, I8 = 0, 1, 2, 3
OK, INVALID_ARGUMENT, RESOURCE_EXHAUSTED, FAILED_PRECONDITION = 0, 3, 8, 9
OUT_OF_RANGE, UNIMPLEMENTED, INTERNAL, UNAVAILABLE = 11, 12, 13, 14

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmi355_attn.so")
_lib = None


class AttnError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"mi355_attn status {code}: {message}")
        self.code = code
        self.message = message


class Config(ctypes.Structure):
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("num_layers", ctypes.c_int32),
        ("num_q_heads", ctypes.c_int32),
        ("num_kv_heads", ctypes.c_int32),
        ("head_dim", ctypes.c_int32),
        ("max_tokens", ctypes.c_int32),
        ("max_seqs", ctypes.c_int32),
        ("kv_dtype", ctypes.c_int32),
        ("io_dtype", ctypes.c_int32),
        ("scale", ctypes.c_float),
        ("softcap", ctypes.c_float),
        ("layer_window", ctypes.POINTER(ctypes.c_int32)),
        ("device", ctypes.c_int32),
        ("host_io", ctypes.c_int32),
        ("own_stream", ctypes.c_int32),
        ("stream", ctypes.c_void_p),
    ]


class LayerTransform(ctypes.Structure):
    """mi355_attn_layer_transform: the constants of the step before attention."""
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("norm_q", ctypes.c_int32),
        ("norm_k", ctypes.c_int32),
        ("norm_v", ctypes.c_int32),
        ("q_weight", ctypes.c_void_p),
        ("k_weight", ctypes.c_void_p),
        ("eps", ctypes.c_float),
        ("weight_offset", ctypes.c_float),
        ("rope_inv_freq", ctypes.c_void_p),
    ]


_ERR = ctypes.POINTER(ctypes.c_char_p)


def lib() -> ctypes.CDLL:
    """Loads the built library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FileNotFoundError(
            f"{LIB_PATH} is missing: build it with `make -C litert-lm_amd/csrc` "
            "(or __graft_entry__.build()); there is no CPU fallback")
    L = ctypes.CDLL(LIB_PATH)
    vp, i32, c = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int
    i32p = ctypes.POINTER(ctypes.c_int32)
    errp = ctypes.POINTER(ctypes.c_void_p)
    L.mi355_attn_create.argtypes = [ctypes.POINTER(Config), ctypes.POINTER(vp), errp]
    L.mi355_attn_destroy.argtypes = [vp]
    L.mi355_attn_destroy.restype = None
    L.mi355_attn_kv_append.argtypes = [vp, i32, i32, i32, i32, vp, vp, errp]
    L.mi355_attn_kv_set_scales.argtypes = [vp, i32, i32, vp, vp, errp]
    L.mi355_attn_kv_read.argtypes = [vp, i32, i32, i32, i32, vp, vp, errp]
    L.mi355_attn_set_layer_transform.argtypes = [vp, i32, ctypes.POINTER(LayerTransform), errp]
    L.mi355_attn_pre_attention.argtypes = [vp, i32, i32, i32, i32, vp, vp, vp, vp, errp]
    L.mi355_attn_prefill.argtypes = [vp, i32, i32, i32, i32, vp, vp, errp]
    L.mi355_attn_prefill_layers.argtypes = [vp, i32, i32, i32, i32, i32, vp, vp, errp]
    L.mi355_attn_decode.argtypes = [vp, i32, i32p, i32p, i32, vp, vp, i32, errp]
    L.mi355_attn_decode_noalloc.argtypes = [vp, i32, i32p, i32p, i32, vp, vp, i32, errp]
    L.mi355_attn_decode_step.argtypes = [vp, i32, i32p, i32p, i32, vp, vp, vp, vp, i32, errp]
    L.mi355_attn_decode_layers.argtypes = [vp, i32, i32, i32p, i32p, i32, vp, vp, i32, errp]
    L.mi355_attn_stream_probe.argtypes = [vp, ctypes.c_uint64, ctypes.c_uint64, i32, i32, errp]
    L.mi355_attn_reset.argtypes = [vp, i32, errp]
    L.mi355_attn_sync.argtypes = [vp, errp]
    L.mi355_attn_stream.argtypes = [vp]
    L.mi355_attn_stream.restype = vp
    L.mi355_attn_set_timing.argtypes = [vp, i32]
    L.mi355_attn_last_kernel_ms.argtypes = [vp]
    L.mi355_attn_last_kernel_ms.restype = ctypes.c_float
    L.mi355_attn_set_option.argtypes = [vp, ctypes.c_char_p, i32]
    L.mi355_attn_cache_bytes.argtypes = [vp]
    L.mi355_attn_cache_bytes.restype = ctypes.c_uint64
    L.mi355_attn_version.restype = ctypes.c_char_p
    for name in ("create", "kv_append", "kv_set_scales", "kv_read", "set_layer_transform", "pre_attention", "prefill",
                 "prefill_layers", "decode", "decode_layers", "decode_step", "decode_noalloc", "prefill_plan_probe", "stream_probe",
                 "reset", "sync", "set_timing", "set_option"):
        getattr(L, "mi355_attn_" + name).restype = c
    _lib = L
    return L


_libc = ctypes.CDLL(None)
_libc.free.argtypes = [ctypes.c_void_p]


def _check(rc: int, err: ctypes.c_void_p):
    msg = ""
    if err.value:
        msg = ctypes.string_at(err.value).decode("utf-8", "replace")
        _libc.free(err.value)
    if rc != OK:
        raise AttnError(rc, msg)


def _ptr(x):
    """Address of a torch tensor or numpy array (must be contiguous)."""
    if x is None:
        return None
    if isinstance(x, np.ndarray):
        if not x.flags["C_CONTIGUOUS"]:
            raise ValueError("numpy array must be C-contiguous")
        return x.ctypes.data
    if not x.is_contiguous():
        raise ValueError("tensor must be contiguous")
    return x.data_ptr()


def _i32_array(xs):
    if xs is None:
        return None
    xs = [int(v) for v in xs]
    return (ctypes.c_int32 * len(xs))(*xs)


class Attn:
    """One attention stack (all layers) with its KV cache in HBM."""

    def __init__(self, num_layers, num_q_heads, num_kv_heads, head_dim, max_tokens, max_seqs, kv_dtype, io_dtype,
                 layer_window=None, scale=0.0, softcap=0.0, device=0, host_io=False, stream=None,
                 own_stream=False):
        L = lib()
        self._win = _i32_array(layer_window)
        if layer_window is not None and len(layer_window) != num_layers:
            raise ValueError("layer_window needs one entry per layer")
        cfg = Config(ctypes.sizeof(Config), num_layers, num_q_heads, num_kv_heads, head_dim, max_tokens, max_seqs,
                     kv_dtype, io_dtype, scale, softcap,
                     ctypes.cast(self._win, ctypes.POINTER(ctypes.c_int32)) if self._win is not None else None,
                     device, int(bool(host_io)), int(bool(own_stream)), stream)
        self.num_layers, self.hq, self.hkv, self.d = num_layers, num_q_heads, num_kv_heads, head_dim
        self.kv_dtype, self.io_dtype, self.host_io = kv_dtype, io_dtype, bool(host_io)
        self._h = ctypes.c_void_p()
        err = ctypes.c_void_p()
        _check(L.mi355_attn_create(ctypes.byref(cfg), ctypes.byref(self._h), ctypes.byref(err)), err)

    def close(self):
        if getattr(self, "_h", None) is not None and self._h.value:
            lib().mi355_attn_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    # -- cache
    def kv_append(self, layer, seq, pos, k, v, n=None):
        n = int(k.shape[0]) if n is None else n
        err = ctypes.c_void_p()
        _check(lib().mi355_attn_kv_append(self._h, layer, seq, pos, n, _ptr(k), _ptr(v), ctypes.byref(err)), err)

    def kv_set_scales(self, layer, seq, k_scale, v_scale):
        err = ctypes.c_void_p()
        _check(lib().mi355_attn_kv_set_scales(self._h, layer, seq, _ptr(k_scale), _ptr(v_scale), ctypes.byref(err)),
               err)

    def kv_read(self, layer, seq, pos, n, k_out, v_out):
        err = ctypes.c_void_p()
        _check(lib().mi355_attn_kv_read(self._h, layer, seq, pos, n, _ptr(k_out), _ptr(v_out), ctypes.byref(err)),
               err)

    def set_layer_transform(self, layer, *, norm_q=False, norm_k=False, norm_v=False, q_weight=None, k_weight=None,
                            eps=1e-6, weight_offset=1.0, rope_inv_freq=None):
        """Constants of the step before attention for one layer; the arrays are
        host float32 ([head_dim] weights, [head_dim / 2] rotary frequencies)."""
        def host(x, count, name):
            if x is None:
                return None
            arr = np.ascontiguousarray(np.asarray(x, dtype=np.float32))
            if arr.shape != (count,):
                raise ValueError(f"{name} must hold {count} float32 values")
            return arr
        qw, kw = host(q_weight, self.d, "q_weight"), host(k_weight, self.d, "k_weight")
        fr = host(rope_inv_freq, self.d // 2, "rope_inv_freq")
        t = LayerTransform(ctypes.sizeof(LayerTransform), int(bool(norm_q)), int(bool(norm_k)), int(bool(norm_v)),
                           _ptr(qw), _ptr(kw), float(eps), float(weight_offset), _ptr(fr))
        err = ctypes.c_void_p()
        _check(lib().mi355_attn_set_layer_transform(self._h, layer, ctypes.byref(t), ctypes.byref(err)), err)

    def pre_attention(self, layer, seq, pos, q, k, v, q_out, n=None):
        """Norm + rotary embedding of the n new rows, query into q_out, key /
        value rows into the cache (the step before prefill / decode)."""
        n = int(q.shape[0]) if n is None else n
        err = ctypes.c_void_p()
        _check(lib().mi355_attn_pre_attention(self._h, layer, seq, pos, n, _ptr(q), _ptr(k), _ptr(v), _ptr(q_out),
                                              ctypes.byref(err)), err)

    # -- attention
    def prefill(self, layer, seq, q_pos0, n, q, out, n_layers=1):
        err = ctypes.c_void_p()
        if n_layers == 1:
            rc = lib().mi355_attn_prefill(self._h, layer, seq, q_pos0, n, _ptr(q), _ptr(out), ctypes.byref(err))
        else:
            rc = lib().mi355_attn_prefill_layers(self._h, layer, n_layers, seq, q_pos0, n, _ptr(q), _ptr(out),
                                                 ctypes.byref(err))
        _check(rc, err)

    def decode(self, layer, kv_lens, q, out, seq_ids=None, num_splits=0, n_layers=1, batch=None):
        lens = kv_lens if isinstance(kv_lens, ctypes.Array) else _i32_array(kv_lens)
        sids = seq_ids if isinstance(seq_ids, ctypes.Array) or seq_ids is None else _i32_array(seq_ids)
        batch = len(lens) if batch is None else batch
        err = ctypes.c_void_p()
        if n_layers == 1:
            rc = lib().mi355_attn_decode(self._h, layer, sids, lens, batch, _ptr(q), _ptr(out), num_splits,
                                         ctypes.byref(err))
        else:
            rc = lib().mi355_attn_decode_layers(self._h, layer, n_layers, sids, lens, batch, _ptr(q), _ptr(out),
                                                num_splits, ctypes.byref(err))
        _check(rc, err)

    def decode_step(self, layer, kv_lens, q, k, v, out, seq_ids=None, num_splits=0, batch=None):
        """mi355_attn_decode_step: the step before attention for each sequence's one new token (row
        kv_lens[b] - 1; q, k, v are the raw projections) and decode attention, in one launch."""
        lens = kv_lens if isinstance(kv_lens, ctypes.Array) else _i32_array(kv_lens)
        sids = seq_ids if isinstance(seq_ids, ctypes.Array) or seq_ids is None else _i32_array(seq_ids)
        batch = len(lens) if batch is None else batch
        err = ctypes.c_void_p()
        _check(lib().mi355_attn_decode_step(self._h, layer, sids, lens, batch, _ptr(q), _ptr(k), _ptr(v), _ptr(out),
                                            num_splits, ctypes.byref(err)), err)

    def decode_noalloc(self, layer, kv_lens, q, out, seq_ids=None, num_splits=0, batch=None):
        """mi355_attn_decode_noalloc: one layer, partials in the library's fixed workspace, no allocation."""
        lens = kv_lens if isinstance(kv_lens, ctypes.Array) else _i32_array(kv_lens)
        sids = seq_ids if isinstance(seq_ids, ctypes.Array) or seq_ids is None else _i32_array(seq_ids)
        batch = len(lens) if batch is None else batch
        err = ctypes.c_void_p()
        _check(lib().mi355_attn_decode_noalloc(self._h, layer, sids, lens, batch, _ptr(q), _ptr(out), num_splits,
                                               ctypes.byref(err)), err)

    def stream_probe(self, offset, nbytes, workgroups, waves):
        """mi355_attn_stream_probe: a read of `nbytes` of the cache in the decode kernel's load pattern, nothing else."""
        err = ctypes.c_void_p()
        _check(lib().mi355_attn_stream_probe(self._h, offset, nbytes, workgroups, waves, ctypes.byref(err)), err)

    # -- control
    def reset(self, seq=-1):
        err = ctypes.c_void_p()
        _check(lib().mi355_attn_reset(self._h, seq, ctypes.byref(err)), err)

    def sync(self):
        err = ctypes.c_void_p()
        _check(lib().mi355_attn_sync(self._h, ctypes.byref(err)), err)

    def set_timing(self, on=True):
        lib().mi355_attn_set_timing(self._h, int(on))

    def last_kernel_ms(self) -> float:
        return float(lib().mi355_attn_last_kernel_ms(self._h))

    def set_option(self, name: str, value: int):
        rc = lib().mi355_attn_set_option(self._h, name.encode(), int(value))
        if rc != OK:
            raise AttnError(rc, f"set_option({name}, {value})")

    @property
    def stream(self):
        return lib().mi355_attn_stream(self._h)

    @property
    def cache_bytes(self) -> int:
        return int(lib().mi355_attn_cache_bytes(self._h))


def version() -> str:
    return lib().mi355_attn_version().decode()
