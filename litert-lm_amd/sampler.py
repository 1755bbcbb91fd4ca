"""ctypes binding of libmi355_sampler.so, the C ABI declared in include/mi355_sampler.h.

Mirrors the reference's Sampler interface (runtime/components/sampler.h:10-25):
`Sampler.sample_to_id_and_score_buffer(logits, ids, scores)`. No fallback: if the
library is missing or no gfx950 device is usable the calls raise.
"""
from __future__ import annotations

import ctypes
import os

from .attn import _check, _ptr  # same status / error-message conventions

TYPE_UNSPECIFIED, TOP_K, TOP_P, GREEDY = 0, 1, 2, 3
MAX_K = 256

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmi355_sampler.so")
_lib = None


class Config(ctypes.Structure):
    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("batch_size", ctypes.c_int32),
        ("vocab_size", ctypes.c_int32),
        ("type", ctypes.c_int32),
        ("k", ctypes.c_int32),
        ("p", ctypes.c_float),
        ("temperature", ctypes.c_float),
        ("seed", ctypes.c_int32),
        ("device", ctypes.c_int32),
        ("host_io", ctypes.c_int32),
        ("own_stream", ctypes.c_int32),
        ("stream", ctypes.c_void_p),
    ]


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FileNotFoundError(
            f"{LIB_PATH} is missing: build it with `make -C litert-lm_amd/csrc all` "
            "(or __graft_entry__.build()); there is no CPU fallback")
    L = ctypes.CDLL(LIB_PATH)
    vp, c = ctypes.c_void_p, ctypes.c_int
    errp = ctypes.POINTER(ctypes.c_void_p)
    L.mi355_sampler_create.argtypes = [ctypes.POINTER(Config), ctypes.POINTER(vp), errp]
    L.mi355_sampler_destroy.argtypes = [vp]
    L.mi355_sampler_destroy.restype = None
    L.mi355_sampler_sample.argtypes = [vp, vp, vp, vp, errp]
    L.mi355_sampler_sample_with_uniforms.argtypes = [vp, vp, vp, vp, vp, errp]
    L.mi355_sampler_top_k.argtypes = [vp, vp, vp, vp, errp]
    L.mi355_sampler_sync.argtypes = [vp, errp]
    L.mi355_sampler_set_timing.argtypes = [vp, ctypes.c_int32]
    L.mi355_sampler_last_kernel_ms.argtypes = [vp]
    L.mi355_sampler_last_kernel_ms.restype = ctypes.c_float
    for name in ("create", "sample", "sample_with_uniforms", "top_k", "sync", "set_timing"):
        getattr(L, "mi355_sampler_" + name).restype = c
    _lib = L
    return L


class Sampler:
    """TopPSampler::Create(k, p, temperature, batch_size, seed) plus the vocabulary
    size, as the reference's GPU sampler plugin takes it."""

    def __init__(self, k, p, temperature, batch_size, seed, vocab_size, type=TOP_P, device=0, host_io=False,
                 stream=None, own_stream=False):
        L = lib()
        cfg = Config(ctypes.sizeof(Config), batch_size, vocab_size, type, k, p, temperature, seed, device,
                     int(bool(host_io)), int(bool(own_stream)), stream)
        self.batch_size, self.vocab_size, self.k = batch_size, vocab_size, (1 if type == GREEDY else k)
        self._h = ctypes.c_void_p()
        err = ctypes.c_void_p()
        _check(L.mi355_sampler_create(ctypes.byref(cfg), ctypes.byref(self._h), ctypes.byref(err)), err)

    def close(self):
        if self._h:
            lib().mi355_sampler_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def sample_to_id_and_score_buffer(self, logits, ids, scores=None, uniforms=None):
        err = ctypes.c_void_p()
        if uniforms is None:
            rc = lib().mi355_sampler_sample(self._h, _ptr(logits), _ptr(ids), _ptr(scores), ctypes.byref(err))
        else:
            rc = lib().mi355_sampler_sample_with_uniforms(self._h, _ptr(logits), _ptr(uniforms), _ptr(ids),
                                                          _ptr(scores), ctypes.byref(err))
        _check(rc, err)

    def top_k(self, logits, indices, probabilities):
        err = ctypes.c_void_p()
        _check(lib().mi355_sampler_top_k(self._h, _ptr(logits), _ptr(indices), _ptr(probabilities), ctypes.byref(err)),
               err)

    def sync(self):
        err = ctypes.c_void_p()
        _check(lib().mi355_sampler_sync(self._h, ctypes.byref(err)), err)

    def set_timing(self, on: bool):
        lib().mi355_sampler_set_timing(self._h, int(on))

    def last_kernel_ms(self) -> float:
        return float(lib().mi355_sampler_last_kernel_ms(self._h))
