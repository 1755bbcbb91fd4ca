"""ctypes loader for oracle/liboracle_attn.so (TEST INFRASTRUCTURE).

The library is built by ``make -C oracle`` (also run by
``__graft_entry__.build()``); nothing here is on the product path.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_attn.so")
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_i32p = ctypes.POINTER(ctypes.c_int32)


def build() -> str:
    subprocess.run(["make", "-C", _HERE, "-B", "liboracle_attn.so"], check=True, capture_output=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_sdpa_f64.restype = ctypes.c_int
        _lib.oracle_sdpa_ref_f32.restype = ctypes.c_int
        _lib.oracle_decode_batch_ref_f32.restype = ctypes.c_int
        _lib.oracle_num_threads.restype = ctypes.c_int
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def sdpa_f64(q, k, v, scale, q_pos0=0, window=0, softcap=0.0, kv_len=None):
    q, k, v = _f32(q), _f32(k), _f32(v)
    n_q, hq, d = q.shape
    hkv = k.shape[1]
    kv_len = k.shape[0] if kv_len is None else kv_len
    out = np.zeros((n_q, hq, d), dtype=np.float64)
    rc = lib().oracle_sdpa_f64(q.ctypes.data_as(_f32p), k.ctypes.data_as(_f32p), v.ctypes.data_as(_f32p),
                               n_q, hq, hkv, d, kv_len, ctypes.c_float(scale), ctypes.c_float(softcap),
                               q_pos0, window, out.ctypes.data_as(_f64p))
    if rc:
        raise RuntimeError(f"oracle_sdpa_f64 rc={rc}")
    return out


def fill_mask(rows, ctx, start, steps, is_f16=True):
    m = np.empty((rows, ctx), dtype=np.float32)
    lib().oracle_fill_mask_f32(m.ctypes.data_as(_f32p), rows, ctx, start, steps, int(is_f16))
    return m


def sdpa_ref_f32(q, k, v, scale, mask=None, threads=0):
    q, k, v = _f32(q), _f32(k), _f32(v)
    n_q, hq, d = q.shape
    ctx, hkv = k.shape[0], k.shape[1]
    out = np.zeros((n_q, hq, d), dtype=np.float32)
    mp = None
    if mask is not None:
        mask = _f32(mask).reshape(n_q, ctx)
        mp = mask.ctypes.data_as(_f32p)
    rc = lib().oracle_sdpa_ref_f32(q.ctypes.data_as(_f32p), k.ctypes.data_as(_f32p), v.ctypes.data_as(_f32p),
                                   n_q, hq, hkv, d, ctx, mp, ctypes.c_float(scale), threads,
                                   out.ctypes.data_as(_f32p))
    if rc:
        raise RuntimeError(f"oracle_sdpa_ref_f32 rc={rc}")
    return out


def decode_batch_ref_f32(q, ks, vs, scale, threads=0):
    """q [B,Hq,D]; ks, vs lists of [L_b,Hkv,D] float32 arrays."""
    q = _f32(q)
    b, hq, d = q.shape
    ks = [_f32(x) for x in ks]
    vs = [_f32(x) for x in vs]
    hkv = ks[0].shape[1]
    lens = np.array([x.shape[0] for x in ks], dtype=np.int32)
    kp = (_f32p * b)(*[x.ctypes.data_as(_f32p) for x in ks])
    vp = (_f32p * b)(*[x.ctypes.data_as(_f32p) for x in vs])
    out = np.zeros((b, hq, d), dtype=np.float32)
    rc = lib().oracle_decode_batch_ref_f32(q.ctypes.data_as(_f32p), kp, vp, lens.ctypes.data_as(_i32p), b, hq, hkv,
                                           d, ctypes.c_float(scale), threads, out.ctypes.data_as(_f32p))
    if rc:
        raise RuntimeError(f"oracle_decode_batch_ref_f32 rc={rc}")
    return out


def num_threads() -> int:
    return int(lib().oracle_num_threads())
