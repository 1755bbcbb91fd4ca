"""CPU restatement of the step right before attention: per-head RMS norm of the
query / key (/ value) projections, rotary position embedding of query and key,
and the write of the new key / value rows into the cache (optionally quantised
to int8 with fixed per-(kv head, channel) scales).

TEST INFRASTRUCTURE ONLY: imported by tests/ and __graft_entry__.smoke();
nothing of the product path may import it.

Where this sits in the reference: the NPU executor runs it as separate
signatures around the transformer stack -- a RoPE signature that turns
`input_pos` into cos / sin tables for local and global layers
(runtime/executor/llm_litert_npu_compiled_model_executor.cc:82-94,1209-1219), and
a cache-update signature that merges the new `kv_slice_{k,v}_i` rows into the
cache at `input_pos` (:96-110,1294-1333); the CPU/GPU executor has all of it
inside the .tflite graph behind compiled_model_.Run
(llm_litert_compiled_model_executor.cc:271,407,522). The int8 write follows the
quantise idiom of llm_litert_npu_compiled_model_executor.cc:116-148
(multiply by the reciprocal scale, std::round, clamp).

PARITY UNPINNED against the reference: the arithmetic of the norm and of the
rotation lives in model files that are not in the reference tree, and no test
or fixture of the reference holds a value of it. What is restated here is the
published Gemma 3 definition (RMS norm `x / sqrt(mean(x^2) + eps) * (offset +
w)`, rotation of the pairs `(d, d + D/2)` by `pos * theta^(-2d/D) / factor`),
pinned by what the mathematics fixes (rotation at position 0 is the identity,
norms of pairs are kept, scores depend on relative positions only, rotations
compose, the complex-number form gives the same numbers; unit RMS, scale
invariance) and by a library cross-check against the Gemma 3 building blocks of
the `transformers` package (tests/test_pre_attention_oracle.py).
"""
from __future__ import annotations

import numpy as np


def rope_inv_freq(head_dim: int, theta: float, factor: float = 1.0) -> np.ndarray:
    """[head_dim / 2] float32: theta^(-2d / head_dim) / factor, computed in float64
    and rounded once (the table the device receives; both sides use these bits)."""
    d = np.arange(0, head_dim, 2, dtype=np.float64)
    return (1.0 / (float(theta) ** (d / head_dim)) / float(factor)).astype(np.float32)


def rms_norm(x: np.ndarray, weight, eps: float, weight_offset: float, dtype=np.float32) -> np.ndarray:
    """Over the last axis: x * 1/sqrt(mean(x^2) + eps) * (weight_offset + weight);
    weight None = no learned scale."""
    x = np.asarray(x, dtype=dtype)
    ms = np.mean(x * x, axis=-1, keepdims=True, dtype=dtype)
    y = x * (dtype(1.0) / np.sqrt(ms + dtype(eps)))
    if weight is not None:
        y = y * (dtype(weight_offset) + np.asarray(weight, dtype=dtype))
    return y.astype(dtype)


def apply_rope(x: np.ndarray, positions: np.ndarray, inv_freq: np.ndarray, dtype=np.float32) -> np.ndarray:
    """x [n][heads][D], positions [n] -> rotated copy. The angle is the float32
    product position * inv_freq (as the device forms it); cos / sin of that
    float32 angle are taken in `dtype`."""
    x = np.asarray(x, dtype=dtype)
    half = x.shape[-1] // 2
    ang32 = np.asarray(positions, dtype=np.float32)[:, None] * np.asarray(inv_freq, dtype=np.float32)[None, :]
    ang = ang32.astype(np.float64)
    c = np.cos(ang).astype(dtype)[:, None, :]
    s = np.sin(ang).astype(dtype)[:, None, :]
    lo, hi = x[..., :half], x[..., half:]
    return np.concatenate([lo * c - hi * s, hi * c + lo * s], axis=-1).astype(dtype)


def quantize_rows(x: np.ndarray, scale: np.ndarray) -> np.ndarray:
    """x [n][Hkv][D] float32, scale [Hkv][D] float32 -> int8: round-half-away of
    x * (1 / scale), clamped to +-127; channels with scale 0 store 0."""
    x = np.asarray(x, dtype=np.float32)
    scale = np.asarray(scale, dtype=np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(scale != 0, np.float32(1.0) / scale, np.float32(0.0)).astype(np.float32)
    t = (x * inv[None]).astype(np.float32)
    r = np.sign(t) * np.floor(np.abs(t) + np.float32(0.5))  # std::round
    return np.clip(r, -127, 127).astype(np.int8)


def pre_attention(q, k, v, pos0: int, *, q_weight=None, k_weight=None, norm_q=False, norm_k=False, norm_v=False,
                  eps=1e-6, weight_offset=1.0, inv_freq=None, dtype=np.float32):
    """q [n][Hq][D], k / v [n][Hkv][D] (any float dtype; computed in `dtype`) for
    the tokens at positions pos0 .. pos0 + n - 1.
    Returns (q_out, k_rows, v_rows) in `dtype`: what attention reads as the query
    and what the cache holds for these rows (before any cast / quantisation)."""
    q = np.asarray(q).astype(dtype)
    k = np.asarray(k).astype(dtype)
    v = np.asarray(v).astype(dtype)
    if norm_q:
        q = rms_norm(q, q_weight, eps, weight_offset, dtype)
    if norm_k:
        k = rms_norm(k, k_weight, eps, weight_offset, dtype)
    if norm_v:
        v = rms_norm(v, None, eps, weight_offset, dtype)
    if inv_freq is not None:
        positions = pos0 + np.arange(q.shape[0])
        q = apply_rope(q, positions, inv_freq, dtype)
        k = apply_rope(k, positions, inv_freq, dtype)
    return q, k, v
