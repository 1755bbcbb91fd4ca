"""Pins oracle/pre_attention_oracle.py (RMS norm, rotary embedding, int8 row
quantisation) without the reference's model graph, which is not in its tree:
what the mathematics fixes, brute force, and the Gemma 3 building blocks of the
`transformers` package as a library cross-check."""
import math

import numpy as np
import pytest

from oracle import pre_attention_oracle as po


def rng_rows(seed, n, heads, d):
    return np.random.default_rng(seed).standard_normal((n, heads, d)).astype(np.float32)


# ----------------------------------------------------------------- rotary embedding
def test_inv_freq_closed_form():
    f = po.rope_inv_freq(256, 10000.0)
    assert f.shape == (128,) and f.dtype == np.float32
    assert f[0] == 1.0
    assert f[64] == np.float32(10000.0 ** -0.5) == np.float32(0.01)
    assert np.all(np.diff(f) < 0)
    # linear position scaling divides every frequency
    assert np.array_equal(po.rope_inv_freq(256, 1e6, 8.0), (po.rope_inv_freq(256, 1e6).astype(np.float64) / 8).astype(np.float32))
    # theta = 2^16, D = 32: exact powers of two
    assert np.array_equal(po.rope_inv_freq(32, 65536.0), (2.0 ** -np.arange(16)).astype(np.float32))


def test_rope_position_zero_is_identity_and_pairs_keep_their_norm():
    x = rng_rows(1, 5, 3, 64)
    f = po.rope_inv_freq(64, 10000.0)
    assert np.array_equal(po.apply_rope(x, np.zeros(5, int), f), x)
    y = po.apply_rope(x, np.array([0, 1, 17, 900, 4095]), f, dtype=np.float64)
    n_in = x[..., :32].astype(np.float64) ** 2 + x[..., 32:].astype(np.float64) ** 2
    n_out = y[..., :32] ** 2 + y[..., 32:] ** 2
    np.testing.assert_allclose(n_out, n_in, rtol=1e-12)


def test_rope_brute_force_loops():
    x = rng_rows(2, 3, 2, 8)
    f = po.rope_inv_freq(8, 100.0)
    pos = [3, 7, 12]
    got = po.apply_rope(x, np.array(pos), f, dtype=np.float64)
    for i in range(3):
        for h in range(2):
            for d in range(4):
                ang = float(np.float32(pos[i]) * f[d])
                lo, hi = float(x[i, h, d]), float(x[i, h, d + 4])
                assert got[i, h, d] == pytest.approx(lo * math.cos(ang) - hi * math.sin(ang), abs=1e-14)
                assert got[i, h, d + 4] == pytest.approx(hi * math.cos(ang) + lo * math.sin(ang), abs=1e-14)


def test_rope_is_multiplication_by_a_unit_complex_number():
    x = rng_rows(3, 6, 2, 32)
    f = po.rope_inv_freq(32, 10000.0)
    pos = np.array([0, 1, 2, 100, 1000, 4000])
    z = x[..., :16].astype(np.complex128) + 1j * x[..., 16:].astype(np.complex128)
    ang = (pos.astype(np.float32)[:, None] * f[None, :]).astype(np.float64)
    w = z * np.exp(1j * ang)[:, None, :]
    got = po.apply_rope(x, pos, f, dtype=np.float64)
    np.testing.assert_allclose(got[..., :16], w.real, atol=1e-13)
    np.testing.assert_allclose(got[..., 16:], w.imag, atol=1e-13)


def test_rope_scores_depend_on_relative_position_only_and_rotations_compose():
    # frequencies that are powers of two: every angle product is exact in float32
    f = po.rope_inv_freq(32, 65536.0)
    q, k = rng_rows(4, 1, 1, 32), rng_rows(5, 1, 1, 32)
    def score(p, j):
        a = po.apply_rope(q, np.array([p]), f, dtype=np.float64)
        b = po.apply_rope(k, np.array([j]), f, dtype=np.float64)
        return float((a * b).sum())
    base = score(9, 0)
    for shift in (1, 50, 1000):
        assert score(9 + shift, shift) == pytest.approx(base, abs=1e-11)
    assert score(9, 0) != pytest.approx(score(10, 0), abs=1e-6)  # and they do depend on it
    once = po.apply_rope(q, np.array([11]), f, dtype=np.float64)
    twice = po.apply_rope(po.apply_rope(q, np.array([4]), f, dtype=np.float64), np.array([7]), f, dtype=np.float64)
    np.testing.assert_allclose(twice, once, atol=1e-13)


# ----------------------------------------------------------------- RMS norm
def test_rms_norm_closed_forms():
    x = rng_rows(6, 4, 2, 256)
    y = po.rms_norm(x, None, 0.0, 1.0, dtype=np.float64)
    np.testing.assert_allclose(np.sqrt((y ** 2).mean(-1)), 1.0, rtol=1e-12)       # unit RMS
    np.testing.assert_allclose(po.rms_norm(7.5 * x, None, 0.0, 1.0, dtype=np.float64), y, rtol=1e-6)  # scale invariance
    ones = np.ones((1, 1, 256), np.float32)
    w = np.linspace(-0.5, 0.5, 256).astype(np.float32)
    # all-ones row: mean square 1, so the result is offset + weight up to eps
    np.testing.assert_allclose(po.rms_norm(ones, w, 0.0, 1.0)[0, 0], 1.0 + w, rtol=1e-7)
    np.testing.assert_allclose(po.rms_norm(ones, w, 0.0, 0.0)[0, 0], w, rtol=1e-7)
    np.testing.assert_allclose(po.rms_norm(ones, w, 3.0, 1.0)[0, 0], (1.0 + w) / 2.0, rtol=1e-6)  # eps inside the root
    assert np.all(po.rms_norm(np.zeros((1, 1, 256), np.float32), w, 1e-6, 1.0) == 0)


def test_rms_norm_matches_torch():
    torch = pytest.importorskip("torch")
    x = rng_rows(7, 8, 4, 256)
    w = np.random.default_rng(8).standard_normal(256).astype(np.float32) * 0.2
    want = torch.nn.functional.rms_norm(torch.from_numpy(x), (256,), torch.from_numpy(1.0 + w), eps=1e-6).numpy()
    np.testing.assert_allclose(po.rms_norm(x, w, 1e-6, 1.0), want, rtol=2e-6, atol=1e-6)


# ----------------------------------------------------------------- library cross-check
def test_matches_gemma3_building_blocks_of_transformers():
    torch = pytest.importorskip("torch")
    m = pytest.importorskip("transformers.models.gemma3.modeling_gemma3")
    n, hq, hkv, d = 12, 4, 1, 256
    q, k, v = rng_rows(10, n, hq, d), rng_rows(11, n, hkv, d), rng_rows(12, n, hkv, d)
    g = np.random.default_rng(13)
    qw, kw = (g.standard_normal(d) * 0.3).astype(np.float32), (g.standard_normal(d) * 0.3).astype(np.float32)
    pos0 = 1000
    for theta in (10000.0, 1000000.0):
        f = po.rope_inv_freq(d, theta)
        got_q, got_k, got_v = po.pre_attention(q, k, v, pos0, q_weight=qw, k_weight=kw, norm_q=True, norm_k=True,
                                               eps=1e-6, weight_offset=1.0, inv_freq=f)
        qn, kn = m.Gemma3RMSNorm(d, eps=1e-6), m.Gemma3RMSNorm(d, eps=1e-6)
        with torch.no_grad():
            qn.weight.copy_(torch.from_numpy(qw))
            kn.weight.copy_(torch.from_numpy(kw))
            # [batch, heads, tokens, head_dim], as the attention module holds them
            tq = qn(torch.from_numpy(q).permute(1, 0, 2)[None])
            tk = kn(torch.from_numpy(k).permute(1, 0, 2)[None])
            ang = (torch.arange(pos0, pos0 + n, dtype=torch.float32)[:, None] * torch.from_numpy(f)[None, :])
            emb = torch.cat([ang, ang], dim=-1)[None]
            rq, rk = m.apply_rotary_pos_emb(tq, tk, emb.cos(), emb.sin())
        np.testing.assert_allclose(got_q, rq[0].permute(1, 0, 2).numpy(), rtol=0, atol=3e-6 * np.abs(got_q).max())
        np.testing.assert_allclose(got_k, rk[0].permute(1, 0, 2).numpy(), rtol=0, atol=3e-6 * np.abs(got_k).max())
        assert np.array_equal(got_v, v)


def test_inv_freq_matches_gemma3_rotary_embedding_of_transformers():
    pytest.importorskip("torch")
    m = pytest.importorskip("transformers.models.gemma3.modeling_gemma3")
    fn = getattr(m.Gemma3RotaryEmbedding, "compute_default_rope_parameters", None)
    if fn is None:
        pytest.skip("this transformers version has no Gemma3RotaryEmbedding.compute_default_rope_parameters")

    class Cfg:
        head_dim = 256
        hidden_size = 1024
        num_attention_heads = 4
        rope_parameters = {"sliding_attention": {"rope_theta": 10000.0}, "full_attention": {"rope_theta": 1000000.0}}
    for layer_type, theta in (("sliding_attention", 10000.0), ("full_attention", 1000000.0)):
        inv, factor = fn(Cfg(), "cpu", layer_type=layer_type)
        assert factor == 1.0
        # theirs is formed in float32, ours in float64 and rounded once
        np.testing.assert_allclose(po.rope_inv_freq(256, theta), inv.numpy(), rtol=2e-6)


# ----------------------------------------------------------------- int8 rows
def test_quantize_rows_known_answers():
    scale = np.array([[0.5, 0.5, 0.5, 0.5, 0.5, 0.5, 0.0, 2.0]], np.float32)
    x = np.array([[[0.25, -0.25, 0.75, 1.25, 1000.0, -1000.0, 3.0, 2.9]]], np.float32)
    #             0.5->1  -0.5->-1  1.5->2  2.5->3 (half away from zero, not to even)  clamp  clamp  zero scale  1.45->1
    assert po.quantize_rows(x, scale).tolist() == [[[1, -1, 2, 3, 127, -127, 0, 1]]]


def test_quantize_rows_round_trip_error_is_half_a_step():
    x = rng_rows(14, 64, 2, 256)
    scale = (np.abs(x).max(axis=0) / np.float32(127)).astype(np.float32)
    qv = po.quantize_rows(x, scale)
    assert qv.dtype == np.int8 and np.abs(qv).max() == 127
    err = np.abs(qv.astype(np.float32) * scale[None] - x)
    assert np.all(err <= scale[None] * 0.5 * (1 + 1e-5))


def test_pre_attention_without_constants_is_a_plain_append():
    q, k, v = rng_rows(15, 3, 4, 256), rng_rows(16, 3, 1, 256), rng_rows(17, 3, 1, 256)
    a, b, c = po.pre_attention(q, k, v, 5)
    assert np.array_equal(a, q) and np.array_equal(b, k) and np.array_equal(c, v)


# ----------------------------------------------------------------- golden fixture
def test_oracle_matches_gemma3_fixture():
    """tests/golden/gemma3_pre_attention.npz: float64 results of the transformers
    Gemma 3 blocks (written by tests/golden/make_golden.py)."""
    import os
    c = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gemma3_pre_attention.npz"))
    v = np.zeros_like(c["k"])
    for kind in ("sliding_attention", "full_attention"):
        for dtype, tol in ((np.float64, 2e-7), (np.float32, 1e-5)):  # (the fixture is stored as float32)
            q, k, _ = po.pre_attention(c["q"], c["k"], v, int(c["pos0"]), q_weight=c["q_weight"], k_weight=c["k_weight"],
                                       norm_q=True, norm_k=True, eps=float(c["eps"]), weight_offset=1.0,
                                       inv_freq=c[f"inv_freq_{kind}"], dtype=dtype)
            assert np.abs(q - c[f"q_out_{kind}"]).max() / np.abs(c[f"q_out_{kind}"]).max() < tol
            assert np.abs(k - c[f"k_out_{kind}"]).max() / np.abs(c[f"k_out_{kind}"]).max() < tol
