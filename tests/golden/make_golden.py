"""Writes the small golden vectors under tests/golden/.

The reference holds no attention values (its graphs and kernels are third-party
and absent), so these vectors come from an independent library, not from the
oracle they later check: torch.nn.functional.scaled_dot_product_attention on
the CPU in float64 with an explicit boolean mask, the KV heads repeated by
hand. Inputs are N(0,1) from numpy's default_rng(seed), rounded to values that
float32, float16 and bfloat16 all represent exactly. Each case is
one .npz (no pickles): inputs, the parameters and the expected output (computed
in float64, stored as float32).

    python tests/golden/make_golden.py

gemma3_pre_attention.npz holds the step before attention (per-head RMS norm with
the (1 + weight) scale, rotary embedding) as the Gemma 3 building blocks of the
`transformers` package compute it in float64 (Gemma3RMSNorm, apply_rotary_pos_emb,
frequencies from Gemma3RotaryEmbedding.compute_default_rope_parameters): again
an independent library, not the oracle it checks.

softmax_kat.json is different in kind: the inputs and expected values that the
reference's own test holds (runtime/components/sampling_cpu_util_test.cc:82-97),
typed in as data.
"""
import json
import os

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))


def visible(q_pos, n_keys, window):
    """[len(q_pos), n_keys] bool: key j visible to position p iff j <= p and, for
    a window W > 0, p - j < W."""
    p = np.asarray(q_pos)[:, None]
    j = np.arange(n_keys)[None, :]
    m = j <= p
    if window > 0:
        m &= (p - j) < window
    return m


def sdpa64(q, k, v, mask, scale, softcap):
    """q [S,Hq,D], k/v [L,Hkv,D] float32 -> [S,Hq,D] float64 via torch CPU SDPA."""
    hq, hkv = q.shape[1], k.shape[1]
    tq = torch.from_numpy(q).double().permute(1, 0, 2)[None]                 # [1,Hq,S,D]
    tk = torch.from_numpy(k).double().permute(1, 0, 2).repeat_interleave(hq // hkv, 0)[None]
    tv = torch.from_numpy(v).double().permute(1, 0, 2).repeat_interleave(hq // hkv, 0)[None]
    tm = torch.from_numpy(mask)[None, None]
    if softcap > 0:
        # SDPA has no soft cap: scores by hand, the rest (mask, softmax, P.V) through the same routine
        s = torch.einsum("bhsd,bhld->bhsl", tq, tk) * scale
        s = softcap * torch.tanh(s / softcap)
        s = s.masked_fill(~tm, float("-inf"))
        o = torch.einsum("bhsl,bhld->bhsd", torch.softmax(s, dim=-1), tv)
    else:
        o = F.scaled_dot_product_attention(tq, tk, tv, attn_mask=tm, scale=scale)
    return o[0].permute(1, 0, 2).contiguous().numpy()


def exact(x):
    """Rounds to values that float32, float16 and bfloat16 all hold exactly (8
    significant bits, magnitudes below 2^-10 flushed to zero), so that one
    expected output serves every cache dtype."""
    t = torch.from_numpy(x).bfloat16().float()
    t[t.abs() < 2.0 ** -10] = 0.0
    return t.numpy()


def case(name, seed, hq, hkv, d, n_keys, q_pos, window=0, scale=None, softcap=0.0):
    rng = np.random.default_rng(seed)
    q = exact(rng.standard_normal((len(q_pos), hq, d), dtype=np.float32))
    k = exact(rng.standard_normal((n_keys, hkv, d), dtype=np.float32))
    v = exact(rng.standard_normal((n_keys, hkv, d), dtype=np.float32))
    scale = d ** -0.5 if scale is None else scale
    out = sdpa64(q, k, v, visible(q_pos, n_keys, window), scale, softcap)
    np.savez_compressed(os.path.join(HERE, name + ".npz"), q=q, k=k, v=v, out=out.astype(np.float32),
                        q_pos=np.asarray(q_pos, np.int32), window=np.int32(window),
                        scale=np.float64(scale), softcap=np.float64(softcap))
    print(name, out.shape, float(np.abs(out).max()))


def gemma3_pre_attention():
    from transformers.models.gemma3 import modeling_gemma3 as m

    class Cfg:
        head_dim = 256
        hidden_size = 1024
        num_attention_heads = 4
        rope_parameters = {"sliding_attention": {"rope_theta": 10000.0}, "full_attention": {"rope_theta": 1000000.0}}

    n, hq, hkv, d, pos0 = 24, 4, 1, 256, 3000
    rng = np.random.default_rng(0xC0FFEE + 21)
    q = exact(rng.standard_normal((n, hq, d), dtype=np.float32) * 2)
    k = exact(rng.standard_normal((n, hkv, d), dtype=np.float32) * 2)
    q_weight = exact((rng.standard_normal(d, dtype=np.float32) * 0.3))
    k_weight = exact((rng.standard_normal(d, dtype=np.float32) * 0.3))
    out = {"q": q, "k": k, "q_weight": q_weight, "k_weight": k_weight, "pos0": np.int32(pos0), "eps": np.float64(1e-6)}
    for kind in ("sliding_attention", "full_attention"):
        inv_freq, _ = m.Gemma3RotaryEmbedding.compute_default_rope_parameters(Cfg(), "cpu", layer_type=kind)
        qn, kn = m.Gemma3RMSNorm(d, eps=1e-6).double(), m.Gemma3RMSNorm(d, eps=1e-6).double()
        with torch.no_grad():
            qn.weight.copy_(torch.from_numpy(q_weight).double())
            kn.weight.copy_(torch.from_numpy(k_weight).double())
            tq = qn(torch.from_numpy(q).double().permute(1, 0, 2)[None])
            tk = kn(torch.from_numpy(k).double().permute(1, 0, 2)[None])
            # the angle as the model forms it: float32 position times float32 frequency
            ang = (torch.arange(pos0, pos0 + n, dtype=torch.float32)[:, None] * inv_freq.float()[None, :]).double()
            emb = torch.cat([ang, ang], dim=-1)[None]
            rq, rk = m.apply_rotary_pos_emb(tq, tk, emb.cos(), emb.sin())
        out[f"inv_freq_{kind}"] = inv_freq.float().numpy()
        out[f"q_out_{kind}"] = rq[0].permute(1, 0, 2).contiguous().numpy().astype(np.float32)
        out[f"k_out_{kind}"] = rk[0].permute(1, 0, 2).contiguous().numpy().astype(np.float32)
    np.savez_compressed(os.path.join(HERE, "gemma3_pre_attention.npz"), **out)
    print("gemma3_pre_attention", out["q_out_full_attention"].shape, float(np.abs(out["q_out_full_attention"]).max()))


def main():
    torch.set_num_threads(1)
    gemma3_pre_attention()
    # decode rows (one query at the last position), shapes of configs 1 and 3 reduced in length
    case("decode_c1_like", 0xC0FFEE + 0, 4, 1, 256, 64, [63])
    case("decode_c3_like", 0xC0FFEE + 2, 8, 2, 256, 96, [95])
    case("decode_window", 0xC0FFEE + 12, 8, 2, 256, 80, [79], window=37)
    case("decode_softcap", 0xC0FFEE + 13, 8, 2, 256, 48, [47], scale=0.11, softcap=30.0)
    # prefill chunks: causal, causal + window (config 2's two layer kinds, reduced), a later chunk
    case("prefill_global", 0xC0FFEE + 1, 4, 1, 256, 32, list(range(32)))
    case("prefill_local", 0xC0FFEE + 11, 4, 1, 256, 32, list(range(32)), window=12)
    case("prefill_second_chunk", 0xC0FFEE + 14, 4, 2, 256, 48, list(range(20, 48)), window=24)
    kat = {
        "source": "runtime/components/sampling_cpu_util_test.cc:82-97 (values as held by the reference test)",
        "cases": [
            {"logits": [0.1, 0.1], "probabilities": [0.5, 0.5]},
            {"logits": [0.0, 5.0], "probabilities": [0.00669285096, 0.993307173]},
            {"logits": [1.0, 0.0], "probabilities": [0.731058598, 0.268941432]},
        ],
    }
    with open(os.path.join(HERE, "softmax_kat.json"), "w") as f:
        json.dump(kat, f, indent=1)


if __name__ == "__main__":
    main()
