"""GPU parity of the step before attention (RMS norm + rotary embedding + cache
write, mi355_attn_pre_attention) through the C ABI against
oracle/pre_attention_oracle.py on identical seeded inputs.

Tolerances (max|a-b| / max|ref| per tensor): fp32 <= 1e-5; fp16 / bf16 <= 2e-3
(the rounding of the output format); int8 rows: bit-exact where the rows pass
through unchanged, else at most one step on at most 0.1 % of the values (the
device's sine / cosine differ from the oracle's in the last bit, which can tip a
value that sits on a rounding boundary).
"""
import os
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from __graft_entry__ import load_package  # noqa: E402
from oracle import attn_oracle as orc  # noqa: E402
from oracle import pre_attention_oracle as po  # noqa: E402

A = load_package().attn
DEV = "cuda:0"
TOL = {A.F32: 1e-5, A.F16: 2e-3, A.BF16: 2e-3}
TDT = {A.F32: torch.float32, A.F16: torch.float16, A.BF16: torch.bfloat16, A.I8: torch.int8}
D = 256


def say(*a):
    print(*a, flush=True)


def make(num_layers, hq, hkv, max_tokens, max_seqs, kv, io=None, **kw):
    io = (A.F16 if kv == A.I8 else kv) if io is None else io
    return A.Attn(num_layers, hq, hkv, D, max_tokens, max_seqs, kv, io,
                  stream=torch.cuda.current_stream().cuda_stream, **kw)


def dev(x, dt):
    t = torch.from_numpy(np.ascontiguousarray(x)).to(DEV).to(TDT[dt]).contiguous()
    return t, t.float().cpu().numpy()


def gen(seed, *shape):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


def weights(seed):
    g = np.random.default_rng(seed)
    return (g.standard_normal(D) * 0.3).astype(np.float32), (g.standard_normal(D) * 0.3).astype(np.float32)


def rel(got, ref):
    return float(np.abs(got.astype(np.float64) - ref.astype(np.float64)).max() / np.abs(ref).max())


@pytest.mark.parametrize("dt", [A.F32, A.F16, A.BF16])
@pytest.mark.parametrize("hq,hkv", [(4, 1), (8, 2)])
def test_norm_rope_append_matches_oracle(dt, hq, hkv):
    say(f"pre_attention dt={dt} hq={hq} hkv={hkv}")
    cap, n1, n2 = 700, 133, 500  # two ragged chunks: positions 0..132 and 133..632
    qw, kw = weights(3)
    local, glob = po.rope_inv_freq(D, 10000.0), po.rope_inv_freq(D, 1000000.0)
    with make(2, hq, hkv, cap, 2, dt) as at:
        at.set_layer_transform(0, norm_q=True, norm_k=True, q_weight=qw, k_weight=kw, eps=1e-6, weight_offset=1.0,
                               rope_inv_freq=local)
        at.set_layer_transform(1, norm_q=True, norm_k=True, norm_v=True, q_weight=qw, k_weight=kw, eps=1e-6,
                               weight_offset=0.0, rope_inv_freq=glob)
        for layer, f, off, nv in ((0, local, 1.0, False), (1, glob, 0.0, True)):
            qd, q = dev(gen(10 + layer, n1 + n2, hq, D) * 3, dt)
            kd, k = dev(gen(20 + layer, n1 + n2, hkv, D) * 3, dt)
            vd, v = dev(gen(30 + layer, n1 + n2, hkv, D), dt)
            q_out = torch.zeros_like(qd)
            at.pre_attention(layer, 1, 0, qd[:n1].contiguous(), kd[:n1].contiguous(), vd[:n1].contiguous(), q_out[:n1])
            at.pre_attention(layer, 1, n1, qd[n1:].contiguous(), kd[n1:].contiguous(), vd[n1:].contiguous(), q_out[n1:])
            ko, vo = torch.zeros_like(kd), torch.zeros_like(vd)
            at.kv_read(layer, 1, 0, n1 + n2, ko, vo)
            torch.cuda.synchronize()
            want_q, want_k, want_v = po.pre_attention(q, k, v, 0, q_weight=qw, k_weight=kw, norm_q=True, norm_k=True,
                                                      norm_v=nv, eps=1e-6, weight_offset=off, inv_freq=f,
                                                      dtype=np.float64)
            for name, got, want in (("q", q_out, want_q), ("k", ko, want_k), ("v", vo, want_v)):
                e = rel(got.float().cpu().numpy(), want)
                say(f"  layer {layer} {name}: rel err {e:.2e}")
                if dt == A.BF16:
                    assert orc.rel_err_beyond_bf16_rounding(got.float().cpu().numpy(), want.astype(np.float32)) < TOL[dt]
                else:
                    assert e < TOL[dt], (layer, name, e)
        # the other sequence's planes were not touched
        k0, v0 = torch.ones(cap, hkv, D, device=DEV, dtype=TDT[dt]), torch.ones(cap, hkv, D, device=DEV, dtype=TDT[dt])
        at.kv_read(0, 0, 0, cap, k0, v0)
        torch.cuda.synchronize()
        assert not k0.any() and not v0.any()


@pytest.mark.parametrize("dt", [A.F32, A.F16, A.BF16])
def test_layer_without_constants_is_a_plain_append(dt):
    say(f"pre_attention passthrough dt={dt}")
    n, hq, hkv = 70, 4, 2
    with make(1, hq, hkv, 128, 1, dt) as at, make(1, hq, hkv, 128, 1, dt) as ref:
        qd, _ = dev(gen(1, n, hq, D), dt)
        kd, _ = dev(gen(2, n, hkv, D), dt)
        vd, _ = dev(gen(3, n, hkv, D), dt)
        q_out = torch.zeros_like(qd)
        at.pre_attention(0, 0, 9, qd, kd, vd, q_out)
        ref.kv_append(0, 0, 9, kd, vd)
        outs = []
        for h in (at, ref):
            ko, vo = torch.zeros_like(kd), torch.zeros_like(vd)
            h.kv_read(0, 0, 9, n, ko, vo)
            outs.append((ko, vo))
        torch.cuda.synchronize()
        assert torch.equal(q_out.view(torch.uint8), qd.view(torch.uint8))
        assert torch.equal(outs[0][0].view(torch.uint8), outs[1][0].view(torch.uint8))
        assert torch.equal(outs[0][1].view(torch.uint8), outs[1][1].view(torch.uint8))
        assert torch.equal(outs[0][0].view(torch.uint8), kd.view(torch.uint8))


def test_query_in_place():
    n, hq, hkv = 33, 8, 2
    f = po.rope_inv_freq(D, 10000.0)
    with make(1, hq, hkv, 64, 1, A.F32) as at:
        at.set_layer_transform(0, norm_q=True, norm_k=True, eps=1e-6, rope_inv_freq=f)
        qd, q = dev(gen(4, n, hq, D), A.F32)
        kd, k = dev(gen(5, n, hkv, D), A.F32)
        vd, v = dev(gen(6, n, hkv, D), A.F32)
        at.pre_attention(0, 0, 20, qd, kd, vd, qd)
        torch.cuda.synchronize()
        want_q, _, _ = po.pre_attention(q, k, v, 20, norm_q=True, norm_k=True, eps=1e-6, inv_freq=f, dtype=np.float64)
        assert rel(qd.cpu().numpy(), want_q) < 1e-5


def test_int8_rows():
    say("pre_attention int8 cache")
    n, hq, hkv = 300, 8, 2
    with make(2, hq, hkv, 512, 1, A.I8) as at:
        kf, vf = gen(7, n, hkv, D), gen(8, n, hkv, D)
        qd, q = dev(gen(9, n, hq, D), A.F16)
        kd, k = dev(kf, A.F16)
        vd, v = dev(vf, A.F16)
        k_scale = (np.abs(k).max(axis=0) / np.float32(127)).astype(np.float32)
        v_scale = (np.abs(v).max(axis=0) / np.float32(127)).astype(np.float32)
        v_scale[1, 17] = 0.0  # a dead channel stores zeros
        for layer in (0, 1):
            at.kv_set_scales(layer, 0, torch.from_numpy(k_scale).to(DEV), torch.from_numpy(v_scale).to(DEV))
        # layer 0: no constants -> the rows are quantised as they are: bit-exact
        q_out = torch.zeros_like(qd)
        at.pre_attention(0, 0, 0, qd, kd, vd, q_out)
        ko = torch.zeros(n, hkv, D, dtype=torch.int8, device=DEV)
        vo = torch.zeros_like(ko)
        at.kv_read(0, 0, 0, n, ko, vo)
        torch.cuda.synchronize()
        assert np.array_equal(ko.cpu().numpy(), po.quantize_rows(k, k_scale))
        assert np.array_equal(vo.cpu().numpy(), po.quantize_rows(v, v_scale))
        assert not vo[:, 1, 17].any()
        assert torch.equal(q_out, qd)
        # layer 1: norm + rotation first; scales for unit-RMS rows
        f = po.rope_inv_freq(D, 10000.0)
        at.set_layer_transform(1, norm_q=True, norm_k=True, eps=1e-6, rope_inv_freq=f)
        _, want_k, _ = po.pre_attention(q, k, v, 100, norm_q=True, norm_k=True, eps=1e-6, inv_freq=f)
        k_scale2 = (np.abs(want_k).max(axis=0) / np.float32(127)).astype(np.float32)
        at.kv_set_scales(1, 0, torch.from_numpy(k_scale2).to(DEV), torch.from_numpy(v_scale).to(DEV))
        at.pre_attention(1, 0, 100, qd, kd, vd, q_out)
        at.kv_read(1, 0, 100, n, ko, vo)
        torch.cuda.synchronize()
        want = po.quantize_rows(want_k, k_scale2).astype(np.int32)
        diff = np.abs(ko.cpu().numpy().astype(np.int32) - want)
        say(f"  int8 K after norm + rotation: {int((diff != 0).sum())} of {diff.size} values differ, max {int(diff.max())}")
        assert diff.max() <= 1 and (diff != 0).mean() < 1e-3
        assert np.array_equal(vo.cpu().numpy(), po.quantize_rows(v, v_scale))


def test_attention_over_rows_written_by_pre_attention():
    """The rows land where the attention kernels read them: prefill and decode over
    a cache filled by pre_attention equal the oracle's attention over the oracle's rows."""
    n, hq, hkv, dt = 200, 4, 1, A.F16
    f = po.rope_inv_freq(D, 10000.0)
    qw, kw = weights(11)
    with make(1, hq, hkv, 256, 1, dt, layer_window=[64]) as at:
        at.set_layer_transform(0, norm_q=True, norm_k=True, q_weight=qw, k_weight=kw, eps=1e-6, rope_inv_freq=f)
        qd, q = dev(gen(12, n, hq, D), dt)
        kd, k = dev(gen(13, n, hkv, D), dt)
        vd, v = dev(gen(14, n, hkv, D), dt)
        q_rot = torch.zeros_like(qd)
        at.pre_attention(0, 0, 0, qd, kd, vd, q_rot)
        out = torch.zeros_like(qd)
        at.prefill(0, 0, 0, n, q_rot, out)
        out1 = torch.zeros(1, hq, D, dtype=TDT[dt], device=DEV)
        at.decode(0, [n], q_rot[n - 1:n].contiguous(), out1)
        torch.cuda.synchronize()
        want_q, want_k, want_v = po.pre_attention(q, k, v, 0, q_weight=qw, k_weight=kw, norm_q=True, norm_k=True,
                                                  eps=1e-6, inv_freq=f)
        r16 = lambda x: x.astype(np.float16).astype(np.float32)
        want = orc.sdpa(r16(want_q), r16(want_k), r16(want_v), D ** -0.5, q_pos0=0, window=64)
        assert orc.rel_err(out.float().cpu().numpy(), want) < 2e-3
        assert orc.rel_err(out1.float().cpu().numpy()[0], want[n - 1]) < 2e-3


def test_argument_checks():
    with make(2, 4, 1, 64, 1, A.F16) as at:
        q = torch.zeros(4, 4, D, dtype=torch.float16, device=DEV)
        kv = torch.zeros(4, 1, D, dtype=torch.float16, device=DEV)
        with pytest.raises(A.AttnError) as e:
            at.pre_attention(0, 0, 62, q, kv, kv, q)
        assert e.value.code == A.OUT_OF_RANGE
        with pytest.raises(A.AttnError) as e:
            at.pre_attention(2, 0, 0, q, kv, kv, q)
        assert e.value.code == A.INVALID_ARGUMENT
        with pytest.raises(A.AttnError) as e:
            at.pre_attention(0, 1, 0, q, kv, kv, q)
        assert e.value.code == A.INVALID_ARGUMENT
        with pytest.raises(A.AttnError) as e:
            at.set_layer_transform(0, eps=-1.0)
        assert e.value.code == A.INVALID_ARGUMENT
        bad = np.full(D // 2, np.nan, np.float32)
        with pytest.raises(A.AttnError) as e:
            at.set_layer_transform(0, rope_inv_freq=bad)
        assert e.value.code == A.INVALID_ARGUMENT
        at.pre_attention(0, 0, 0, q, kv, kv, q, n=0)  # nothing to do


@pytest.mark.parametrize("dt", [A.F32, A.F16, A.BF16])
def test_gemma3_fixture(dt):
    """The HIP path against tests/golden/gemma3_pre_attention.npz (float64 results of
    the transformers Gemma 3 blocks; inputs exact in every dtype)."""
    c = np.load(os.path.join(ROOT, "tests", "golden", "gemma3_pre_attention.npz"))
    n, hq, _ = c["q"].shape
    pos0 = int(c["pos0"])
    with make(2, hq, c["k"].shape[1], pos0 + n, 1, dt) as at:
        for layer, kind in enumerate(("sliding_attention", "full_attention")):
            at.set_layer_transform(layer, norm_q=True, norm_k=True, q_weight=c["q_weight"], k_weight=c["k_weight"],
                                   eps=float(c["eps"]), weight_offset=1.0, rope_inv_freq=c[f"inv_freq_{kind}"])
            qd, _ = dev(c["q"], dt)
            kd, _ = dev(c["k"], dt)
            vd = torch.zeros_like(kd)
            q_out, ko, vo = torch.zeros_like(qd), torch.zeros_like(kd), torch.ones_like(kd)
            at.pre_attention(layer, 0, pos0, qd, kd, vd, q_out)
            at.kv_read(layer, 0, pos0, n, ko, vo)
            torch.cuda.synchronize()
            for got, want in ((q_out, c[f"q_out_{kind}"]), (ko, c[f"k_out_{kind}"])):
                g = got.float().cpu().numpy()
                e = orc.rel_err_beyond_bf16_rounding(g, want) if dt == A.BF16 else rel(g, want)
                say(f"  gemma3 fixture dt={dt} {kind}: {e:.2e}")
                assert e < TOL[dt]
            assert not vo.any()
