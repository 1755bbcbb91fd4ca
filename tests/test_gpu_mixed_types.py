"""GPU parity where the activation type (queries in, attention out) differs from the cache's type.

float32 activations over a 16-bit cache is the reference's own split (ActivationDataType::FLOAT32 over the
fp16 cache of its GPU path, runtime/executor/executor_settings_base.h:54-66,
llm_litert_compiled_model_executor.cc:609-617). It is also where the stated tolerance can be read
literally for a bfloat16 cache: with float32 output nothing is lost to the output format, so the plain
norm-wise error max|a-b| / max|ref| of the bfloat16 arithmetic itself is held to 2e-3, no allowance. The
bfloat16-output result is then shown to be that float32 result rounded once, bit for bit.
"""
import glob
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
from oracle import c_oracle  # noqa: E402

A = load_package().attn
DEV = "cuda:0"
TDT = {A.F32: torch.float32, A.F16: torch.float16, A.BF16: torch.bfloat16, A.I8: torch.int8}
D = 256
TOL16 = 2e-3  # the stated bound for fp16 / bf16 arithmetic, applied to the plain norm-wise error


def say(*a):
    print(*a, flush=True)


def make(num_layers, hq, hkv, max_tokens, max_seqs, kv, io, **kw):
    return A.Attn(num_layers, hq, hkv, D, max_tokens, max_seqs, kv, io,
                  stream=torch.cuda.current_stream().cuda_stream, **kw)


def gen(seed, *shape):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


def rounded(x, dt):
    """fp32 numpy -> (device tensor in dt, the values it holds as fp32 numpy)."""
    t = torch.from_numpy(np.ascontiguousarray(x)).to(DEV).to(TDT[dt]).contiguous()
    return t, t.float().cpu().numpy()


def append(at, kv, layer, seq, k, v):
    kd, kr = rounded(k, kv)
    vd, vr = rounded(v, kv)
    at.kv_append(layer, seq, 0, kd, vd)
    return kr, vr


def match_note(got16, ref):
    share, worst = orc.bf16_output_match(got16, ref)
    return f"equal to the correctly rounded result on {100 * share:.2f} % of the elements, others within {worst} bfloat16 step(s)"


# ------------------------------------------------------------------ decode, config 3 at full size
@pytest.mark.parametrize("kv", [A.BF16, A.F16])
def test_c3_decode_fp32_activations_meet_the_stated_bound_literally(kv):
    seed = orc.SEED_BASE + 2
    q = gen(seed, 1, 8, D)
    k, v = gen(seed + 100, 4096, 2, D), gen(seed + 200, 4096, 2, D)
    with make(1, 8, 2, 4096, 1, kv, A.F32) as at32, make(1, 8, 2, 4096, 1, kv, kv) as at16:
        kr, vr = append(at32, kv, 0, 0, k, v)
        append(at16, kv, 0, 0, k, v)
        q16, qr = rounded(q, kv)          # queries that the cache's type holds exactly ...
        q32 = q16.float().contiguous()    # ... handed over as float32
        ref = c_oracle.sdpa_f64(qr[0:1], kr, vr, D ** -0.5, q_pos0=4095, kv_len=4096)[0]
        for waves in (4, 2, 1):
            at32.set_option("decode_waves", waves)
            at16.set_option("decode_waves", waves)
            for ns in (16, 1, 5, 0):
                out32 = torch.full((1, 8, D), float("nan"), device=DEV)
                at32.decode(0, [4096], q32, out32, num_splits=ns)
                out16 = torch.empty_like(q16)
                at16.decode(0, [4096], q16, out16, num_splits=ns)
                torch.cuda.synchronize()
                err = orc.rel_err(out32.cpu().numpy()[0], ref)
                say(f"C3 kv={kv} fp32 out waves={waves} splits={ns}: plain rel_err {err:.3e}")
                assert err < TOL16
                # the 16-bit output is the float32 one rounded once
                assert torch.equal(out16, out32.to(TDT[kv])), (waves, ns)
        if kv == A.BF16:
            say("  bf16 output: " + match_note(out16.float().cpu().numpy()[0], ref))
        # float32 queries that the cache's type does not hold exactly are rounded to it on the way in:
        # the result is that of the rounded queries, and the distance to the oracle on the unrounded ones is
        # reported (fp16 keeps 11 significant bits of a query, bf16 8)
        qx = torch.from_numpy(q).to(DEV)
        outx = torch.empty((1, 8, D), device=DEV)
        at32.decode(0, [4096], qx, outx, num_splits=16)
        at32.decode(0, [4096], q32, out32, num_splits=16)
        torch.cuda.synchronize()
        assert torch.equal(outx, out32)
        refx = c_oracle.sdpa_f64(q[0:1], kr, vr, D ** -0.5, q_pos0=4095, kv_len=4096)[0]
        errx = orc.rel_err(outx.cpu().numpy()[0], refx)
        say(f"  unrounded float32 queries against the oracle on them: {errx:.3e}")
        assert errx < (TOL16 if kv == A.F16 else 2.0 ** -8 + TOL16)


# ------------------------------------------------------------------ prefill, config 2: the launch bench.py times
@pytest.mark.parametrize("kv", [A.BF16, A.F16])
def test_c2_benched_launch_fp32_activations_every_layer_literal_bound(kv):
    layers, n, hq, hkv = 26, 1024, 4, 1
    windows = [0 if (l + 1) % 6 == 0 else 512 for l in range(layers)]
    seed = orc.SEED_BASE + 1
    with make(layers, hq, hkv, n, 1, kv, A.F32, layer_window=windows) as at32, \
            make(layers, hq, hkv, n, 1, kv, kv, layer_window=windows) as at16:
        krs, vrs = [], []
        for layer in range(layers):
            kr, vr = append(at32, kv, layer, 0, gen(seed + 100 + layer, n, hkv, D), gen(seed + 200 + layer, n, hkv, D))
            append(at16, kv, layer, 0, gen(seed + 100 + layer, n, hkv, D), gen(seed + 200 + layer, n, hkv, D))
            krs.append(kr)
            vrs.append(vr)
        q16, qr = rounded(gen(seed + 300, layers, n, hq, D), kv)
        q32 = q16.float().contiguous()
        out32 = torch.full_like(q32, float("nan"))
        out16 = torch.full_like(q16, float("nan"))
        at32.prefill(0, 0, 0, n, q32, out32, n_layers=layers)
        at16.prefill(0, 0, 0, n, q16, out16, n_layers=layers)
        torch.cuda.synchronize()
        got = out32.cpu().numpy()
        assert np.isfinite(got).all()
        worst, shares = 0.0, []
        for layer, w in enumerate(windows):
            ref = c_oracle.sdpa_f64(qr[layer], krs[layer], vrs[layer], D ** -0.5, window=w)
            err = orc.rel_err(got[layer], ref)
            worst = max(worst, err)
            assert err < TOL16, (kv, layer, w, err)
            if kv == A.BF16:
                shares.append(orc.bf16_output_match(out16[layer].float().cpu().numpy(), ref))
        say(f"C2 benched launch kv={kv}, float32 activations: worst layer plain rel_err {worst:.3e}")
        # same arithmetic, one rounding: the 16-bit launch returns the float32 result rounded to its type
        assert torch.equal(out16, out32.to(TDT[kv]))
        if shares:
            say(f"  bf16 output equals the correctly rounded oracle result on {100 * min(s for s, _ in shares):.2f} % "
                f"(worst layer) of the elements; others within {max(d for _, d in shares)} bfloat16 step(s)")


@pytest.mark.parametrize("rows16", [0, 1], ids=["mfma32", "mfma16"])
@pytest.mark.parametrize("kv", [A.BF16, A.F16])
@pytest.mark.parametrize("hq,hkv", [(4, 1), (8, 2), (3, 1)])
def test_prefill_fp32_activations_small_shapes_both_kernels(kv, hq, hkv, rows16):
    """Ragged chunks, windows, later chunks of a longer context, key splits (the merge kernel writes the
    float32 output then) and the row-wise path, float32 in and out over a 16-bit cache."""
    windows = [0, 40, 1, 33]
    L = 400
    with make(len(windows), hq, hkv, L, 1, kv, A.F32, layer_window=windows) as at:
        at.set_option("prefill_rows16", rows16)
        k, v = gen(61, L, hkv, D), gen(62, L, hkv, D)
        for layer, w in enumerate(windows):
            kr, vr = append(at, kv, layer, 0, k, v)
            for q_pos0, n in ((0, 1), (0, 33), (0, 257), (70, 64), (129, 200), (399, 1)):
                q16, qr = rounded(gen(1000 + n + q_pos0, n, hq, D), kv)
                q32 = q16.float().contiguous()
                ref = c_oracle.sdpa_f64(qr, kr, vr, D ** -0.5, q_pos0=q_pos0, window=w, kv_len=q_pos0 + n)
                for split, rowwise in ((0, 0), (2, 0), (0, 1)):
                    at.set_option("prefill_key_split", split)
                    at.set_option("rowwise_prefill", rowwise)
                    out = torch.full_like(q32, float("nan"))
                    at.prefill(layer, 0, q_pos0, n, q32, out)
                    torch.cuda.synchronize()
                    err = orc.rel_err(out.cpu().numpy(), ref)
                    assert err < TOL16, (kv, hq, hkv, w, q_pos0, n, split, rowwise, err)
        at.set_option("prefill_key_split", -1)
        at.set_option("rowwise_prefill", 0)
    say(f"prefill float32 activations kv={kv} hq={hq} hkv={hkv} rows16={rows16}: ok")


def test_prefill_fp32_activations_softcap():
    with make(1, 4, 1, 300, 1, A.F16, A.F32, scale=0.11, softcap=3.0) as at:
        kr, vr = append(at, A.F16, 0, 0, gen(21, 300, 1, D), gen(22, 300, 1, D))
        q16, qr = rounded(3.0 * gen(23, 300, 4, D), A.F16)
        ref = orc.sdpa(qr, kr, vr, 0.11, softcap=3.0)
        for rows16 in (0, 1):
            at.set_option("prefill_rows16", rows16)
            out = torch.empty((300, 4, D), device=DEV)
            at.prefill(0, 0, 0, 300, q16.float().contiguous(), out)
            torch.cuda.synchronize()
            assert orc.rel_err(out.cpu().numpy(), ref) < TOL16


# ------------------------------------------------------------------ golden vectors
GOLDEN = sorted(glob.glob(os.path.join(ROOT, "tests", "golden", "decode_*.npz")) +
                glob.glob(os.path.join(ROOT, "tests", "golden", "prefill_*.npz")))


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
@pytest.mark.parametrize("kv", [A.BF16, A.F16])
def test_golden_vectors_fp32_activations_literal_bound(path, kv):
    """The committed vectors (inputs exact in every type, expected output from an independent float64
    routine) through a 16-bit cache with float32 activations: plain error under 2e-3."""
    z = np.load(path)
    q, k, v, want = z["q"], z["k"], z["v"], z["out"]
    q_pos0, n, L = int(z["q_pos"][0]), q.shape[0], k.shape[0]
    window, scale, softcap = int(z["window"]), float(z["scale"]), float(z["softcap"])
    hq, hkv = q.shape[1], k.shape[1]
    with make(1, hq, hkv, L, 1, kv, A.F32, layer_window=[window], scale=scale, softcap=softcap) as at:
        kr, vr = append(at, kv, 0, 0, k, v)
        assert np.array_equal(kr, k) and np.array_equal(vr, v)
        qd = torch.from_numpy(q).to(DEV)
        out = torch.empty_like(qd)
        if n == 1:
            for splits in (0, 1, 2):
                at.decode(0, [L], qd, out, num_splits=splits)
                torch.cuda.synchronize()
                err = orc.rel_err(out.cpu().numpy(), want)
                assert err < TOL16, (os.path.basename(path), kv, splits, err)
        else:
            for rows16 in (0, 1):
                at.set_option("prefill_rows16", rows16)
                at.prefill(0, 0, q_pos0, n, qd, out)
                torch.cuda.synchronize()
                err = orc.rel_err(out.cpu().numpy(), want)
                assert err < TOL16, (os.path.basename(path), kv, rows16, err)
        say(f"golden {os.path.basename(path)} kv={kv} float32 activations: plain rel_err {err:.3e}")


# ------------------------------------------------------------------ int8 cache with any activation type
@pytest.mark.parametrize("io", [A.F16, A.BF16, A.F32])
def test_int8_cache_with_each_activation_type(io):
    lens = [1000, 65, 2048]
    with make(1, 8, 2, 2048, 3, A.I8, io) as at:
        kvs = []
        for b, n in enumerate(lens):
            kq, ks = orc.quantize_kv_int8(gen(300 + b, n, 2, D))
            vq, vs = orc.quantize_kv_int8(gen(400 + b, n, 2, D))
            at.kv_append(0, b, 0, torch.from_numpy(kq).to(DEV), torch.from_numpy(vq).to(DEV))
            at.kv_set_scales(0, b, torch.from_numpy(ks).to(DEV), torch.from_numpy(vs).to(DEV))
            kvs.append((orc.dequantize_kv_int8(kq, ks), orc.dequantize_kv_int8(vq, vs)))
        qd, qr = rounded(gen(9, len(lens), 8, D), io)
        for ns in (1, 7):
            out = torch.empty_like(qd)
            at.decode(0, lens, qd, out, num_splits=ns)
            torch.cuda.synchronize()
            got = out.float().cpu().numpy()
            for b, n in enumerate(lens):
                ref = c_oracle.sdpa_f64(qr[b:b + 1], kvs[b][0], kvs[b][1], D ** -0.5, q_pos0=n - 1, kv_len=n)[0]
                if io == A.BF16:  # a bfloat16 output: format-aware figures, as everywhere else
                    assert orc.l2_rel_err(got[b], ref) < TOL16
                    err = orc.rel_err_beyond_bf16_rounding(got[b], ref)
                else:
                    err = orc.rel_err(got[b], ref)
                assert err < TOL16, (io, ns, b, err)
        # a prefill chunk over the int8 cache in this activation type
        n = 130
        qd, qr = rounded(gen(19, n, 8, D), io)
        out = torch.empty_like(qd)
        at.prefill(0, 0, 1000 - n, n, qd, out)
        torch.cuda.synchronize()
        ref = c_oracle.sdpa_f64(qr, kvs[0][0], kvs[0][1], D ** -0.5, q_pos0=1000 - n, kv_len=1000)
        got = out.float().cpu().numpy()
        err = orc.rel_err_beyond_bf16_rounding(got, ref) if io == A.BF16 else orc.rel_err(got, ref)
        say(f"int8 cache, activations {io}: prefill rel_err {err:.3e}")
        assert err < TOL16


# ------------------------------------------------------------------ the fused decode step with mixed types
@pytest.mark.parametrize("kv,io", [(A.BF16, A.F32), (A.F16, A.F32), (A.I8, A.BF16), (A.I8, A.F32)])
def test_decode_step_equals_two_calls_with_mixed_types(kv, io):
    hq, hkv, L = 8, 2, 300
    lens = [L, 77, 129]
    inv_freq = (10000.0 ** (-np.arange(0, D, 2, dtype=np.float64) / D)).astype(np.float32)
    qw, kw = gen(5, D) * 0.1, gen(6, D) * 0.1
    outs = []
    for fused in (0, 1):
        with make(1, hq, hkv, L, len(lens), kv, io) as at:
            at.set_layer_transform(0, norm_q=True, norm_k=True, norm_v=True, q_weight=qw, k_weight=kw, rope_inv_freq=inv_freq)
            for b, n in enumerate(lens):
                if kv == A.I8:
                    sc = torch.full((hkv, D), 0.03, device=DEV)
                    at.kv_set_scales(0, b, sc, sc)
                # rows [0, n - 1) through the step before attention, in the activation type
                qa, _ = rounded(gen(50 + b, n - 1, hq, D), io)
                ka, _ = rounded(gen(60 + b, n - 1, hkv, D), io)
                va, _ = rounded(gen(70 + b, n - 1, hkv, D), io)
                if n > 1:
                    at.pre_attention(0, b, 0, qa, ka, va, torch.empty_like(qa))
            q, _ = rounded(gen(80, len(lens), hq, D), io)
            k, _ = rounded(gen(81, len(lens), hkv, D), io)
            v, _ = rounded(gen(82, len(lens), hkv, D), io)
            out = torch.full_like(q, float("nan"))
            if fused:
                at.decode_step(0, lens, q, k, v, out, num_splits=3)
            else:
                qn = torch.empty_like(q)
                for b, n in enumerate(lens):
                    at.pre_attention(0, b, n - 1, q[b:b + 1].contiguous(), k[b:b + 1].contiguous(), v[b:b + 1].contiguous(),
                                     qn[b:b + 1])
                at.decode(0, lens, qn, out, num_splits=3)
            kc = torch.empty((L, hkv, D), dtype=TDT[kv], device=DEV)
            vc = torch.empty_like(kc)
            at.kv_read(0, 0, 0, L, kc, vc)
            torch.cuda.synchronize()
            assert torch.isfinite(out.float()).all()
            outs.append((out.clone(), kc.clone(), vc.clone()))
    assert torch.equal(outs[0][0], outs[1][0])
    assert torch.equal(outs[0][1].view(torch.uint8), outs[1][1].view(torch.uint8))
    assert torch.equal(outs[0][2].view(torch.uint8), outs[1][2].view(torch.uint8))


def test_unsupported_pairs_are_rejected_at_creation():
    for kv, io in ((A.F32, A.F16), (A.F32, A.BF16), (A.F16, A.BF16), (A.BF16, A.F16)):
        with pytest.raises(A.AttnError) as e:
            A.Attn(1, 4, 1, D, 16, 1, kv, io)
        assert e.value.code == A.UNIMPLEMENTED
