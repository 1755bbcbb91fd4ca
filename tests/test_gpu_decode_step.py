"""GPU tests of mi355_attn_decode_step (the step before attention for the one new
token of every sequence and decode attention in one launch) through the C ABI.

The entry point promises the bits of mi355_attn_pre_attention (n = 1, per
sequence) followed by mi355_attn_decode: outputs and the new cache rows are
compared bit for bit between a handle driven one way and a handle driven the
other, over several consecutive steps (the new row crosses block and partition
boundaries), dtypes, head groupings, windows, ragged batches, split counts and
workgroup shapes; one case is also checked against the oracles
(oracle/pre_attention_oracle.py rows, oracle/attn_oracle.py attention) to the
tolerance of the decode tests (2e-3 of the largest reference value for fp16).
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
TDT = {A.F32: torch.float32, A.F16: torch.float16, A.BF16: torch.bfloat16, A.I8: torch.int8}
D = 256


def say(*a):
    print(*a, flush=True)


def make(num_layers, hq, hkv, max_tokens, max_seqs, kv, **kw):
    io = A.F16 if kv == A.I8 else kv
    return A.Attn(num_layers, hq, hkv, D, max_tokens, max_seqs, kv, io,
                  stream=torch.cuda.current_stream().cuda_stream, **kw)


def rows(seed, dt, *shape):
    g = torch.Generator(device=DEV).manual_seed(seed)
    io = torch.float16 if dt == A.I8 else TDT[dt]
    return torch.randn(shape, generator=g, device=DEV).to(io)


def set_up_layers(at, kv, n_layers, max_seqs, hkv, seed):
    """Gemma-3-like constants on layer 0, norms without weights and a value norm on layer 1, none on layer 2."""
    g = np.random.default_rng(seed)
    qw, kw = (g.standard_normal(D) * 0.3).astype(np.float32), (g.standard_normal(D) * 0.3).astype(np.float32)
    at.set_layer_transform(0, norm_q=True, norm_k=True, q_weight=qw, k_weight=kw, eps=1e-6,
                           rope_inv_freq=po.rope_inv_freq(D, 10000.0))
    if n_layers > 1:
        at.set_layer_transform(1, norm_q=True, norm_k=True, norm_v=True, eps=1e-5, weight_offset=0.0,
                               rope_inv_freq=po.rope_inv_freq(D, 1000000.0))
    if kv == A.I8:
        for layer in range(n_layers):
            for s in range(max_seqs):
                ks = torch.from_numpy((g.random((hkv, D)) * 0.02 + 0.02).astype(np.float32)).to(DEV)
                vs = torch.from_numpy((g.random((hkv, D)) * 0.02 + 0.02).astype(np.float32)).to(DEV)
                at.kv_set_scales(layer, s, ks, vs)


def drive_both(kv, hq, hkv, lens0, steps, windows, splits, waves, seq_ids=None, seed=1):
    """Two handles with the same prefix; `steps` decode steps: one by pre_attention + decode, one by decode_step.
    Returns nothing; asserts equal outputs and equal new cache rows at every step and layer."""
    n_layers = len(windows)
    B = len(lens0)
    max_seqs = (max(seq_ids) + 1) if seq_ids else B
    cap = max(lens0) + steps + 1
    sids = seq_ids or list(range(B))
    io = torch.float16 if kv == A.I8 else TDT[kv]
    with make(n_layers, hq, hkv, cap, max_seqs, kv, layer_window=windows) as two, \
            make(n_layers, hq, hkv, cap, max_seqs, kv, layer_window=windows) as one:
        for at in (two, one):
            set_up_layers(at, kv, n_layers, max_seqs, hkv, seed)
            at.set_option("decode_waves", waves)
            for layer in range(n_layers):
                for b, n in enumerate(lens0):
                    q0 = rows(seed * 1000 + layer * 100 + b, kv, n, hq, D)
                    k0 = rows(seed * 1000 + layer * 100 + b + 50, kv, n, hkv, D)
                    v0 = rows(seed * 1000 + layer * 100 + b + 75, kv, n, hkv, D)
                    at.pre_attention(layer, sids[b], 0, q0, k0, v0, torch.empty_like(q0))
        for step in range(steps):
            lens = [n + step + 1 for n in lens0]
            for layer in range(n_layers):
                q = rows(seed * 7 + step * 13 + layer, kv, B, hq, D)
                k = rows(seed * 7 + step * 13 + layer + 3, kv, B, hkv, D)
                v = rows(seed * 7 + step * 13 + layer + 5, kv, B, hkv, D)
                q_rot = torch.empty_like(q)
                for b in range(B):
                    two.pre_attention(layer, sids[b], lens[b] - 1, q[b:b + 1], k[b:b + 1], v[b:b + 1], q_rot[b:b + 1])
                want = torch.full((B, hq, D), 7.0, device=DEV).to(io)
                two.decode(layer, lens, q_rot, want, seq_ids=seq_ids, num_splits=splits)
                got = torch.full((B, hq, D), -7.0, device=DEV).to(io)
                one.decode_step(layer, lens, q, k, v, got, seq_ids=seq_ids, num_splits=splits)
                torch.cuda.synchronize()
                assert torch.isfinite(want.float()).all()
                assert torch.equal(got, want), (f"step {step} layer {layer}: "
                                                f"{int((got != want).sum())} of {got.numel()} outputs differ")
                for b in range(B):
                    ka, va = (torch.zeros(1, hkv, D, dtype=TDT[kv], device=DEV) for _ in range(2))
                    kb, vb = torch.ones_like(ka), torch.ones_like(va)
                    two.kv_read(layer, sids[b], lens[b] - 1, 1, ka, va)
                    one.kv_read(layer, sids[b], lens[b] - 1, 1, kb, vb)
                    torch.cuda.synchronize()
                    assert torch.equal(ka, kb) and torch.equal(va, vb), f"step {step} layer {layer} seq {b}: cache rows"


@pytest.mark.parametrize("kv", [A.F16, A.BF16, A.F32, A.I8])
@pytest.mark.parametrize("waves", [0, 1, 2, 4])
def test_one_sequence_over_block_boundaries(kv, waves):
    say(f"decode_step kv {kv} waves {waves}: one sequence, the new row crosses blocks and partitions")
    # 126 -> rows 126 .. 131: the end of one 64-row partition, the start of the next, all block sizes (16 / 32 / 64)
    drive_both(kv, 4, 1, [126], 6, [0, 48, 0], 0, waves)


@pytest.mark.parametrize("kv", [A.F16, A.I8])
@pytest.mark.parametrize("splits", [0, 1, 3, 16])
def test_ragged_batch_and_sequence_ids(kv, splits):
    say(f"decode_step kv {kv} splits {splits}: ragged batch, permuted cache slots, 8 query heads on 2 KV heads")
    drive_both(kv, 8, 2, [1, 63, 64, 200, 517, 31], 3, [0, 128], splits, 0, seq_ids=[5, 0, 3, 2, 1, 4], seed=2)


def test_sixteen_heads_per_kv_head_from_an_empty_cache():
    say("decode_step: 16 query heads on 1 KV head, first token of an empty sequence")
    drive_both(A.F16, 16, 1, [0], 4, [0], 0, 0, seed=3)
    drive_both(A.BF16, 16, 1, [0, 40], 2, [32], 2, 1, seed=4)


def test_full_batch_of_64():
    say("decode_step: 64 sequences")
    lens = [int(x) for x in np.random.default_rng(5).integers(1, 300, size=64)]
    drive_both(A.F16, 4, 1, lens, 2, [0], 0, 0, seed=5)


def test_more_sequences_than_one_launch_holds():
    say("decode_step: 150 sequences (three launches behind one call), permuted cache slots")
    g = np.random.default_rng(9)
    lens = [int(x) for x in g.integers(1, 120, size=150)]
    drive_both(A.F16, 8, 2, lens, 2, [0, 40], 0, 0, seq_ids=[int(x) for x in g.permutation(150)], seed=9)


@pytest.mark.parametrize("kv", [A.F16, A.BF16, A.I8])
def test_long_context(kv):
    say(f"decode_step kv {kv}: context 4090 -> 4096, positions where the angles are thousands of radians")
    drive_both(kv, 8, 2, [4090], 6, [0, 512], 0, 0, seed=6)
    drive_both(kv, 8, 2, [4090, 2047], 2, [0], 16, 0, seed=7)


def test_against_the_oracles():
    """Rows and attention of one fused step against the CPU oracles (fp16, window 64)."""
    n, hq, hkv, dt = 200, 4, 1, A.F16
    f = po.rope_inv_freq(D, 10000.0)
    g = np.random.default_rng(11)
    qw, kw = (g.standard_normal(D) * 0.3).astype(np.float32), (g.standard_normal(D) * 0.3).astype(np.float32)
    with make(1, hq, hkv, 256, 1, dt, layer_window=[64]) as at:
        at.set_layer_transform(0, norm_q=True, norm_k=True, q_weight=qw, k_weight=kw, eps=1e-6, rope_inv_freq=f)
        q, k, v = rows(12, dt, n, hq, D), rows(13, dt, n, hkv, D), rows(14, dt, n, hkv, D)
        at.pre_attention(0, 0, 0, q[:n - 1], k[:n - 1], v[:n - 1], torch.empty_like(q[:n - 1]))
        out = torch.zeros(1, hq, D, dtype=TDT[dt], device=DEV)
        at.decode_step(0, [n], q[n - 1:], k[n - 1:], v[n - 1:], out)
        torch.cuda.synchronize()
        host = lambda x: x.float().cpu().numpy()
        want_q, want_k, want_v = po.pre_attention(host(q), host(k), host(v), 0, q_weight=qw, k_weight=kw, norm_q=True,
                                                  norm_k=True, eps=1e-6, inv_freq=f)
        r16 = lambda x: x.astype(np.float16).astype(np.float32)
        want = orc.sdpa(r16(want_q), r16(want_k), r16(want_v), D ** -0.5, q_pos0=0, window=64)
        err = orc.rel_err(host(out)[0], want[n - 1])
        say(f"  fused step against the oracles: {err:.2e}")
        assert err < 2e-3
        ko, vo = (torch.zeros(1, hkv, D, dtype=TDT[dt], device=DEV) for _ in range(2))
        at.kv_read(0, 0, n - 1, 1, ko, vo)
        torch.cuda.synchronize()
        assert orc.rel_err(host(ko)[0], want_k[n - 1]) < 2e-3
        assert orc.rel_err(host(vo)[0], want_v[n - 1]) < 2e-3


def test_replayed_from_a_hip_graph():
    """Three layers' steps captured into one HIP graph (the calls allocate nothing once the split-KV workspace
    exists) and replayed several times, with eager work and synchronisations in between: every replay leaves
    what the eager calls left."""
    hq, hkv, dt, n, layers = 8, 2, A.F16, 333, 3
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with A.Attn(layers, hq, hkv, D, 512, 1, dt, dt, layer_window=[0, 64, 0], stream=side.cuda_stream) as at:
            for layer in range(layers):
                at.set_layer_transform(layer, norm_q=True, norm_k=True, eps=1e-6,
                                       rope_inv_freq=po.rope_inv_freq(D, 10000.0))
                q0, k0, v0 = rows(31 + layer, dt, n - 1, hq, D), rows(41 + layer, dt, n - 1, hkv, D), rows(51 + layer, dt, n - 1, hkv, D)
                at.pre_attention(layer, 0, 0, q0, k0, v0, torch.empty_like(q0))
            q, k, v = rows(61, dt, layers, 1, hq, D), rows(62, dt, layers, 1, hkv, D), rows(63, dt, layers, 1, hkv, D)
            out = torch.zeros_like(q)

            def steps():
                for layer in range(layers):
                    at.decode_step(layer, [n], q[layer], k[layer], v[layer], out[layer])

            steps()  # eager: the workspace is allocated here
            side.synchronize()
            want = out.clone()
            assert torch.isfinite(want.float()).all() and want.float().abs().max() > 0
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                steps()
            for replay in range(4):
                out.zero_()
                side.synchronize()
                graph.replay()
                side.synchronize()
                assert torch.equal(out, want), f"replay {replay}"
                steps()  # eager work between the replays
                side.synchronize()
                assert torch.equal(out, want)
            del graph


def test_host_pointers():
    """A handle that stages host buffers (host_io = 1) gives the same step."""
    hq, hkv, dt, n = 4, 1, A.F16, 70
    outs = []
    for host_io in (False, True):
        with A.Attn(1, hq, hkv, D, 128, 1, dt, dt, host_io=host_io,
                    stream=torch.cuda.current_stream().cuda_stream) as at:
            at.set_layer_transform(0, norm_q=True, norm_k=True, eps=1e-6, rope_inv_freq=po.rope_inv_freq(D, 10000.0))
            q, k, v = rows(21, dt, n, hq, D), rows(22, dt, n, hkv, D), rows(23, dt, n, hkv, D)
            place = (lambda x: x.cpu().contiguous()) if host_io else (lambda x: x)
            q, k, v = place(q), place(k), place(v)
            at.pre_attention(0, 0, 0, q[:n - 1], k[:n - 1], v[:n - 1], torch.empty_like(q[:n - 1]))
            out = torch.zeros_like(q[:1])
            at.decode_step(0, [n], q[n - 1:], k[n - 1:], v[n - 1:], out)
            at.sync()
            outs.append(out.cpu())
    assert torch.equal(outs[0], outs[1])


def test_argument_checks_and_row_accounting():
    hq, hkv, dt = 4, 1, A.F16
    with make(1, hq, hkv, 128, 70, dt) as at:
        q = torch.zeros(70, hq, D, dtype=torch.float16, device=DEV)
        kv = torch.zeros(70, hkv, D, dtype=torch.float16, device=DEV)
        out = torch.zeros_like(q)
        with pytest.raises(A.AttnError) as e:  # rows [0, 4) were never appended
            at.decode_step(0, [5], q[:1], kv[:1], kv[:1], out[:1])
        assert e.value.code == A.OUT_OF_RANGE
        with pytest.raises(A.AttnError) as e:
            at.decode_step(0, [1, 1], q[:2], kv[:2], kv[:2], out[:2], seq_ids=[3, 3])
        assert e.value.code == A.INVALID_ARGUMENT
        with pytest.raises(A.AttnError) as e:  # a batch cut into two launches is checked as a whole before the first
            at.decode_step(0, [1] * 64 + [2], q[:65], kv[:65], kv[:65], out[:65])
        assert e.value.code == A.OUT_OF_RANGE
        with pytest.raises(A.AttnError) as e:
            at.decode_step(0, [1] * 65, q[:65], kv[:65], kv[:65], out[:65], seq_ids=list(range(64)) + [5])
        assert e.value.code == A.INVALID_ARGUMENT
        at.decode_step(0, [1] * 64, q[:64], kv[:64], kv[:64], out[:64])  # (nothing of the refused calls was written)
        at.reset()
        with pytest.raises(A.AttnError) as e:
            at.decode_step(1, [1], q[:1], kv[:1], kv[:1], out[:1])
        assert e.value.code == A.INVALID_ARGUMENT
        # the step's row counts as appended: the next step and a plain decode over it are accepted
        at.decode_step(0, [1], q[:1], kv[:1], kv[:1], out[:1])
        at.decode_step(0, [2], q[:1], kv[:1], kv[:1], out[:1])
        at.decode(0, [2], q[:1], out[:1])
        with pytest.raises(A.AttnError) as e:
            at.decode(0, [3], q[:1], out[:1])
        assert e.value.code == A.OUT_OF_RANGE
        torch.cuda.synchronize()
