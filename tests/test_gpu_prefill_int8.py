"""GPU parity of prefill over an int8 cache on the matrix cores.

The cache holds int8 K / V with per-(head, channel) float32 scales (the reference's quantised KV cache:
runtime/executor/llm_litert_compiled_model_executor.cc builds it when the model's cache tensors are int8);
the expected values are the float64 oracle on the dequantised K / V. A prefill call turns the planes it reads
into half planes once (half(int8 value x scale)) and runs the kernels of a half cache on them; calls of a few
rows, and calls that find no room while a graph is recorded, take the row-wise path, which converts in
registers (K scales folded into the queries, V scales applied to the result). Both are held to the same
bound here, against the oracle and against each other.
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
from oracle import c_oracle  # noqa: E402

A = load_package().attn
DEV = "cuda:0"
TDT = {A.F32: torch.float32, A.F16: torch.float16, A.BF16: torch.bfloat16}
D = 256
TOL = 2e-3  # plain norm-wise error max|a - b| / max|ref|, float32 and half activations
# bfloat16 activations: the output format alone costs up to 2^-9 of an element, so those are compared with the
# float32-activation result of the same call rounded once (which must match bit for bit) instead of with the
# oracle directly


def say(*a):
    print(*a, flush=True)


def make(num_layers, hq, hkv, max_tokens, max_seqs, io, **kw):
    return A.Attn(num_layers, hq, hkv, D, max_tokens, max_seqs, A.I8, io,
                  stream=torch.cuda.current_stream().cuda_stream, **kw)


def gen(seed, *shape):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


def fill_int8(at, layer, seq, k, v):
    """Quantises fp32 rows as the oracle does, appends them, returns the dequantised fp32 values."""
    kq, ks = orc.quantize_kv_int8(k)
    vq, vs = orc.quantize_kv_int8(v)
    at.kv_append(layer, seq, 0, torch.from_numpy(kq).to(DEV), torch.from_numpy(vq).to(DEV))
    at.kv_set_scales(layer, seq, torch.from_numpy(ks).to(DEV), torch.from_numpy(vs).to(DEV))
    return orc.dequantize_kv_int8(kq, ks), orc.dequantize_kv_int8(vq, vs)


def queries(q, io):
    t = torch.from_numpy(np.ascontiguousarray(q)).to(DEV).to(TDT[io]).contiguous()
    return t, t.float().cpu().numpy()


def prefill(at, layer, seq, q_pos0, qd, rowwise=False, n_layers=1):
    out = torch.empty_like(qd)
    at.set_option("rowwise_prefill", int(rowwise))
    n = qd.shape[-3]
    at.prefill(layer, seq, q_pos0, n, qd, out, n_layers=n_layers)
    torch.cuda.synchronize()
    at.set_option("rowwise_prefill", 0)
    return out


def plain_err(got, ref):
    return float(np.abs(got - ref).max() / np.abs(ref).max())


@pytest.mark.parametrize("rows16", [1, 0], ids=["mfma16", "mfma32"])
def test_chunks_of_1024_rows_against_the_oracle_and_the_rowwise_path(rows16):
    # 8 query heads over 2 KV heads, two chunks of 1,024 rows of one sequence
    L, hq, hkv = 2048, 8, 2
    with make(1, hq, hkv, L, 1, A.F16) as at:
        at.set_option("prefill_rows16", rows16)
        kr, vr = fill_int8(at, 0, 0, gen(11, L, hkv, D), gen(12, L, hkv, D))
        for q_pos0 in (0, 1024):
            qd, qr = queries(gen(13 + q_pos0, 1024, hq, D), A.F16)
            out = prefill(at, 0, 0, q_pos0, qd).float().cpu().numpy()
            row = prefill(at, 0, 0, q_pos0, qd, rowwise=True).float().cpu().numpy()
            ref = c_oracle.sdpa_f64(qr, kr, vr, D ** -0.5, q_pos0=q_pos0, kv_len=q_pos0 + 1024)
            e, er, between = plain_err(out, ref), plain_err(row, ref), plain_err(out, row)
            say(f"int8 prefill q_pos0={q_pos0} rows16={rows16}: matrix cores {e:.3e}, row-wise {er:.3e}, "
                f"between them {between:.3e}")
            assert e < TOL and er < TOL and between < TOL


@pytest.mark.parametrize("io", [A.F32, A.F16, A.BF16], ids=["f32", "f16", "bf16"])
def test_activation_types_windows_layers_and_sequences(io):
    # three layers (global, window 100, window 33), three sequences in the cache, the call on sequence 2;
    # ragged row counts and starts
    windows = [0, 100, 33]
    L, hq, hkv = 600, 4, 2
    with make(3, hq, hkv, L, 3, io, layer_window=windows) as at, \
            make(3, hq, hkv, L, 3, A.F32, layer_window=windows) as at32:
        kv = []
        for layer in range(3):
            k, v = gen(20 + layer, L, hkv, D), gen(30 + layer, L, hkv, D)
            kv.append(fill_int8(at, layer, 2, k, v))
            fill_int8(at32, layer, 2, k, v)
            # another sequence of the same layer holds other values, which must not show up
            fill_int8(at, layer, 1, gen(40 + layer, L, hkv, D), gen(50 + layer, L, hkv, D))
        for q_pos0, n in ((0, 16), (0, 33), (0, 257), (70, 64), (129, 200), (341, 259)):
            q = gen(60 + n, 3, n, hq, D)
            qd, qr = queries(q, io)
            out = prefill(at, 0, 2, q_pos0, qd, n_layers=3)
            if io == A.BF16:
                # (the float32-activation call on the same rounded queries)
                q32 = torch.from_numpy(qr).to(DEV)
                out32 = prefill(at32, 0, 2, q_pos0, q32, n_layers=3)
                share, ulps = orc.bf16_output_match(out.float().cpu().numpy(), out32.cpu().numpy())
                assert share == 1.0, (q_pos0, n, share, ulps)
                got = out32.cpu().numpy()
            else:
                got = out.float().cpu().numpy()
            for layer in range(3):
                ref = c_oracle.sdpa_f64(qr[layer], kv[layer][0], kv[layer][1], D ** -0.5, q_pos0=q_pos0,
                                        window=windows[layer], kv_len=q_pos0 + n)
                e = plain_err(got[layer], ref)
                assert e < TOL, (io, layer, q_pos0, n, e)
        say(f"int8 prefill io={io}: layers, windows, sequences ok")


def test_passes_over_layers_when_the_staging_area_is_limited():
    # 1 MiB holds the half planes of one layer of this call (2 KV heads x 2 planes x 512 rows x 512 bytes): the call
    # over four layers runs in four passes. A pass of one layer is another launch shape than the call over four (its
    # tiles' keys may be split over work items and merged), so the two agree to rounding, not bit for bit; both
    # are held against the oracle, layer by layer.
    L, hq, hkv, n = 512, 8, 2, 512
    windows = [0, 64, 0, 200]
    with make(4, hq, hkv, L, 1, A.F16, layer_window=windows) as at:
        kv = [fill_int8(at, layer, 0, gen(70 + layer, L, hkv, D), gen(80 + layer, L, hkv, D)) for layer in range(4)]
        qd, qr = queries(gen(90, 4, n, hq, D), A.F16)
        at.set_option("prefill_i8_stage_mib", 1)
        one_by_one = prefill(at, 0, 0, 0, qd, n_layers=4).float().cpu().numpy()
        at.set_option("prefill_i8_stage_mib", 2048)
        at_once = prefill(at, 0, 0, 0, qd, n_layers=4).float().cpu().numpy()
        # a call over layers 1..2 only
        part = prefill(at, 1, 0, 0, qd[1:3].contiguous(), n_layers=2).float().cpu().numpy()
        for layer in range(4):
            ref = c_oracle.sdpa_f64(qr[layer], kv[layer][0], kv[layer][1], D ** -0.5, q_pos0=0, window=windows[layer],
                                    kv_len=n)
            e1, e4 = plain_err(one_by_one[layer], ref), plain_err(at_once[layer], ref)
            assert e1 < TOL and e4 < TOL, (layer, e1, e4)
            if layer in (1, 2):
                assert plain_err(part[layer - 1], ref) < TOL
        say(f"int8 prefill in passes: one layer at a time against all at once {plain_err(one_by_one, at_once):.3e}")


def test_few_rows_take_the_rowwise_path_and_the_rule_can_be_moved():
    L, hq, hkv = 300, 8, 2
    with make(1, hq, hkv, L, 1, A.F16) as at:
        kr, vr = fill_int8(at, 0, 0, gen(101, L, hkv, D), gen(102, L, hkv, D))
        qd, qr = queries(gen(103, 15, hq, D), A.F16)
        by_rule = prefill(at, 0, 0, 285, qd)
        rowwise = prefill(at, 0, 0, 285, qd, rowwise=True)
        assert torch.equal(by_rule, rowwise)  # 15 rows: under the rule's 16
        at.set_option("prefill_i8_min_rows", 1)
        mfma = prefill(at, 0, 0, 285, qd)
        ref = c_oracle.sdpa_f64(qr, kr, vr, D ** -0.5, q_pos0=285, kv_len=300)
        assert plain_err(mfma.float().cpu().numpy(), ref) < TOL
        assert plain_err(rowwise.float().cpu().numpy(), ref) < TOL
        assert not torch.equal(mfma, rowwise)  # (two different kernels did run)
        with pytest.raises(A.AttnError):
            at.set_option("prefill_i8_min_rows", 0)


def test_softcap_and_scale():
    L, hq, hkv = 384, 4, 1
    with make(1, hq, hkv, L, 1, A.F32, softcap=30.0, scale=0.11) as at:
        kr, vr = fill_int8(at, 0, 0, 3.0 * gen(111, L, hkv, D), gen(112, L, hkv, D))
        qd, qr = queries(2.0 * gen(113, L, hq, D), A.F32)
        out = prefill(at, 0, 0, 0, qd).cpu().numpy()
        ref = c_oracle.sdpa_f64(qr, kr, vr, 0.11, q_pos0=0, softcap=30.0, kv_len=L)
        e = plain_err(out, ref)
        say(f"int8 prefill softcap: {e:.3e}")
        assert e < TOL


def test_key_split_for_few_long_tiles():
    # one layer, one KV head, 64 rows deep into a long context: fewer work items than compute units, so the keys
    # of a tile are split over several items and merged
    L, hq, hkv = 8192, 4, 1
    with make(1, hq, hkv, L, 1, A.F16) as at:
        kr, vr = fill_int8(at, 0, 0, gen(121, L, hkv, D), gen(122, L, hkv, D))
        qd, qr = queries(gen(123, 64, hq, D), A.F16)
        ref = c_oracle.sdpa_f64(qr, kr, vr, D ** -0.5, q_pos0=L - 64, kv_len=L)
        for split in (-1, 0, 16):
            at.set_option("prefill_key_split", split)
            e = plain_err(prefill(at, 0, 0, L - 64, qd).float().cpu().numpy(), ref)
            say(f"int8 prefill key split {split}: {e:.3e}")
            assert e < TOL


def test_recorded_into_a_graph_without_room_it_takes_the_rowwise_path():
    L, hq, hkv, n = 256, 8, 2, 128
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with A.Attn(1, hq, hkv, D, L, 1, A.I8, A.F16, stream=side.cuda_stream) as at:
            kr, vr = fill_int8(at, 0, 0, gen(131, L, hkv, D), gen(132, L, hkv, D))
            qd, qr = queries(gen(133, n, hq, D), A.F16)
            out = torch.zeros_like(qd)
            side.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                at.prefill(0, 0, 0, n, qd, out)  # (no call before it: no staging area yet)
            ref = c_oracle.sdpa_f64(qr, kr, vr, D ** -0.5, q_pos0=0, kv_len=n)
            for _ in range(3):
                out.zero_()
                g.replay()
                side.synchronize()
                assert plain_err(out.float().cpu().numpy(), ref) < TOL
            eager = prefill(at, 0, 0, 0, qd, rowwise=True)
            assert torch.equal(out, eager)
            del g


def test_passes_with_different_windows_do_not_share_a_work_plan():
    # two passes of four layers each through the planned kernel: global layers first, then narrow windows. The
    # passes' launches have the same shape (layers counted from the staged planes' first), so the plan cache must
    # tell them apart by the handle's layer they start at.
    L, hq, hkv, n = 512, 8, 2, 512
    windows = [0, 0, 0, 0, 40, 40, 40, 40]
    with make(8, hq, hkv, L, 1, A.F16, layer_window=windows) as at:
        kv = [fill_int8(at, layer, 0, gen(140 + layer, L, hkv, D), gen(150 + layer, L, hkv, D)) for layer in range(8)]
        qd, qr = queries(gen(160, 8, n, hq, D), A.F16)
        at.set_option("prefill_rows16", 1)
        at.set_option("prefill_key_split", 4)  # (tiles of the global layers in up to four parts, the windowed ones whole)
        at.set_option("prefill_i8_stage_mib", 4)
        for _ in range(2):  # (the second call finds both plans cached)
            out = prefill(at, 0, 0, 0, qd, n_layers=8).float().cpu().numpy()
            for layer in range(8):
                ref = c_oracle.sdpa_f64(qr[layer], kv[layer][0], kv[layer][1], D ** -0.5, q_pos0=0,
                                        window=windows[layer], kv_len=n)
                assert plain_err(out[layer], ref) < TOL, layer


@pytest.mark.parametrize("io", [A.F32, A.BF16], ids=["f32", "bf16"])
def test_passes_with_staged_queries(io):
    # float32 / bfloat16 activations are staged as halves (with the K scales) pass by pass: the staging rows of a
    # pass start at its first layer's queries, wherever that layer sits in the call
    L, hq, hkv, n = 256, 4, 2, 256
    windows = [0, 50, 0, 0, 70]
    with make(5, hq, hkv, L, 1, io, layer_window=windows) as at, make(5, hq, hkv, L, 1, A.F32, layer_window=windows) as at32:
        kv = []
        for layer in range(5):
            k, v = gen(170 + layer, L, hkv, D), gen(180 + layer, L, hkv, D)
            kv.append(fill_int8(at, layer, 0, k, v))
            fill_int8(at32, layer, 0, k, v)
        qd, qr = queries(gen(190, 5, n, hq, D), io)
        at.set_option("prefill_i8_stage_mib", 1)   # one layer's planes are 0.5 MiB: two layers per pass, three passes
        out = prefill(at, 0, 0, 0, qd, n_layers=5)
        if io == A.BF16:
            out32 = prefill(at32, 0, 0, 0, torch.from_numpy(qr).to(DEV), n_layers=5)
            share, _ = orc.bf16_output_match(out.float().cpu().numpy(), out32.cpu().numpy())
            # (the float32 twin stages all five layers at once: other launch shapes, so rounding-level differences
            # may flip a last bit here and there)
            assert share > 0.99, share
            got = out32.cpu().numpy()
        else:
            got = out.cpu().numpy()
        for layer in range(5):
            ref = c_oracle.sdpa_f64(qr[layer], kv[layer][0], kv[layer][1], D ** -0.5, q_pos0=0, window=windows[layer],
                                    kv_len=n)
            assert plain_err(got[layer], ref) < TOL, (io, layer)


def test_host_pointers():
    L, hq, hkv, n = 192, 8, 2, 192
    with A.Attn(1, hq, hkv, D, L, 1, A.I8, A.F16, host_io=True) as at:
        k, v = gen(201, L, hkv, D), gen(202, L, hkv, D)
        kq, ks = orc.quantize_kv_int8(k)
        vq, vs = orc.quantize_kv_int8(v)
        at.kv_append(0, 0, 0, torch.from_numpy(kq), torch.from_numpy(vq))
        at.kv_set_scales(0, 0, torch.from_numpy(ks), torch.from_numpy(vs))
        q = torch.from_numpy(gen(203, n, hq, D)).half()
        out = torch.zeros_like(q)
        at.prefill(0, 0, 0, n, q, out)
        ref = c_oracle.sdpa_f64(q.float().numpy(), orc.dequantize_kv_int8(kq, ks), orc.dequantize_kv_int8(vq, vs),
                                D ** -0.5, q_pos0=0, kv_len=n)
        assert plain_err(out.float().numpy(), ref) < TOL
