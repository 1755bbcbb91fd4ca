"""What the library does when its stream is being captured into a HIP graph, and the no-alloc entry point
called from two streams: cases where the C ABI has to refuse, fall back or order work itself."""
import os
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from __graft_entry__ import load_package  # noqa: E402

A = load_package().attn
DEV = "cuda:0"
D = 256


def say(*a):
    print(*a, flush=True)


def rnd(seed, *shape, dtype=torch.float16):
    g = torch.Generator(device=DEV).manual_seed(seed)
    return torch.randn(shape, generator=g, device=DEV).to(dtype)


def test_prefill_shapes_first_seen_under_capture_and_more_captured_shapes_than_plan_slots():
    """The planned prefill kernel keeps its work plans in four slots, and a slot whose launch a graph holds is
    never reused. A shape met for the first time while the stream is being captured, and any shape once all
    slots belong to graphs, run on the kernel that needs no plan: every capture succeeds, every replay gives
    the eager result (to the tolerance where the kernels differ), and eager calls of new shapes keep working."""
    layers, hq, hkv, n = 12, 4, 1, 512
    windows = [0 if (l + 1) % 6 == 0 else 128 for l in range(layers)]
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with A.Attn(layers, hq, hkv, D, 1024, 1, A.F16, A.F16, layer_window=windows, stream=side.cuda_stream) as at:
            for layer in range(layers):
                at.kv_append(layer, 0, 0, rnd(10 + layer, 1024, hkv, D), rnd(40 + layer, 1024, hkv, D))
            q = rnd(5, layers, n, hq, D)
            graphs = []
            # six chunk positions = six launch shapes: the first is new under capture, the others are run eagerly
            # first (their plans get slots, captured launches pin them: after four, no slot is left)
            for i, pos0 in enumerate((0, 64, 128, 192, 256, 320)):
                eager = torch.full_like(q, float("nan"))
                if i > 0:
                    at.prefill(0, 0, pos0, n, q, eager, n_layers=layers)
                side.synchronize()
                out = torch.full_like(q, float("nan"))
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=side):
                    at.prefill(0, 0, pos0, n, q, out, n_layers=layers)
                if i == 0:
                    at.prefill(0, 0, pos0, n, q, eager, n_layers=layers)  # (eager after the capture: a plan now)
                    side.synchronize()
                graphs.append((g, out, eager.clone(), pos0))
            for rep in range(2):
                for g, out, eager, pos0 in graphs:
                    out.fill_(float("nan"))
                    g.replay()
                    side.synchronize()
                    assert torch.isfinite(out.float()).all(), pos0
                    err = float((out.float() - eager.float()).abs().max() / eager.float().abs().max())
                    assert err < 2e-3, (pos0, rep, err)
            # a new shape, eagerly, with every slot held by a graph
            eager = torch.full_like(q, float("nan"))
            at.prefill(0, 0, 448, n, q, eager, n_layers=layers)
            side.synchronize()
            assert torch.isfinite(eager.float()).all()
            del graphs


def test_decode_of_more_than_64_sequences_is_refused_under_capture():
    B, hq, hkv = 70, 4, 1
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with A.Attn(1, hq, hkv, D, 64, B, A.F16, A.F16, stream=side.cuda_stream) as at:
            kv = rnd(1, 64, hkv, D)
            for b in range(B):
                at.kv_append(0, b, 0, kv, kv)
            q = rnd(2, B, hq, D)
            out = torch.zeros_like(q)
            at.decode(0, [64] * B, q, out, num_splits=2)  # eager: fine (and the split workspace exists now)
            side.synchronize()
            want = out.clone()
            g = torch.cuda.CUDAGraph()
            codes = []
            with torch.cuda.graph(g, stream=side):
                for call in (lambda: at.decode(0, [64] * B, q, out, num_splits=2),
                             lambda: at.decode_noalloc(0, [64] * B, q, out, num_splits=2)):
                    try:
                        call()
                        codes.append(0)
                    except A.AttnError as e:
                        codes.append(e.code)
                at.decode(0, [64] * 64, q[:64], out[:64], num_splits=2)  # 64 sequences: captured
            assert codes == [A.FAILED_PRECONDITION, A.FAILED_PRECONDITION]
            out.zero_()
            g.replay()
            side.synchronize()
            assert torch.equal(out[:64], want[:64]) and not out[64:].any()
            del g


def test_noalloc_calls_on_two_streams_are_ordered_by_the_library():
    """Two handles on two streams share the GPU's fixed workspace; the library makes each call wait for the
    previous one's event, so alternating calls without any synchronisation by the caller give what
    mi355_attn_decode gives."""
    hq, hkv, ctx, B = 8, 2, 1024, 8
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    at1 = A.Attn(1, hq, hkv, D, ctx, B, A.F16, A.F16, stream=s1.cuda_stream)
    at2 = A.Attn(1, hq, hkv, D, ctx, B, A.F16, A.F16, stream=s2.cuda_stream)
    try:
        qs, wants, gots = {}, {}, {}
        for i, (at, s) in enumerate(((at1, s1), (at2, s2))):
            with torch.cuda.stream(s):
                for b in range(B):
                    at.kv_append(0, b, 0, rnd(100 * i + b, ctx, hkv, D), rnd(100 * i + 50 + b, ctx, hkv, D))
                qs[i] = rnd(7 + i, B, hq, D)
                wants[i] = torch.empty_like(qs[i])
                at.decode(0, [ctx] * B, qs[i], wants[i], num_splits=16)
                gots[i] = [torch.full_like(qs[i], float("nan")) for _ in range(20)]
        torch.cuda.synchronize()
        for rep in range(20):  # alternating, back to back, no synchronisation in between
            for i, (at, s) in enumerate(((at1, s1), (at2, s2))):
                with torch.cuda.stream(s):
                    at.decode_noalloc(0, [ctx] * B, qs[i], gots[i][rep], num_splits=16)
        torch.cuda.synchronize()
        for i in (0, 1):
            for rep in range(20):
                assert torch.equal(gots[i][rep], wants[i]), (i, rep)
    finally:
        at1.close()
        at2.close()


def test_stream_probe_reads_without_touching_the_cache_and_checks_its_range():
    with A.Attn(2, 4, 1, D, 1024, 2, A.F16, A.F16, stream=torch.cuda.current_stream().cuda_stream) as at:
        k, v = rnd(3, 1024, 1, D), rnd(4, 1024, 1, D)
        at.kv_append(1, 1, 0, k, v)
        total = at.cache_bytes  # 2 layers x 2 sequences x 2 planes x 512 KiB = 4 MiB
        assert total == 2 * 2 * 2 * 1024 * D * 2
        at.set_timing(True)
        at.stream_probe(0, total, 32, 1)
        ms = at.last_kernel_ms()
        at.stream_probe(32768, total // 2, 8, 4)
        at.set_timing(False)
        assert ms > 0
        for off, nbytes, wgs, waves, code in ((0, total + 32 * 32768, 32, 1, A.OUT_OF_RANGE), (8, 1024, 1, 1, A.OUT_OF_RANGE),
                                              (total - 1024, 32768, 1, 1, A.OUT_OF_RANGE), (0, 1024, 0, 1, A.INVALID_ARGUMENT),
                                              (0, 1024, 1, 17, A.INVALID_ARGUMENT)):
            with pytest.raises(A.AttnError) as e:
                at.stream_probe(off, nbytes, wgs, waves)
            assert e.value.code == code, (off, nbytes, wgs, waves)
        ko, vo = torch.zeros_like(k), torch.zeros_like(v)
        at.kv_read(1, 1, 0, 1024, ko, vo)
        torch.cuda.synchronize()
        assert torch.equal(ko, k) and torch.equal(vo, v)
