"""mi355_attn_decode_noalloc (the entry point for callers that cannot allocate) against
mi355_attn_decode, through the C ABI: same kernels, so the outputs must be bit-identical."""
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
D = 256


def say(*a):
    print(*a, flush=True)


def test_decode_noalloc_matches_decode_two_calls_second_smaller():
    hq, hkv, ctx, B = 8, 2, 2048, 6
    rng = np.random.default_rng(77)
    stream = torch.cuda.current_stream().cuda_stream
    with A.Attn(2, hq, hkv, D, ctx, B, A.F16, A.F16, layer_window=[0, 300], stream=stream) as at:
        lens_big = [2048, 1500, 1999, 777, 2048, 64]
        kvs = []
        for layer in range(2):
            for b in range(B):
                k = torch.from_numpy(rng.standard_normal((ctx, hkv, D)).astype(np.float32)).to(DEV).half()
                v = torch.from_numpy(rng.standard_normal((ctx, hkv, D)).astype(np.float32)).to(DEV).half()
                at.kv_append(layer, b, 0, k, v)
                if layer == 0:
                    kvs.append((k.float().cpu().numpy(), v.float().cpu().numpy()))
        q = torch.from_numpy(rng.standard_normal((B, hq, D)).astype(np.float32)).to(DEV).half()
        qr = q.float().cpu().numpy()
        # first call: the whole batch, 16 partitions; second call: fewer and shorter sequences, another split count;
        # then a windowed layer and the library's own choice of partitions
        for layer, lens, seq_ids, splits in ((0, lens_big, None, 16), (0, [300, 65, 1], [3, 0, 5], 4),
                                            (1, lens_big, None, 0), (1, [2048], [4], 1)):
            n = len(lens)
            say(f"decode_noalloc layer={layer} lens={lens} seq_ids={seq_ids} splits={splits}")
            want = torch.full((n, hq, D), 7.0, dtype=torch.float16, device=DEV)
            got = torch.full((n, hq, D), 9.0, dtype=torch.float16, device=DEV)
            at.decode(layer, lens, q[:n].contiguous(), want, seq_ids=seq_ids, num_splits=splits)
            at.decode_noalloc(layer, lens, q[:n].contiguous(), got, seq_ids=seq_ids, num_splits=splits)
            torch.cuda.synchronize()
            assert torch.equal(got, want)
            if layer == 0:  # and both are right
                for j, L in enumerate(lens):
                    b = j if seq_ids is None else seq_ids[j]
                    ref = c_oracle.sdpa_f64(qr[j:j + 1], kvs[b][0], kvs[b][1], D ** -0.5, q_pos0=L - 1, kv_len=L)[0]
                    assert orc.rel_err(got[j].float().cpu().numpy(), ref) < 2e-3


def test_decode_noalloc_limits():
    stream = torch.cuda.current_stream().cuda_stream
    with A.Attn(1, 8, 2, D, 4096, 64, A.F16, A.F16, stream=stream) as at:
        k = torch.zeros((4096, 2, D), dtype=torch.float16, device=DEV)
        for b in range(64):
            at.kv_append(0, b, 0, k, k)
        q = torch.zeros((64, 8, D), dtype=torch.float16, device=DEV)
        out = torch.empty_like(q)
        with pytest.raises(A.AttnError) as e:
            at.decode_noalloc(0, [4096] * 64, q, out, num_splits=32)  # 64 x 8 x 32 = 16384 partial results > 8192
        assert e.value.code == A.RESOURCE_EXHAUSTED and "8192" in e.value.message
        at.decode_noalloc(0, [4096] * 64, q, out, num_splits=16)       # exactly the limit
        at.decode_noalloc(0, [4096] * 64, q, out, num_splits=0)        # the library's choice stays inside it
        torch.cuda.synchronize()
        assert not out.float().abs().max().item() > 0  # zero values in, zero out (and finite)
    with A.Attn(1, 4, 1, D, 64, 1, A.F32, A.F32, host_io=True) as at:
        x = np.zeros((1, 4, D), np.float32)
        with pytest.raises(A.AttnError) as e:
            at.decode_noalloc(0, [1], x, x)
        assert e.value.code == A.FAILED_PRECONDITION
