"""End to end through the C++ HipLlmExecutor on the GPU: chunked prefill and
greedy decode over the synthetic decoder layers must reproduce, step by step,
the logits of a whole-sequence numpy forward pass that uses the CPU oracle for
attention. This exercises what the attention-level tests cannot: KV rows
landing at the right cache positions across chunks and steps, the deferred
last token, local and global layers inside one stack."""
import os
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from __graft_entry__ import load_package  # noqa: E402
from synthetic_twin import Twin  # noqa: E402

X = load_package().executor


def rel(a, b):
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


@pytest.mark.parametrize("device_resident", [False, True])
@pytest.mark.parametrize("pre_attention", [False, True])
@pytest.mark.parametrize("fp16", [False, True])
def test_prefill_chunks_then_greedy_decode_match_whole_sequence_reference(fp16, pre_attention, device_resident):
    # device_resident: activations, logits and the sampled id stay in device memory, the layers run as kernels and
    # nothing waits between layers; else float32 host rows are staged through the boundary per call
    # pre_attention: the layers hand over raw projections and the fused device step
    # (RMS norm + rotary embedding + cache write) runs before every attention call
    layers, hq, hkv, vocab = 3, 4, 1, 48
    windows = [0, 24, 0]
    rng = np.random.default_rng(11)
    prompt = [int(x) for x in rng.integers(0, vocab, size=71)]
    tol = 2e-3 if fp16 else 2e-5
    twin = Twin(layers, hq, hkv, vocab, windows, pre_attention=pre_attention)
    with X.HipLlmExecutor(layers, hq, hkv, vocab, 256, runner_lengths=(32, 8), layer_window=windows, fp16=fp16,
                          pre_attention=pre_attention, device_resident=device_resident) as ex:
        assert "MI355X" in ex.backend_name() and ex.is_device_resident() == device_resident
        ex.prefill(prompt[:40])   # chunks of 32 and 8, last id deferred
        ex.prefill(prompt[40:])   # pending id goes first
        assert ex.current_step() == len(prompt)
        seq = list(prompt)
        for step in range(6):
            logits = ex.decode_logits()  # executes the pending token at position len(seq)-1
            ref = twin.forward_all(seq, round_io=np.float16 if fp16 else None)[-1]
            err = rel(logits, ref)
            print(f"fp16={fp16} pre_attention={pre_attention} device_resident={device_resident} step {step}: logits rel_err {err:.2e}", flush=True)
            assert err < tol
            assert int(np.argmax(logits)) == int(np.argmax(ref))
            nxt = int(np.argmax(logits))
            seq.append(nxt)
            # feed the greedy token explicitly for the next step
            if step < 5:
                logits2 = ex.decode_logits(explicit_id=nxt)
                ref2 = twin.forward_all(seq, round_io=np.float16 if fp16 else None)[-1]
                assert rel(logits2, ref2) < tol
                seq.append(int(np.argmax(logits2)))
                ex.prefill([seq[-1]])  # a one-id prefill just parks the id
        # Decode(tokens) samples greedily and parks the id itself
        ex.reset()
        ex.prefill(prompt[:10])
        t1 = ex.decode()
        ref = twin.forward_all(prompt[:10], round_io=np.float16 if fp16 else None)[-1]
        assert t1 == int(np.argmax(ref))
        t2 = ex.decode()
        ref = twin.forward_all(prompt[:10] + [t1], round_io=np.float16 if fp16 else None)[-1]
        assert t2 == int(np.argmax(ref))


@pytest.mark.parametrize("fp16", [False, True])
def test_device_resident_executor_follows_the_host_staged_one_step_by_step(fp16):
    """The same calls on a device-resident and on a host-staged executor: logits of every step agree to rounding
    (the layers' sums of squares and logits are reduced by a tree on the device, in sequence on the host), the
    sampled ids and the step counters agree exactly. Prefill is queued without waiting (wait_for_completion
    false, the default of the parameters) on the device-resident one."""
    layers, hq, hkv, vocab = 6, 8, 2, 96
    windows = [0 if (l + 1) % 3 == 0 else 48 for l in range(layers)]
    rng = np.random.default_rng(5)
    prompt = [int(x) for x in rng.integers(0, vocab, size=150)]
    tol = 1e-3 if fp16 else 1e-5
    kw = dict(runner_lengths=(64, 16), layer_window=windows, fp16=fp16, pre_attention=True)
    with X.HipLlmExecutor(layers, hq, hkv, vocab, 512, device_resident=True, **kw) as dev, \
            X.HipLlmExecutor(layers, hq, hkv, vocab, 512, device_resident=False, **kw) as host:
        assert dev.is_device_resident() and not host.is_device_resident()
        dev.prefill(prompt[:100], wait_for_completion=False)
        dev.prefill(prompt[100:], wait_for_completion=False)   # queued behind the first, no wait in between
        host.prefill(prompt[:100])
        host.prefill(prompt[100:], wait_for_completion=True)
        assert dev.current_step() == host.current_step() == len(prompt)
        assert dev.runs() == host.runs()
        for step in range(12):
            if step % 3 == 2:   # the logits route
                a, b = dev.decode_logits(), host.decode_logits()
                err = rel(a, b)
                print(f"fp16={fp16} step {step}: device-resident vs host-staged logits rel_err {err:.2e}", flush=True)
                assert err < tol
                nxt = int(np.argmax(b))
                assert int(np.argmax(a)) == nxt
                dev.prefill([nxt]); host.prefill([nxt])   # park the id
            else:               # the sampled route: only the id returns from the device
                ta, tb = dev.decode(), host.decode()
                print(f"fp16={fp16} step {step}: sampled {ta} / {tb}", flush=True)
                assert ta == tb
            assert dev.current_step() == host.current_step()
        # a cancelled prefill executes nothing; the next one runs as usual
        with pytest.raises(X.ExecutorError) as e:
            dev.prefill([1, 2, 3], cancel=True)
        assert e.value.code == 1
        dev.reset(); host.reset()
        dev.prefill(prompt[:33], wait_for_completion=True); host.prefill(prompt[:33])
        assert dev.decode() == host.decode()


def test_readme_benchmark_protocol_in_the_reference_report_format():
    """`litert_lm_main --benchmark --benchmark_prefill_tokens=1024 --benchmark_decode_tokens=256`
    (README.md:390-400 of the reference) on the HIP executor: Gemma-3-like attention stack
    (26 layers, 5 local : 1 global, window 512, Hq4 / Hkv1, fp16), synthetic layers around it."""
    import re
    layers, hq, hkv, vocab = 26, 4, 1, 64
    windows = [0 if (l + 1) % 6 == 0 else 512 for l in range(layers)]
    with X.HipLlmExecutor(layers, hq, hkv, vocab, 2048, runner_lengths=(1024,), layer_window=windows, fp16=True,
                          pre_attention=True) as ex:
        r = X.run_benchmark(ex, [3, 1, 4, 1, 5, 9, 2, 6], 1024, 256)
        print(r["report"], flush=True)
        assert len(r["tokens"]) == 256 and r["current_step"] == 1024 + 256
        assert all(0 <= t < vocab for t in r["tokens"])
        runs = ex.runs()
        assert [len(t) for k, t, _ in runs if k == "prefill"] == [1023]   # the 1024th id is the first decode step
        assert sum(1 for k, _, _ in runs if k == "decode") == 256
        assert re.search(r"Prefill Turn 1: Processed 1024 tokens in \S+ duration\.\n      Prefill Speed: \d+\.\d\d tokens/sec\.",
                         r["report"])
        assert re.search(r"Decode Turn 1: Processed 256 tokens in \S+ duration\.\n      Decode Speed: \d+\.\d\d tokens/sec\.",
                         r["report"])
