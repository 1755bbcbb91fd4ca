"""Host logic of the C++ HipLlmExecutor, no GPU: the executor runs over a
recording attention backend and its forward-pass trace, step counter, chunk
plan and status codes are compared with the oracle's restatement of the
reference executor (oracle.attn_oracle.OracleExecutor / prefill_work_groups)."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from __graft_entry__ import load_package  # noqa: E402
from oracle import attn_oracle as orc  # noqa: E402

X = load_package().executor
INVALID_ARGUMENT, OUT_OF_RANGE, INTERNAL = 3, 11, 13


def make(runners=(1024,), max_tokens=4096, fix=False, **kw):
    return X.HipLlmExecutor(2, 4, 1, 16, max_tokens, runner_lengths=runners, recording_backend=True,
                            execute_pending_on_single_id_chunk=fix, **kw)


def test_plan_matches_reference_strategy():
    runners = [32, 1024, 256]
    for n in (1, 26, 32, 33, 255, 256, 257, 1023, 1024, 1025, 1050, 1100, 1300, 2048, 5000):
        assert X.plan(runners, n) == orc.prefill_work_groups(runners, n), n
    assert X.plan(runners, 1300) == [(1024, 1024), (1024, 276)]
    assert X.plan(runners, 1100) == [(1024, 1024), (256, 76)]
    assert X.plan(runners, 1050) == [(1024, 1024), (32, 26)]
    assert X.plan([128], 300) == [(128, 128), (128, 128), (128, 44)]


def test_backend_selector():
    assert X.backend_from_string("hip") == 6  # Backend::GPU_HIP, the new enumerator
    assert X.backend_from_string("cpu") == 2 and X.backend_from_string("gpu") == 3
    assert X.backend_from_string("tpu") == -INVALID_ARGUMENT


def test_deferred_last_token_and_steps():
    with make(runners=(4,)) as ex:
        assert ex.backend_name() == "MI355X HIP attention"
        assert ex.vocab_size() == 16 and ex.max_num_tokens() == 4096 and ex.current_step() == 0
        ex.prefill([10, 11, 12])
        assert ex.runs() == [("prefill", [10, 11], [0, 1])]
        assert ex.current_step() == 3  # user-visible step counts the deferred token
        ex.prefill([13, 14, 15, 16, 17, 18])
        assert ex.runs()[1:] == [("prefill", [12, 13, 14, 15], [2, 3, 4, 5]), ("prefill", [16, 17], [6, 7])]
        tok = ex.decode()
        assert ex.runs()[-1] == ("decode", [18], [8]) and ex.current_step() == 10  # sampled token is pending again
        ex.decode_logits()
        assert ex.runs()[-1] == ("decode", [tok], [9]) and ex.current_step() == 10
        with pytest.raises(X.ExecutorError) as e:
            ex.decode_logits()
        assert e.value.code == INVALID_ARGUMENT and "No id available to be decoded" in e.value.message
        ex.decode_logits(explicit_id=7)
        assert ex.runs()[-1] == ("decode", [7], [10])
        ex.reset()
        assert ex.current_step() == 0 and ex.runs() == []


def test_benchmark_shape_1024_ids():
    # README protocol: 1024 ids -> 1023 executed by prefill, the last by the first decode step
    with make(runners=(1024,)) as ex:
        ex.prefill(list(range(1024)))
        (kind, toks, pos), = ex.runs()
        assert kind == "prefill" and len(toks) == 1023 and pos == list(range(1023)) and ex.current_step() == 1024
        ex.decode()
        assert ex.runs()[-1] == ("decode", [1023], [1023])


def test_single_id_chunk_quirk_and_fix():
    with X.HipLlmExecutor(2, 4, 1, 16, 64, runner_lengths=(4,), recording_backend=True) as dflt:
        dflt.prefill([1, 2]); dflt.prefill([3])  # the default is the reference's behaviour
        assert dflt.runs() == [("prefill", [1], [0]), ("prefill", [], [])] and dflt.current_step() == 2
    with make(runners=(4,), fix=False) as ref:  # reference behaviour: the pending token is dropped
        ref.prefill([1, 2]); ref.prefill([3])
        assert ref.runs() == [("prefill", [1], [0]), ("prefill", [], [])] and ref.current_step() == 2
    with make(runners=(4,), fix=True) as fix:
        fix.prefill([1, 2]); fix.prefill([3])
        assert fix.runs() == [("prefill", [1], [0]), ("prefill", [2], [1])] and fix.current_step() == 3


@pytest.mark.parametrize("seed", range(8))
def test_random_call_sequences_match_oracle_state_machine(seed):
    rng = np.random.default_rng(seed)
    runners = tuple(int(x) for x in rng.choice([1, 2, 3, 5, 8, 13, 32], size=int(rng.integers(1, 4)), replace=False))
    fix = bool(seed % 2)
    oracle = orc.OracleExecutor(runner_lengths=runners, execute_single_pending=fix)
    with make(runners=runners, fix=fix, max_tokens=100000) as ex:
        for _ in range(40):
            op = rng.integers(0, 10)
            if op < 5:
                ids = [int(x) for x in rng.integers(0, 16, size=int(rng.integers(1, 70)))]
                ex.prefill(ids)
                oracle.prefill(ids)
            elif op < 8:
                if oracle.next_input_token_id == -1:
                    with pytest.raises(X.ExecutorError):
                        ex.decode()
                    continue
                tok = ex.decode()
                oracle.decode()
                oracle.next_input_token_id = tok  # Decode(tokens) parks the sampled id
            elif op < 9:
                ex.decode_logits(explicit_id=3)
                oracle.decode(explicit_id=3)
            else:
                ex.reset()
                oracle.reset()
                oracle.calls.clear()
            assert ex.current_step() == oracle.get_current_step()
        assert ex.runs() == [(k, t, p) for k, t, p in oracle.calls]


def test_error_paths():
    with make(runners=(8,), max_tokens=10) as ex:
        with pytest.raises(X.ExecutorError) as e:
            ex.prefill([1, 2, 3, 4], batch=2)  # batch must be 1: RET_CHECK -> kInternal
        assert e.value.code == INTERNAL
        with pytest.raises(X.ExecutorError) as e:
            ex.prefill([], batch=1)
        assert e.value.code == INTERNAL and "non-empty" in e.value.message
        with pytest.raises(X.ExecutorError) as e:
            ex.decode()
        assert e.value.code == INVALID_ARGUMENT
        ex.prefill(list(range(8)))  # 7 executed + 1 pending
        ex.decode(); ex.decode(); ex.decode()  # positions 7, 8, 9
        with pytest.raises(X.ExecutorError) as e:
            ex.decode()             # position 10 does not exist
        assert e.value.code == OUT_OF_RANGE
    with pytest.raises(X.ExecutorError) as e:
        X.HipLlmExecutor(2, 4, 1, 16, 0, recording_backend=True)
    assert e.value.code == INVALID_ARGUMENT


def test_fused_step_before_attention_keeps_the_step_logic():
    # raw projections + norm / rotary constants per layer: same chunks, positions and steps
    with make(runners=(4,), pre_attention=True) as ex, make(runners=(4,)) as plain:
        for e in (ex, plain):
            e.prefill([10, 11, 12, 13, 14, 15, 16])
            e.decode()
        assert ex.runs() == plain.runs() and ex.current_step() == plain.current_step() == 8


def test_interface_matches_the_reference_header_method_for_method():
    # names, return types, parameter types, constness and purity of every virtual method, in declaration order
    import json
    from cpp_interface import virtual_methods
    with open(os.path.join(ROOT, "tests", "golden", "llm_executor_base_methods.json")) as f:
        want = json.load(f)["methods"]
    with open(os.path.join(ROOT, "litert-lm_amd", "executor", "llm_executor_base.h")) as f:
        got = virtual_methods(f.read(), "LlmExecutorBase")
    assert [m["name"] for m in want] == ["Prefill", "Prefill", "Decode", "Decode", "DecodeLogits", "ExecutorBackendName",
                                         "GetVocabSize", "GetCurrentStep", "GetExecutorSettings", "FillVisionEmbeddings",
                                         "Reset"]
    assert got == want


def test_vision_entry_point_keeps_the_base_class_default():
    with make(runners=(4,)) as ex:
        with pytest.raises(X.ExecutorError) as e:
            ex.fill_vision_embeddings(0)
        assert e.value.code == 12  # kUnimplemented
        assert e.value.message == "FillVisionEmbeddings not implemented for backend: MI355X HIP attention"


def test_prefill_params_cancel_and_wait():
    with make(runners=(4,)) as ex:
        assert not ex.is_device_resident()          # the recording backend is host-staged
        with pytest.raises(X.ExecutorError) as e:
            ex.prefill([1, 2, 3, 4, 5, 6], cancel=True)
        assert e.value.code == 1 and "cancelled" in e.value.message   # kCancelled before the first chunk
        assert ex.runs() == [] and ex.current_step() == 0
        ex.prefill([1, 2, 3, 4, 5, 6], wait_for_completion=True, cancel=False)
        assert ex.current_step() == 6 and len(ex.runs()) == 2
        ex.wait_for_completion()                    # nothing is ever pending on a host-staged executor


def test_device_resident_needs_a_device_resident_backend():
    with pytest.raises(X.ExecutorError) as e:
        make(device_resident=True)
    assert e.value.code == INVALID_ARGUMENT and "device-resident" in e.value.message
