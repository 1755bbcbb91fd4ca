"""The reference's benchmark report, stop-token detection and prefill / decode loop
(executor/benchmark_info.h, stop_token_detector.h, pipeline.h) held to what the
reference's own tests hold: runtime/engine/io_types_test.cc:120-275,
runtime/components/stop_token_detector_test.cc:15-118, runtime/core/pipeline_test.cc:47-141
(token ids instead of text: tokenisation is not part of this build). CPU only."""
import os
import re
import sys
import time

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from __graft_entry__ import load_package  # noqa: E402

X = load_package().executor
INVALID_ARGUMENT, ALREADY_EXISTS, INTERNAL = 3, 6, 13


# ------------------------------------------------------------------ BenchmarkInfo (io_types_test.cc)
def test_init_phases():
    b = X.BenchmarkInfo(100, 100)
    b.time_init_phase_start("Model Load")
    b.time_init_phase_start("Tokenizer Load")
    time.sleep(0.05)
    b.time_init_phase_end("Tokenizer Load")
    time.sleep(0.05)
    b.time_init_phase_end("Model Load")
    assert b.num_init_phases() == 2
    assert b.init_phase_seconds("Tokenizer Load") > 0.05
    assert b.init_phase_seconds("Model Load") > 0.10


def test_init_phase_twice_or_unstarted_is_internal():
    b = X.BenchmarkInfo(100, 100)
    b.time_init_phase_start("Model Load")
    with pytest.raises(X.ExecutorError) as e:
        b.time_init_phase_start("Model Load")
    assert e.value.code == INTERNAL
    with pytest.raises(X.ExecutorError) as e:
        b.time_init_phase_end("Tokenizer Load")
    assert e.value.code == INTERNAL


@pytest.mark.parametrize("kind", ["prefill", "decode"])
def test_turns(kind):
    b = X.BenchmarkInfo(100, 100)
    start = getattr(b, f"time_{kind}_turn_start")
    end = getattr(b, f"time_{kind}_turn_end")
    total = getattr(b, f"total_{kind}_turns")
    start(); end(100); start(); end(200)
    assert total() == 2
    b = X.BenchmarkInfo(100, 100)
    start = getattr(b, f"time_{kind}_turn_start")
    end = getattr(b, f"time_{kind}_turn_end")
    start()
    with pytest.raises(X.ExecutorError) as e:   # started twice
        start()
    assert e.value.code == INTERNAL
    end(100)
    with pytest.raises(X.ExecutorError) as e:   # ended without a start
        end(200)
    assert e.value.code == INTERNAL


def test_marks():
    b = X.BenchmarkInfo(100, 100)
    b.time_mark_delta("sampling")
    time.sleep(0.2)
    b.time_mark_delta("sampling")
    time.sleep(0.2)
    b.time_mark_delta("sampling")
    assert b.num_marks() == 1
    assert 0.2 < b.mark_seconds("sampling") < 0.4   # between the 2nd and 3rd call, not the 1st and 3rd
    b = X.BenchmarkInfo(100, 100)
    b.time_mark_delta("tokenize")
    b.time_mark_delta("sampling")
    time.sleep(0.05)
    b.time_mark_delta("sampling")
    time.sleep(0.05)
    b.time_mark_delta("tokenize")
    assert b.num_marks() == 2
    assert b.mark_seconds("sampling") > 0.05 and b.mark_seconds("tokenize") > 0.10


def test_report_matches_the_reference_tests_pattern():
    b = X.BenchmarkInfo(100, 100)
    b.time_init_phase_start("Load Model")
    b.time_init_phase_start("Load Tokenizer")
    b.time_init_phase_end("Load Model")
    b.time_init_phase_end("Load Tokenizer")
    b.time_prefill_turn_start(); b.time_prefill_turn_end(100)
    b.time_prefill_turn_start(); b.time_prefill_turn_end(200)
    b.time_decode_turn_start(); b.time_decode_turn_end(100)
    expected = r"""BenchmarkInfo:
  Init Phases \(2\):
    - Load Model: .* ms
    - Load Tokenizer: .* ms
    Total init time: .* ms
--------------------------------------------------
  Prefill Turns \(Total: 2\):
    Prefill Turn 1: Processed 100 tokens in .* duration.
      Prefill Speed: .* tokens/sec.
    Prefill Turn 2: Processed 200 tokens in .* duration.
      Prefill Speed: .* tokens/sec.
--------------------------------------------------
  Decode Turns \(Total: 1\):
    Decode Turn 1: Processed 100 tokens in .* duration.
      Decode Speed: .* tokens/sec.
--------------------------------------------------
"""  # the pattern of io_types_test.cc:255-272
    text = b.report()
    assert re.search(expected, text), text
    assert text.endswith("-" * 50 + "\n" + "-" * 50 + "\n")  # no marks: the two closing rules follow each other
    assert re.search(r"Prefill Speed: \d+\.\d\d tokens/sec\.", text)  # fixed, two decimals
    empty = X.BenchmarkInfo().report()
    assert "    No init phases recorded.\n" in empty and "    No prefill turns recorded.\n" in empty
    assert "    No decode turns recorded.\n" in empty


def test_duration_text():
    # absl::FormatDuration's documented examples and unit rules
    assert X.format_duration(0) == "0"
    assert X.format_duration(1) == "1ns"
    assert X.format_duration(1500) == "1.5us"
    assert X.format_duration(1_500_000) == "1.5ms"
    assert X.format_duration(72_345_678) == "72.345678ms"
    assert X.format_duration(999_999_999) == "999.999999ms"
    assert X.format_duration(1_000_000_000) == "1s"
    assert X.format_duration(3_500_000_000) == "3.5s"
    assert X.format_duration(60_000_000_000) == "1m"
    assert X.format_duration(72 * 60_000_000_000 + 3_500_000_000) == "1h12m3.5s"
    assert X.format_duration(3_600_000_000_000 + 250_000_000) == "1h0.25s"
    assert X.format_duration(-1_500_000) == "-1.5ms"


# ------------------------------------------------------------------ StopTokenDetector (stop_token_detector_test.cc)
def test_stop_sequences_added():
    _, codes, _, _ = X.stop_detector_run(1, [[1, 2, 3], [1, 2, 3], [9]], [])
    assert codes == [0, ALREADY_EXISTS, 0]


def test_single_stop_token_two_items():
    toks = list(zip([3, 4, 5, 6, 7], [1, 0, 6, 5, 99]))
    step, _, before, _ = X.stop_detector_run(2, [[5]], toks)
    assert step == 3 and before == [2, 1]


def test_multi_token_stop_sequence():
    toks = list(zip([3, 6, 7, 8, 9, 10, 11, 12], [1, 0, 0, 0, 0, 6, 5, 99]))
    step, _, before, _ = X.stop_detector_run(2, [[5], [7, 8, 9]], toks)
    assert step == 6 and before == [5, 1]


def test_reset_batch():
    step, _, before, done = X.stop_detector_run(1, [[1]], [[0], [2], [3], [1], [5]], reset=True)
    assert step == 3 and done is False and before == [0]


def test_partial_match_restarts_on_the_same_token():
    # 7 7 8 9: the second 7 must start the sequence anew
    step, _, before, _ = X.stop_detector_run(1, [[7, 8, 9]], [[7], [7], [8], [9], [1]])
    assert step == 3 and before == [3]


# ------------------------------------------------------------------ prefill / decode loop (pipeline_test.cc)
PROMPT = [90, 547, 58, 735, 210, 466, 2294]          # "Hello World!" in the reference's test vocabulary
PREFILL = [2] + PROMPT                                # with the bos id in front
DECODE = [224, 24, 8, 66, 246, 18, 2295, 2294]        # "How's it going?!" then the stop token


def test_prefill_too_long():
    with pytest.raises(X.ExecutorError) as e:
        X.fake_loop(PROMPT, PREFILL, DECODE, max_num_tokens=3, stop_sequence=[2294])
    assert e.value.code == INVALID_ARGUMENT and "8 >= 3" in e.value.message


def test_prefill_then_decode_until_the_stop_token():
    r = X.fake_loop(PROMPT, PREFILL, DECODE, stop_sequence=[2294])
    assert r["last_prefill_id"] == 2294
    assert r["tokens"] == DECODE and r["current_step"] == len(PREFILL) + len(DECODE)
    assert r["report"] == ""


@pytest.mark.parametrize("streaming", [False, True])
def test_decode_reaches_max_num_tokens(streaming):
    # no prefill, limit 3: three ids (" How", "'", "s" in the reference's test), then the loop ends
    r = X.fake_loop([], [], DECODE, max_num_tokens=3, stop_sequence=[2294], do_prefill=False, streaming=streaming)
    assert r["tokens"] == [224, 24, 8]
    assert r["cache_full_error"] is streaming  # only the streaming form reports it to its observer


def test_wrong_prefill_ids_are_rejected_by_the_fake():
    with pytest.raises(X.ExecutorError) as e:
        X.fake_loop([90, 547], PREFILL, DECODE, stop_sequence=[2294])
    assert e.value.code == INVALID_ARGUMENT and "Expected token size is 8 but got 3" in e.value.message


def test_benchmark_mode_fixes_both_counts():
    # prefill ids resized to the benchmark's count (no bos), decode runs the requested steps through the stop token
    script = [5, 2294, 6, 7, 8, 9]
    r = X.fake_loop([11, 12, 13], [11, 12, 13, 0, 0], script, stop_sequence=[2294], bench_prefill=5, bench_decode=4)
    assert r["last_prefill_id"] == 0 and r["tokens"] == script[:4] and r["current_step"] == 9
    assert "Prefill Turn 1: Processed 5 tokens in " in r["report"]
    assert "Decode Turn 1: Processed 4 tokens in " in r["report"]
    # the step marks land in the caller's record (the reference times them into a copy that it drops)
    assert "- executor_decode_and_sample: " in r["report"]
    r = X.fake_loop([11, 12, 13, 14, 15, 16], [11, 12], script, stop_sequence=[2294], bench_prefill=2, bench_decode=1)
    assert r["last_prefill_id"] == 12 and r["tokens"] == [5]


def test_benchmark_protocol_on_the_executor_host_logic():
    # README protocol scaled down, attention recorded instead of run: 64 prefill ids, 16 decode steps
    with X.HipLlmExecutor(2, 4, 1, 32, 256, runner_lengths=(32,), recording_backend=True) as ex:
        r = X.run_benchmark(ex, list(range(1, 20)), 64, 16)
        assert len(r["tokens"]) == 16 and r["current_step"] == 64 + 16
        # 63 ids run in prefill (the last of every chunk is deferred: 31, then the pending one + 31;
        # the 64th goes into the first decode step)
        runs = ex.runs()
        assert [len(t) for k, t, _ in runs if k == "prefill"] == [31, 32]
        assert sum(1 for k, _, _ in runs if k == "decode") == 16
        assert "Prefill Turn 1: Processed 64 tokens in " in r["report"]
        assert "Decode Turn 1: Processed 16 tokens in " in r["report"]
