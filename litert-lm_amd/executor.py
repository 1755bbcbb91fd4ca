"""ctypes binding of libhip_llm_executor.so: the C++ HipLlmExecutor driven
through its C test surface (litert-lm_amd/executor/executor_c_api.cc)."""
from __future__ import annotations

import ctypes
import os

import numpy as np

from . import attn as _attn

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libhip_llm_executor.so")
_lib = None
# HipLlmExecutor(device_resident=True): activations, logits and sampling stay on the GPU for the whole pass.
HAS_DEVICE_RESIDENT = True


class ExecutorError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"executor status {code}: {message}")
        self.code = code
        self.message = message


class _Config(ctypes.Structure):
    _fields_ = [
        ("num_layers", ctypes.c_int32), ("num_q_heads", ctypes.c_int32), ("num_kv_heads", ctypes.c_int32),
        ("vocab", ctypes.c_int32), ("max_num_tokens", ctypes.c_int32),
        ("layer_window", ctypes.POINTER(ctypes.c_int32)),
        ("runner_lengths", ctypes.POINTER(ctypes.c_int32)),
        ("num_runners", ctypes.c_int32), ("fp16_activations", ctypes.c_int32),
        ("recording_backend", ctypes.c_int32), ("execute_pending_on_single_id_chunk", ctypes.c_int32),
        ("softcap", ctypes.c_float), ("pre_attention", ctypes.c_int32), ("device_resident", ctypes.c_int32),
        ("two_call_decode_step", ctypes.c_int32),
    ]


class LoopResult(ctypes.Structure):
    _fields_ = [("last_prefill_id", ctypes.c_int32), ("n_tokens", ctypes.c_int32),
                ("cache_full_error", ctypes.c_int32), ("current_step", ctypes.c_int32)]


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(f"{LIB_PATH} is missing: build it with `make -C litert-lm_amd/executor`")
        _attn.lib()  # dependency, loaded first so that the rpath-less case still resolves
        L = ctypes.CDLL(LIB_PATH)
        vp, i32 = ctypes.c_void_p, ctypes.c_int32
        i32p = ctypes.POINTER(ctypes.c_int32)
        errp = ctypes.POINTER(ctypes.c_void_p)
        L.hle_create.argtypes = [ctypes.POINTER(_Config), ctypes.POINTER(vp), errp]
        L.hle_destroy.argtypes = [vp]
        L.hle_destroy.restype = None
        L.hle_prefill.argtypes = [vp, i32p, i32, i32, errp]
        L.hle_prefill_with_params.argtypes = [vp, i32p, i32, i32, i32, i32, errp]
        L.hle_is_device_resident.argtypes = [vp]
        L.hle_wait_for_completion.argtypes = [vp, errp]
        L.hle_decode.argtypes = [vp, i32p, errp]
        L.hle_decode_logits.argtypes = [vp, i32, ctypes.POINTER(ctypes.c_float), errp]
        for n in ("hle_current_step", "hle_vocab_size", "hle_max_num_tokens", "hle_num_runs"):
            getattr(L, n).argtypes = [vp]
        L.hle_reset.argtypes = [vp, errp]
        L.hle_fill_vision_embeddings.argtypes = [vp, i32, errp]
        L.hle_backend_name.argtypes = [vp]
        L.hle_backend_name.restype = ctypes.c_char_p
        L.hle_get_run.argtypes = [vp, i32, i32p, i32p, i32p, i32]
        L.hle_backend_from_string.argtypes = [ctypes.c_char_p]
        L.hle_plan.argtypes = [i32p, i32, i32, i32p, i32p, i32]
        L.hle_bi_create.argtypes = [i32, i32]
        L.hle_bi_create.restype = vp
        L.hle_bi_destroy.argtypes = [vp]
        L.hle_bi_destroy.restype = None
        L.hle_bi_call.argtypes = [vp, i32, ctypes.c_char_p, ctypes.c_uint64, errp]
        L.hle_bi_count.argtypes = [vp, i32]
        L.hle_bi_value.argtypes = [vp, i32, ctypes.c_char_p, i32]
        L.hle_bi_value.restype = ctypes.c_double
        L.hle_bi_report.argtypes = [vp]
        L.hle_bi_report.restype = vp
        L.hle_format_duration.argtypes = [ctypes.c_int64]
        L.hle_format_duration.restype = vp
        L.hle_stop_detector_run.argtypes = [i32, i32p, i32p, i32, i32p, i32, i32p, i32p, i32, i32p]
        resp = ctypes.POINTER(LoopResult)
        L.hle_fake_loop.argtypes = [i32p, i32, i32, i32p, i32, i32p, i32, i32, i32p, i32, i32, i32, i32, i32, i32p, i32,
                                    resp, errp, errp]
        L.hle_run_benchmark.argtypes = [vp, i32p, i32, i32, i32, i32p, i32, resp, errp, errp]
        L.hle_litertlm_header.argtypes = [ctypes.c_char_p, vp, ctypes.c_uint64, errp, errp]
        L.hle_litertlm_read.argtypes = [ctypes.c_char_p, i32, i32, i32, errp, ctypes.POINTER(ctypes.c_uint64), errp]
        _lib = L
    return _lib


def _check(rc, err):
    msg = ""
    if err.value:
        msg = ctypes.string_at(err.value).decode("utf-8", "replace")
        _attn._libc.free(err.value)
    if rc != 0:
        raise ExecutorError(rc, msg)


def _arr(xs):
    xs = [int(x) for x in xs]
    return (ctypes.c_int32 * len(xs))(*xs)


class HipLlmExecutor:
    """HipLlmExecutor over the synthetic decoder layers (test scaffolding)."""

    def __init__(self, num_layers, num_q_heads, num_kv_heads, vocab, max_num_tokens, runner_lengths=(1024,),
                 layer_window=None, fp16=False, recording_backend=False, execute_pending_on_single_id_chunk=False,
                 softcap=0.0, pre_attention=False, device_resident=None, two_call_decode_step=False):
        """device_resident: True / False, or None to let the executor decide (device-resident on its own MI355X
        backend, host-staged on the recording backend). two_call_decode_step: device-resident decode keeps the step
        before attention and the attention as two calls per layer instead of one (comparisons)."""
        self._win = _arr(layer_window) if layer_window is not None else None
        self._runners = _arr(runner_lengths)
        cfg = _Config(num_layers, num_q_heads, num_kv_heads, vocab, max_num_tokens,
                      ctypes.cast(self._win, ctypes.POINTER(ctypes.c_int32)) if self._win is not None else None,
                      ctypes.cast(self._runners, ctypes.POINTER(ctypes.c_int32)), len(runner_lengths), int(fp16),
                      int(recording_backend), int(execute_pending_on_single_id_chunk), softcap, int(pre_attention),
                      -1 if device_resident is None else int(bool(device_resident)), int(bool(two_call_decode_step)))
        self._h = ctypes.c_void_p()
        err = ctypes.c_void_p()
        _check(lib().hle_create(ctypes.byref(cfg), ctypes.byref(self._h), ctypes.byref(err)), err)
        self.vocab = vocab

    def close(self):
        if getattr(self, "_h", None) is not None and self._h.value:
            lib().hle_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def prefill(self, ids, batch=1, wait_for_completion=None, cancel=None):
        """Prefill(inputs), or Prefill(inputs, params) when wait_for_completion or cancel (the value the cancel
        flag holds during the call) is given."""
        ids = list(ids)
        n = len(ids) // batch if batch else 0
        err = ctypes.c_void_p()
        if wait_for_completion is None and cancel is None:
            _check(lib().hle_prefill(self._h, _arr(ids), batch, n, ctypes.byref(err)), err)
        else:
            _check(lib().hle_prefill_with_params(self._h, _arr(ids), batch, n, int(bool(wait_for_completion)),
                                                 -1 if cancel is None else int(bool(cancel)), ctypes.byref(err)), err)

    def is_device_resident(self) -> bool:
        return bool(lib().hle_is_device_resident(self._h))

    def wait_for_completion(self):
        err = ctypes.c_void_p()
        _check(lib().hle_wait_for_completion(self._h, ctypes.byref(err)), err)

    def decode(self) -> int:
        tok = ctypes.c_int32(-7)
        err = ctypes.c_void_p()
        _check(lib().hle_decode(self._h, ctypes.byref(tok), ctypes.byref(err)), err)
        return tok.value

    def decode_logits(self, explicit_id=None) -> np.ndarray:
        out = np.zeros(self.vocab, dtype=np.float32)
        err = ctypes.c_void_p()
        _check(lib().hle_decode_logits(self._h, -1 if explicit_id is None else int(explicit_id),
                                       out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), ctypes.byref(err)), err)
        return out

    def current_step(self) -> int:
        return lib().hle_current_step(self._h)

    def vocab_size(self) -> int:
        return lib().hle_vocab_size(self._h)

    def max_num_tokens(self) -> int:
        return lib().hle_max_num_tokens(self._h)

    def backend_name(self) -> str:
        return lib().hle_backend_name(self._h).decode()

    def reset(self):
        err = ctypes.c_void_p()
        _check(lib().hle_reset(self._h, ctypes.byref(err)), err)

    def fill_vision_embeddings(self, image_index: int = 0):
        """LlmExecutorBase::FillVisionEmbeddings with empty vision data (not implemented by this executor)."""
        err = ctypes.c_void_p()
        _check(lib().hle_fill_vision_embeddings(self._h, image_index, ctypes.byref(err)), err)

    def runs(self):
        """[(kind, tokens, positions)] of every forward pass since the last reset."""
        out = []
        cap = 1 << 16
        toks = (ctypes.c_int32 * cap)()
        pos = (ctypes.c_int32 * cap)()
        for i in range(lib().hle_num_runs(self._h)):
            dec = ctypes.c_int32()
            n = lib().hle_get_run(self._h, i, ctypes.byref(dec), toks, pos, cap)
            out.append(("decode" if dec.value else "prefill", list(toks[:n]), list(pos[:n])))
        return out


def _take_text(ptr) -> str:
    if not ptr:
        return ""
    text = ctypes.string_at(ptr).decode("utf-8", "replace")
    _attn._libc.free(ptr)
    return text


class BenchmarkInfo:
    """The C++ BenchmarkInfo (executor/benchmark_info.h) behind its test surface."""
    INIT_START, INIT_END, PREFILL_START, PREFILL_END, DECODE_START, DECODE_END, MARK = range(7)

    def __init__(self, num_prefill_tokens=0, num_decode_tokens=0):
        self._h = ctypes.c_void_p(lib().hle_bi_create(num_prefill_tokens, num_decode_tokens))

    def __del__(self):
        if getattr(self, "_h", None) is not None and self._h.value:
            lib().hle_bi_destroy(self._h)
            self._h = ctypes.c_void_p()

    def _call(self, what, name=b"", tokens=0):
        err = ctypes.c_void_p()
        _check(lib().hle_bi_call(self._h, what, name.encode() if isinstance(name, str) else name, tokens,
                                 ctypes.byref(err)), err)

    def time_init_phase_start(self, name): self._call(self.INIT_START, name)
    def time_init_phase_end(self, name): self._call(self.INIT_END, name)
    def time_prefill_turn_start(self): self._call(self.PREFILL_START)
    def time_prefill_turn_end(self, tokens): self._call(self.PREFILL_END, tokens=tokens)
    def time_decode_turn_start(self): self._call(self.DECODE_START)
    def time_decode_turn_end(self, tokens): self._call(self.DECODE_END, tokens=tokens)
    def time_mark_delta(self, name): self._call(self.MARK, name)

    def num_init_phases(self): return lib().hle_bi_count(self._h, 0)
    def total_prefill_turns(self): return lib().hle_bi_count(self._h, 1)
    def total_decode_turns(self): return lib().hle_bi_count(self._h, 2)
    def num_marks(self): return lib().hle_bi_count(self._h, 3)
    def init_phase_seconds(self, name): return lib().hle_bi_value(self._h, 0, name.encode(), 0)
    def mark_seconds(self, name): return lib().hle_bi_value(self._h, 3, name.encode(), 0)
    def prefill_tokens_per_sec(self, i): return lib().hle_bi_value(self._h, 1, b"", i)
    def decode_tokens_per_sec(self, i): return lib().hle_bi_value(self._h, 2, b"", i)

    def report(self) -> str:
        return _take_text(lib().hle_bi_report(self._h))


def format_duration(ns: int) -> str:
    return _take_text(lib().hle_format_duration(int(ns)))


def stop_detector_run(batch, sequences, tokens, reset=False):
    """tokens: [steps][batch]. Returns (step at which every item had stopped, add status codes,
    steps-before-stop per item, all-done after the optional reset)."""
    flat = [t for seq in sequences for t in seq]
    lens = [len(seq) for seq in sequences]
    steps = len(tokens)
    toks = [t for row in tokens for t in row]
    codes = (ctypes.c_int32 * max(1, len(sequences)))()
    before = (ctypes.c_int32 * batch)()
    done = ctypes.c_int32(-1)
    i = lib().hle_stop_detector_run(batch, _arr(flat) if flat else None, _arr(lens) if lens else None, len(sequences),
                                    _arr(toks) if toks else None, steps, codes, before, int(reset), ctypes.byref(done))
    if i < 0:
        raise ExecutorError(-i, "ProcessTokens")
    return i, list(codes[:len(sequences)]), list(before), (None if not reset else bool(done.value))


def _loop_outputs(rc, err, out, res, report):
    text = _take_text(report.value)
    _check(rc, err)
    return {"tokens": list(out[:res.n_tokens]), "last_prefill_id": res.last_prefill_id,
            "cache_full_error": bool(res.cache_full_error), "current_step": res.current_step, "report": text}


def fake_loop(prompt, expected_prefill, decode_script, *, bos=2, max_num_tokens=0, stop_sequence=(), bench_prefill=0,
              bench_decode=0, streaming=False, do_prefill=True):
    """Prefill + decode loop of executor/pipeline.h over the scripted FakeLlmExecutor."""
    cap = 4096
    out = (ctypes.c_int32 * cap)()
    res = LoopResult()
    err, report = ctypes.c_void_p(), ctypes.c_void_p()
    stop = list(stop_sequence)
    rc = lib().hle_fake_loop(_arr(prompt) if prompt else None, len(prompt), bos,
                             _arr(expected_prefill) if expected_prefill else None, len(expected_prefill),
                             _arr(decode_script) if decode_script else None, len(decode_script), max_num_tokens,
                             _arr(stop) if stop else None, len(stop), bench_prefill, bench_decode, int(streaming),
                             int(do_prefill), out, cap, ctypes.byref(res), ctypes.byref(report), ctypes.byref(err))
    return _loop_outputs(rc, err, out, res, report)


def run_benchmark(executor: "HipLlmExecutor", prompt, bench_prefill, bench_decode):
    """The reference's benchmark protocol (prefill turn of `bench_prefill` ids, `bench_decode` decode
    steps) on a HipLlmExecutor; returns the ids, the step counter and the BenchmarkInfo text."""
    cap = max(16, bench_decode + 16)
    out = (ctypes.c_int32 * cap)()
    res = LoopResult()
    err, report = ctypes.c_void_p(), ctypes.c_void_p()
    rc = lib().hle_run_benchmark(executor._h, _arr(prompt) if prompt else None, len(prompt), bench_prefill, bench_decode,
                                 out, cap, ctypes.byref(res), ctypes.byref(report), ctypes.byref(err))
    return _loop_outputs(rc, err, out, res, report)


# AnySectionDataType of the .litertlm container
SECTION_NONE, SECTION_BINARY, SECTION_DEPRECATED, SECTION_TFLITE, SECTION_SP_TOKENIZER, SECTION_LLM_METADATA, \
    SECTION_HF_TOKENIZER_ZLIB = range(7)


def model_file(path, preset_max_num_tokens=0) -> dict:
    """What an executor takes from a .litertlm file: the section map by kind and the token capacity (the settings'
    own value if `preset_max_num_tokens` is set, else the file's LlmMetadata.max_num_tokens, else 4096)."""
    import json
    lib().hle_model_file.argtypes = [ctypes.c_char_p, ctypes.c_int32, ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_void_p)]
    text, err = ctypes.c_void_p(), ctypes.c_void_p()
    rc = lib().hle_model_file(str(path).encode(), preset_max_num_tokens, ctypes.byref(text), ctypes.byref(err))
    out = _take_text(text.value)
    _check(rc, err)
    return json.loads(out)


def proto_int32_field(message: bytes, field_number: int) -> int:
    lib().hle_proto_int32_field.argtypes = [ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int32, ctypes.POINTER(ctypes.c_int32),
                                            ctypes.POINTER(ctypes.c_void_p)]
    buf = ctypes.create_string_buffer(bytes(message), len(message))
    value, err = ctypes.c_int32(), ctypes.c_void_p()
    _check(lib().hle_proto_int32_field(ctypes.cast(buf, ctypes.c_void_p), len(message), field_number, ctypes.byref(value),
                                       ctypes.byref(err)), err)
    return value.value


def litertlm_header(path=None, data=None) -> dict:
    """Header of a .litertlm file (or of a bytes object): version, system metadata, section map."""
    import json
    text, err = ctypes.c_void_p(), ctypes.c_void_p()
    if path is not None:
        rc = lib().hle_litertlm_header(str(path).encode(), None, 0, ctypes.byref(text), ctypes.byref(err))
    else:
        buf = ctypes.create_string_buffer(bytes(data), len(data))
        rc = lib().hle_litertlm_header(None, ctypes.cast(buf, ctypes.c_void_p), len(data), ctypes.byref(text),
                                       ctypes.byref(err))
    out = _take_text(text.value)
    _check(rc, err)
    return json.loads(out)


def _litertlm_read(path, what, idx=0, expected_type=0) -> bytes:
    data, err, n = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_uint64()
    rc = lib().hle_litertlm_read(str(path).encode(), what, idx, expected_type, ctypes.byref(data), ctypes.byref(n),
                                 ctypes.byref(err))
    _check(rc, err)
    out = ctypes.string_at(data.value, n.value)
    _attn._libc.free(data.value)
    return out


def litertlm_section(path, idx, expected_type) -> bytes:
    return _litertlm_read(path, 0, idx, expected_type)


def litertlm_hf_tokenizer_json(path, idx=None) -> bytes:
    return _litertlm_read(path, 2) if idx is None else _litertlm_read(path, 1, idx)


def litertlm_any_binary(path) -> bytes:
    return _litertlm_read(path, 3)


def backend_from_string(s: str) -> int:
    return lib().hle_backend_from_string(s.encode())


def plan(runner_lengths, n):
    cap = 4096
    lens = (ctypes.c_int32 * cap)()
    counts = (ctypes.c_int32 * cap)()
    k = lib().hle_plan(_arr(runner_lengths), len(runner_lengths), n, lens, counts, cap)
    if k < 0:
        raise ExecutorError(-k, "plan")
    return [(lens[i], counts[i]) for i in range(k)]
