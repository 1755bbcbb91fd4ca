"""CPU-side checks of the C ABI: the library loads, exports every symbol the
header declares, and reports kUnavailable (never a silent fallback) when no
GPU can be used. No compute call is made."""
import ctypes
import os
import re
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from __graft_entry__ import load_package  # noqa: E402

A = load_package().attn


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "mi355_attn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi355_attn_[a-z_0-9]+)\s*\(", text)))


def test_header_symbols_are_exported():
    names = declared_symbols()
    assert len(names) >= 15 and "mi355_attn_decode" in names and "mi355_attn_prefill" in names
    L = ctypes.CDLL(A.LIB_PATH)
    for name in names:
        assert hasattr(L, name), f"{name} declared in include/mi355_attn.h but not exported"


def test_config_struct_matches_header_size():
    # struct_size is checked by the library; a mismatch would mean the binding drifted from the header
    assert ctypes.sizeof(A.Config) == 80


def test_version_and_no_silent_fallback():
    assert "gfx950" in A.version()
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present: covered by the gpu tests")
    with pytest.raises(A.AttnError) as e:
        A.Attn(1, 4, 1, 256, 128, 1, A.F16, A.F16)
    assert e.value.code == A.UNAVAILABLE


def test_argument_validation_precedes_device_use():
    L = A.lib()
    err = ctypes.c_void_p()
    h = ctypes.c_void_p()
    cfg = A.Config(4, 1, 4, 1, 256, 16, 1, A.F16, A.F16, 0.0, 0.0, None, 0, 0, 0, None)  # wrong struct_size
    assert L.mi355_attn_create(ctypes.byref(cfg), ctypes.byref(h), ctypes.byref(err)) == A.INVALID_ARGUMENT
    assert b"struct_size" in ctypes.string_at(err.value)
    assert L.mi355_attn_create(None, ctypes.byref(h), None) == A.INVALID_ARGUMENT
    assert L.mi355_attn_sync(None, None) == A.INVALID_ARGUMENT
    assert L.mi355_attn_decode(None, 0, None, None, 1, None, None, 1, None) == A.INVALID_ARGUMENT


# ---------------------------------------------------------------- sampler library
S = load_package().sampler


def test_sampler_header_symbols_are_exported():
    text = open(os.path.join(ROOT, "include", "mi355_sampler.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(mi355_sampler_[a-z_0-9]+)\s*\(", text)))
    assert len(names) >= 8 and "mi355_sampler_sample" in names and "mi355_sampler_create" in names
    L = ctypes.CDLL(S.LIB_PATH)
    for name in names:
        assert hasattr(L, name), f"{name} declared in include/mi355_sampler.h but not exported"
    assert ctypes.sizeof(S.Config) == 56


def test_sampler_argument_checks_follow_the_reference():
    """TopPSampler::Create (runtime/components/top_p_cpu_sampler.cc:40-57): k <= 0, p outside [0, 1],
    batch_size <= 0 and temperature <= 0 are kInvalidArgument, before any device is touched."""
    for kw, text in ((dict(k=0), "k must be positive."), (dict(p=1.5), "p must be in [0, 1]."),
                     (dict(p=-0.5), "p must be in [0, 1]."), (dict(batch_size=0), "batch_size must be positive."),
                     (dict(temperature=0.0), "Temperature must be positive")):
        args = dict(k=4, p=0.5, temperature=1.0, batch_size=1, seed=1, vocab_size=100)
        args.update(kw)
        with pytest.raises(A.AttnError) as e:
            S.Sampler(**args)
        assert e.value.code == A.INVALID_ARGUMENT and text in e.value.message
    with pytest.raises(A.AttnError) as e:
        S.Sampler(k=1000, p=0.5, temperature=1.0, batch_size=1, seed=1, vocab_size=5000)
    assert e.value.code == A.UNIMPLEMENTED
    import torch
    if not torch.cuda.is_available():
        with pytest.raises(A.AttnError) as e:
            S.Sampler(k=4, p=0.5, temperature=1.0, batch_size=1, seed=1, vocab_size=100)
        assert e.value.code == A.UNAVAILABLE  # the code on which the reference falls back to its CPU sampler
