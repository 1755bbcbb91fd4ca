"""The oracle against the committed golden vectors (tests/golden/, written by
tests/golden/make_golden.py from an independent library routine) and against
the softmax values the reference's own test holds."""
import glob
import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from oracle import attn_oracle as orc  # noqa: E402
from oracle import c_oracle  # noqa: E402

GOLDEN = os.path.join(ROOT, "tests", "golden")
CASES = sorted(glob.glob(os.path.join(GOLDEN, "decode_*.npz")) + glob.glob(os.path.join(GOLDEN, "prefill_*.npz")))


def load(path):
    z = np.load(path)  # allow_pickle stays False
    q_pos = z["q_pos"]
    assert np.array_equal(q_pos, q_pos[0] + np.arange(len(q_pos)))
    return dict(q=z["q"], k=z["k"], v=z["v"], out=z["out"], q_pos0=int(q_pos[0]), window=int(z["window"]),
                scale=float(z["scale"]), softcap=float(z["softcap"]))


def test_fixtures_present():
    names = {os.path.basename(p) for p in CASES}
    assert {"decode_c1_like.npz", "decode_c3_like.npz", "decode_window.npz", "decode_softcap.npz",
            "prefill_global.npz", "prefill_local.npz", "prefill_second_chunk.npz"} <= names


@pytest.mark.parametrize("path", CASES, ids=[os.path.basename(p)[:-4] for p in CASES])
def test_numpy_oracle_matches_golden(path):
    c = load(path)
    got = orc.sdpa(c["q"], c["k"], c["v"], c["scale"], q_pos0=c["q_pos0"], window=c["window"], softcap=c["softcap"])
    assert orc.rel_err(got, c["out"]) < 1e-6


@pytest.mark.parametrize("path", CASES, ids=[os.path.basename(p)[:-4] for p in CASES])
def test_c_oracle_matches_golden(path):
    c = load(path)
    got = c_oracle.sdpa_f64(c["q"], c["k"], c["v"], c["scale"], q_pos0=c["q_pos0"], window=c["window"],
                            softcap=c["softcap"])
    assert orc.rel_err(got, c["out"]) < 1e-6


def test_split_kv_oracle_matches_golden_decode():
    c = load(os.path.join(GOLDEN, "decode_c3_like.npz"))
    n = c["k"].shape[0]
    for splits in (1, 2, 3, 16):
        got = orc.decode_attn_split(c["q"][0], c["k"], c["v"], c["scale"], n, splits)
        got = got[0] if isinstance(got, tuple) else got
        assert orc.rel_err(got, c["out"][0]) < 1e-6, splits


def test_reference_softmax_values():
    with open(os.path.join(GOLDEN, "softmax_kat.json")) as f:
        kat = json.load(f)
    for case in kat["cases"]:
        p = orc.softmax_rows(np.array([case["logits"]], dtype=np.float32), dtype=np.float32)[0]
        np.testing.assert_allclose(p, case["probabilities"], rtol=1e-6)
