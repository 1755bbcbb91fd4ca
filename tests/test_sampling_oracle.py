"""Pins of oracle/sampling_oracle.py: the values held by the reference's own
tests (runtime/components/sampling_cpu_util_test.cc, top_p_cpu_sampler_test.cc),
brute force, closed forms, and the published known answers of Philox4x32-10."""
import math
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from oracle import sampling_oracle as so  # noqa: E402

FLT_MIN, FLT_MAX = float(np.finfo(np.float32).tiny), float(np.finfo(np.float32).max)


# ---- sampling_cpu_util_test.cc:16-31
def test_top_k_indices_reference_values():
    idx = so.top_k_indices(np.array([[0.1, 0.5, 0.4, 0.2]], np.float32), 2)
    assert sorted(idx[0].tolist()) == [1, 2]
    idx = so.top_k_indices(np.array([[0.1, 0.5], [0.4, 0.2]], np.float32), 1)
    assert idx[:, 0].tolist() == [1, 0]


# ---- sampling_cpu_util_test.cc:33-97
def test_softmax_reference_values():
    p, m = so.softmax_top_k(np.array([[0.1, 0.1]], np.float32), np.array([[0, 1]]), 1.0)
    assert p[0].tolist() == [0.5, 0.5] and m.tolist() == [np.float32(0.1)]
    p, m = so.softmax_top_k(np.array([[0.0, 0.0]], np.float32), np.array([[0, 1]]), 1.0)
    assert p[0].tolist() == [0.5, 0.5] and m.tolist() == [0.0]
    p, m = so.softmax_top_k(np.array([[0.0, 1.0, 2.0]], np.float32), np.array([[0, 1, 2]]), 0.00000001)
    assert p[0].tolist() == [0.0, 0.0, 1.0] and m.tolist() == [2.0]
    p, m = so.softmax_top_k(np.array([[0.0, 1.0, 2.0, 3.0]], np.float32), np.array([[0, 1, 2, 3]]), 100000000000.0)
    assert p[0].tolist() == [0.25, 0.25, 0.25, 0.25] and m.tolist() == [3.0]
    logits = np.array([[0.1, 0.1], [0.0, 5.0], [1.0, 0.0]], np.float32)
    p, m = so.softmax_top_k(logits, np.array([[0, 1]] * 3), 1.0)
    np.testing.assert_allclose(p.ravel(), [0.5, 0.5, 0.00669285096, 0.993307173, 0.731058598, 0.268941432], rtol=2e-7)
    assert m.tolist() == [np.float32(0.1), 5.0, 1.0]
    with pytest.raises(ValueError):
        so.softmax_top_k(logits, np.array([[0, 1]] * 3), 0.0)


# ---- sampling_cpu_util_test.cc:99-143
@pytest.mark.parametrize("as_written", [False, True])
def test_top_k_top_p_sampling_reference_values(as_written):
    probs = np.array([[0.0, 0.0, 0.3]], np.float32)
    with pytest.raises(ValueError):
        so.top_k_top_p_sample(probs, -1, 0.5, 1.0, np.zeros(1), as_written)
    with pytest.raises(ValueError):
        so.top_k_top_p_sample(probs, 1, -0.5, 1.0, np.zeros(1), as_written)
    ids, sc = so.top_k_top_p_sample(probs, 1, 0.5, 1.0, np.array([0.7]), as_written)
    assert ids.tolist() == [2] and sc.tolist() == [1.0]
    logits = np.array([[0.0, 0.0, 1.0], [0.0, 1.0, 0.0], [1.0, 0.0, 0.0]], np.float32)
    for u in (0.0, 0.31, 0.999999):
        ids, sc = so.top_k_top_p_sample(logits, 2, 0.5, 0.00001, np.full(3, u), as_written)
        assert ids.tolist() == [2, 1, 0] and sc.tolist() == [1.0, 1.0, 1.0]
    if as_written:  # whichever way nth_element leaves the two candidates
        for order in ([[2, 0], [1, 0], [0, 1]], [[0, 2], [2, 1], [2, 0]], [[1, 2], [0, 1], [1, 0]]):
            ids, sc = so.top_k_top_p_sample(logits, 2, 0.5, 0.00001, np.full(3, 0.5), True, np.array(order))
            assert ids.tolist() == [2, 1, 0] and sc.tolist() == [1.0, 1.0, 1.0]


# ---- top_p_cpu_sampler_test.cc:20-76
def test_top_p_sampler_reference_values():
    logits = np.array([[0.0, 0.0, 10.0, 0.0], [11.0, 12.0, 1.0, 2.0]], np.float32)
    ids, sc = so.top_k_top_p_sample(logits, 1, 0.5, 1.0, np.array([0.1, 0.9]))
    assert ids.tolist() == [2, 1]
    logits = np.array([[FLT_MIN, FLT_MIN, FLT_MAX, FLT_MIN], [FLT_MIN, FLT_MAX, FLT_MIN, FLT_MIN]], np.float32)
    ids, sc = so.top_k_top_p_sample(logits, 1, 0.5, 1.0, np.array([0.1, 0.9]))
    assert ids.tolist() == [2, 1]
    assert so.log_scores(sc).tolist() == [math.log(1.0), math.log(1.0)]


# ---- brute force and closed forms
def brute_sample(row, k, p, temperature, u):
    """Independent float64 formulation: sort everything, inverse CDF over the nucleus."""
    order = sorted(range(len(row)), key=lambda i: (-float(row[i]), i))[:k]
    m = max(float(row[i]) for i in order)
    w = [math.exp((float(row[i]) - m) / temperature) for i in order]
    tot = sum(w)
    pr = [x / tot for x in w]
    cum, n = 0.0, 0
    for i, x in enumerate(pr):
        cum += x
        n = i + 1
        if cum >= p:
            break
    draw, cur = u * cum, 0.0
    for i in range(n):
        cur += pr[i]
        if draw <= cur:
            return order[i]
    return order[n - 1]


def test_intended_mode_matches_brute_force():
    rng = np.random.default_rng(5)
    for trial in range(200):
        v = int(rng.integers(2, 40))
        k = int(rng.integers(2, v + 1))
        p = float(rng.choice([0.0, 0.3, 0.5, 0.9, 1.0]))
        t = float(rng.choice([0.5, 1.0, 2.0]))
        logits = (rng.standard_normal((3, v)) * 3).astype(np.float32)
        # keep the draw away from the cumulative boundaries (float32 vs float64 probabilities)
        u = rng.random(3)
        ids, _ = so.top_k_top_p_sample(logits, k, p, t, u)
        for r in range(3):
            want = brute_sample(logits[r], k, p, t, u[r])
            if ids[r] != want:
                lo = brute_sample(logits[r], k, p, t, max(u[r] - 1e-5, 0.0))
                hi = brute_sample(logits[r], k, p, t, min(u[r] + 1e-5, 1.0))
                assert ids[r] in (lo, hi), (trial, r)


def test_inverse_cdf_closed_form():
    # p = 1, k = V: the draw follows the softmax itself; the boundaries are the cumulative sums
    logits = np.log(np.array([[0.5, 0.25, 0.125, 0.125]], np.float32))
    for u, want in ((0.0, 0), (0.49, 0), (0.51, 1), (0.74, 1), (0.76, 2), (0.874, 2), (0.876, 3), (0.999, 3)):
        ids, sc = so.top_k_top_p_sample(logits, 4, 1.0, 1.0, np.array([u]))
        assert ids.tolist() == [want], u
        np.testing.assert_allclose(sc[0], [1.0, 0.5, 0.25, 0.25][want], rtol=1e-6)
    # p = 0.6: the nucleus is {0, 1} (0.5 < 0.6 <= 0.75) and the draw is scaled by its mass
    for u, want in ((0.0, 0), (0.66, 0), (0.67, 1), (0.999, 1)):
        ids, _ = so.top_k_top_p_sample(logits, 4, 0.6, 1.0, np.array([u]))
        assert ids.tolist() == [want], u
    # as written: the last candidate of the nucleus, whatever the draw
    for u in (0.0, 0.3, 0.9):
        ids, _ = so.top_k_top_p_sample(logits, 4, 0.6, 1.0, np.array([u]), as_written=True)
        assert ids.tolist() == [1]
    # ties: lower index first; k limits the candidates
    ids, _ = so.top_k_top_p_sample(np.zeros((1, 8), np.float32), 4, 1.0, 1.0, np.array([0.3]))
    assert ids.tolist() == [1]


def test_philox_known_answers():
    assert so.philox4x32_10([0, 0, 0, 0], [0, 0]) == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    assert so.philox4x32_10([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2) == [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]
    assert so.philox4x32_10([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0]) == \
        [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]
    us = [so.device_uniform(7, c, r) for c in range(50) for r in range(20)]
    assert 0.0 <= min(us) and max(us) < 1.0 and 0.4 < float(np.mean(us)) < 0.6 and len(set(us)) == len(us)
