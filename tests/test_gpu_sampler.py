"""GPU parity of the HIP sampler, called through the C ABI, against
oracle/sampling_oracle.py and the values the reference's own tests hold.

Index work is held to exact equality; probabilities and scores to 1e-6
relative (float32 exp / log of the device library against numpy's)."""
import math
import os
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from __graft_entry__ import load_package  # noqa: E402
from oracle import sampling_oracle as so  # noqa: E402

S = load_package().sampler
DEV = "cuda:0"
FLT_MIN, FLT_MAX = float(np.finfo(np.float32).tiny), float(np.finfo(np.float32).max)


def say(*a):
    print(*a, flush=True)


def run(logits, k, p, temperature, u=None, seed=1, type=S.TOP_P, want_scores=True):
    """logits [B, V] float32 numpy -> (ids, log scores) from the device."""
    b, v = logits.shape
    with S.Sampler(k, p, temperature, b, seed, v, type=type, stream=torch.cuda.current_stream().cuda_stream) as s:
        lg = torch.from_numpy(np.ascontiguousarray(logits)).to(DEV)
        ids = torch.full((b,), -1, dtype=torch.int32, device=DEV)
        sc = torch.full((b,), 123.0, dtype=torch.float32, device=DEV) if want_scores else None
        ud = torch.from_numpy(np.asarray(u, np.float32)).to(DEV) if u is not None else None
        s.sample_to_id_and_score_buffer(lg, ids, sc, ud)
        torch.cuda.synchronize()
        return ids.cpu().numpy(), (sc.cpu().numpy() if want_scores else None)


def top_k(logits, k, temperature):
    b, v = logits.shape
    kk = min(k, v)
    with S.Sampler(k, 1.0, temperature, b, 1, v, stream=torch.cuda.current_stream().cuda_stream) as s:
        lg = torch.from_numpy(np.ascontiguousarray(logits)).to(DEV)
        idx = torch.full((b, kk), -1, dtype=torch.int32, device=DEV)
        pr = torch.zeros((b, kk), dtype=torch.float32, device=DEV)
        s.top_k(lg, idx, pr)
        torch.cuda.synchronize()
        return idx.cpu().numpy(), pr.cpu().numpy()


def test_reference_held_values():
    # sampling_cpu_util_test.cc:16-31 (TopKIndicies)
    idx, _ = top_k(np.array([[0.1, 0.5, 0.4, 0.2]], np.float32), 2, 1.0)
    assert sorted(idx[0].tolist()) == [1, 2]
    ids, _ = run(np.array([[0.1, 0.5], [0.4, 0.2]], np.float32), 1, 0.5, 1.0)
    assert ids.tolist() == [1, 0]
    # :33-97 (Softmax), probabilities of the candidates in descending order
    _, pr = top_k(np.array([[0.1, 0.1]], np.float32), 2, 1.0)
    assert pr[0].tolist() == [0.5, 0.5]
    _, pr = top_k(np.array([[0.0, 0.0]], np.float32), 2, 1.0)
    assert pr[0].tolist() == [0.5, 0.5]
    idx, pr = top_k(np.array([[0.0, 1.0, 2.0]], np.float32), 3, 0.00000001)
    assert idx[0].tolist() == [2, 1, 0] and pr[0].tolist() == [1.0, 0.0, 0.0]
    _, pr = top_k(np.array([[0.0, 1.0, 2.0, 3.0]], np.float32), 4, 100000000000.0)
    assert pr[0].tolist() == [0.25, 0.25, 0.25, 0.25]
    idx, pr = top_k(np.array([[0.1, 0.1], [0.0, 5.0], [1.0, 0.0]], np.float32), 2, 1.0)
    assert idx.tolist() == [[0, 1], [1, 0], [0, 1]]
    np.testing.assert_allclose(pr.ravel(), [0.5, 0.5, 0.993307173, 0.00669285096, 0.731058598, 0.268941432], rtol=1e-6)
    # :116-143 (TopKTopPSampling)
    ids, sc = run(np.array([[0.0, 0.0, 0.3]], np.float32), 1, 0.5, 1.0)
    assert ids.tolist() == [2] and sc.tolist() == [0.0]
    logits = np.array([[0.0, 0.0, 1.0], [0.0, 1.0, 0.0], [1.0, 0.0, 0.0]], np.float32)
    for u in (0.0, 0.31, 0.999999):
        ids, sc = run(logits, 2, 0.5, 0.00001, u=[u] * 3)
        assert ids.tolist() == [2, 1, 0] and sc.tolist() == [0.0, 0.0, 0.0]
    # top_p_cpu_sampler_test.cc:20-76
    ids, _ = run(np.array([[0.0, 0.0, 10.0, 0.0], [11.0, 12.0, 1.0, 2.0]], np.float32), 1, 0.5, 1.0, want_scores=False)
    assert ids.tolist() == [2, 1]
    ids, sc = run(np.array([[FLT_MIN, FLT_MIN, FLT_MAX, FLT_MIN], [FLT_MIN, FLT_MAX, FLT_MIN, FLT_MIN]], np.float32),
                  1, 0.5, 1.0)
    assert ids.tolist() == [2, 1] and sc.tolist() == [math.log(1.0), math.log(1.0)]
    say("sampler: reference-held values ok")


@pytest.mark.parametrize("vocab,k", [(262144, 64), (300001, 50), (524288, 256), (262144, 40), (32000, 256), (50257, 8), (1000, 1000), (7, 3), (4099, 2)])
def test_top_k_and_probabilities_match_oracle(vocab, k):
    rng = np.random.default_rng(vocab + k)
    b = 5
    logits = (rng.standard_normal((b, vocab)) * 4).astype(np.float32)
    logits[1, ::3] = logits[1, 0]          # long runs of equal values
    logits[2] = np.round(logits[2])        # heavy ties at the top
    logits[3, : vocab // 2] = -np.inf
    if k > S.MAX_K:
        with pytest.raises(Exception):
            top_k(logits, k, 0.8)
        return
    idx, pr = top_k(logits, k, 0.8)
    want_idx = so.top_k_indices(logits, min(k, vocab))
    assert np.array_equal(idx, want_idx), (vocab, k)
    want_pr, _ = so.softmax_top_k(logits, want_idx, 0.8)
    np.testing.assert_allclose(pr, want_pr, rtol=2e-6, atol=1e-30)
    say(f"sampler top-k vocab={vocab} k={k}: ok")


def test_all_equal_and_fallback_paths():
    # every logit equal: the bound from the thread maxima admits the whole row -> radix descent,
    # exact ties taken in ascending index order
    for vocab in (262144, 5000, 70000, 400000):
        for value in (0.0, -3.5, 7.25):
            logits = np.full((2, vocab), value, np.float32)
            logits[1, vocab - 5:] = value + 1.0     # five winners at the very end, then ties from index 0
            idx, pr = top_k(logits, 64, 1.0)
            assert idx[0].tolist() == list(range(64))
            assert idx[1].tolist() == list(range(vocab - 5, vocab)) + list(range(59))
            np.testing.assert_allclose(pr[0], 1.0 / 64, rtol=1e-6)
    # two crowded levels: many values sharing the top 24 bits of the key
    base = np.float32(3.0)
    vals = base + np.arange(200, dtype=np.float32) * np.float32(2.0 ** -22)
    logits = np.tile(vals, (1, 40)).astype(np.float32)
    idx, _ = top_k(logits, 50, 1.0)
    assert np.array_equal(idx, so.top_k_indices(logits, 50))
    say("sampler: tie / fallback paths ok")


@pytest.mark.parametrize("k,p,temperature", [(64, 0.95, 1.0), (40, 0.5, 0.7), (8, 1.0, 2.0), (256, 0.0, 1.0), (2, 0.9, 0.1)])
def test_sampling_matches_oracle_for_given_uniforms(k, p, temperature):
    rng = np.random.default_rng(k)
    b, vocab = 64, 32768
    logits = (rng.standard_normal((b, vocab)) * 2.5).astype(np.float32)
    u = rng.random(b).astype(np.float32)
    u[0], u[1] = 0.0, np.float32(1.0 - 2.0 ** -24)
    ids, sc = run(logits, k, p, temperature, u=u)
    want_ids, want_sc = so.top_k_top_p_sample(logits, k, p, temperature, u)
    near = 0
    for r in range(b):
        if ids[r] != want_ids[r]:
            # a draw within float32 rounding of a cumulative boundary may fall to the neighbour
            lo, _ = so.top_k_top_p_sample(logits[r:r + 1], k, p, temperature, np.array([max(u[r] - 1e-5, 0.0)]))
            hi, _ = so.top_k_top_p_sample(logits[r:r + 1], k, p, temperature, np.array([min(u[r] + 1e-5, 1.0)]))
            assert ids[r] in (lo[0], hi[0]), (r, ids[r], want_ids[r])
            near += 1
        else:
            np.testing.assert_allclose(sc[r], so.log_scores(want_sc[r:r + 1])[0], rtol=1e-5, atol=1e-6)
    assert near <= 1
    say(f"sampler k={k} p={p} T={temperature}: ids exact ({near} boundary cases)")


def test_type_switches_and_philox_draws():
    rng = np.random.default_rng(3)
    b, vocab = 16, 4096
    logits = (rng.standard_normal((b, vocab)) * 2).astype(np.float32)
    ids, sc = run(logits, 50, 0.3, 1.0, type=S.GREEDY)
    assert ids.tolist() == np.argmax(logits, axis=1).tolist() and sc.tolist() == [0.0] * b
    u = rng.random(b).astype(np.float32)
    ids, _ = run(logits, 20, 0.01, 1.0, u=u, type=S.TOP_K)        # TOP_K ignores p
    want, _ = so.top_k_top_p_sample(logits, 20, 1.0, 1.0, u)
    assert (ids == want).sum() >= b - 1
    # own draws: call n of a handle uses Philox4x32-10(counter = {row, n, 0, 0}, key = {seed, const})
    seed = 12345
    with S.Sampler(20, 0.9, 1.0, b, seed, vocab, stream=torch.cuda.current_stream().cuda_stream) as s:
        lg = torch.from_numpy(logits).to(DEV)
        out = torch.zeros((b,), dtype=torch.int32, device=DEV)
        for call in range(3):
            s.sample_to_id_and_score_buffer(lg, out)
            torch.cuda.synchronize()
            u = np.array([so.device_uniform(seed, call, r) for r in range(b)], np.float32)
            want, _ = so.top_k_top_p_sample(logits, 20, 0.9, 1.0, u)
            assert (out.cpu().numpy() == want).sum() >= b - 1, call
    say("sampler: type switches and Philox draws ok")


def test_distribution_of_draws():
    # p = 1, k = V = 4: the frequencies follow the softmax itself
    probs = np.array([0.5, 0.25, 0.125, 0.125])
    b = 4096
    logits = np.tile(np.log(probs).astype(np.float32), (b, 1))
    with S.Sampler(4, 1.0, 1.0, b, 99, 4, stream=torch.cuda.current_stream().cuda_stream) as s:
        lg = torch.from_numpy(logits).to(DEV)
        out = torch.zeros((b,), dtype=torch.int32, device=DEV)
        counts = np.zeros(4)
        for _ in range(8):
            s.sample_to_id_and_score_buffer(lg, out)
            torch.cuda.synchronize()
            counts += np.bincount(out.cpu().numpy(), minlength=4)
    freq = counts / counts.sum()
    assert np.abs(freq - probs).max() < 0.01, freq
    say(f"sampler: empirical frequencies {freq}")


def test_host_io_and_large_batch():
    rng = np.random.default_rng(9)
    b, vocab = 3, 262144
    logits = (rng.standard_normal((b, vocab)) * 3).astype(np.float32)
    u = rng.random(b).astype(np.float32)
    with S.Sampler(64, 0.95, 1.0, b, 1, vocab, host_io=True) as s:
        ids = np.zeros(b, np.int32)
        sc = np.zeros(b, np.float32)
        s.sample_to_id_and_score_buffer(logits, ids, sc, u)
    want, want_sc = so.top_k_top_p_sample(logits, 64, 0.95, 1.0, u)
    assert ids.tolist() == want.tolist()
    np.testing.assert_allclose(sc, so.log_scores(want_sc), rtol=1e-5, atol=1e-6)


# Calls of many rows: segments four times as long (64 logits per thread in registers, sample_kernel<64>), chosen when
# rows x 16,384-logit segments would be more than two workgroups per compute unit.
@pytest.mark.parametrize("vocab,k,b", [(262144, 64, 40), (262144, 256, 33), (250001, 50, 48), (131072, 1, 80),
                                       (70000, 17, 160)])
def test_many_rows_take_wide_segments_and_match_oracle(vocab, k, b):
    rng = np.random.default_rng(vocab + k + b)
    logits = (rng.standard_normal((b, vocab)) * 4).astype(np.float32)
    logits[1, ::3] = logits[1, 0]          # long runs of equal values: the radix descent
    logits[2] = np.round(logits[2])        # heavy ties at the top
    logits[3, : vocab // 2] = -np.inf
    logits[4, 5::7] = np.nan               # NaNs never win
    logits[5] = 1.5                        # every logit equal: ties in ascending index order
    logits[6, : vocab - 3] = -np.inf       # fewer than k finite values (k > 3)
    idx, pr = top_k(logits, k, 0.8)
    want_idx = so.top_k_indices(logits, k)
    assert np.array_equal(idx, want_idx), (vocab, k, b, np.argwhere((idx != want_idx).any(axis=1)).ravel()[:8])
    want_pr, _ = so.softmax_top_k(logits, want_idx, 0.8)
    np.testing.assert_allclose(pr, want_pr, rtol=2e-6, atol=1e-30)
    # and a draw with given uniforms, twice on the same sampler (the rows' tickets must be back at zero)
    u = rng.random(b).astype(np.float32)
    with S.Sampler(k, 0.9, 0.8, b, 1, vocab, stream=torch.cuda.current_stream().cuda_stream) as s:
        lg = torch.from_numpy(logits).to(DEV)
        ud = torch.from_numpy(u).to(DEV)
        want, _ = so.top_k_top_p_sample(logits, k, 0.9, 0.8, u)
        for _ in range(3):
            ids = torch.full((b,), -1, dtype=torch.int32, device=DEV)
            s.sample_to_id_and_score_buffer(lg, ids, None, ud)
            torch.cuda.synchronize()
            assert ids.cpu().numpy().tolist() == want.tolist()
    say(f"sampler wide segments vocab={vocab} k={k} rows={b}: ok")
