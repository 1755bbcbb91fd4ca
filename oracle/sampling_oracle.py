"""CPU restatement of the reference's token sampling (top-k -> softmax with
temperature -> top-p nucleus -> draw), the checker for the HIP sampler.

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py; nothing of the product path may import it.

Follows runtime/components/sampling_cpu_util.cc:
  top_k_indices        TopKIndicies            :21-64
  softmax_top_k        Softmax                 :66-134
  top_k_top_p_sample   TopKTopPSampling        :136-233
  log_scores           TopPSampler::SampleToIdAndScoreBuffer, top_p_cpu_sampler.cc:96-107

Pinned by the values the reference's own tests hold
(sampling_cpu_util_test.cc:16-145, top_p_cpu_sampler_test.cc:20-79), by brute
force on tiny inputs and by closed forms (tests/test_sampling_oracle.py).

Two places where the reference's code does not do what its comments say; both
modes are restated (`as_written=True` / default intended behaviour):
  * :186-187 sorts the empty range [b*k, (b*1)*k): the top-k candidates are
    walked in whatever order std::nth_element left them, not by descending
    probability;
  * :222-229 has no break after the first cumulative sum that reaches the random
    draw, so the last candidate of the nucleus always wins.
The HIP sampler implements the intended behaviour (descending order, first
crossing). PARITY UNPINNED: the candidate order of std::nth_element is
implementation-defined, so "as written" results are only defined where they do
not depend on it (k = 1, one candidate holding all the mass: exactly the cases
the reference's tests cover); the random stream of absl::BitGen is not
reproducible by design, the draw is therefore an explicit input `u` here.
"""
from __future__ import annotations

import numpy as np

F32_EPS = float(np.finfo(np.float32).eps)


def top_k_indices(logits: np.ndarray, k: int) -> np.ndarray:
    """[B, V] -> [B, k] indices of the k largest logits per row, by descending
    logit, equal logits by ascending index. (The reference returns the same set
    in unspecified order; for k == 1 it is std::max_element: the first maximum.)"""
    logits = np.asarray(logits, dtype=np.float32)
    if logits.ndim != 2:
        raise ValueError("logits must be [batch, vocab]")
    order = np.argsort(-logits.astype(np.float64), axis=1, kind="stable")
    return order[:, :k].astype(np.int32)


def softmax_top_k(logits: np.ndarray, idx: np.ndarray, temperature: float):
    """Probabilities over the selected candidates, float32 arithmetic in the
    reference's op order. Returns (probabilities [B, k], max_logit [B])."""
    if temperature <= 0.0:
        raise ValueError(f"Temperature must be positive, but got {temperature}")
    logits = np.asarray(logits, dtype=np.float32)
    b, k = idx.shape
    probs = np.zeros((b, k), dtype=np.float32)
    max_logit = np.zeros(b, dtype=np.float32)
    t = np.float32(max(np.float32(temperature), np.float32(F32_EPS)))
    for r in range(b):
        sel = logits[r, idx[r]]
        max_logit[r] = sel.max()
        with np.errstate(over="ignore", under="ignore"):
            e = np.exp(((sel - max_logit[r]) / t).astype(np.float32)).astype(np.float32)
        s = np.float32(0.0)
        for x in e:  # sequential float32 sum, as the reference
            s = np.float32(s + x)
        if s <= F32_EPS:
            probs[r] = np.float32(1.0 / k)
        elif np.isinf(s):
            probs[r] = 0.0
            probs[r, int(np.argmax(sel))] = 1.0
        else:
            probs[r] = e * np.float32(np.float32(1.0) / s)
    return probs, max_logit


def top_k_top_p_sample(logits: np.ndarray, k: int, p: float, temperature: float, u: np.ndarray,
                       as_written: bool = False, candidate_order: np.ndarray | None = None):
    """Returns (ids [B] int32, sampled_scores [B] float32 = exp((logit - max) / T), 1.0 for k == 1).

    u [B] in [0, 1): the uniform draw, scaled by the nucleus mass as the
    reference scales its uniform_real_distribution(0, nucleus_sum).
    candidate_order [B, k]: the order in which the candidates are walked when
    `as_written` (stands in for what std::nth_element leaves behind)."""
    logits = np.asarray(logits, dtype=np.float32)
    if logits.size == 0:
        raise ValueError("Logits vector cannot be empty.")
    if k <= 0:
        raise ValueError("k must be greater than 0.")
    if p < 0.0 or p > 1.0:
        raise ValueError("p must be in the range [0.0, 1.0].")
    b, v = logits.shape
    k = min(k, v)
    idx = top_k_indices(logits, k)
    if as_written and candidate_order is not None:
        idx = np.asarray(candidate_order, dtype=np.int32)
    probs, max_logit = softmax_top_k(logits, idx, temperature)
    if k == 1:
        return idx[:, 0].copy(), np.ones(b, dtype=np.float32)
    ids = np.zeros(b, dtype=np.int32)
    scores = np.zeros(b, dtype=np.float32)
    t = np.float32(temperature)
    for r in range(b):
        order = np.arange(k)
        if not as_written:
            order = np.argsort(-probs[r].astype(np.float64), kind="stable")
        pr = probs[r, order].astype(np.float64)
        cum = 0.0
        n = 0
        for i in range(k):
            cum += pr[i]
            n = i + 1
            if cum >= p:
                break
        nucleus_sum = cum

        def score_of(i):
            with np.errstate(under="ignore"):
                return np.float32(np.exp(np.float32((logits[r, idx[r, order[i]]] - max_logit[r]) / t)))

        if nucleus_sum <= np.finfo(np.float64).eps:
            ids[r] = idx[r, order[0]]
            scores[r] = score_of(0)
            continue
        draw = float(u[r]) * nucleus_sum
        cur = 0.0
        chosen = n - 1
        for i in range(n):
            cur += pr[i]
            if draw <= cur:
                chosen = i
                if not as_written:
                    break
        ids[r] = idx[r, order[chosen]]
        scores[r] = score_of(chosen)
    return ids, scores


def log_scores(sampled_scores: np.ndarray) -> np.ndarray:
    """What the reference's sampler writes into the scores tensor."""
    with np.errstate(divide="ignore"):
        return np.log(np.asarray(sampled_scores, dtype=np.float32)).astype(np.float32)


# ---------------------------------------------------------------- Philox4x32-10
# Counter-based generator (Salmon et al., "Parallel random numbers: as easy as
# 1, 2, 3", SC'11) the HIP sampler draws its uniforms from; restated so that
# tests can predict the device's draws. Pinned by the published known answers.
_M0, _M1 = 0xD2511F53, 0xCD9E8D57
_W0, _W1 = 0x9E3779B9, 0xBB67AE85


def philox4x32_10(counter, key):
    c = [int(x) & 0xFFFFFFFF for x in counter]
    k = [int(x) & 0xFFFFFFFF for x in key]
    for _ in range(10):
        p0, p1 = _M0 * c[0], _M1 * c[2]
        c = [(p1 >> 32) ^ c[1] ^ k[0], p1 & 0xFFFFFFFF, (p0 >> 32) ^ c[3] ^ k[1], p0 & 0xFFFFFFFF]
        k = [(k[0] + _W0) & 0xFFFFFFFF, (k[1] + _W1) & 0xFFFFFFFF]
    return c


def device_uniform(seed: int, call_index: int, row: int) -> float:
    """The draw of the HIP sampler for (seed, number of sample calls so far,
    batch row): 24 high bits of the first Philox word, in [0, 1)."""
    w = philox4x32_10([row, call_index & 0xFFFFFFFF, (call_index >> 32) & 0xFFFFFFFF, 0], [seed & 0xFFFFFFFF, 0x4D493335])
    return (w[0] >> 8) * (1.0 / (1 << 24))
