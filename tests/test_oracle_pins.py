"""Pins the CPU oracle before anything is compared against it.

Each check is chosen so that a plausible mistake in the oracle (dropped scale,
wrong GQA map, off-by-one in the causal or window rule, transposed operand,
mis-merged partitions) makes it fail. Sources of truth, in order: the
reference's own known-answer values, closed forms and invariants of the
mathematics, a pure-Python brute force on tiny shapes, and torch's CPU SDPA as
an independent library cross-check.
"""
import math

import numpy as np
import pytest

from oracle import attn_oracle as orc
from oracle import c_oracle


def rng(seed=0):
    return np.random.default_rng(seed)


# ---------------------------------------------------------------- softmax KATs
# Values held by the reference: runtime/components/sampling_cpu_util_test.cc:32-97
def test_softmax_known_answers():
    p = orc.softmax_rows(np.array([[0.1, 0.1], [0.0, 5.0], [1.0, 0.0]], dtype=np.float32), dtype=np.float32)
    np.testing.assert_allclose(p[0], [0.5, 0.5], rtol=1e-6)
    np.testing.assert_allclose(p[1], [0.00669285096, 0.993307173], rtol=1e-6)
    np.testing.assert_allclose(p[2], [0.731058598, 0.268941432], rtol=1e-6)
    np.testing.assert_allclose(orc.softmax_rows(np.zeros((1, 2), np.float32)), [[0.5, 0.5]])


def test_softmax_temperature_limits():
    # sampling_cpu_util_test.cc:56-80: tiny temperature -> greedy, huge -> uniform
    p = orc.softmax_rows(np.array([0.0, 1.0, 2.0]), temperature=1e-8)
    np.testing.assert_array_equal(p, [0.0, 0.0, 1.0])
    p = orc.softmax_rows(np.array([0.0, 1.0, 2.0, 3.0]), temperature=1e11)
    np.testing.assert_allclose(p, [0.25] * 4, rtol=1e-6)
    with pytest.raises(ValueError):
        orc.softmax_rows(np.array([1.0]), temperature=0.0)


# ---------------------------------------------------------------- mask rule
def test_fill_attention_mask_rule():
    m = orc.fill_attention_mask(orc.init_attention_mask(4, 8), start_timestep=2, steps=3)
    assert m.shape == (1, 1, 4, 8)
    rows = m[0, 0]
    for i in range(3):
        assert (rows[i, : 2 + i + 1] == 0.0).all()
        assert (rows[i, 2 + i + 1:] == np.float32(-45824)).all()
    assert (rows[3] == np.float32(-45824)).all()  # row beyond `steps` stays masked
    mb = orc.fill_attention_mask(orc.init_attention_mask(4, 8, boolean=True), 2, 3)[0, 0]
    np.testing.assert_array_equal(mb, rows == 0.0)
    m32 = orc.init_attention_mask(1, 4, is_f16=False)
    assert m32[0, 0, 0, 0] == np.float32(-0.7) * np.finfo(np.float32).max
    with pytest.raises(ValueError):
        orc.fill_attention_mask(np.zeros((2, 2), np.float32), 0, 1)
    # the C twin builds the same mask
    np.testing.assert_array_equal(c_oracle.fill_mask(4, 8, 2, 3), rows)


def test_additive_bool_and_predicate_masks_agree():
    r = rng(1)
    S, L, Hq, Hkv, D, start = 5, 16, 4, 2, 8, 7
    q = r.standard_normal((S, Hq, D))
    k = r.standard_normal((L, Hkv, D))
    v = r.standard_normal((L, Hkv, D))
    add = orc.fill_attention_mask(orc.init_attention_mask(S, L), start, S)[0, 0]
    boo = orc.fill_attention_mask(orc.init_attention_mask(S, L, boolean=True), start, S)[0, 0]
    o_add = orc.sdpa_masked(q, k, v, 0.3, add)
    o_boo = orc.sdpa_masked(q, k, v, 0.3, boo)
    o_pred = orc.sdpa(q, k, v, 0.3, q_pos0=start)
    # exp(-45824 + ...) underflows to exactly 0 in fp64 as well
    np.testing.assert_array_equal(o_add, o_boo)
    np.testing.assert_array_equal(o_boo, o_pred)
    # fp32 evaluation of the additive form stays within 1e-6 of the fp64 one
    o32 = orc.sdpa_masked(q, k, v, 0.3, add, dtype=np.float32)
    assert orc.rel_err(o32, o_add) < 1e-6


# ---------------------------------------------------------------- closed forms
def test_closed_forms():
    r = rng(2)
    L, Hq, Hkv, D = 12, 4, 2, 8
    q = r.standard_normal((1, Hq, D))
    k = r.standard_normal((L, Hkv, D))
    v = r.standard_normal((L, Hkv, D))
    p = 8
    # (i) identical keys -> mean of the visible values
    k_same = np.broadcast_to(k[:1], k.shape)
    o = orc.sdpa(q, k_same, v, 0.5, q_pos0=p)
    exp = np.repeat(v[: p + 1].mean(axis=0), Hq // Hkv, axis=0)
    np.testing.assert_allclose(o[0], exp, rtol=1e-12)
    # (ii) a single visible key -> that value row
    o = orc.sdpa(q, k, v, 0.5, q_pos0=0)
    np.testing.assert_allclose(o[0], np.repeat(v[0], Hq // Hkv, axis=0), rtol=1e-12)
    # (iii) one dominant key
    k_dom = k.copy()
    k_dom[5] = 0
    q_big = np.zeros_like(q)
    q_big[..., 0] = 1.0
    k_dom[:, :, 0] = 0.0
    k_dom[5, :, 0] = 1e4
    o = orc.sdpa(q_big, k_dom, v, 1.0, q_pos0=p)
    np.testing.assert_allclose(o[0], np.repeat(v[5], Hq // Hkv, axis=0), rtol=1e-9)
    # (iv) zero query -> uniform average
    o = orc.sdpa(np.zeros_like(q), k, v, 0.5, q_pos0=p)
    np.testing.assert_allclose(o[0], exp, rtol=1e-12)
    # (v) constant values -> constant output
    o = orc.sdpa(q, k, np.full_like(v, 3.25), 0.5, q_pos0=p)
    np.testing.assert_allclose(o, 3.25, rtol=1e-12)


def test_two_key_closed_form_pins_scale_and_sign():
    # o = sigmoid(scale * q.(k1-k0)) v1 + (1 - ...) v0: catches a dropped or
    # squared scale, a sign error and a K/V swap.
    q = np.array([[[1.0, 2.0]]])
    k = np.array([[[0.5, -1.0]], [[2.0, 0.25]]])
    v = np.array([[[10.0, 0.0]], [[0.0, 20.0]]])
    scale = 0.37
    s0, s1 = scale * (0.5 - 2.0), scale * (2.0 + 0.5)
    w1 = 1.0 / (1.0 + math.exp(s0 - s1))
    o = orc.sdpa(q, k, v, scale, q_pos0=1)
    np.testing.assert_allclose(o[0, 0], [10.0 * (1 - w1), 20.0 * w1], rtol=1e-12)


# ---------------------------------------------------------------- invariants
def test_invariants():
    r = rng(3)
    S, L, Hq, Hkv, D = 3, 20, 8, 2, 16
    q = r.standard_normal((S, Hq, D))
    k = r.standard_normal((L, Hkv, D))
    v = r.standard_normal((L, Hkv, D))
    base = orc.sdpa(q, k, v, 0.25, q_pos0=L - S)
    # scaling K by c and the scale by 1/c
    np.testing.assert_allclose(orc.sdpa(q, 4.0 * k, v, 0.25 / 4.0, q_pos0=L - S), base, rtol=1e-12)
    # a per-row constant added to the scores (through an additive mask)
    vis = orc.visibility(L - S + np.arange(S), L)
    add = np.where(vis, 0.0, -np.inf) + np.array([[1.5], [-2.0], [7.0]])
    np.testing.assert_allclose(orc.sdpa_masked(q, k, v, 0.25, add), base, rtol=1e-12)
    # permuting (k, v) pairs together: compare the last row, which sees all keys
    perm = r.permutation(L)
    o_perm = orc.sdpa_masked(q[-1:], k[perm], v[perm], 0.25, np.ones((1, L), bool))
    np.testing.assert_allclose(o_perm[0], base[-1], rtol=1e-11)
    # GQA == MHA over explicitly repeated KV heads
    k_rep, v_rep = np.repeat(k, Hq // Hkv, axis=1), np.repeat(v, Hq // Hkv, axis=1)
    np.testing.assert_array_equal(orc.sdpa(q, k_rep, v_rep, 0.25, q_pos0=L - S), base)
    # and a wrong map (kv = q_head % Hkv) must differ
    wrong = orc.sdpa(q, np.tile(k, (1, Hq // Hkv, 1)), np.tile(v, (1, Hq // Hkv, 1)), 0.25, q_pos0=L - S)
    assert np.abs(wrong - base).max() > 1e-3


def test_sliding_window_rule():
    r = rng(4)
    L, Hq, Hkv, D = 24, 4, 1, 8
    q = r.standard_normal((L, Hq, D))
    k = r.standard_normal((L, Hkv, D))
    v = r.standard_normal((L, Hkv, D))
    glob = orc.sdpa(q, k, v, 0.3)
    np.testing.assert_array_equal(orc.sdpa(q, k, v, 0.3, window=L), glob)
    np.testing.assert_array_equal(orc.sdpa(q, k, v, 0.3, window=10 * L), glob)
    # window 1: only the token itself
    np.testing.assert_allclose(orc.sdpa(q, k, v, 0.3, window=1), np.repeat(v, Hq, axis=1), rtol=1e-12)
    # window W: row p equals global attention over keys p-W+1..p
    W = 5
    loc = orc.sdpa(q, k, v, 0.3, window=W)
    for p in (0, 3, 4, 5, 17, 23):
        lo = max(0, p - W + 1)
        ref = orc.sdpa_masked(q[p:p + 1], k[lo:p + 1], v[lo:p + 1], 0.3, np.ones((1, p + 1 - lo), bool))
        np.testing.assert_allclose(loc[p], ref[0], rtol=1e-12)
    vis = orc.visibility(np.arange(L), L, W)
    assert vis.sum(axis=1).tolist() == [min(p + 1, W) for p in range(L)]


def test_split_kv_merge_equals_unsplit():
    r = rng(5)
    Hq, Hkv, D = 8, 2, 16
    for kv_len, window in ((37, 0), (64, 0), (5, 0), (50, 7), (50, 1)):
        q = r.standard_normal((Hq, D))
        k = r.standard_normal((kv_len, Hkv, D))
        v = r.standard_normal((kv_len, Hkv, D))
        ref = orc.decode_attn(q, k, v, 0.25, kv_len, window=window)
        for ns in (1, 2, 3, 16, 64):  # 64 > kv_len gives empty partitions
            out, lse = orc.decode_attn_split(q, k, v, 0.25, kv_len, ns, window=window)
            np.testing.assert_allclose(out, ref, rtol=1e-11, atol=1e-13)
        # lse against the direct definition
        kk = np.repeat(k, Hq // Hkv, axis=1)
        s = 0.25 * np.einsum("hd,lhd->hl", q, kk)
        s = np.where(orc.visibility(np.array([kv_len - 1]), kv_len, window), s, -np.inf)
        direct = np.log(np.exp(s - s.max(-1, keepdims=True)).sum(-1)) + s.max(-1)
        np.testing.assert_allclose(lse, direct, rtol=1e-11)


def test_int8_kv_equals_dequantised_and_folded_scales():
    r = rng(6)
    L, Hq, Hkv, D = 40, 8, 2, 16
    q = r.standard_normal((Hq, D))
    k = r.standard_normal((L, Hkv, D)).astype(np.float32)
    v = r.standard_normal((L, Hkv, D)).astype(np.float32)
    kq, ks = orc.quantize_kv_int8(k)
    vq, vs = orc.quantize_kv_int8(v)
    assert kq.dtype == np.int8 and np.abs(kq).max() == 127 and ks.shape == (Hkv, D)
    np.testing.assert_allclose(ks, np.abs(k).max(axis=0) / 127.0, rtol=1e-7)
    assert np.abs(orc.dequantize_kv_int8(kq, ks) - k).max() <= 0.5 * ks.max() * (1 + 1e-6)
    ref = orc.decode_attn(q, orc.dequantize_kv_int8(kq, ks), orc.dequantize_kv_int8(vq, vs), 0.25, L)
    # fold k_scale into q and v_scale into the output: algebraically the same
    g = Hq // Hkv
    q_fold = q * np.repeat(ks.astype(np.float64), g, axis=0)
    o_fold = orc.decode_attn(q_fold, kq.astype(np.float64), vq.astype(np.float64), 0.25, L)
    o_fold = o_fold * np.repeat(vs.astype(np.float64), g, axis=0)
    # dequantisation rounds q*s to fp32 once per element; the folded form does not
    assert orc.rel_err(o_fold, ref) < 1e-6
    # all-zero channel: scale 0 must not produce NaN
    z = np.zeros((4, 1, 2), np.float32)
    zq, zs = orc.quantize_kv_int8(z)
    assert (zq == 0).all() and (zs == 0).all()


# ---------------------------------------------------------------- brute force
def _brute(q, k, v, scale, q_pos0, window, softcap=0.0):
    S, Hq, D = q.shape
    L, Hkv, _ = k.shape
    g = Hq // Hkv
    out = [[[0.0] * D for _ in range(Hq)] for _ in range(S)]
    for i in range(S):
        p = q_pos0 + i
        for h in range(Hq):
            scores = []
            for j in range(L):
                if j > p or (window > 0 and p - j >= window):
                    continue
                s = sum(float(q[i, h, c]) * float(k[j, h // g, c]) for c in range(D)) * scale
                if softcap > 0:
                    s = softcap * math.tanh(s / softcap)
                scores.append((j, s))
            if not scores:
                continue
            m = max(s for _, s in scores)
            den = sum(math.exp(s - m) for _, s in scores)
            for j, s in scores:
                w = math.exp(s - m) / den
                for c in range(D):
                    out[i][h][c] += w * float(v[j, h // g, c])
    return np.array(out)


@pytest.mark.parametrize("seed", range(6))
def test_brute_force_tiny(seed):
    r = rng(100 + seed)
    S = int(r.integers(1, 5))
    L = int(r.integers(S, 17))
    Hkv = int(r.integers(1, 3))
    Hq = Hkv * int(r.integers(1, 4))
    D = int(r.integers(1, 9))
    window = int(r.integers(0, 6))
    softcap = float(r.choice([0.0, 0.0, 5.0]))
    q = r.standard_normal((S, Hq, D))
    k = r.standard_normal((L, Hkv, D))
    v = r.standard_normal((L, Hkv, D))
    q_pos0 = L - S
    ref = _brute(q, k, v, 0.7, q_pos0, window, softcap)
    np.testing.assert_allclose(orc.sdpa(q, k, v, 0.7, q_pos0=q_pos0, window=window, softcap=softcap), ref,
                               rtol=1e-11, atol=1e-13)
    got_c = c_oracle.sdpa_f64(q, k, v, 0.7, q_pos0=q_pos0, window=window, softcap=softcap)
    q32, k32, v32 = (x.astype(np.float32) for x in (q, k, v))
    ref32 = _brute(q32, k32, v32, float(np.float32(0.7)), q_pos0, window, softcap)
    np.testing.assert_allclose(got_c, ref32, rtol=1e-6, atol=1e-8)


# ---------------------------------------------------------------- library cross-check
def test_against_torch_cpu_sdpa():
    torch = pytest.importorskip("torch")
    r = rng(7)
    S, L, Hq, Hkv, D = 9, 33, 8, 2, 32
    q = r.standard_normal((S, Hq, D))
    k = r.standard_normal((L, Hkv, D))
    v = r.standard_normal((L, Hkv, D))
    for window in (0, 6):
        vis = orc.visibility(L - S + np.arange(S), L, window)
        tq = torch.from_numpy(q).permute(1, 0, 2)[None]
        tk = torch.from_numpy(np.repeat(k, Hq // Hkv, axis=1)).permute(1, 0, 2)[None]
        tv = torch.from_numpy(np.repeat(v, Hq // Hkv, axis=1)).permute(1, 0, 2)[None]
        ref = torch.nn.functional.scaled_dot_product_attention(
            tq, tk, tv, attn_mask=torch.from_numpy(vis)[None, None], scale=0.2)[0].permute(1, 0, 2).numpy()
        np.testing.assert_allclose(orc.sdpa(q, k, v, 0.2, q_pos0=L - S, window=window), ref, rtol=1e-10)


# ---------------------------------------------------------------- C twin vs numpy
def test_c_oracle_matches_numpy_oracle():
    r = rng(8)
    S, L, Hq, Hkv, D = 7, 70, 8, 2, 64
    q = r.standard_normal((S, Hq, D)).astype(np.float32)
    k = r.standard_normal((L, Hkv, D)).astype(np.float32)
    v = r.standard_normal((L, Hkv, D)).astype(np.float32)
    scale = float(D) ** -0.5
    for window in (0, 9):
        ref = orc.sdpa(q, k, v, scale, q_pos0=L - S, window=window)
        got = c_oracle.sdpa_f64(q, k, v, scale, q_pos0=L - S, window=window)
        assert orc.rel_err(got, ref) < 1e-7  # scale is fp32 in C, fp64 in numpy
        vis = orc.visibility(L - S + np.arange(S), L, window)
        mask = np.where(vis, 0.0, orc.MASK_NEG_F16).astype(np.float32)
        got32 = c_oracle.sdpa_ref_f32(q, k, v, scale, mask=mask, threads=2)
        assert orc.rel_err(got32, ref) < 1e-5
    # batched decode entry
    lens = [5, 70, 33]
    ks = [k[:n] for n in lens]
    vs = [v[:n] for n in lens]
    qb = q[:3]
    got = c_oracle.decode_batch_ref_f32(qb, ks, vs, scale, threads=2)
    for b, n in enumerate(lens):
        ref = orc.decode_attn(qb[b], ks[b], vs[b], scale, n)
        assert orc.rel_err(got[b], ref) < 1e-5


# ---------------------------------------------------------------- planner + state machine
def test_prefill_work_groups_hand_worked():
    runners = [32, 1024, 256]
    assert orc.prefill_work_groups(runners, 1300) == [(1024, 1024), (1024, 276)]
    assert orc.prefill_work_groups(runners, 1100) == [(1024, 1024), (256, 76)]
    assert orc.prefill_work_groups(runners, 1050) == [(1024, 1024), (32, 26)]
    assert orc.prefill_work_groups(runners, 26) == [(32, 26)]
    assert orc.prefill_work_groups(runners, 32) == [(32, 32)]
    assert orc.prefill_work_groups(runners, 33) == [(256, 33)]
    assert orc.prefill_work_groups(runners, 2048) == [(1024, 1024), (1024, 1024)]
    assert orc.prefill_work_groups([128], 300) == [(128, 128), (128, 128), (128, 44)]


def test_executor_state_machine_hand_worked():
    ex = orc.OracleExecutor(runner_lengths=(4,), execute_single_pending=True)
    ex.prefill([10, 11, 12])
    # last id is deferred: executor.cc:182-203,244
    assert ex.calls == [("prefill", [10, 11], [0, 1])]
    assert ex.current_step == 2 and ex.next_input_token_id == 12 and ex.get_current_step() == 3
    ex.prefill([13, 14, 15, 16, 17, 18])  # chunks of 4 and 2; pending 12 goes first
    assert ex.calls[1] == ("prefill", [12, 13, 14, 15], [2, 3, 4, 5])
    assert ex.calls[2] == ("prefill", [16, 17], [6, 7])
    assert ex.next_input_token_id == 18 and ex.get_current_step() == 9
    assert ex.decode() == 18
    assert ex.calls[3] == ("decode", [18], [8]) and ex.current_step == 9
    with pytest.raises(ValueError):
        ex.decode()  # nothing pending: kInvalidArgument in the reference (:432-434)
    assert ex.decode(explicit_id=99) == 99 and ex.calls[-1] == ("decode", [99], [9])
    ex.reset()
    assert ex.get_current_step() == 0 and ex.next_input_token_id == -1
    # README benchmark shape: 1024 ids -> 1023 executed in prefill, 1 in decode
    ex = orc.OracleExecutor(runner_lengths=(1024,))
    ex.prefill(list(range(1024)))
    assert len(ex.calls[0][1]) == 1023 and ex.get_current_step() == 1024
    # single-id chunk with a pending token: reference drops it, HIP executor runs it
    ref = orc.OracleExecutor(runner_lengths=(4,), execute_single_pending=False)
    ref.prefill([1, 2]); ref.prefill([3])
    assert ref.calls[-1] == ("prefill", [], []) and ref.current_step == 1
    fix = orc.OracleExecutor(runner_lengths=(4,), execute_single_pending=True)
    fix.prefill([1, 2]); fix.prefill([3])
    assert fix.calls[-1] == ("prefill", [2], [1]) and fix.current_step == 2 and fix.next_input_token_id == 3
