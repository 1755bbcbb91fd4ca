"""Pins the helpers through which every bfloat16 verdict of the GPU parity tests is computed
(oracle/attn_oracle.py: round_bf16, half_ulp_bf16, rel_err_beyond_bf16_rounding, l2_rel_err,
bf16_bits, bf16_ulp_distance, bf16_output_match). Nothing here restates their formulas: they are
held against the definition of the format (every bfloat16 number is a fixed point, midpoints go to
the even neighbour), against torch.bfloat16 as an independent implementation, and against cases
worked by hand."""
import numpy as np
import pytest
import torch

from oracle import attn_oracle as orc


def all_finite_bf16():
    bits = np.arange(1 << 16, dtype=np.uint32)
    vals = (bits << 16).view(np.float32)
    keep = np.isfinite(vals)
    return bits[keep].astype(np.uint16), vals[keep]


def test_every_finite_bf16_number_is_a_fixed_point_of_round_bf16():
    bits, vals = all_finite_bf16()
    assert len(vals) == 65280
    out = orc.round_bf16(vals)
    assert out.dtype == np.float64
    assert np.array_equal(out, vals.astype(np.float64))
    assert np.array_equal(np.signbit(out), np.signbit(vals))  # -0 stays -0
    assert np.array_equal(orc.bf16_bits(vals), bits)


def test_midpoints_round_to_the_even_neighbour_and_off_midpoints_to_the_nearest():
    # 1 + 2^-8 lies halfway between 1 (mantissa even) and 1 + 2^-7: down. 1 + 3*2^-8 halfway between
    # 1 + 2^-7 (odd) and 1 + 2^-6 (even): up.
    assert orc.round_bf16(np.float32(1 + 2.0 ** -8)) == 1.0
    assert orc.round_bf16(np.float32(1 + 3 * 2.0 ** -8)) == 1 + 2.0 ** -6
    assert orc.round_bf16(np.float32(-(1 + 2.0 ** -8))) == -1.0
    # one float32 step off the midpoint decides by distance
    mid = np.float32(1 + 2.0 ** -8)
    assert orc.round_bf16(np.nextafter(mid, np.float32(2))) == 1 + 2.0 ** -7
    assert orc.round_bf16(np.nextafter(mid, np.float32(0))) == 1.0
    # across a power of two: 2 - 2^-8 is halfway between 2 - 2^-7 (odd mantissa 0x7F) and 2 (even)
    assert orc.round_bf16(np.float32(2 - 2.0 ** -8)) == 2.0
    # every midpoint between neighbouring positive normal bfloat16 numbers, all at once
    bits, vals = all_finite_bf16()
    pos = (vals > 0) & (bits >= 0x0080) & (bits < 0x7F7F)
    lo = vals[pos].astype(np.float64)
    hi = ((bits[pos].astype(np.uint32) + 1) << 16).view(np.float32).astype(np.float64)
    mids = ((lo + hi) / 2).astype(np.float32)
    assert np.array_equal(mids.astype(np.float64), (lo + hi) / 2)  # representable in float32
    want = np.where(bits[pos] % 2 == 0, lo, hi)
    assert np.array_equal(orc.round_bf16(mids), want)


def test_round_bf16_agrees_with_torch_on_random_float32():
    rng = np.random.default_rng(17)
    x = np.concatenate([rng.standard_normal(200_000).astype(np.float32),
                        (rng.standard_normal(50_000) * 1e-30).astype(np.float32),
                        (rng.standard_normal(50_000) * 1e30).astype(np.float32),
                        rng.integers(0, 1 << 32, 200_000, dtype=np.uint64).astype(np.uint32).view(np.float32)])
    x = x[np.isfinite(x)]
    x = x[np.isfinite(torch.from_numpy(x).bfloat16().float().numpy())]  # (values that round to infinity: not outputs of attention)
    want = torch.from_numpy(x).bfloat16().float().numpy().astype(np.float64)
    assert np.array_equal(orc.round_bf16(x), want)
    want_bits = (torch.from_numpy(x).bfloat16().view(torch.int16).numpy().astype(np.int32) & 0xFFFF).astype(np.uint16)
    assert np.array_equal(orc.bf16_bits(x), want_bits)


def test_half_ulp_at_and_around_powers_of_two():
    # bfloat16 has 8 significant bits: in [2^e, 2^(e+1)) neighbours are 2^(e-7) apart, half of that is 2^(e-8)
    for e in (-20, -1, 0, 1, 7, 30):
        p = 2.0 ** e
        assert orc.half_ulp_bf16(p) == 2.0 ** (e - 8)
        assert orc.half_ulp_bf16(-p) == 2.0 ** (e - 8)
        assert orc.half_ulp_bf16(np.nextafter(p, 0)) == 2.0 ** (e - 9)        # just below: the finer grid
        assert orc.half_ulp_bf16(p * 1.9999) == 2.0 ** (e - 8)                # up to the next power: the same grid
    assert orc.half_ulp_bf16(0.0) == 0.0
    np.testing.assert_array_equal(orc.half_ulp_bf16(np.array([1.0, 3.0, -0.75, 0.0])), [2.0 ** -8, 2.0 ** -7, 2.0 ** -9, 0.0])


def test_half_ulp_bounds_the_rounding_error_of_round_bf16_and_is_reached():
    rng = np.random.default_rng(3)
    x = (rng.standard_normal(300_000) * np.exp(rng.uniform(-20, 20, 300_000))).astype(np.float32).astype(np.float64)
    err = np.abs(orc.round_bf16(x) - x)
    hu = orc.half_ulp_bf16(x)
    assert (err <= hu).all()
    assert (err / hu).max() > 0.999  # not a loose bound
    # a midpoint reaches it exactly
    x = np.float32(1 + 2.0 ** -8)
    assert abs(orc.round_bf16(x) - float(x)) == orc.half_ulp_bf16(x)


def test_rel_err_beyond_bf16_rounding_hand_worked():
    ref = np.array([1.0, -4.0, 0.3])  # half ulps: 2^-8, 2^-6, 2^-10 ; max|ref| = 4
    hu = np.array([2.0 ** -8, 2.0 ** -6, 2.0 ** -10])
    assert orc.rel_err_beyond_bf16_rounding(ref, ref) == 0.0
    # an error of exactly half an ulp on every element is forgiven
    assert orc.rel_err_beyond_bf16_rounding(ref + hu, ref) == 0.0
    assert orc.rel_err_beyond_bf16_rounding(ref - hu, ref) == 0.0
    # half an ulp + delta on one element leaves delta / max|ref|
    delta = 2.0 ** -7
    for i in range(3):
        got = ref.copy()
        got[i] += hu[i] + delta
        assert orc.rel_err_beyond_bf16_rounding(got, ref) == delta / 4.0
        got[i] = ref[i] - hu[i] - delta
        assert orc.rel_err_beyond_bf16_rounding(got, ref) == delta / 4.0
    # the allowance is taken from the reference element, not from the largest one: the same absolute
    # error that is forgiven on -4 is not on 0.3
    got = ref.copy()
    got[2] += 2.0 ** -6
    assert orc.rel_err_beyond_bf16_rounding(got, ref) == (2.0 ** -6 - 2.0 ** -10) / 4.0
    # and it never exceeds the plain figure
    rng = np.random.default_rng(5)
    a, b = rng.standard_normal(1000), rng.standard_normal(1000)
    assert 0 < orc.rel_err_beyond_bf16_rounding(a, b) <= orc.rel_err(a, b)
    # a correctly rounded result has nothing beyond the rounding
    assert orc.rel_err_beyond_bf16_rounding(orc.round_bf16(b), b) == 0.0


def test_rel_err_and_l2_rel_err_hand_worked():
    ref = np.array([[3.0, -4.0]])
    got = np.array([[3.0, -3.0]])
    assert orc.rel_err(got, ref) == 0.25          # 1 / 4
    assert orc.l2_rel_err(got, ref) == 0.2        # 1 / 5
    assert orc.l2_rel_err(ref, ref) == 0.0
    assert orc.l2_rel_err(2 * ref, ref) == 1.0
    assert orc.l2_rel_err(np.array([1.0]), np.array([0.0])) == 1.0  # zero reference: absolute
    # rounding N(0,1) data to bfloat16 costs about 2^-9 * sqrt(1/3) * (mean-square mantissa factor) in L2 terms:
    # between 1.3e-3 and 2e-3, which is why a bf16 output sits so close to a 2e-3 L2 bound
    x = np.random.default_rng(9).standard_normal(100_000)
    assert 1.3e-3 < orc.l2_rel_err(orc.round_bf16(x), x) < 2.0e-3


def test_bf16_ulp_distance_and_output_match():
    one = np.float32(1.0)
    up = np.float32(1 + 2.0 ** -7)       # next bfloat16 above 1
    down = np.float32(1 - 2.0 ** -8)     # next bfloat16 below 1
    assert orc.bf16_ulp_distance(one, one) == 0
    assert orc.bf16_ulp_distance(one, up) == 1
    assert orc.bf16_ulp_distance(one, down) == 1
    assert orc.bf16_ulp_distance(up, down) == 2
    assert orc.bf16_ulp_distance(np.float32(0.0), np.float32(-0.0)) == 0
    tiny = (np.array([1], dtype=np.uint32) << 16).view(np.float32)[0]  # smallest positive bfloat16 (subnormal)
    assert orc.bf16_ulp_distance(tiny, np.float32(0.0)) == 1
    assert orc.bf16_ulp_distance(tiny, -tiny) == 2
    # consecutive bit patterns of one sign are neighbours, all of them
    bits, vals = all_finite_bf16()
    pos = vals[(bits & 0x8000) == 0]
    assert (orc.bf16_ulp_distance(pos[:-1], pos[1:]) == 1).all()
    # output match: the exact result rounded is a full match; one element moved one step is seen
    ref = np.random.default_rng(2).standard_normal(1000)
    got = orc.round_bf16(ref)
    assert orc.bf16_output_match(got, ref) == (1.0, 0)
    got2 = got.copy()
    got2[7] = float(torch.nextafter(torch.tensor(got[7]).bfloat16(), torch.tensor(10.0).bfloat16()).float())
    share, worst = orc.bf16_output_match(got2, ref)
    assert share == 0.999 and worst == 1
    got2[8] = 2 * got[8]  # far off: 128 steps (one binade)
    assert orc.bf16_output_match(got2, ref)[1] == 128
