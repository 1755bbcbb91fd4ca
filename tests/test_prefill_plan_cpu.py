"""CPU tests of the prefill work planner (host code of libmi355_attn.so, no device needed) through
mi355_attn_prefill_plan_probe: every work item of a launch is planned exactly once (the probe itself
answers < 0 otherwise), the key blocks it accounts for equal a brute-force count over visible
(query, key) pairs, and the packed plan of the benchmarked launch is balanced the way its clock says.
"""
import ctypes
import os

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "litert-lm_amd", "libmi355_attn.so")
i32 = ctypes.c_int32


def lib():
    L = ctypes.CDLL(LIB)  # (a missing library is a failure, not a skip: the build comes first)
    L.mi355_attn_prefill_plan_probe.restype = ctypes.c_int
    return L


def probe(layers_windows, n, q_pos0, hq, hkv, wgs, cus):
    L = lib()
    nl = len(layers_windows)
    win = (i32 * nl)(*layers_windows)
    ipw, bpw, off = (i32 * wgs)(), (i32 * wgs)(), i32()
    r = L.mi355_attn_prefill_plan_probe(nl, n, q_pos0, hq, hkv, win, wgs, cus, ipw, bpw, ctypes.byref(off))
    return r, np.array(ipw[:]), np.array(bpw[:]), off.value


def rows_per_tile(hq, hkv):
    g = hq // hkv
    hpb = 4 if g % 4 == 0 else (2 if g % 2 == 0 else 1)
    return 32 * (4 // hpb), hkv * (g // hpb)


def brute_force_blocks(windows, n, q_pos0, hq, hkv):
    """Key blocks (32 keys) that hold at least one key some query of the tile sees, summed over tiles, head
    blocks and layers: key j is visible to the query at position p when j <= p and (window 0 or p - j < window).
    Every (query, key) pair is looked at."""
    rpt, per_layer = rows_per_tile(hq, hkv)
    total = 0
    keys = np.arange(q_pos0 + n)
    for w in windows:
        for p0 in range(q_pos0, q_pos0 + n, rpt):
            qs = np.arange(p0, min(p0 + rpt, q_pos0 + n))
            visible = keys[None, :] <= qs[:, None]
            if w > 0:
                visible &= qs[:, None] - keys[None, :] < w
            total += len(set((keys[visible.any(axis=0)] // 32).tolist())) * per_layer
    return total


def test_benchmarked_launch():
    windows = [0 if (l + 1) % 6 == 0 else 512 for l in range(26)]
    r, items, blocks, off = probe(windows, 1024, 0, 4, 1, 512, 256)
    assert r == 26 * 32 == items.sum()
    assert blocks.sum() == 4 * (32 * 33 // 2) + 22 * (sum(range(1, 17)) + 16 * 17) == brute_force_blocks(windows, 1024, 0, 4, 1)
    assert (items > 0).all()
    # the workgroups placed first on a compute unit are the faster ones: they get more key blocks
    assert blocks[:256].mean() > 1.3 * blocks[256:].mean()
    # by the planner's own clock (0.05 us units) nobody is far behind the rest
    done = np.where(np.arange(512) < 256, 162 + 28 * blocks + 100 * items, 141 + 44 * blocks + 100 * items)
    assert done.max() <= 1.02 * np.sort(done)[-64:].mean()
    assert done.max() * 0.05 < 61.0  # us
    # a layer's items mostly stay on one XCD
    assert off < 0.25 * r


@pytest.mark.parametrize("seed", range(12))
def test_every_item_once_and_blocks_by_brute_force(seed):
    rng = np.random.default_rng(seed)
    nl = int(rng.integers(1, 30))
    hq, hkv = [(4, 1), (8, 2), (2, 2), (16, 2), (6, 3), (3, 1)][int(rng.integers(0, 6))]
    n = int(rng.integers(1, 1400))
    q_pos0 = int(rng.integers(0, 3)) * int(rng.integers(0, 900))
    windows = [int(rng.choice([0, 0, 1, 33, 64, 100, 512])) for _ in range(nl)]
    cus = int(rng.choice([256, 256, 64, 8]))
    wgs = int(rng.choice([2 * cus, cus, max(1, cus // 2), 1]))
    r, items, blocks, _ = probe(windows, n, q_pos0, hq, hkv, wgs, cus)
    rpt, per_layer = rows_per_tile(hq, hkv)
    assert r == nl * per_layer * ((n + rpt - 1) // rpt) == items.sum(), (r, items.sum())
    assert blocks.sum() == brute_force_blocks(windows, n, q_pos0, hq, hkv)


def test_bad_arguments():
    L = lib()
    win = (i32 * 1)(0)
    buf = (i32 * 4)()
    assert L.mi355_attn_prefill_plan_probe(0, 10, 0, 4, 1, win, 4, 2, buf, buf, None) == -1
    assert L.mi355_attn_prefill_plan_probe(1, 10, 0, 4, 3, win, 4, 2, buf, buf, None) == -1
    assert L.mi355_attn_prefill_plan_probe(1, 10, 0, 4, 1, None, 4, 2, buf, buf, None) == -1
    assert L.mi355_attn_prefill_plan_probe(1, 10, 0, 4, 1, win, 4, 2, buf, buf, None) == 1
