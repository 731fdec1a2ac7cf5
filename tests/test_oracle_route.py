"""Pins of the oracle's tile router (oracle/mx_route.py) and of attn_mx's routed mode.

The routing rule is this build's own, so what is pinned is that the integer formulation computes what it says it
stands for (the ratio of score-magnitude bounds, evaluated independently in exact rational arithmetic), the
exemptions, the list layout handed to the kernel, and that routed attention equals the dense float64 attention on the
same map and reproduces the fixed modes on the maps that describe them."""
from fractions import Fraction

import numpy as np
import torch

import oracle as O
from oracle.mx_route import SKIP, FP4, FP8, NOT_VISITED
from conftest import make_qkv


def _random_scales(rng, B, H, N, nb, lo=118, hi=132):
    return rng.integers(lo, hi, size=(B, H, N, nb), dtype=np.uint8)


def _tiled_scales(rng, B, H, nt, tile, nb, lo, hi):
    """Scale bytes whose per-tile maxima are drawn uniformly from [lo, hi): rows lie 0..3 below their tile's maximum."""
    top = rng.integers(lo, hi, size=(B, H, nt, 1, nb))
    rows = top - rng.integers(0, 4, size=(B, H, nt, tile, nb))
    rows[:, :, :, 0, :] = top[:, :, :, 0, :]
    return rows.reshape(B, H, nt * tile, nb).astype(np.uint8)


def test_tile_scale_stats_against_loops():
    rng = np.random.default_rng(0)
    s = _random_scales(rng, 2, 3, 256, 4, 100, 130)
    m, f = O.tile_scale_stats(s, 64)
    for b in range(2):
        for h in range(3):
            for t in range(4):
                for c in range(4):
                    col = [int(s[b, h, 64 * t + r, c]) for r in range(64)]
                    assert m[b, h, t, c] == max(col)
                    assert f[b, h, t, c] == sum((1 << (10 - (max(col) - e))) if max(col) - e <= 10 else 0 for e in col)
    # 2^(M-10) * F is the exact sum of 2^e whenever no row lies more than 10 below the maximum
    s = _tiled_scales(rng, 1, 1, 3, 32, 2, 110, 130)
    m, f = O.tile_scale_stats(s, 32)
    for t in range(3):
        for c in range(2):
            exact = sum(Fraction(2) ** int(e) for e in s[0, 0, 32 * t:32 * t + 32, c])
            assert Fraction(2) ** int(m[0, 0, t, c] - 10) * int(f[0, 0, t, c]) == exact


def _exact_bound(sq, sk):
    """sum_c (sum over query rows of 2^e) * (sum over key rows of 2^e) as an exact integer: proportional to the summed
    magnitude bound sum_c sum_r sum_r' 32 * (6*2^(eq-127)) * (6*2^(ek-127)) of the tile's scores."""
    return sum(sum(1 << int(e) for e in sq[:, c]) * sum(1 << int(e) for e in sk[:, c]) for c in range(sq.shape[1]))


def test_route_follows_exact_bound_ratio():
    # rows within 3 of their tile's maximum and exponent sums within 12 of each other: nothing is dropped, only the
    # two floors act, so T/Tmax equals the exact bound ratio to ~1e-5; tiles nearer than 1e-3 to a threshold are not judged
    rng = np.random.default_rng(1)
    tile, group, nt = 32, 2, 6
    qs = _tiled_scales(rng, 1, 4, nt, tile, 4, 120, 126)
    ks = _tiled_scales(rng, 1, 2, nt, tile, 4, 120, 126)
    hi_t, lo_t = 0.5, 0.125
    for causal in (False, True):
        cls = O.route_tiles(qs, ks, tile, causal, hi_thresh=hi_t, skip_thresh=lo_t)
        seen, judged = set(), 0
        for h in range(4):
            for i in range(nt):
                last = i if causal else nt - 1
                bounds = [_exact_bound(qs[0, h, i * tile:(i + 1) * tile], ks[0, h // group, j * tile:(j + 1) * tile])
                          for j in range(last + 1)]
                bmax = max(bounds)
                for j in range(nt):
                    if j > last:
                        assert cls[0, h, i, j] == NOT_VISITED
                        continue
                    ratio = Fraction(bounds[j], bmax)
                    if min(abs(ratio - Fraction(hi_t)), abs(ratio - Fraction(lo_t))) < Fraction(1, 1000):
                        continue
                    if ratio >= Fraction(hi_t):
                        want = FP8
                    elif ratio < Fraction(lo_t) and j != 0 and not (causal and j == i):
                        want = SKIP
                    else:
                        want = FP4
                    assert cls[0, h, i, j] == want, (causal, h, i, j, float(ratio))
                    seen.add(want)
                    judged += 1
        assert {FP4, FP8, SKIP} <= seen and judged > 60


def test_route_hand_worked():
    # one head, D = 64 (two blocks), tile = 2 rows, three key tiles.  Query tile 0: rows [130,120],[100,100] ->
    # M = [130,120], F = [1024 + 0, 1024 + 0] (rows 30 and 20 below the maximum are dropped).
    qs = np.array([[130, 120], [100, 100]] * 3, dtype=np.uint8).reshape(1, 1, 6, 2)
    # key tiles: M = [130,120] / [126,130] / [110,141], each F = [1024,1024] except tile 1 block 0: rows 126 and 125
    # -> F = 1024 + 512
    ks = np.array([[130, 120], [1, 1], [126, 130], [125, 2], [110, 141], [3, 3]], dtype=np.uint8).reshape(1, 1, 6, 2)
    # s = [260,240] / [256,250] / [240,261]; smax = 261; w = 2^20 except tile 1 block 0: 1.5 * 2^20
    # T0 = (2^20 >> 1  + 2^20 >> 21) >> 13 = 64;  T1 = (1.5*2^20 >> 5 + 2^20 >> 11) >> 13 = (49152 + 512) >> 13 = 6
    # T2 = (2^20 >> 21 + 2^20) >> 13 = 128
    m, f = O.tile_scale_stats(ks, 2)
    assert f[0, 0].tolist() == [[1024, 1024], [1536, 1024], [1024, 1024]]
    cls = O.route_tiles(qs, ks, 2, False, hi_thresh=0.5, skip_thresh=0.05)
    assert cls[0, 0, 0].tolist() == [FP8, SKIP, FP8]          # T1/Tmax = 0.047 < 0.05
    cls = O.route_tiles(qs, ks, 2, False, hi_thresh=0.75, skip_thresh=0.04)
    assert cls[0, 0, 0].tolist() == [FP4, FP4, FP8]
    cls = O.route_tiles(qs, ks, 2, True, hi_thresh=0.75, skip_thresh=0.04)
    assert cls[0, 0, 0].tolist() == [FP8, NOT_VISITED, NOT_VISITED]


def test_route_exemptions_and_switches():
    rng = np.random.default_rng(2)
    qs = _tiled_scales(rng, 1, 2, 8, 16, 2, 100, 140)
    ks = _tiled_scales(rng, 1, 1, 8, 16, 2, 100, 140)
    off = O.route_tiles(qs, ks, 16, False, None, None)
    assert (off == FP4).all()
    for causal in (False, True):
        cls = O.route_tiles(qs, ks, 16, causal, hi_thresh=None, skip_thresh=1.0)    # everything below the max is skippable
        assert (cls[:, :, :, 0] != SKIP).all()                                       # the sink tile never is
        assert (cls == FP8).sum() == 0
        if causal:
            for i in range(8):
                assert (cls[:, :, i, i] == FP4).all()
                assert (cls[:, :, i, i + 1:] == NOT_VISITED).all()
        assert (cls == SKIP).sum() > 0
    # the largest tile of every row is 8-bit as soon as hi_thresh is on, whatever its value <= 1
    cls = O.route_tiles(qs, ks, 16, False, hi_thresh=1.0, skip_thresh=None)
    assert ((cls == FP8).sum(axis=3) >= 1).all()


def test_route_order_layout():
    rng = np.random.default_rng(3)
    tile, n_keys = 16, 7 * 16 + 5                      # ragged: the last key tile needs a mask
    cls = rng.choice(np.array([SKIP, FP4, FP8], dtype=np.uint8), size=(2, 3, 8, 8))
    for causal in (False, True):
        c = cls.copy()
        if causal:
            for i in range(8):
                c[:, :, i, i + 1:] = NOT_VISITED
        order, counts = O.route_order(c, n_keys, tile, causal)
        for b in range(2):
            for h in range(3):
                for i in range(8):
                    n4p, n4m, n8p, n8m = counts[b, h, i]
                    total = n4p + n4m + n8p + n8m
                    lst = order[b, h, i]
                    assert (lst[total:] == -1).all()
                    kept = [j for j in range(8) if c[b, h, i, j] in (FP4, FP8)]
                    assert sorted(lst[:total].tolist()) == kept
                    runs = (lst[:n4p], lst[n4p:n4p + n4m], lst[n4p + n4m:n4p + n4m + n8p], lst[n4p + n4m + n8p:total])
                    for k, run in enumerate(runs):
                        assert list(run) == sorted(run)
                        for j in run:
                            assert c[b, h, i, j] == (FP8 if k >= 2 else FP4)
                            assert ((causal and j == i) or j == 7) == bool(k & 1)


def test_routed_attention_against_dense_and_fixed_modes():
    q, k, v = make_qkv(1, 2, 1, 4 * 32 + 9, 64, seed=11)
    tile, nt = 32, 5
    rng = np.random.default_rng(4)
    for causal in (True, False):
        route = rng.choice(np.array([SKIP, FP4, FP8], dtype=np.uint8), size=(1, 2, nt, nt), p=[0.2, 0.4, 0.4])
        route[:, :, :, 0] = FP4
        for i in range(nt):
            route[:, :, i, i] = FP8
            if causal:
                route[:, :, i, i + 1:] = NOT_VISITED
        got = O.attn_mx(q, k, v, tile=tile, causal=causal, mode="routed", route=route, out_dtype=torch.float32)
        want = O.attn_dense_f64(q, k, v, tile=tile, causal=causal, mode="routed", route=route)
        m = O.precision_metric(got, want)
        assert m["cos"] > 0.99999 and m["max_abs"] < 2e-2, m            # 16-bit P only
        # the maps that describe the fixed modes reproduce them exactly
        visited = np.full((1, 2, nt, nt), FP4, dtype=np.uint8)
        if causal:
            for i in range(nt):
                visited[:, :, i, i + 1:] = NOT_VISITED
        assert torch.equal(O.attn_mx(q, k, v, tile=tile, causal=causal, mode="routed", route=visited),
                           O.attn_mx(q, k, v, tile=tile, causal=causal, mode="mxfp4"))
        diag = visited.copy()
        for i in range(nt):
            diag[:, :, i, i] = FP8
        assert torch.equal(O.attn_mx(q, k, v, tile=tile, causal=causal, mode="routed", route=diag),
                           O.attn_mx(q, k, v, tile=tile, causal=causal, mode="diag"))


def test_routed_attention_all_skipped_row_is_zero():
    q, k, v = make_qkv(1, 1, 1, 64, 64, seed=12)
    route = np.array([[[[FP4, FP4], [SKIP, SKIP]]]], dtype=np.uint8)
    out = O.attn_mx(q, k, v, tile=32, causal=False, mode="routed", route=route)
    assert (out[0, 0, 32:] == 0).all() and out[0, 0, :32].abs().max() > 0


def test_route_golden_vectors():
    """The committed vectors (tests/golden/route_vectors.npz, written by make_route_vectors.py) pin the rule."""
    import os
    d = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "route_vectors.npz"))
    for name in "abcde":
        tile, D, n_keys, causal = (int(x) for x in d[name + "_meta"])
        hi, lo = (float(x) for x in d[name + "_thresh"])
        cls = O.route_tiles(d[name + "_qs"], d[name + "_ks"], tile, bool(causal), hi, lo)
        order, counts = O.route_order(cls, n_keys, tile, bool(causal))
        assert np.array_equal(cls, d[name + "_cls"]), name
        assert np.array_equal(order, d[name + "_order"]), name
        assert np.array_equal(counts, d[name + "_counts"]), name

