"""Per-tile precision routing from the E8M0 scale bytes, restated on the CPU.

TEST INFRASTRUCTURE ONLY (see the package docstring).

The reference's online routing is a keep / skip test per score tile (``ours/online_routing.py:87-112``: a tile is
kept iff its statistic reaches ``skip_thresh`` times the reference tile's).  The benchmark contract extends it to a
precision choice (8-bit, 4-bit or skip per tile) taken from per-block absolute maxima of Q and K -- which the MX
quantizer has already produced: the E8M0 byte of a block is ``floor(log2(amax)) - emax_elem + 127``.  The rule is this
build's own (the reference has no precision router), stated here in integers so that every implementation gives the
same map:

* per tile (of Q: query tile I, of K: key tile J) and per 32-wide block c of the head dimension, over the tile's rows
  r of the padded scale array (padding rows carry byte 0): ``M[c] = max_r e[r][c]`` and
  ``F[c] = sum_r 2^(10 - (M[c] - e[r][c]))`` with terms below 1 dropped -- ``2^(M-137) * F`` is the sum over the rows of
  ``2^(e-127)``, i.e. (up to the constant 6) of the rows' magnitude bounds in that block;
* ``s[c] = Mq[I][c] + Mk[J][c]``, ``w[c] = Fq[I][c] * Fk[J][c]``; ``smax[I]`` = largest ``s[c]`` over the visited key
  tiles and all c;
* ``T[I][J] = floor(sum_c floor(w[c] / 2^(smax[I] - s[c])) / 2^13)`` (shifts above 40 give 0): proportional to
  ``sum_c (sum over query rows of their bound) * (sum over key rows of their bound)``, i.e. to the summed magnitude
  bound of the tile's scores -- and so to the absolute error a 4-bit product makes there; it fits 24 bits;
* with ``Tmax[I]`` the largest ``T[I][J]``: a tile is 8-bit if ``float32(T) >= hi_thresh * float32(Tmax)``;
  otherwise it is skipped if ``float32(T) < skip_thresh * float32(Tmax)`` unless it is key tile 0 (the reference's
  always-kept "sink" tile) or the diagonal tile of a causal run; otherwise 4-bit.  A threshold <= 0 switches its
  class off.  Causal runs visit key tiles J <= I only; the others are marked NOT_VISITED.
"""

import numpy as np

SKIP, FP4, FP8, NOT_VISITED = 0, 1, 2, 255
ROW_BITS, OUT_SHIFT, MAX_SHIFT = 10, 13, 40


def tile_scale_stats(scales, tile):
    """scales ``[B,H,Npad,D/32]`` uint8 (Npad a multiple of ``tile``) -> ``(M, F)``, each ``[B,H,Npad/tile,D/32]`` int64."""
    s = np.asarray(scales).astype(np.int64)
    B, H, Np, nb = s.shape
    assert Np % tile == 0
    s = s.reshape(B, H, Np // tile, tile, nb)
    m = s.max(axis=3)
    d = m[:, :, :, None, :] - s
    f = np.where(d <= ROW_BITS, 1 << np.clip(ROW_BITS - d, 0, ROW_BITS), 0).sum(axis=3)
    return m, f


def tile_statistic(mq, fq, mk, fk, smax):
    """T of one query tile (``mq``, ``fq``: ``[nb]``) against key tiles (``mk``, ``fk``: ``[J, nb]``)."""
    d = smax - (mq[None, :] + mk)
    w = fq[None, :] * fk
    return (np.where(d <= MAX_SHIFT, w >> np.clip(d, 0, MAX_SHIFT), 0).sum(axis=1)) >> OUT_SHIFT


def route_tiles(qs4, ks4, tile, causal, hi_thresh, skip_thresh):
    """Class map ``[B,Hq,ntq,ntk]`` uint8 from the padded 4-bit scale bytes of Q ``[B,Hq,Nq_pad,D/32]`` and K
    ``[B,Hkv,Nk_pad,D/32]``."""
    mq, fq = tile_scale_stats(qs4, tile)
    mk, fk = tile_scale_stats(ks4, tile)
    B, Hq, ntq, nb = mq.shape
    Hkv, ntk = mk.shape[1], mk.shape[2]
    group = Hq // Hkv
    hi = np.float32(0.0 if hi_thresh is None else hi_thresh)
    lo = np.float32(0.0 if skip_thresh is None else skip_thresh)
    cls = np.full((B, Hq, ntq, ntk), NOT_VISITED, dtype=np.uint8)
    for b in range(B):
        for h in range(Hq):
            for i in range(ntq):
                last = i if causal else ntk - 1
                mkj, fkj = mk[b, h // group, :last + 1], fk[b, h // group, :last + 1]
                smax = (mq[b, h, i][None, :] + mkj).max()
                t = tile_statistic(mq[b, h, i], fq[b, h, i], mkj, fkj, smax)
                tf = t.astype(np.float32)
                tmax = np.float32(t.max())
                row = np.full(last + 1, FP4, dtype=np.uint8)
                if lo > 0:
                    skip = tf < lo * tmax
                    skip[0] = False
                    if causal:
                        skip[i] = False
                    row[skip] = SKIP
                if hi > 0:
                    row[tf >= hi * tmax] = FP8
                cls[b, h, i, :last + 1] = row
    return cls


def route_order(cls, n_keys, tile, causal):
    """The visiting lists the attention kernel consumes: ``order[B,Hq,ntq,ntk]`` int32 holds, per query tile, the
    4-bit key tiles that need no mask (ascending), the 4-bit ones that do, then the 8-bit ones likewise; the rest is
    -1.  ``counts[B,Hq,ntq,4]`` = lengths of the four runs.  A tile needs a mask if it is the diagonal tile of a
    causal run or holds the end of a sequence that is not a whole number of tiles."""
    B, Hq, ntq, ntk = cls.shape
    order = np.full((B, Hq, ntq, ntk), -1, dtype=np.int32)
    counts = np.zeros((B, Hq, ntq, 4), dtype=np.int32)
    ragged = n_keys % tile != 0
    for b in range(B):
        for h in range(Hq):
            for i in range(ntq):
                runs = [[], [], [], []]
                for j in range(ntk):
                    c = cls[b, h, i, j]
                    if c not in (FP4, FP8):
                        continue
                    masked = (causal and j == i) or (ragged and j == ntk - 1)
                    runs[(2 if c == FP8 else 0) + (1 if masked else 0)].append(j)
                flat = [j for r in runs for j in r]
                order[b, h, i, :len(flat)] = flat
                counts[b, h, i] = [len(r) for r in runs]
    return order, counts
