"""Diagonal-tiled mixed-precision MXFP attention, restated on the CPU.

TEST INFRASTRUCTURE ONLY (see the package docstring).

Loop structure and numerics follow the reference's fused kernel
(``ours/mxfp_attn_kernel.py:216-359``: exp2 online softmax, float32 running max / sum, P summed
in float32 before the down-cast, low-precision P.V, ``acc / l`` epilogue); the causal
decomposition (tiles left of the diagonal unmasked, the diagonal tile masked ``row >= col``,
tiles right of it never visited) follows ``ours/online_routing.py:68-77, :113-118``; the
grouped-query head mapping follows ``ours/online_routing.py:160-171``.  The benchmark contract
adds per-tile precision: tile ``j == i`` uses the 8-bit operands, every other tile the 4-bit
ones.
"""

import torch
import torch.nn.functional as Fnn

from .mx_quantize import FMT_E2M1, FMT_E4M3, quantize_mx, dequantize_mx, q_pre_scale, smooth_k as _smooth_k

MODES = ("mxfp4", "mxfp8", "diag", "routed", "mixed")


def _tile_is_8bit(mode: str, i: int, j: int, route=None) -> bool:
    if mode == "routed":
        return int(route[i, j]) == 2
    if mode == "mxfp8":
        return True
    if mode == "mxfp4":
        return False
    if mode == "diag":
        return i == j
    raise ValueError(f"unknown block_scale_type {mode}")


def _tile_tags(mode: str, i: int, j: int, route=None):
    """(precision of the Q operand, of the K operand) for tile (i, j).  ``"mixed"`` is the reference's 8-bit Q against
    4-bit K on every tile (ELEM_PER_BYTE_A = 1, ELEM_PER_BYTE_B = 2: ours/mxfp_attn_kernel.py:264-269, :448-449)."""
    if mode == "mixed":
        return "8", "4"
    tag = "8" if _tile_is_8bit(mode, i, j, route) else "4"
    return tag, tag


def _prepare(q, k, mode, scale, fmt8):
    """Quantize + dequantize Q and K in the formats the mode needs (float32 fake-quant)."""
    D = q.shape[-1]
    pre = q_pre_scale(D, scale)
    ops = {}
    if mode in ("mxfp4", "diag", "routed"):
        ops["q4"] = dequantize_mx(*quantize_mx(q, pre, FMT_E2M1), FMT_E2M1)
    if mode in ("mxfp4", "diag", "routed", "mixed"):
        ops["k4"] = dequantize_mx(*quantize_mx(k, 1.0, FMT_E2M1), FMT_E2M1)
    if mode in ("mxfp8", "diag", "routed", "mixed"):
        ops["q8"] = dequantize_mx(*quantize_mx(q, pre, fmt8), fmt8)
    if mode in ("mxfp8", "diag", "routed"):
        ops["k8"] = dequantize_mx(*quantize_mx(k, 1.0, fmt8), fmt8)
    return ops


def attn_mx(q, k, v, tile=128, causal=True, mode="diag", scale=None, smooth_k=False,
            fmt8=FMT_E4M3, out_dtype=None, heads=None, q_tiles=None, skip_thresh=None, return_skipped=False,
            ratios_out=None, route=None, score8=None):
    """Tile-by-tile MXFP attention.  q ``[B,Hq,N,D]``, k/v ``[B,Hkv,N,D]`` in bf16 or fp16.

    P is rounded to v's dtype before P.V and the product of a tile is accumulated in float32
    (ours/mxfp_attn_kernel.py:339-340).  ``heads`` restricts the computation to a list of query
    heads (the output then has ``len(heads)`` heads).  N need not be a multiple of ``tile``:
    the last key tile is cut at N.  ``q_tiles`` restricts the computation to a list of query tiles (all
    keys are still visited); the output then holds only those tiles' rows, concatenated in list order.

    ``skip_thresh``: the reference's tile skipping (ours/mxfp_attn_kernel.py:272-297, with the pointer advance
    a skipped tile needs): the statistic of a score tile is the mean over its query rows of the row maximum; key
    tile 0 is always kept and sets the reference value, tile j > 0 is kept iff its statistic is at least
    ``skip_thresh`` times that; the diagonal tile of a causal run is always kept too (the reference's causal loop,
    ours/online_routing.py:68-77, walks it as a stage of its own whose first tile is exempt).  ``return_skipped`` adds an int32 ``[B, heads, tiles]`` count of skipped tiles;
    a list passed as ``ratios_out`` collects statistic(j) / statistic(0) of every tile j > 0 examined.

    ``mode="routed"``: ``route`` ``[B,Hq,tiles,key tiles]`` gives every tile's class (0 skip, 1 4-bit, 2 8-bit, 255 not
    visited), see :mod:`oracle.mx_route`; a query row whose every tile is skipped returns zeros.

    ``score8``: optional callable ``(q_tile, k_tile) -> scores`` that replaces the float32 product ``q_tile @ k_tile.T`` for
    tiles whose two operands are 8-bit -- the tests use it to put a model of a matrix unit's accumulation in place of the
    exact product; the default is the reference's arithmetic."""
    B, Hq, N, D = q.shape
    Hkv, Nk = k.shape[1], k.shape[2]
    assert Hq % Hkv == 0
    assert Nk == N or (not causal and mode != "diag"), "cross attention: non-causal, single precision"
    assert (mode == "routed") == (route is not None)
    group = Hq // Hkv
    if smooth_k:
        k = _smooth_k(k)
    lp = v.dtype
    assert lp in (torch.bfloat16, torch.float16)
    out_dtype = out_dtype or lp
    head_list = list(range(Hq)) if heads is None else list(heads)
    ops = _prepare(q[:, head_list], k, mode, scale, fmt8)
    vf = v.to(torch.float32)
    nt = (N + tile - 1) // tile
    ntk = (Nk + tile - 1) // tile
    tile_list = list(range(nt)) if q_tiles is None else list(q_tiles)
    starts, n_out = {}, 0
    for i in tile_list:
        starts[i] = n_out
        n_out += min((i + 1) * tile, N) - i * tile
    out = torch.empty((B, len(head_list), n_out, D), dtype=out_dtype)
    skipped = torch.zeros((B, len(head_list), len(tile_list)), dtype=torch.int32)
    for b in range(B):
        for hi_, h in enumerate(head_list):
            kvh = h // group
            for i in tile_list:
                r0, r1 = i * tile, min((i + 1) * tile, N)
                rows = r1 - r0
                m = torch.full((rows,), float("-inf"))
                l = torch.zeros((rows,))
                acc = torch.zeros((rows, D))
                last = i if causal else ntk - 1
                for j in range(last + 1):
                    c0, c1 = j * tile, min((j + 1) * tile, Nk)
                    if mode == "routed" and int(route[b, h, i, j]) not in (1, 2):
                        continue
                    qtag, ktag = _tile_tags(mode, i, j, None if route is None else route[b, h])
                    qt = ops["q" + qtag][b, hi_, r0:r1]
                    kt = ops["k" + ktag][b, kvh, c0:c1]
                    if score8 is not None and qtag == "8" and ktag == "8":
                        s = score8(qt, kt)
                    else:
                        s = qt @ kt.T                                # float32, already in log2 units
                    if causal and j == i:
                        rr = torch.arange(r0, r1).unsqueeze(1)
                        cc = torch.arange(c0, c1).unsqueeze(0)
                        s = torch.where(cc > rr, torch.tensor(float("-inf")), s)
                    if skip_thresh is not None:
                        stat = s.amax(dim=1).sum() / rows
                        if j == 0:
                            sink = stat
                        elif ratios_out is not None:
                            ratios_out.append(float(stat / sink))
                        exempt = j == 0 or (causal and j == i)       # ours/online_routing.py:68-77: the diagonal stage's first tile
                        if not exempt and not bool(stat >= sink * skip_thresh):
                            skipped[b, hi_, tile_list.index(i)] += 1
                            continue
                    m_new = torch.maximum(m, s.amax(dim=1))
                    p = torch.exp2(s - m_new.unsqueeze(1))
                    alpha = torch.exp2(m - m_new)
                    l = l * alpha + p.sum(dim=1)
                    pv = p.to(lp).to(torch.float32) @ vf[b, kvh, c0:c1]
                    acc = acc * alpha.unsqueeze(1) + pv
                    m = m_new
                if mode == "routed":
                    acc = torch.where(l.unsqueeze(1) > 0, acc, torch.zeros(()))
                    l = torch.where(l > 0, l, torch.ones(()))
                out[b, hi_, starts[i]:starts[i] + rows] = (acc / l.unsqueeze(1)).to(out_dtype)
    if return_skipped:
        return out, skipped
    return out


def attn_dense_f64(q, k, v, tile=128, causal=True, mode="diag", scale=None, smooth_k=False,
                   fmt8=FMT_E4M3, heads=None, route=None) -> torch.Tensor:
    """Brute-force check of :func:`attn_mx`: the full score matrix is assembled tile by tile from
    the per-tile-precision dequantised operands, then a dense base-2 softmax and P.V in float64
    (no online rescaling, no low-precision P)."""
    B, Hq, N, D = q.shape
    Hkv = k.shape[1]
    group = Hq // Hkv
    if smooth_k:
        k = _smooth_k(k)
    head_list = list(range(Hq)) if heads is None else list(heads)
    ops = {n: t.double() for n, t in _prepare(q[:, head_list], k, mode, scale, fmt8).items()}
    nt = (N + tile - 1) // tile
    out = torch.empty((B, len(head_list), N, D), dtype=torch.float64)
    for b in range(B):
        for hi_, h in enumerate(head_list):
            kvh = h // group
            s = torch.full((N, N), float("-inf"), dtype=torch.float64)
            for i in range(nt):
                for j in range((i if causal else nt - 1) + 1):
                    if mode == "routed" and int(route[b, h, i, j]) not in (1, 2):
                        continue                                     # skipped: the tile's scores stay -inf
                    qtag, ktag = _tile_tags(mode, i, j, None if route is None else route[b, h])
                    r = slice(i * tile, min((i + 1) * tile, N))
                    c = slice(j * tile, min((j + 1) * tile, N))
                    s[r, c] = ops["q" + qtag][b, hi_, r] @ ops["k" + ktag][b, kvh, c].T
            if causal:
                s = s.masked_fill(torch.ones(N, N, dtype=torch.bool).triu(1), float("-inf"))
            p = torch.exp2(s - s.amax(dim=1, keepdim=True))
            out[b, hi_] = (p / p.sum(dim=1, keepdim=True)) @ v[b, kvh].double()
    return out


def precision_metric(x: torch.Tensor, ref: torch.Tensor) -> dict:
    """Cosine similarity over the flattened tensors, relative L1, RMSE and max-abs error.
    Definition of the first three: spas_sage_attn/utils.py:25-36."""
    a, b = x.double().reshape(1, -1), ref.double().reshape(1, -1)
    return {
        "cos": Fnn.cosine_similarity(a, b).item(),
        "l1": ((a - b).abs().sum() / b.abs().sum()).item(),
        "rmse": torch.sqrt(torch.mean((a - b) ** 2)).item(),
        "max_abs": (a - b).abs().max().item(),
    }


def v_fragment_order(v: torch.Tensor, tile: int) -> torch.Tensor:
    """Value-tile layout the HIP attention kernel consumes, restated for checking the repack kernel.

    v ``[B,H,N,D]`` -> ``[B,H,Npad/tile, tile/32, 2, D/32, 64, 8]`` with
    ``out[.., kb, c, db, lane, t] = v[key, dim]`` where ``lane = 32*h + r``, ``dim = 32*db + r`` and
    ``key = tile*it + 32*kb + 16*c + 8*(t//4) + 4*h + t%4``; keys past N read as zero.  (This is the
    build's own operand layout, not a reference format: it lets a 64-lane wave fetch one
    32x16 value block for the matrix core with a single 16-byte load per lane.)"""
    B, H, N, D = v.shape
    nt = (N + tile - 1) // tile
    vp = torch.zeros((B, H, nt * tile, D), dtype=v.dtype)
    vp[:, :, :N] = v
    # key index decomposition: key = tile*it + 32*kb + 16*c + 8*t1 + 4*h + t0
    x = vp.reshape(B, H, nt, tile // 32, 2, 2, 2, 4, D // 32, 32)    # it kb c t1 h t0 db r
    x = x.permute(0, 1, 2, 3, 4, 8, 6, 9, 5, 7)                       # it kb c db h r t1 t0
    return x.reshape(B, H, nt, tile // 32, 2, D // 32, 64, 8).contiguous()
