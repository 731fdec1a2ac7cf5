"""Fused MXFP attention -- the reference's ``ours/mxfp_attn_kernel.py::mxfp_attn_kernel`` on HIP kernels.

Pipeline per call (all on torch's current stream, no host synchronisation):
  1. MX-quantize Q (with ``scale*log2e`` folded in) and K, repack V into matrix-core operand order -- one launch,
     ``mpsa_attn_prepare`` (preceded by ``mpsa_seq_mean`` when ``smooth_k``);
  2. fused attention -- ``mpsa_attn_fwd`` / ``mpsa_attn_fwd_skip``; for ``block_scale_type="routed"`` the tile router
     (``mpsa_route_tiles``, integer work on the scale bytes) followed by ``mpsa_attn_fwd_routed``.
"""

import torch

from . import _lib
from .quant_mxint8 import seq_mean, pre_scale_q, _as_bhnd, _check_input

_MODES = {"mxfp4": _lib.MODE_MXFP4, "mxfp8": _lib.MODE_MXFP8, "mxfp8e5": _lib.MODE_MXFP8, "diag": _lib.MODE_DIAG,
          "diag_e5": _lib.MODE_DIAG, "routed": _lib.MODE_ROUTED, "routed_e5": _lib.MODE_ROUTED}


def prepare_operands(q, k, v, tile, block_scale_type, scale=None, smooth_k=False):
    """Quantize Q/K (K minus its mean over the sequence if ``smooth_k``) and repack V for one attention call.
    q ``[B,Hq,Nq,D]``, k/v ``[B,Hkv,Nk,D]`` of one 16-bit dtype.  Returns a dict of device tensors (rows padded to
    whole tiles) the launcher consumes."""
    if block_scale_type not in _MODES:
        raise ValueError(f"Invalid block scale type: {block_scale_type}")
    mode = _MODES[block_scale_type]
    fmt8 = _lib.FMT_E5M2 if block_scale_type.endswith("e5") else _lib.FMT_E4M3
    B, Hq, Nq, D = q.shape
    Hkv, N = k.shape[1], k.shape[2]
    nt = (N + tile - 1) // tile
    n_pad = nt * tile
    nq_pad = (Nq + tile - 1) // tile * tile
    pre = pre_scale_q(D, scale)
    ops = {"mode": mode, "fmt8": fmt8, "tile": tile, "n": N, "q4": None, "qs4": None, "q8": None, "qs8": None,
           "k4": None, "ks4": None, "k8": None, "ks8": None}
    # smooth-K (ours/mxfp_attn_kernel.py:33-34): the mean over the sequence is subtracted inside the K quantizer
    kmean = seq_mean(k) if smooth_k else None
    q, k = _check_input(q), _check_input(k)
    dev = q.device
    need4, need8 = mode != _lib.MODE_MXFP8, mode != _lib.MODE_MXFP4
    u8 = lambda *shape: torch.empty(shape, dtype=torch.uint8, device=dev)
    if need4:
        ops["q4"], ops["qs4"] = u8(B, Hq, nq_pad, D // 2), u8(B, Hq, nq_pad, D // 32)
        ops["k4"], ops["ks4"] = u8(B, Hkv, n_pad, D // 2), u8(B, Hkv, n_pad, D // 32)
    if need8:
        ops["q8"], ops["qs8"] = u8(B, Hq, nq_pad, D), u8(B, Hq, nq_pad, D // 32)
        ops["k8"], ops["ks8"] = u8(B, Hkv, n_pad, D), u8(B, Hkv, n_pad, D // 32)
    v_tiles = torch.empty((B, Hkv, nt, tile * D), dtype=v.dtype, device=v.device)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mpsa_attn_prepare(
            _lib.ptr(q), _lib.strides4(q), _lib.ptr(k), _lib.strides4(k), _lib.ptr(v), _lib.strides4(v),
            _lib.dtype_id(q.dtype), B, Hq, Hkv, Nq, N, D, tile, mode, fmt8, pre, _lib.ptr(kmean),
            _lib.ptr(ops["q4"]), _lib.ptr(ops["qs4"]), _lib.ptr(ops["q8"]), _lib.ptr(ops["qs8"]),
            _lib.ptr(ops["k4"]), _lib.ptr(ops["ks4"]), _lib.ptr(ops["k8"]), _lib.ptr(ops["ks8"]),
            _lib.ptr(v_tiles), _lib.stream_ptr(dev)))
    ops["v_tiles"] = v_tiles
    ops["shape"] = (B, Hq, Hkv, Nq, N, D)
    return ops


def route_tiles(ops, is_causal, route_thresh=None, skip_thresh=None):
    """Run the tile router on prepared operands.  Returns ``(cls, order, counts)``: the uint8 class map
    ``[B,Hq,ntq,ntk]`` (0 skipped, 1 4-bit, 2 8-bit, 255 not visited) and the visiting lists
    ``mpsa_attn_fwd_routed`` walks.  ``route_thresh`` / ``skip_thresh``: a tile whose score bound reaches
    ``route_thresh`` times the largest of its query tile runs in 8-bit, one below ``skip_thresh`` times it is skipped
    (None switches the class off)."""
    B, Hq, Hkv, Nq, N, D = ops["shape"]
    tile = ops["tile"]
    dev = ops["qs4"].device
    ntq, ntk = (Nq + tile - 1) // tile, (N + tile - 1) // tile
    with torch.cuda.device(dev):
        work = torch.empty(_lib.lib().mpsa_route_workspace(B, Hq, Hkv, Nq, N, D, tile), dtype=torch.uint8, device=dev)
        cls = torch.empty((B, Hq, ntq, ntk), dtype=torch.uint8, device=dev)
        order = torch.empty((B, Hq, ntq, ntk), dtype=torch.int32, device=dev)
        counts = torch.empty((B, Hq, ntq, 4), dtype=torch.int32, device=dev)
        _lib.check(_lib.lib().mpsa_route_tiles(
            _lib.ptr(ops["qs4"]), _lib.ptr(ops["ks4"]), B, Hq, Hkv, Nq, N, D, tile, 1 if is_causal else 0,
            0.0 if route_thresh is None else float(route_thresh), 0.0 if skip_thresh is None else float(skip_thresh),
            _lib.ptr(work), _lib.ptr(cls), _lib.ptr(order), _lib.ptr(counts), _lib.stream_ptr(dev)))
    return cls, order, counts


def attention_from_operands(ops, out, is_causal, skip_thresh=None, skipped=None, route=None):
    """Launch ``mpsa_attn_fwd`` on prepared operands; ``out`` is a ``[B,Hq,Nq,D]`` view (last dim contiguous).
    With ``skip_thresh`` the tile-skipping entry point runs instead (``skipped``: optional int32 ``[B,Hq,nt]``
    that receives the number of skipped key tiles per query tile).  Routed operands take ``route`` = the
    ``(cls, order, counts)`` of :func:`route_tiles`."""
    B, Hq, Hkv, Nq, N, D = ops["shape"]
    dev = out.device
    if ops["mode"] == _lib.MODE_ROUTED:
        if route is None:
            raise ValueError("routed operands need route=(cls, order, counts) from route_tiles()")
        _, order, counts = route
        with torch.cuda.device(dev):
            _lib.check(_lib.lib().mpsa_attn_fwd_routed(
                _lib.ptr(ops["q4"]), _lib.ptr(ops["qs4"]), _lib.ptr(ops["q8"]), _lib.ptr(ops["qs8"]),
                _lib.ptr(ops["k4"]), _lib.ptr(ops["ks4"]), _lib.ptr(ops["k8"]), _lib.ptr(ops["ks8"]), ops["fmt8"],
                _lib.ptr(ops["v_tiles"]), _lib.dtype_id(ops["v_tiles"].dtype), _lib.ptr(out), _lib.dtype_id(out.dtype),
                _lib.strides4(out), B, Hq, Hkv, Nq, N, D, ops["tile"], 1 if is_causal else 0,
                _lib.ptr(order), _lib.ptr(counts), _lib.stream_ptr(dev)))
        return out
    if skip_thresh is not None:
        with torch.cuda.device(dev):
            _lib.check(_lib.lib().mpsa_attn_fwd_skip(
                _lib.ptr(ops["q4"]), _lib.ptr(ops["qs4"]), _lib.ptr(ops["q8"]), _lib.ptr(ops["qs8"]),
                _lib.ptr(ops["k4"]), _lib.ptr(ops["ks4"]), _lib.ptr(ops["k8"]), _lib.ptr(ops["ks8"]), ops["fmt8"],
                _lib.ptr(ops["v_tiles"]), _lib.dtype_id(ops["v_tiles"].dtype), _lib.ptr(out), _lib.dtype_id(out.dtype),
                _lib.strides4(out), B, Hq, Hkv, Nq, N, D, ops["tile"], 1 if is_causal else 0, ops["mode"],
                float(skip_thresh), _lib.ptr(skipped), _lib.stream_ptr(dev)))
        return out
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mpsa_attn_fwd(
            _lib.ptr(ops["q4"]), _lib.ptr(ops["qs4"]), _lib.ptr(ops["q8"]), _lib.ptr(ops["qs8"]),
            _lib.ptr(ops["k4"]), _lib.ptr(ops["ks4"]), _lib.ptr(ops["k8"]), _lib.ptr(ops["ks8"]), ops["fmt8"],
            _lib.ptr(ops["v_tiles"]), _lib.dtype_id(ops["v_tiles"].dtype), _lib.ptr(out), _lib.dtype_id(out.dtype),
            _lib.strides4(out), B, Hq, Hkv, Nq, N, D, ops["tile"], 1 if is_causal else 0, ops["mode"],
            _lib.stream_ptr(dev)))
    return out


def _normalise(q, k, v):
    """Reference prologue (ours/mxfp_attn_kernel.py:27-31): fp32/fp16 inputs run in fp16, everything else in
    bf16.  V follows Q/K's 16-bit dtype here (the reference always used fp16 for V)."""
    lp = torch.float16 if q.dtype in (torch.float32, torch.float16) else torch.bfloat16
    return q.to(lp), k.to(lp), v.to(lp)


def _reject_unsupported(attn_mask, dropout_p, attention_sink, block_scale_type, skip_thresh):
    if attn_mask is not None or dropout_p != 0.0 or attention_sink:
        raise NotImplementedError("attn_mask, dropout_p and attention_sink are not implemented "
                                  "(the reference accepts and ignores them)")
    if skip_thresh is not None and block_scale_type in _MODES and _MODES[block_scale_type] == _lib.MODE_DIAG:
        raise NotImplementedError("tile skipping (skip_thresh) needs a single-precision block_scale_type "
                                  "(mxfp4, mxfp8, mxfp8e5): its reference tile is the first key tile; "
                                  "\"routed\" skips by its own statistic")


@torch.compiler.disable
def mxfp_attn_kernel(q, k, v, attn_mask=None, dropout_p=0.0,
                     is_causal=False, scale=None, smooth_k=False, attention_sink=False, tensor_layout="HND",
                     output_dtype=torch.float16, return_sparsity=False, block_scale_type="mxfp4", skip_thresh=None,
                     tile=128, route_thresh=None):
    """Attention output ``[B,Hq,N,D]`` (``"NHD"``: ``[B,N,Hq,D]``) from MX-quantized Q.K^T and 16-bit P.V.

    Signature of the reference (ours/mxfp_attn_kernel.py:19-22) plus ``tile`` (score tile edge, 64 or 128).
    ``block_scale_type``: ``"mxfp4"``, ``"mxfp8"`` (E4M3), ``"mxfp8e5"`` (E5M2, the reference's 8-bit format),
    ``"diag"`` (tile j == i in MXFP8, the rest in MXFP4) or ``"diag_e5"``.  K/V may have fewer heads than Q
    (grouped-query attention); ``is_causal`` is honoured.  ``skip_thresh`` switches on the reference's tile
    skipping (ours/mxfp_attn_kernel.py:272-297; single-precision types only); ``return_sparsity`` adds the share of
    skipped tiles as a second result.

    ``block_scale_type="routed"`` (``"routed_e5"``): per-tile precision from the tile router -- a tile whose score
    bound (from the E8M0 bytes of Q and K) reaches ``route_thresh`` times the largest of its query tile runs in
    MXFP8, one below ``skip_thresh`` times it is skipped, the rest runs in MXFP4."""
    _lib.require_device(q, k, v)
    _reject_unsupported(attn_mask, dropout_p, attention_sink, block_scale_type, skip_thresh)
    torch.cuda.set_device(v.device)
    q, k, v = _normalise(q, k, v)
    q, k, v = _as_bhnd(q, tensor_layout), _as_bhnd(k, tensor_layout), _as_bhnd(v, tensor_layout)
    B, Hq, N, D = q.shape
    assert D in [64, 128], "headdim should be in [64, 128]."
    Nk = k.shape[2]
    assert v.shape[2] == Nk, "k and v must have the same sequence length"
    if Nk != N:                      # cross attention: the reference's kernel takes M and N apart as well
        assert not is_causal, "causal masking needs q and k of the same sequence length"
        assert _MODES.get(block_scale_type) != _lib.MODE_DIAG, "the diag types need q and k of the same sequence length"
    assert k.shape[1] == v.shape[1] and Hq % k.shape[1] == 0, "query heads must be a multiple of key/value heads"
    assert tile in (64, 128), "tile must be 64 or 128"
    if output_dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise ValueError(f"Unsupported dtype: {output_dtype}")       # ours/mxfp_attn_kernel.py:389
    if v.stride(-1) != 1:
        v = v.contiguous()
    ops = prepare_operands(q, k, v, tile, block_scale_type, scale, smooth_k=smooth_k)
    nt, ntk = (N + tile - 1) // tile, (Nk + tile - 1) // tile       # query tiles, key tiles
    skipped = None
    routed = ops["mode"] == _lib.MODE_ROUTED
    route = route_tiles(ops, is_causal, route_thresh, skip_thresh) if routed else None
    if routed:
        skip_thresh = None
    elif route_thresh is not None:
        raise ValueError("route_thresh needs block_scale_type=\"routed\"")
    if skip_thresh is not None and return_sparsity:
        skipped = torch.zeros((B, Hq, nt), dtype=torch.int32, device=q.device)
    if tensor_layout == "HND":
        out = torch.empty((B, Hq, N, D), dtype=output_dtype, device=q.device)
        attention_from_operands(ops, out, is_causal, skip_thresh, skipped, route)
    else:
        out = torch.empty((B, N, Hq, D), dtype=output_dtype, device=q.device)
        attention_from_operands(ops, out.transpose(1, 2), is_causal, skip_thresh, skipped, route)
    if not return_sparsity:
        return out
    # share of the visited (query tile, key tile) pairs that were skipped
    visited = B * Hq * (nt * (nt + 1) // 2 if is_causal else nt * ntk)
    if routed:
        return out, (route[0] == 0).sum().to(torch.float32) / visited
    if skipped is None:
        return out, torch.zeros((), dtype=torch.float32, device=q.device)
    return out, skipped.sum().to(torch.float32) / visited
