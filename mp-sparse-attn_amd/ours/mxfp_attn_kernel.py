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
          "diag_e5": _lib.MODE_DIAG, "routed": _lib.MODE_ROUTED, "routed_e5": _lib.MODE_ROUTED,
          "mixed": _lib.MODE_MIXED, "mixed_e5": _lib.MODE_MIXED}


def q_fusable(q, k, tile, block_scale_type, is_causal):
    """True when the attention kernel can take this Q unquantized and quantize it itself (``mpsa_attn_fwd_q16``: the
    paired-tile kernel's shapes -- D = 128, tile = 128, every type but the routed ones; causal from two tiles on, unmasked
    from six tiles on, any length)."""
    mode = _MODES.get(block_scale_type)
    if mode not in (_lib.MODE_DIAG, _lib.MODE_MXFP4, _lib.MODE_MIXED, _lib.MODE_MXFP8) or q.shape[2] != k.shape[2]:
        return False
    B, Hq, N, D = q.shape
    return bool(_lib.lib().mpsa_attn_fwd_q16_supported(B, Hq, k.shape[1], N, D, tile, 1 if is_causal else 0, mode))


def prepare_operands(q, k, v, tile, block_scale_type, scale=None, smooth_k=False, reuse=None, fuse_q=False):
    """Quantize Q/K (K minus its mean over the sequence if ``smooth_k``) and repack V for one attention call.
    q ``[B,Hq,Nq,D]``, k/v ``[B,Hkv,Nk,D]`` of one 16-bit dtype.  Returns a dict of device tensors (rows padded to
    whole tiles) the launcher consumes.  ``reuse``: the dict a previous call returned for the same shapes, dtype, tile
    and type -- its buffers are written again instead of allocating new ones (a serving loop's steady state).
    ``fuse_q`` (only where :func:`q_fusable` says so): Q is left unquantized for ``mpsa_attn_fwd_q16``; only K and V are
    prepared."""
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
    key = (mode, fmt8, tile, tuple(q.shape), tuple(k.shape), q.dtype, v.dtype, q.device, bool(fuse_q))
    # smooth-K (ours/mxfp_attn_kernel.py:33-34): the mean over the sequence is subtracted inside the K quantizer
    kmean = seq_mean(k) if smooth_k else None
    q, k = _check_input(q), _check_input(k)
    dev = q.device
    if reuse is not None and reuse.get("key") == key:
        ops = reuse
        v_tiles = ops["v_tiles"]
    else:
        ops = {"mode": mode, "fmt8": fmt8, "tile": tile, "n": N, "q4": None, "qs4": None, "q8": None, "qs8": None,
               "k4": None, "ks4": None, "k8": None, "ks8": None, "key": key}
        need4, need8 = mode != _lib.MODE_MXFP8, mode != _lib.MODE_MXFP4
        u8 = lambda *shape: torch.empty(shape, dtype=torch.uint8, device=dev)
        if need4:
            if not fuse_q:
                ops["q4"], ops["qs4"] = u8(B, Hq, nq_pad, D // 2), u8(B, Hq, nq_pad, D // 32)
            ops["k4"], ops["ks4"] = u8(B, Hkv, n_pad, D // 2), u8(B, Hkv, n_pad, D // 32)
        if need8:
            if not fuse_q:
                ops["q8"], ops["qs8"] = u8(B, Hq, nq_pad, D), u8(B, Hq, nq_pad, D // 32)
            ops["k8"], ops["ks8"] = u8(B, Hkv, n_pad, D), u8(B, Hkv, n_pad, D // 32)
        v_tiles = torch.empty((B, Hkv, nt, tile * D), dtype=v.dtype, device=v.device)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mpsa_attn_prepare(
            _lib.ptr(None if fuse_q else q), _lib.strides4(q), _lib.ptr(k), _lib.strides4(k), _lib.ptr(v), _lib.strides4(v),
            _lib.dtype_id(q.dtype), B, Hq, Hkv, Nq, N, D, tile, mode, fmt8, pre, _lib.ptr(kmean),
            _lib.ptr(ops["q4"]), _lib.ptr(ops["qs4"]), _lib.ptr(ops["q8"]), _lib.ptr(ops["qs8"]),
            _lib.ptr(ops["k4"]), _lib.ptr(ops["ks4"]), _lib.ptr(ops["k8"]), _lib.ptr(ops["ks8"]),
            _lib.ptr(v_tiles), _lib.stream_ptr(dev)))
    ops["v_tiles"] = v_tiles
    ops["shape"] = (B, Hq, Hkv, Nq, N, D)
    ops["q_raw"], ops["pre"] = (q, pre) if fuse_q else (None, pre)
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


def skip_route(ops, is_causal, skip_thresh, skipped=None, want_cls=False):
    """The reference's tile-skipping rule decided ahead of the attention kernel (``mpsa_skip_route``): a score-product-only
    pass takes every tile's statistic, the rule turns them into the visiting lists ``mpsa_attn_fwd_routed`` walks.  Returns
    ``(cls or None, order, counts)``; ``skipped`` (int32 ``[B,Hq,ntq]``) receives the number of skipped key tiles per query
    tile.  Only where :func:`skip_routable` says so."""
    B, Hq, Hkv, Nq, N, D = ops["shape"]
    tile = ops["tile"]
    dev = ops["v_tiles"].device
    ntq, ntk = (Nq + tile - 1) // tile, (N + tile - 1) // tile
    with torch.cuda.device(dev):
        work = torch.empty(_lib.lib().mpsa_skip_route_workspace(B, Hq, Nq, N, tile), dtype=torch.uint8, device=dev)
        cls = torch.empty((B, Hq, ntq, ntk), dtype=torch.uint8, device=dev) if want_cls else None
        order = torch.empty((B, Hq, ntq, ntk), dtype=torch.int32, device=dev)
        counts = torch.empty((B, Hq, ntq, 4), dtype=torch.int32, device=dev)
        _lib.check(_lib.lib().mpsa_skip_route(
            _lib.ptr(ops["q4"]), _lib.ptr(ops["qs4"]), _lib.ptr(ops["q8"]), _lib.ptr(ops["qs8"]),
            _lib.ptr(ops["k4"]), _lib.ptr(ops["ks4"]), _lib.ptr(ops["k8"]), _lib.ptr(ops["ks8"]), ops["fmt8"],
            B, Hq, Hkv, Nq, N, D, tile, 1 if is_causal else 0, ops["mode"], float(skip_thresh),
            _lib.ptr(work), _lib.ptr(cls), _lib.ptr(order), _lib.ptr(counts), _lib.ptr(skipped), _lib.stream_ptr(dev)))
    return cls, order, counts


def skip_routable(ops, is_causal):
    """True when tile skipping can be decided ahead of the attention kernel for these operands (D = 128, tile = 128, the
    mxfp4 / mxfp8 / diag types, quantized Q)."""
    B, Hq, Hkv, Nq, N, D = ops["shape"]
    return ops.get("q_raw") is None and bool(_lib.lib().mpsa_skip_route_supported(Nq, N, D, ops["tile"], 1 if is_causal else 0, ops["mode"]))


def attention_from_operands(ops, out, is_causal, skip_thresh=None, skipped=None, route=None, skip_in_kernel=False):
    """Launch ``mpsa_attn_fwd`` on prepared operands; ``out`` is a ``[B,Hq,Nq,D]`` view (last dim contiguous).
    With ``skip_thresh`` the reference's tile skipping runs (``skipped``: optional int32 ``[B,Hq,nt]`` that receives the
    number of skipped key tiles per query tile): decided ahead of the attention kernel where :func:`skip_routable` says so
    (the attention kernel then visits the kept tiles only), inside the attention kernel otherwise or with
    ``skip_in_kernel`` (``mpsa_attn_fwd_skip``) -- same rule, same decisions.  Routed operands take ``route`` = the
    ``(cls, order, counts)`` of :func:`route_tiles`."""
    B, Hq, Hkv, Nq, N, D = ops["shape"]
    dev = out.device
    if skip_thresh is not None and not skip_in_kernel and ops["mode"] != _lib.MODE_ROUTED and skip_routable(ops, is_causal):
        _, order, counts = skip_route(ops, is_causal, skip_thresh, skipped)
        with torch.cuda.device(dev):
            _lib.check(_lib.lib().mpsa_attn_fwd_routed(
                _lib.ptr(ops["q4"]), _lib.ptr(ops["qs4"]), _lib.ptr(ops["q8"]), _lib.ptr(ops["qs8"]),
                _lib.ptr(ops["k4"]), _lib.ptr(ops["ks4"]), _lib.ptr(ops["k8"]), _lib.ptr(ops["ks8"]), ops["fmt8"],
                _lib.ptr(ops["v_tiles"]), _lib.dtype_id(ops["v_tiles"].dtype), _lib.ptr(out), _lib.dtype_id(out.dtype),
                _lib.strides4(out), B, Hq, Hkv, Nq, N, D, ops["tile"], 1 if is_causal else 0,
                _lib.ptr(order), _lib.ptr(counts), _lib.stream_ptr(dev)))
        return out
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
    if ops.get("q_raw") is not None:
        if skip_thresh is not None:
            raise ValueError("tile skipping needs quantized Q operands (prepare_operands without fuse_q)")
        q = ops["q_raw"]
        with torch.cuda.device(dev):
            _lib.check(_lib.lib().mpsa_attn_fwd_q16(
                _lib.ptr(q), _lib.strides4(q), _lib.dtype_id(q.dtype), ops["pre"],
                _lib.ptr(ops["k4"]), _lib.ptr(ops["ks4"]), _lib.ptr(ops["k8"]), _lib.ptr(ops["ks8"]), ops["fmt8"],
                _lib.ptr(ops["v_tiles"]), _lib.dtype_id(ops["v_tiles"].dtype), _lib.ptr(out), _lib.dtype_id(out.dtype),
                _lib.strides4(out), B, Hq, Hkv, N, D, ops["tile"], 1 if is_causal else 0, ops["mode"], _lib.stream_ptr(dev)))
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


def initialize_block_scaled_batched_from_tensor(a_tensor, b_tensor, a_scale, b_scale, block_scale_type="mxfp4", compute_reference=False):
    """Operand packaging of the fused attention with the reference's signature (ours/mxfp_attn_kernel.py:426-553).

    ``a_tensor [B,H,M,K]`` (Q) and ``b_tensor [B,Hkv,N,K]`` (K): uint8 codes as the quantizer leaves them (one E2M1
    code per byte, or FP8 bytes) or float values, which are cast element by element; ``a_scale`` / ``b_scale``:
    ``[B,H,rows/128,K/128,32,4,4]`` scale factors, uint8 E8M0 bytes (taken as they are, :505-506) or float (encoded
    with ``MXScaleTensor``).  4-bit codes are packed two per byte along K (the last dim).  Returns
    ``(a, a_scale, b, b_scale, configs, reference)``; ``reference`` is ``(None, None, None)``, or with
    ``compute_reference`` the reference's triple (:508-551): the float32 scores ``dq(A) @ dq(B)^T`` ``[B,H,M,N]`` (codes
    decoded, E8M0 bytes decoded and repeated over their 32 elements, ``torch.matmul``, all on the device) and the
    decoded codes of A and B without their scale factors, as the reference returns them."""
    from .block_scaled_matmul import _TYPES, _fmts_of, _package_operand, _package_scale, _expanded_scales, make_configs, VEC_SIZE
    if block_scale_type == "nvfp4":
        raise NotImplementedError("nvfp4 (16-element blocks, FP8 scale factors) is not available: the gfx950 scaled matrix "
                                  "instructions take one E8M0 scale per 32 elements")
    assert block_scale_type in _TYPES, f"Invalid block scale type: {block_scale_type}"
    B, H, M, K = a_tensor.shape
    B_b, H_b, N, K_b = b_tensor.shape
    assert B == B_b, f"batch sizes do not match: A.shape[0]={B} != B.shape[0]={B_b}"
    assert H % H_b == 0, f"head counts do not match: A.shape[1]={H}, B.shape[1]={H_b}"
    assert K == K_b, f"matrix dimensions do not match: A.shape[3]={K} != B.shape[3]={K_b}"
    expected_a = (B, H, M // 128, K // VEC_SIZE // 4, 32, 4, 4)
    expected_b = (B, H_b, N // 128, K // VEC_SIZE // 4, 32, 4, 4)
    assert tuple(a_scale.shape) == expected_a, f"a_scale shape mismatch: expected {expected_a}, got {tuple(a_scale.shape)}"
    assert tuple(b_scale.shape) == expected_b, f"b_scale shape mismatch: expected {expected_b}, got {tuple(b_scale.shape)}"
    configs = make_configs(block_scale_type)
    configs["BLOCK_SIZE_M"] = configs["BLOCK_SIZE_N"] = 128
    fmt_a, fmt_b = _fmts_of(configs)
    f8 = fmt_a if fmt_a != _lib.FMT_E2M1 else _lib.FMT_E4M3
    a, a_ref = _package_operand(a_tensor, fmt_a == _lib.FMT_E2M1, f8)
    b, b_ref = _package_operand(b_tensor, fmt_b == _lib.FMT_E2M1, f8)
    a_scale, b_scale = _package_scale(a_scale), _package_scale(b_scale)
    reference = (None, None, None)
    if compute_reference:
        a_dec, b_dec = a_ref(), b_ref()
        a_dq = a_dec * _expanded_scales(a_scale, K)
        b_dq = (b_dec * _expanded_scales(b_scale, K)).repeat_interleave(H // H_b, dim=1)     # grouped heads
        reference = (torch.matmul(a_dq, b_dq.transpose(-1, -2)), a_dec, b_dec)
    return a, a_scale, b, b_scale, configs, reference


def block_scaled_batched_attn(a_desc, a_scale, b_desc, b_scale, v_ori, dtype_dst, B, H, M, N, K, configs, STAGE=1, skip_thresh=None):
    """Fused attention on packaged operands -- the reference's launcher (ours/mxfp_attn_kernel.py:362-423).

    ``a_desc`` / ``b_desc``: Q ``[B,H,M,K']`` and K ``[B,Hkv,N,K']`` codes (``K' = K/2`` packed E2M1 or ``K`` FP8 bytes)
    with ``sm_scale*log2(e)`` already folded into Q; ``a_scale`` / ``b_scale``: E8M0 bytes, packed
    ``[B,H,rows/128,K/128,32,4,4]`` or linear ``[B,H,rows,K/32]``; ``v_ori [B,Hkv,N,K]`` bf16/fp16.  The precision comes
    from ``configs`` (``ELEM_PER_BYTE_A`` / ``_B``: 2,2 = mxfp4; 1,1 = mxfp8; 1,2 = mixed).  ``STAGE``: 1 = every key
    tile (what the reference's kernel does), 3 = causal.  Returns ``[B,H,M,K]`` of ``dtype_dst``."""
    from .block_scaled_matmul import _fmts_of, unpack_scale_5d
    if dtype_dst not in (torch.float32, torch.float16, torch.bfloat16):
        raise ValueError(f"Unsupported dtype: {dtype_dst}")            # ours/mxfp_attn_kernel.py:389
    if STAGE not in (1, 3):
        raise ValueError(f"STAGE must be 1 (all key tiles) or 3 (causal), got {STAGE}")
    _lib.require_device(a_desc, a_scale, b_desc, b_scale, v_ori)
    fmt_a, fmt_b = _fmts_of(configs)
    if fmt_a == _lib.FMT_E2M1 and fmt_b != _lib.FMT_E2M1:
        raise ValueError("a 4-bit Q with an 8-bit K is not a type of the reference (mixed is 8-bit Q x 4-bit K)")
    mode = _lib.MODE_MXFP4 if fmt_a == _lib.FMT_E2M1 else (_lib.MODE_MXFP8 if fmt_b != _lib.FMT_E2M1 else _lib.MODE_MIXED)
    fmt8 = fmt_a if fmt_a != _lib.FMT_E2M1 else _lib.FMT_E4M3
    Hkv = b_desc.shape[1]
    tile = 128
    assert M % tile == 0 and N % tile == 0, "M and N must be multiples of 128 (the packaged scale layout's chunk)"
    assert K in [64, 128], "headdim should be in [64, 128]."
    a_desc, b_desc = a_desc.view(torch.uint8).contiguous(), b_desc.view(torch.uint8).contiguous()
    if a_scale.dim() == 7:
        a_scale = unpack_scale_5d(a_scale)
    if b_scale.dim() == 7:
        b_scale = unpack_scale_5d(b_scale)
    a_scale, b_scale = a_scale.contiguous(), b_scale.contiguous()
    wa = K // 2 if fmt_a == _lib.FMT_E2M1 else K
    wb = K // 2 if fmt_b == _lib.FMT_E2M1 else K
    assert a_desc.shape == (B, H, M, wa) and b_desc.shape == (B, Hkv, N, wb), "operand shapes do not match B, H, M, N, K"
    assert a_scale.shape == (B, H, M, K // 32) and b_scale.shape == (B, Hkv, N, K // 32), "scale shapes do not match"
    assert v_ori.shape == (B, Hkv, N, K) and v_ori.dtype in (torch.float16, torch.bfloat16), "v must be [B,Hkv,N,K] bf16/fp16"
    if v_ori.stride(-1) != 1:
        v_ori = v_ori.contiguous()
    dev = a_desc.device
    v_tiles = torch.empty((B, Hkv, N // tile, tile * K), dtype=v_ori.dtype, device=dev)
    out = torch.empty((B, H, M, K), dtype=dtype_dst, device=dev)
    q4 = a_desc if fmt_a == _lib.FMT_E2M1 else None
    q8 = a_desc if fmt_a != _lib.FMT_E2M1 else None
    k4 = b_desc if fmt_b == _lib.FMT_E2M1 else None
    k8 = b_desc if fmt_b != _lib.FMT_E2M1 else None
    common = (_lib.ptr(q4), _lib.ptr(a_scale if q4 is not None else None), _lib.ptr(q8), _lib.ptr(a_scale if q8 is not None else None),
              _lib.ptr(k4), _lib.ptr(b_scale if k4 is not None else None), _lib.ptr(k8), _lib.ptr(b_scale if k8 is not None else None), fmt8,
              _lib.ptr(v_tiles), _lib.dtype_id(v_ori.dtype), _lib.ptr(out), _lib.dtype_id(dtype_dst), _lib.strides4(out),
              B, H, Hkv, M, N, K, tile, 1 if STAGE == 3 else 0, mode)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mpsa_v_tiles(_lib.ptr(v_ori), _lib.dtype_id(v_ori.dtype), B, Hkv, N, K, _lib.strides4(v_ori), tile,
                                           _lib.ptr(v_tiles), _lib.stream_ptr(dev)))
        if skip_thresh is not None:
            _lib.check(_lib.lib().mpsa_attn_fwd_skip(*common, float(skip_thresh), None, _lib.stream_ptr(dev)))
        else:
            _lib.check(_lib.lib().mpsa_attn_fwd(*common, _lib.stream_ptr(dev)))
    return out


def _normalise(q, k, v):
    """Reference prologue (ours/mxfp_attn_kernel.py:27-31): fp32/fp16 inputs run in fp16, everything else in
    bf16.  V follows Q/K's 16-bit dtype here (the reference always used fp16 for V)."""
    lp = torch.float16 if q.dtype in (torch.float32, torch.float16) else torch.bfloat16
    return q.to(lp), k.to(lp), v.to(lp)


def _reject_unsupported(attn_mask, dropout_p, attention_sink):
    if attn_mask is not None or dropout_p != 0.0 or attention_sink:
        raise NotImplementedError("attn_mask, dropout_p and attention_sink are not implemented "
                                  "(the reference accepts and ignores them)")


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
    skipping (ours/mxfp_attn_kernel.py:272-297; fixed-precision and diag types); ``return_sparsity`` adds the share of
    skipped tiles as a second result.

    ``block_scale_type="routed"`` (``"routed_e5"``): per-tile precision from the tile router -- a tile whose score
    bound (from the E8M0 bytes of Q and K) reaches ``route_thresh`` times the largest of its query tile runs in
    MXFP8, one below ``skip_thresh`` times it is skipped, the rest runs in MXFP4."""
    _lib.require_device(q, k, v)
    _reject_unsupported(attn_mask, dropout_p, attention_sink)
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
    # shapes of the paired-tile kernel: Q stays unquantized in HBM and the attention kernel quantizes it in registers
    fuse_q = skip_thresh is None and q.stride(-1) == 1 and q.dtype == v.dtype and q_fusable(q, k, tile, block_scale_type, is_causal)
    ops = prepare_operands(q, k, v, tile, block_scale_type, scale, smooth_k=smooth_k, fuse_q=fuse_q)
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
