"""MX quantizer entry points -- the reference's ``ours/quant_mxint8.py`` surface on HIP kernels.

``quant_mxfp4`` / ``quant_mxfp8e5`` keep the reference signatures (ours/quant_mxint8.py:453, :223);
``quant_mxfp8`` is the E4M3 sibling the benchmark contract asks for.  Differences from the
reference, all deliberate:

  * E2M1 codes come back nibble-packed along the head dim (``[..., D/2]``; even element in the low
    nibble) instead of one code per byte -- pass ``packed=False`` for the reference's layout;
  * E2M1 rounding is round-to-nearest-even as in ``MXFP4Tensor._from_float`` (ours/mxfp.py:84-170),
    not the threshold rule of the Triton kernel (ours/quant_mxint8.py:318-331);
  * ``floor(log2(amax))`` is exact (exponent bits); an all-zero block gets scale byte 0, codes 0.

Scales are linear ``[B, H, L, D/32]`` uint8 (E8M0), as in the reference.
"""

import torch

from . import _lib
from .mxfp import MXFP4Tensor

LOG2E = 1.44269504          # ours/quant_mxint8.py:494
EMAX_E2M1 = 3               # ours/quant_mxint8.py:303
EMAX_8BIT = 7               # ours/quant_mxint8.py:191


def _as_bhnd(x, tensor_layout):
    """View x as [B,H,L,D] without copying (reference: stride juggling at ours/quant_mxint8.py:458-474)."""
    if tensor_layout == "HND":
        return x
    if tensor_layout == "NHD":
        return x.transpose(1, 2)
    raise ValueError(f"Unknown tensor layout: {tensor_layout}")


def _check_input(x):
    _lib.require_device(x)
    if x.dim() != 4:
        raise ValueError("expected a 4-D tensor")
    if x.dtype not in (torch.bfloat16, torch.float16):
        raise ValueError(f"the quantizer takes bf16 or fp16, got {x.dtype}")
    if x.stride(-1) != 1 or any(s % 8 for s in x.stride()[:3]) or x.data_ptr() % 16:
        x = x.contiguous()
    return x


def pre_scale_q(head_dim, sm_scale=None):
    """``sm_scale * 1.44269504`` as float32 (ours/quant_mxint8.py:479-480, :494)."""
    if sm_scale is None:
        sm_scale = head_dim ** -0.5
    return float(torch.tensor(sm_scale * LOG2E, dtype=torch.float32).item())


def seq_mean(x):
    """``x.mean(dim=-2)`` of a ``[B,H,L,D]`` bf16/fp16 tensor -> ``[B,H,D]`` in x's dtype, through ``mpsa_seq_mean``
    (float32 sum in a fixed order, times float32 ``1/L``, rounded once).  The mean the smooth-K prologue subtracts
    (ours/mxfp_attn.py:44-45); pass it as ``sub`` to the quantizers."""
    x = _check_input(x)
    B, H, L, D = x.shape
    mean = torch.empty((B, H, D), dtype=x.dtype, device=x.device)
    nbytes = _lib.lib().mpsa_seq_mean_workspace(B, H, L, D)
    work = torch.empty((max(nbytes // 4, 1),), dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().mpsa_seq_mean(_lib.ptr(x), _lib.dtype_id(x.dtype), B, H, L, D, _lib.strides4(x),
                                            _lib.ptr(work), _lib.ptr(mean), _lib.stream_ptr(x.device)))
    return mean


def _sub_ptr(sub, x):
    if sub is None:
        return None
    B, H, _, D = x.shape
    assert sub.shape == (B, H, D) and sub.dtype == x.dtype and sub.device == x.device, "sub must be [B,H,D] of x's dtype"
    return _lib.ptr(sub.contiguous())


def quantize_mx(x, pre_scale, fmt, emax_elem=None, out_rows=None, sub=None):
    """One tensor ``[B,H,L,D]`` -> (codes, scales) through ``mpsa_quantize_mx``.

    ``out_rows`` >= L pads every head with zero rows (the attention kernel wants whole tiles).
    ``sub`` (``[B,H,D]``, x's dtype): quantize ``x - sub[:, :, None]`` (difference rounded to x's dtype)."""
    x = _check_input(x)
    B, H, L, D = x.shape
    rows = L if out_rows is None else int(out_rows)
    if emax_elem is None:
        emax_elem = EMAX_E2M1 if fmt == _lib.FMT_E2M1 else EMAX_8BIT
    width = D // 2 if fmt == _lib.FMT_E2M1 else D
    codes = torch.empty((B, H, rows, width), dtype=torch.uint8, device=x.device)
    scales = torch.empty((B, H, rows, D // 32), dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().mpsa_quantize_mx(
            _lib.ptr(x), _lib.dtype_id(x.dtype), B, H, L, D, _lib.strides4(x), _sub_ptr(sub, x), pre_scale, fmt, emax_elem,
            _lib.ptr(codes), _lib.ptr(scales), rows, _lib.stream_ptr(x.device)))
    return codes, scales


def quantize_mx_dual(x, pre_scale, fmt8=_lib.FMT_E4M3, out_rows=None, sub=None):
    """E2M1 and an 8-bit format in one pass over x -> (codes4, scales4, codes8, scales8).  ``sub`` as in
    :func:`quantize_mx`."""
    x = _check_input(x)
    B, H, L, D = x.shape
    rows = L if out_rows is None else int(out_rows)
    dev = x.device
    c4 = torch.empty((B, H, rows, D // 2), dtype=torch.uint8, device=dev)
    s4 = torch.empty((B, H, rows, D // 32), dtype=torch.uint8, device=dev)
    c8 = torch.empty((B, H, rows, D), dtype=torch.uint8, device=dev)
    s8 = torch.empty((B, H, rows, D // 32), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().mpsa_quantize_mx_dual(
            _lib.ptr(x), _lib.dtype_id(x.dtype), B, H, L, D, _lib.strides4(x), _sub_ptr(sub, x), pre_scale,
            EMAX_E2M1, fmt8, EMAX_8BIT, _lib.ptr(c4), _lib.ptr(s4), _lib.ptr(c8), _lib.ptr(s8), rows,
            _lib.stream_ptr(dev)))
    return c4, s4, c8, s8


def _quant_pair(q, k, fmt, sm_scale, tensor_layout):
    q4 = _as_bhnd(q, tensor_layout)
    k4 = _as_bhnd(k, tensor_layout)
    head_dim = q4.shape[-1]
    qc, qs = quantize_mx(q4, pre_scale_q(head_dim, sm_scale), fmt)
    kc, ks = quantize_mx(k4, 1.0, fmt)
    return qc, qs, kc, ks


def quant_mxfp4(q, k, BLKQ=128, BLKK=64, sm_scale=None, tensor_layout="HND", packed=True):
    """Q (with ``sm_scale*log2e`` folded in) and K to MXFP4: E2M1 codes + E8M0 scales per 32 along D.

    Reference: ours/quant_mxint8.py:453-512.  ``BLKQ``/``BLKK`` were the reference's Triton tile
    heights and do not change the result; they are accepted and ignored.  Returns
    ``(q_codes, q_scale, k_codes, k_scale)`` in ``[B,H,L,*]`` order."""
    qc, qs, kc, ks = _quant_pair(q, k, _lib.FMT_E2M1, sm_scale, tensor_layout)
    if not packed:
        unpack = MXFP4Tensor(size=(1,)).unpack_packed_tensor
        qc = unpack(qc, 3, (*qc.shape[:3], qc.shape[3] * 2))
        kc = unpack(kc, 3, (*kc.shape[:3], kc.shape[3] * 2))
    return qc, qs, kc, ks


def quant_mxfp8(q, k, BLKQ=128, BLKK=64, sm_scale=None, tensor_layout="HND"):
    """As :func:`quant_mxfp4` with E4M3 elements (codes as uint8; view as ``torch.float8_e4m3fn``)."""
    return _quant_pair(q, k, _lib.FMT_E4M3, sm_scale, tensor_layout)


def quant_mxfp8e5(q, k, BLKQ=128, BLKK=64, sm_scale=None, tensor_layout="HND"):
    """As :func:`quant_mxfp4` with E5M2 elements, the reference's 8-bit format
    (ours/quant_mxint8.py:223-272); codes come back as ``torch.float8_e5m2`` like there."""
    qc, qs, kc, ks = _quant_pair(q, k, _lib.FMT_E5M2, sm_scale, tensor_layout)
    return qc.view(torch.float8_e5m2), qs, kc.view(torch.float8_e5m2), ks
