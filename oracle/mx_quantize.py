"""MX quantizer of the path, restated on the CPU.

TEST INFRASTRUCTURE ONLY (see the package docstring).

Follows ``ours/quant_mxint8.py:276-351`` (E2M1) and ``:164-219`` (8-bit) for the
pre-scale, the shared-exponent rule, the power-of-two divide and the clamp, and
``ours/mxfp.py`` (via ``mx_formats``) for the element and scale encodings.
"""

import torch

from . import mx_formats as F

# hardware format selectors of the CDNA4 scaled MFMA double as format ids
FMT_E4M3 = 0
FMT_E5M2 = 1
FMT_E2M1 = 4

# "emax_elem" of the reference: 3 for E2M1 (ours/quant_mxint8.py:303), 7 for the 8-bit
# format (ours/quant_mxint8.py:191).  The OCP MX spec would use 2 and 8 (E4M3) / 15 (E5M2).
EMAX_ELEM = {FMT_E2M1: 3, FMT_E4M3: 7, FMT_E5M2: 7}

LOG2E_F = 1.44269504        # the literal the reference multiplies in (ours/quant_mxint8.py:494)


def q_pre_scale(head_dim: int, scale=None) -> float:
    """Factor folded into Q before quantizing: ``sm_scale * 1.44269504`` rounded to float32.

    ours/quant_mxint8.py:479-480, :494 (``sm_scale = head_dim**-0.5`` when not given; the
    product is formed in Python double precision and handed to the kernel as a float32)."""
    sm = head_dim ** -0.5 if scale is None else float(scale)
    return float(torch.tensor(sm * LOG2E_F, dtype=torch.float32).item())


def quantize_mx(x: torch.Tensor, pre: float, fmt: int, emax_elem=None):
    """Quantize ``x[..., D]`` (bf16 / fp16 / fp32) per 32 consecutive elements of the last dim.

    Steps (ours/quant_mxint8.py:295-351, :183-219):
      x32   = f32(x) * f32(pre)                      (float32 multiply)
      amax  = max |x32| over the block
      se    = floor(log2(amax)) - emax_elem          (true floor, by bit extraction)
      y     = x32 / 2**se                            (exact power-of-two scaling)
      y     = clamp(y, +-6 | +-448 | +-57344)
      codes = encode_fmt(y);  scale byte = clamp(se + 127, 0, 254)
      amax == 0  ->  scale byte 0 and codes +0        (this build's decision)

    Returns ``(codes, scales)``: codes uint8, packed two per byte along the last dim for E2M1
    (``[..., D/2]``) and one per byte otherwise (``[..., D]``); scales uint8 ``[..., D/32]``."""
    assert x.shape[-1] % 32 == 0
    if emax_elem is None:
        emax_elem = EMAX_ELEM[fmt]
    shape = x.shape
    nb = shape[-1] // 32
    x32 = x.to(torch.float32) * torch.tensor(pre, dtype=torch.float32)
    xb = x32.reshape(-1, nb, 32)
    amax = xb.abs().amax(dim=-1)                               # [R, nb]
    zero = amax == 0
    safe = torch.where(zero, torch.ones_like(amax), amax)
    se = F._floor_log2(safe) - int(emax_elem)                    # int32
    # exact scaling in float64, then back to float32 (exact unless the result is far below
    # the smallest code, where every encoder gives zero anyway)
    y = torch.ldexp(xb.to(torch.float64), (-se).unsqueeze(-1).to(torch.int32))
    if fmt == FMT_E2M1:
        y = torch.clamp(y, -6.0, 6.0).to(torch.float32)
        codes = F.encode_e2m1(y)
    elif fmt == FMT_E4M3:
        codes = F.encode_e4m3(torch.clamp(y, -448.0, 448.0).to(torch.float32))
    elif fmt == FMT_E5M2:
        codes = F.encode_e5m2(torch.clamp(y, -57344.0, 57344.0).to(torch.float32))
    else:
        raise ValueError(f"unknown MX element format {fmt}")
    scales = torch.clamp(se + 127, 0, 254).to(torch.uint8)
    codes = torch.where(zero.unsqueeze(-1), torch.zeros_like(codes), codes)
    scales = torch.where(zero, torch.zeros_like(scales), scales)
    codes = codes.reshape(shape)
    if fmt == FMT_E2M1:
        codes = F.pack_fp4(codes)
    return codes, scales.reshape(*shape[:-1], nb)


def dequantize_mx(codes: torch.Tensor, scales: torch.Tensor, fmt: int, dtype=torch.float32) -> torch.Tensor:
    """``decode(codes) * 2**(scale-127)`` per 32-block of the last dim (ours/block_scaled_matmul.py:382-392)."""
    if fmt == FMT_E2M1:
        val = F.decode_e2m1(F.unpack_fp4(codes))
    elif fmt == FMT_E4M3:
        val = F.decode_e4m3(codes)
    elif fmt == FMT_E5M2:
        val = F.decode_e5m2(codes)
    else:
        raise ValueError(f"unknown MX element format {fmt}")
    s = F.decode_e8m0(scales).to(dtype).repeat_interleave(32, dim=-1)
    return val.to(dtype) * s


def seq_mean(k: torch.Tensor) -> torch.Tensor:
    """Mean over the sequence dim in k's 16-bit dtype the way the reference's device computes it: float32
    accumulation, times float32 ``1/N``, one rounding (torch's CUDA mean; its CPU mean for 16-bit inputs rounds
    the sum to 16 bits first, which is not what the reference ran).  ours/mxfp_attn.py:44-45."""
    n = k.shape[-2]
    inv = torch.tensor(1.0, dtype=torch.float32) / torch.tensor(float(n), dtype=torch.float32)
    return (k.to(torch.float32).sum(dim=-2, keepdim=True) * inv).to(k.dtype)


def smooth_k(k: torch.Tensor, mean: torch.Tensor = None) -> torch.Tensor:
    """``k - mean over the sequence dim`` in k's own dtype.  ours/mxfp_attn.py:44-45.  ``mean`` (``[..., 1, D]``
    or ``[..., D]``, k's dtype) replaces the oracle's own mean, for checking the subtraction apart from the
    summation order of the mean."""
    if mean is None:
        mean = seq_mean(k)
    elif mean.dim() == k.dim() - 1:
        mean = mean.unsqueeze(-2)
    return k - mean.to(k.dtype)
