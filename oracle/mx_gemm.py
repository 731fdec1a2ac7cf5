"""Block-scaled matmul of the path, restated on the CPU.

TEST INFRASTRUCTURE ONLY (see the package docstring).

Follows the reference's torch fake-quant reference, ``ours/block_scaled_matmul.py:382-392``:
``C = (decode(A) * 2**(sa-127)) @ (decode(B) * 2**(sb-127))^T`` with A ``[M,K]`` and B ``[N,K]``
row-major and one E8M0 scale per 32 elements along K.
"""

import torch

from .mx_quantize import dequantize_mx


def gemm_mx(a_codes, a_scales, b_codes, b_scales, fmt_a, fmt_b=None, acc_dtype=torch.float32,
            out_dtype=None) -> torch.Tensor:
    """Dequantise both operands and multiply (NT).  ``acc_dtype`` float32 follows the reference;
    float64 gives the tolerance budget.  ``out_dtype`` (e.g. bf16) casts the result."""
    if fmt_b is None:
        fmt_b = fmt_a
    a = dequantize_mx(a_codes, a_scales, fmt_a, acc_dtype)
    b = dequantize_mx(b_codes, b_scales, fmt_b, acc_dtype)
    c = a @ b.transpose(-1, -2)
    return c if out_dtype is None else c.to(out_dtype)


def scales_to_5d(scale: torch.Tensor) -> torch.Tensor:
    """Linear ``[..., rows, K/32]`` scales -> the reference's packed ``[..., rows/128, K/128, 32, 4, 4]``:
    ``reshape(..., rows//128, 4, 32, K//32//4, 4).permute(..., 0, 3, 2, 1, 4)`` -- ours/mxfp_attn_kernel.py:56-57."""
    *lead, rows, kb = scale.shape
    n = len(lead)
    x = scale.reshape(*lead, rows // 128, 4, 32, kb // 4, 4)
    return x.permute(*range(n), n + 0, n + 3, n + 2, n + 1, n + 4).contiguous()


def scales_from_5d(packed: torch.Tensor) -> torch.Tensor:
    """Inverse of :func:`scales_to_5d`: ``permute(0, 3, 2, 1, 4).reshape(chunks_m*128, chunks_k*4)`` --
    ours/block_scaled_matmul.py:384."""
    *lead, cm, ck, r32, r4, c4 = packed.shape
    n = len(lead)
    x = packed.permute(*range(n), n + 0, n + 3, n + 2, n + 1, n + 4)
    return x.reshape(*lead, cm * 128, ck * 4).contiguous()
