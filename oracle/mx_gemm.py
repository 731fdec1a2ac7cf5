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
