"""Batched block-scaled matmul -- the reference's ``ours/batched_block_scaled_matmul.py`` surface.

``block_scaled_batched_matmul(a, a_scale, b, b_scale, dtype_dst, B, H, M, N, K, configs)`` keeps the reference
signature (ours/batched_block_scaled_matmul.py:183): ``C[b,h] = (A[b,h] o 2^(sa-127)) @ (B[b,h] o 2^(sb-127))^T``
for every batch entry and head, the batched Q.K^T the reference's ``mxfp_attn`` ends with (ours/mxfp_attn.py:64-66).
The arithmetic is that of :func:`ours.block_scaled_matmul.block_scaled_matmul` (the reference's batched kernel
is fp8-only and divides by raw scale bytes in its torch check -- work in progress there; the 2-D semantics are
the specification).  B may have fewer heads than A (grouped heads).  Scales may be linear ``[B,H,rows,K/32]`` or
in the reference's packed form ``[B,H,rows/128,K/128,32,4,4]``.
"""

import torch

from . import _lib
from .block_scaled_matmul import VEC_SIZE, _fmts_of, unpack_scale_5d
# the reference defines the batched packaging here (ours/batched_block_scaled_matmul.py:239) and again, identically, next
# to its attention kernel (ours/mxfp_attn_kernel.py:426); both names are one function in this package
from .mxfp_attn_kernel import initialize_block_scaled_batched_from_tensor  # noqa: F401


def block_scaled_batched_matmul(a, a_scale, b, b_scale, dtype_dst, B, H, M, N, K, configs):
    """Reference: ours/batched_block_scaled_matmul.py:183-236.  Returns ``[B, H, M, N]`` of ``dtype_dst``."""
    if dtype_dst not in (torch.float32, torch.float16, torch.bfloat16, torch.float8_e5m2):
        raise ValueError(f"Unsupported dtype: {dtype_dst}")
    fmt_a, fmt_b = _fmts_of(configs)
    _lib.require_device(a, a_scale, b, b_scale)
    packed = a_scale.dim() == 7 and b_scale.dim() == 7      # both packed: the kernel takes them as they are
    if not packed:
        if a_scale.dim() == 7:
            a_scale = unpack_scale_5d(a_scale)
        if b_scale.dim() == 7:
            b_scale = unpack_scale_5d(b_scale)
    width_a = K // 2 if fmt_a == _lib.FMT_E2M1 else K
    width_b = K // 2 if fmt_b == _lib.FMT_E2M1 else K
    a = a.view(torch.uint8).contiguous()
    b = b.view(torch.uint8).contiguous()
    a_scale = a_scale.contiguous()
    b_scale = b_scale.contiguous()
    Hb = b.shape[1]
    assert a.shape == (B, H, M, width_a) and b.shape == (B, Hb, N, width_b), "operand shapes do not match B, H, M, N, K"
    assert H % Hb == 0, "heads of A must be a multiple of heads of B"
    if packed:
        assert a_scale.shape == (B, H, M // 128, K // 128, 32, 4, 4) and b_scale.shape == (B, Hb, N // 128, K // 128, 32, 4, 4), \
            "packed scales must be [B, H, rows/128, K/128, 32, 4, 4]"
    else:
        assert a_scale.shape == (B, H, M, K // VEC_SIZE) and b_scale.shape == (B, Hb, N, K // VEC_SIZE), "scales must be [B, H, rows, K/32]"
    out = torch.empty((B, H, M, N), dtype=dtype_dst, device=a.device)
    entry = _lib.lib().mpsa_gemm_mx_batched_packed if packed else _lib.lib().mpsa_gemm_mx_batched
    with torch.cuda.device(a.device):
        _lib.check(entry(_lib.ptr(a), _lib.ptr(a_scale), fmt_a, _lib.ptr(b), _lib.ptr(b_scale), fmt_b,
                         B, H, Hb, M, N, K, _lib.ptr(out), _lib.dtype_id(dtype_dst), N, _lib.stream_ptr(a.device)))
    return out
