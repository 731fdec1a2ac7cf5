"""Block-scaled matmul entry point -- the reference's ``ours/block_scaled_matmul.py`` surface.

``block_scaled_matmul(a, a_scale, b, b_scale, dtype_dst, M, N, K, configs)`` keeps the reference
signature (ours/block_scaled_matmul.py:271).  Operands are what the quantizer emits: row-major codes
(``[M, K/2]`` packed E2M1 or ``[M, K]`` 8-bit) and linear E8M0 scales ``[M, K/32]`` (the reference's 5-D packed
scales ``[M/128, K/128, 32, 4, 4]`` are accepted too: given for both operands they go to the kernel as they are,
which is its faster path); B is ``[N, K]``
(NT product).  The element format is read from ``configs["ELEM_PER_BYTE_A"]`` (2 = E2M1) and, for
8-bit, ``configs.get("FMT8", "e4m3")``.
"""

import torch

from . import _lib
from .quant_mxint8 import quantize_mx

VEC_SIZE = 32


def make_configs(block_scale_type="mxfp4"):
    """The ``configs`` dict of the reference (ours/block_scaled_matmul.py:394-402) for this build's kernel."""
    if block_scale_type not in ("mxfp4", "mxfp8", "mxfp8e5"):
        raise ValueError(f"Invalid block scale type: {block_scale_type}")
    fp4 = block_scale_type == "mxfp4"
    return {
        "BLOCK_SIZE_M": 256, "BLOCK_SIZE_N": 256, "BLOCK_SIZE_K": 128 if fp4 else 64, "num_stages": 2,
        "ELEM_PER_BYTE_A": 2 if fp4 else 1, "ELEM_PER_BYTE_B": 2 if fp4 else 1, "VEC_SIZE": VEC_SIZE,
        "FMT8": "e5m2" if block_scale_type == "mxfp8e5" else "e4m3",
    }


def _fmt_of(configs):
    if configs["ELEM_PER_BYTE_A"] != configs["ELEM_PER_BYTE_B"]:
        raise ValueError("mixed 8-bit x 4-bit operands are not supported")
    if configs["ELEM_PER_BYTE_A"] == 2:
        return _lib.FMT_E2M1
    return _lib.FMT_E5M2 if configs.get("FMT8", "e4m3") == "e5m2" else _lib.FMT_E4M3


def pack_scale_5d(scale):
    """Linear E8M0 scales ``[..., rows, K/32]`` -> the reference's packed form ``[..., rows/128, K/128, 32, 4, 4]``
    (ours/mxfp_attn_kernel.py:56-57), through ``mpsa_scales_to_5d``."""
    _lib.require_device(scale)
    scale = scale.contiguous()
    rows, kb = scale.shape[-2], scale.shape[-1]
    batch = scale.numel() // max(rows * kb, 1)
    out = torch.empty((*scale.shape[:-2], rows // 128, kb // 4, 32, 4, 4), dtype=torch.uint8, device=scale.device)
    with torch.cuda.device(scale.device):
        _lib.check(_lib.lib().mpsa_scales_to_5d(_lib.ptr(scale), batch, rows, kb, _lib.ptr(out), _lib.stream_ptr(scale.device)))
    return out


def unpack_scale_5d(packed):
    """The reference's packed scales ``[..., rows/128, K/128, 32, 4, 4]`` -> linear ``[..., rows, K/32]``
    (ours/block_scaled_matmul.py:384), through ``mpsa_scales_from_5d``."""
    _lib.require_device(packed)
    assert packed.dim() >= 5 and packed.shape[-3:] == (32, 4, 4), "expected [..., rows/128, K/128, 32, 4, 4]"
    packed = packed.contiguous()
    rows, kb = packed.shape[-5] * 128, packed.shape[-4] * 4
    batch = packed.numel() // max(rows * kb, 1)
    out = torch.empty((*packed.shape[:-5], rows, kb), dtype=torch.uint8, device=packed.device)
    with torch.cuda.device(packed.device):
        _lib.check(_lib.lib().mpsa_scales_from_5d(_lib.ptr(packed), batch, rows, kb, _lib.ptr(out), _lib.stream_ptr(packed.device)))
    return out


def block_scaled_matmul(a, a_scale, b, b_scale, dtype_dst, M, N, K, configs):
    """``C = (A o 2^(sa-127)) @ (B o 2^(sb-127))^T`` with float32 accumulation.

    Reference: ours/block_scaled_matmul.py:271-296 (ValueError for an unsupported output dtype, :280)."""
    if dtype_dst not in (torch.float32, torch.float16, torch.bfloat16, torch.float8_e5m2):
        raise ValueError(f"Unsupported dtype: {dtype_dst}")
    fmt = _fmt_of(configs)
    _lib.require_device(a, a_scale, b, b_scale)
    # the reference's packed scale layout goes to the kernel as it is when both operands come that way
    packed = a_scale.dim() == 5 and b_scale.dim() == 5
    if not packed:
        if a_scale.dim() == 5:
            a_scale = unpack_scale_5d(a_scale)
        if b_scale.dim() == 5:
            b_scale = unpack_scale_5d(b_scale)
    width = K // 2 if fmt == _lib.FMT_E2M1 else K
    a = a.view(torch.uint8).contiguous()
    b = b.view(torch.uint8).contiguous()
    a_scale = a_scale.contiguous()
    b_scale = b_scale.contiguous()
    assert a.shape == (M, width) and b.shape == (N, width), "operand shapes do not match M, N, K"
    if packed:
        assert a_scale.shape == (M // 128, K // 128, 32, 4, 4) and b_scale.shape == (N // 128, K // 128, 32, 4, 4), \
            "packed scales must be [rows/128, K/128, 32, 4, 4]"
    else:
        assert a_scale.shape == (M, K // VEC_SIZE) and b_scale.shape == (N, K // VEC_SIZE), "scales must be [rows, K/32]"
    out = torch.empty((M, N), dtype=dtype_dst, device=a.device)
    entry = _lib.lib().mpsa_gemm_mx_packed if packed else _lib.lib().mpsa_gemm_mx
    with torch.cuda.device(a.device):
        _lib.check(entry(_lib.ptr(a), _lib.ptr(a_scale), _lib.ptr(b), _lib.ptr(b_scale), fmt,
                         M, N, K, _lib.ptr(out), _lib.dtype_id(dtype_dst), N, _lib.stream_ptr(a.device)))
    return out


def initialize_block_scaled_from_tensor(a_tensor, b_tensor, block_scale_type="mxfp4", packed_scales=False):
    """Quantize bf16/fp16 ``A [M,K]`` and ``B [N,K]`` per 32 along K and package them for
    :func:`block_scaled_matmul`: returns ``(a, a_scale, b, b_scale, configs)``.

    Counterpart of the reference's operand packaging (ours/block_scaled_matmul.py:299-406) chained after
    the quantizer as in test_quant.py:296-350; scales stay in the linear ``[rows, K/32]`` layout unless
    ``packed_scales`` asks for the reference's packed one."""
    configs = make_configs(block_scale_type)
    fmt = _fmt_of(configs)
    a, sa = quantize_mx(a_tensor[None, None], 1.0, fmt)
    b, sb = quantize_mx(b_tensor[None, None], 1.0, fmt)
    if packed_scales:                            # the reference packs them at this point (ours/block_scaled_matmul.py:299-406)
        return a[0, 0], pack_scale_5d(sa[0, 0]), b[0, 0], pack_scale_5d(sb[0, 0]), configs
    return a[0, 0], sa[0, 0], b[0, 0], sb[0, 0], configs
