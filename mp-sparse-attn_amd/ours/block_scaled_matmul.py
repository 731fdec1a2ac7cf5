"""Block-scaled matmul entry points -- the reference's ``ours/block_scaled_matmul.py`` surface.

``block_scaled_matmul(a, a_scale, b, b_scale, dtype_dst, M, N, K, configs)`` keeps the reference signature
(ours/block_scaled_matmul.py:271) and ``initialize_block_scaled_from_tensor(a_tensor, b_tensor, a_scale, b_scale,
block_scale_type, compute_reference)`` the reference's operand packaging (ours/block_scaled_matmul.py:299-406).
Operands are row-major codes (``[M, K/2]`` packed E2M1 or ``[M, K]`` 8-bit) with E8M0 scales, either linear
``[M, K/32]`` (what the quantizer emits) or in the reference's 5-D packed form ``[M/128, K/128, 32, 4, 4]``; given
packed for both operands they go to the kernel as they are, which is its faster path.  B is ``[N, K]`` (NT product).
Element formats come from ``configs["ELEM_PER_BYTE_A"]`` / ``configs["ELEM_PER_BYTE_B"]`` (2 = E2M1, 1 = 8-bit; they
may differ: the reference's ``"mixed"`` type) and, for 8-bit operands, ``configs.get("FMT8", "e4m3")``.
"""

import torch

from . import _lib
from .mxfp import MXFP4Tensor, MXScaleTensor
from .quant_mxint8 import quantize_mx

VEC_SIZE = 32

# block_scale_type -> (elements per byte of A, of B, 8-bit format).  As everywhere in this package "mxfp8" is E4M3;
# the reference's own 8-bit format, E5M2 (a_tensor.to(torch.float8_e5m2), ours/block_scaled_matmul.py:334-336), is
# spelled "mxfp8e5".  "mixed" is the reference's 8-bit A x 4-bit B.
_TYPES = {
    "mxfp4": (2, 2, "e4m3"), "mxfp8": (1, 1, "e4m3"), "mixed": (1, 2, "e4m3"),
    "mxfp8e5": (1, 1, "e5m2"), "mixed_e5": (1, 2, "e5m2"),
}


def make_configs(block_scale_type="mxfp4", fmt8=None):
    """The ``configs`` dict of the reference (ours/block_scaled_matmul.py:394-402) for this build's kernels.
    ``fmt8`` overrides the 8-bit element format (``"e4m3"`` | ``"e5m2"``)."""
    if block_scale_type not in _TYPES:
        raise ValueError(f"Invalid block scale type: {block_scale_type}")
    epb_a, epb_b, f8 = _TYPES[block_scale_type]
    return {
        "BLOCK_SIZE_M": 256, "BLOCK_SIZE_N": 256, "BLOCK_SIZE_K": 128 if epb_a == 2 else 64, "num_stages": 4,
        "ELEM_PER_BYTE_A": epb_a, "ELEM_PER_BYTE_B": epb_b, "VEC_SIZE": VEC_SIZE, "FMT8": fmt8 or f8,
    }


def _fmts_of(configs):
    """(fmt_a, fmt_b) of a configs dict."""
    f8 = _lib.FMT_E4M3 if configs.get("FMT8", "e4m3") == "e4m3" else _lib.FMT_E5M2
    pick = lambda epb: _lib.FMT_E2M1 if epb == 2 else f8
    if configs["ELEM_PER_BYTE_A"] not in (1, 2) or configs["ELEM_PER_BYTE_B"] not in (1, 2):
        raise ValueError("ELEM_PER_BYTE_A / ELEM_PER_BYTE_B must be 1 or 2")
    return pick(configs["ELEM_PER_BYTE_A"]), pick(configs["ELEM_PER_BYTE_B"])


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
    fmt_a, fmt_b = _fmts_of(configs)
    _lib.require_device(a, a_scale, b, b_scale)
    # the reference's packed scale layout goes to the kernel as it is when both operands come that way
    packed = a_scale.dim() == 5 and b_scale.dim() == 5
    if not packed:
        if a_scale.dim() == 5:
            a_scale = unpack_scale_5d(a_scale)
        if b_scale.dim() == 5:
            b_scale = unpack_scale_5d(b_scale)
    width_a = K // 2 if fmt_a == _lib.FMT_E2M1 else K
    width_b = K // 2 if fmt_b == _lib.FMT_E2M1 else K
    a = a.view(torch.uint8).contiguous()
    b = b.view(torch.uint8).contiguous()
    a_scale = a_scale.contiguous()
    b_scale = b_scale.contiguous()
    assert a.shape == (M, width_a) and b.shape == (N, width_b), "operand shapes do not match M, N, K"
    if packed:
        assert a_scale.shape == (M // 128, K // 128, 32, 4, 4) and b_scale.shape == (N // 128, K // 128, 32, 4, 4), \
            "packed scales must be [rows/128, K/128, 32, 4, 4]"
    else:
        assert a_scale.shape == (M, K // VEC_SIZE) and b_scale.shape == (N, K // VEC_SIZE), "scales must be [rows, K/32]"
    out = torch.empty((M, N), dtype=dtype_dst, device=a.device)
    entry = _lib.lib().mpsa_gemm_mx_packed if packed else _lib.lib().mpsa_gemm_mx
    with torch.cuda.device(a.device):
        _lib.check(entry(_lib.ptr(a), _lib.ptr(a_scale), fmt_a, _lib.ptr(b), _lib.ptr(b_scale), fmt_b,
                         M, N, K, _lib.ptr(out), _lib.dtype_id(dtype_dst), N, _lib.stream_ptr(a.device)))
    return out


def fp8_cast(x, fmt8):
    """Elementwise float -> FP8 byte (``x.to(torch.float8_e5m2)`` / ``float8_e4m3fn``) through ``mpsa_fp8_encode``."""
    _lib.require_device(x)
    x = x.to(torch.float32).contiguous()
    out = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().mpsa_fp8_encode(_lib.ptr(x), x.numel(), fmt8, _lib.ptr(out), _lib.stream_ptr(x.device)))
    return out


E4M3_MAX = 448.0


def _package_operand(t, four_bit, fmt8):
    """One operand of the reference's packaging: 8-bit -> the elementwise FP8 cast (ours/block_scaled_matmul.py:334-336);
    4-bit -> ``MXFP4Tensor`` codes packed two per byte along K (:338-345; uint8 input is taken as ready-made codes, one
    per byte, which is what the reference's constructor call accepts; float input is encoded first).  Returns
    ``(bytes for the kernel, decoded float32 values)`` -- the second is what the reference calls ``a_ref``.

    The reference's 8-bit cast is E5M2 (largest finite value 57344); under this package's ``"mxfp8"`` / ``"mixed"``
    the cast is E4M3, where torch's cast -- and ``mpsa_fp8_encode`` -- turns every magnitude above 464 into NaN, so
    float input beyond +-448 is refused here with a pointer to the E5M2 types instead of being packaged as NaN."""
    if not four_bit:
        if t.dtype in (torch.float8_e5m2, torch.float8_e4m3fn):
            want = torch.float8_e5m2 if fmt8 == _lib.FMT_E5M2 else torch.float8_e4m3fn
            assert t.dtype == want, f"operand is {t.dtype} but the block scale type asks for {want}"
            codes = t.view(torch.uint8)
        elif t.dtype == torch.uint8:
            codes = t
        else:
            if fmt8 == _lib.FMT_E4M3 and bool((t.abs() > E4M3_MAX).any()):
                raise ValueError("values beyond +-448 do not fit E4M3 (this package's \"mxfp8\" / \"mixed\"); the "
                                 "reference casts to E5M2: use block_scale_type \"mxfp8e5\" / \"mixed_e5\"")
            codes = fp8_cast(t, fmt8)
        return codes, lambda: codes.view(torch.float8_e5m2 if fmt8 == _lib.FMT_E5M2 else torch.float8_e4m3fn).to(torch.float32)
    fp4 = MXFP4Tensor(data=t, dtype=torch.uint8) if t.dtype == torch.uint8 else MXFP4Tensor(data=t.to(torch.float32))
    return fp4.to_packed_tensor(dim=t.dim() - 1), lambda: fp4.to(torch.float32)


def _package_scale(s):
    """Float scale factors -> E8M0 bytes through ``MXScaleTensor`` (ours/block_scaled_matmul.py:370-374); uint8 input
    is taken as ready-made E8M0 bytes (ours/mxfp_attn_kernel.py:505-506)."""
    if s.dtype == torch.uint8:
        return s
    return MXScaleTensor(s.to(torch.float32)).data


def _expanded_scales(packed_bytes, K):
    """E8M0 bytes in the packed layout -> float32 factors, one per element: ``unpack_scale`` + ``repeat_interleave``
    of the reference (ours/block_scaled_matmul.py:382-388), on the device (``mpsa_scales_from_5d``,
    ``mpsa_e8m0_decode``)."""
    holder = MXScaleTensor(size=(1,), device=packed_bytes.device)
    holder.data = unpack_scale_5d(packed_bytes)
    return holder.to(torch.float32).repeat_interleave(VEC_SIZE, dim=-1)[..., :K]


def initialize_block_scaled_from_tensor(a_tensor, b_tensor, a_scale, b_scale, block_scale_type="mxfp4", compute_reference=False):
    """Operand packaging with the reference's signature (ours/block_scaled_matmul.py:299-406).

    ``a_tensor [M,K]``, ``b_tensor [N,K]``: values to cast element by element (no block scale is derived from them);
    ``a_scale``, ``b_scale``: caller-supplied scale factors in the packed ``[rows/128, K/128, 32, 4, 4]`` layout, float
    (encoded to E8M0 with ``MXScaleTensor``) or uint8.  ``block_scale_type``: ``"mxfp4"``, ``"mxfp8"`` (E4M3),
    ``"mixed"`` (8-bit A x 4-bit B), ``"mxfp8e5"`` / ``"mixed_e5"`` (E5M2, the reference's cast).  ``"nvfp4"`` (16-element
    blocks with FP8 scales) has no counterpart on the CDNA4 scaled matrix cores and raises.
    Returns ``(a, a_scale, b, b_scale, configs, reference)``; ``reference`` is None, or with ``compute_reference`` the
    reference's triple ``(dq(A) @ dq(B)^T, dq(A), dq(B))`` in float32 (:376-392, :404), computed on the device from
    the packaged bytes: codes decoded, E8M0 bytes decoded and repeated over their 32 elements, ``torch.matmul``."""
    if block_scale_type == "nvfp4":
        raise NotImplementedError("nvfp4 (16-element blocks, FP8 scale factors) is not available: the gfx950 scaled matrix "
                                  "instructions take one E8M0 scale per 32 elements")
    assert block_scale_type in _TYPES, f"Invalid block scale type: {block_scale_type}"
    M, K = a_tensor.shape
    N, K_b = b_tensor.shape
    assert K == K_b, f"matrix dimensions do not match: A.shape[1]={K} != B.shape[1]={K_b}"
    expected_a = (M // 128, K // VEC_SIZE // 4, 32, 4, 4)
    expected_b = (N // 128, K // VEC_SIZE // 4, 32, 4, 4)
    assert tuple(a_scale.shape) == expected_a, f"a_scale shape mismatch: expected {expected_a}, got {tuple(a_scale.shape)}"
    assert tuple(b_scale.shape) == expected_b, f"b_scale shape mismatch: expected {expected_b}, got {tuple(b_scale.shape)}"
    configs = make_configs(block_scale_type)
    fmt_a, fmt_b = _fmts_of(configs)
    f8 = fmt_a if fmt_a != _lib.FMT_E2M1 else _lib.FMT_E4M3
    a, a_ref = _package_operand(a_tensor, fmt_a == _lib.FMT_E2M1, f8)
    b, b_ref = _package_operand(b_tensor, fmt_b == _lib.FMT_E2M1, f8)
    a_scale, b_scale = _package_scale(a_scale), _package_scale(b_scale)
    reference = None
    if compute_reference:
        a_dq = a_ref() * _expanded_scales(a_scale, K)
        b_dq = b_ref() * _expanded_scales(b_scale, K)
        reference = (torch.matmul(a_dq, b_dq.T), a_dq, b_dq)
    return a, a_scale, b, b_scale, configs, reference


def validate_block_scaled_from_tensor(M, N, K, block_scale_type="mxfp4", device="cuda"):
    """The reference's self-check (ours/block_scaled_matmul.py:409-441): random fp16 operands and float scale factors
    ``rand + 1e-8`` in the packed layout, packaged with ``compute_reference=True``, multiplied to fp16, and compared
    with the fake-quant product under the reference's bound (``assert_close``, atol = rtol = 1e-3).  Returns
    ``(reference, output)``."""
    a_tensor = torch.randn((M, K), dtype=torch.float16, device=device)
    b_tensor = torch.randn((N, K), dtype=torch.float16, device=device)
    epsilon = 1e-8
    a_scale_tensor = torch.rand((M // 128, K // VEC_SIZE // 4, 32, 4, 4), device=device) + epsilon
    b_scale_tensor = torch.rand((N // 128, K // VEC_SIZE // 4, 32, 4, 4), device=device) + epsilon
    a_desc, a_scale, b_desc, b_scale, configs, reference = initialize_block_scaled_from_tensor(
        a_tensor, b_tensor, a_scale_tensor, b_scale_tensor, block_scale_type, compute_reference=True)
    output = block_scaled_matmul(a_desc, a_scale, b_desc, b_scale, torch.float16, M, N, K, configs)
    torch.testing.assert_close(reference[0], output.to(torch.float32), atol=1e-3, rtol=1e-3)
    return reference[0], output


def quantize_block_scaled_from_tensor(a_tensor, b_tensor, block_scale_type="mxfp4", packed_scales=False):
    """MX-quantize bf16/fp16 ``A [M,K]`` and ``B [N,K]`` per 32 along K (scales derived from the data, as the attention
    path does) and package them for :func:`block_scaled_matmul`: returns ``(a, a_scale, b, b_scale, configs)``.
    ``block_scale_type``: ``"mxfp4"``, ``"mxfp8"`` (E4M3), ``"mxfp8e5"`` (E5M2), ``"mixed"`` / ``"mixed_e5"`` (8-bit A,
    4-bit B).  Scales stay in the linear ``[rows, K/32]`` layout unless ``packed_scales`` asks for the reference's
    packed one."""
    if block_scale_type not in ("mxfp4", "mxfp8", "mxfp8e5", "mixed", "mixed_e5"):
        raise ValueError(f"Invalid block scale type: {block_scale_type}")
    configs = make_configs(block_scale_type)
    fmt_a, fmt_b = _fmts_of(configs)
    a, sa = quantize_mx(a_tensor[None, None], 1.0, fmt_a)
    b, sb = quantize_mx(b_tensor[None, None], 1.0, fmt_b)
    if packed_scales:
        return a[0, 0], pack_scale_5d(sa[0, 0]), b[0, 0], pack_scale_5d(sb[0, 0]), configs
    return a[0, 0], sa[0, 0], b[0, 0], sb[0, 0], configs
