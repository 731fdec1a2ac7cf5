"""Element and scale formats of the MX path, restated on the CPU.

TEST INFRASTRUCTURE ONLY (see the package docstring).

Follows the reference's ``ours/mxfp.py``:
  * E2M1 decode            -- ours/mxfp.py:44-77
  * E2M1 encode (RNE)      -- ours/mxfp.py:84-170
  * nibble pack / unpack   -- ours/mxfp.py:172-236
  * E8M0 encode / decode   -- ours/mxfp.py:275-307
E4M3 is the benchmark contract's 8-bit format (the reference stores E5M2,
ours/quant_mxint8.py:203-205); both are provided.
"""

import torch

# index = (E << 1) | M ; code = (S << 3) | index          (ours/mxfp.py:53-77, :103-135)
E2M1_VALUES = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)

_CHUNK = 1 << 20


def decode_e2m1(codes: torch.Tensor) -> torch.Tensor:
    """uint8 codes (one per byte, low nibble ``SEEM``) -> float32.  ours/mxfp.py:44-77.

    ``0bS000`` decodes to +-0.0."""
    assert codes.dtype == torch.uint8
    table = torch.tensor(E2M1_VALUES, dtype=torch.float32)
    mag = table[(codes & 0x7).long()]
    sign = ((codes >> 3) & 1).bool()
    return torch.where(sign, -mag, mag)


def encode_e2m1(values: torch.Tensor) -> torch.Tensor:
    """float32 -> uint8 E2M1 codes, round-to-nearest, ties to even mantissa.  ours/mxfp.py:84-170.

    Restates the reference literally: distance to all eight magnitudes in
    float32, a float32 ``1e-6`` subtracted from the distance to the
    even-mantissa candidates (applied whenever the tensor has two or more
    elements -- ours/mxfp.py:151-158 -- and applied here always), first
    minimal index wins, NaN/Inf take magnitude 6, a zero magnitude takes
    E = M = 0, sign from ``signbit``."""
    assert values.dtype == torch.float32
    flat = values.reshape(-1)
    out = torch.empty(flat.shape, dtype=torch.uint8)
    cand = torch.tensor(E2M1_VALUES, dtype=torch.float32)
    bias = torch.tensor([1, 0, 1, 0, 1, 0, 1, 0], dtype=torch.int32) * 1e-6   # float32, as int32 * python float
    assert bias.dtype == torch.float32
    for s in range(0, flat.numel(), _CHUNK):
        x = flat[s:s + _CHUNK]
        sign = torch.signbit(x).to(torch.uint8)
        a = torch.abs(x)
        is_zero = a == 0
        invalid = torch.isnan(x) | torch.isinf(x)
        a = torch.where(invalid, torch.tensor(6.0), a)
        err = torch.abs(a.unsqueeze(1) - cand.unsqueeze(0))
        err = err - bias.unsqueeze(0)
        idx = torch.argmin(err, dim=1).to(torch.uint8)     # first minimal index on CPU
        idx = torch.where(is_zero, torch.zeros_like(idx), idx)
        out[s:s + _CHUNK] = (sign << 3) | idx
    return out.reshape(values.shape)


def pack_fp4(codes: torch.Tensor) -> torch.Tensor:
    """Two codes per byte along the last dim: ``byte[j] = codes[2j] | codes[2j+1] << 4``.

    ours/mxfp.py:196-205 (``packed = (high << 4) | low``); the 2-D reference use packs
    along K (ours/block_scaled_matmul.py:343-345).  The last dim must be even here."""
    assert codes.dtype == torch.uint8 and codes.shape[-1] % 2 == 0
    lo = codes[..., 0::2]
    hi = codes[..., 1::2]
    return (hi << 4) | lo


def unpack_fp4(packed: torch.Tensor) -> torch.Tensor:
    """Inverse of :func:`pack_fp4`.  ours/mxfp.py:207-236."""
    assert packed.dtype == torch.uint8
    lo = packed & 0xF
    hi = (packed >> 4) & 0xF
    return torch.stack((lo, hi), dim=-1).reshape(*packed.shape[:-1], packed.shape[-1] * 2)


def _floor_log2(v: torch.Tensor) -> torch.Tensor:
    """True ``floor(log2(v))`` of positive finite float32 values (frexp, no rounding)."""
    _, e = torch.frexp(v)          # v = m * 2**e, m in [0.5, 1)
    return e.to(torch.int32) - 1


def encode_e8m0(values: torch.Tensor) -> torch.Tensor:
    """float32 -> E8M0 byte.  ours/mxfp.py:286-307.

    NaN, +-Inf and values <= 0 give 255; otherwise ``clamp(floor(log2 v) + 127, 0, 254)``.
    The reference evaluates ``floor(log2(v))`` in float32; for the exact powers of two the
    quantizer feeds it the two agree."""
    assert values.dtype == torch.float32
    invalid = torch.isnan(values) | torch.isinf(values) | (values <= 0)
    safe = torch.where(invalid, torch.ones_like(values), values)
    e = torch.clamp(_floor_log2(safe) + 127, 0, 254).to(torch.uint8)
    return torch.where(invalid, torch.full_like(e, 255), e)


def decode_e8m0(e: torch.Tensor) -> torch.Tensor:
    """E8M0 byte -> float32 ``2**(e-127)``; 255 -> NaN.  ours/mxfp.py:275-284."""
    assert e.dtype == torch.uint8
    val = torch.ldexp(torch.ones(e.shape, dtype=torch.float64), e.to(torch.int32) - 127).to(torch.float32)
    return torch.where(e == 255, torch.full_like(val, float("nan")), val)


def encode_e4m3(y: torch.Tensor) -> torch.Tensor:
    """float32 -> E4M3 (OCP "fn": no Inf, max 448) byte: clamp to +-448, then round to nearest even.

    Not in the reference (its 8-bit format is E5M2); the benchmark contract names E4M3.
    torch's float8_e4m3fn cast is RNE, keeps subnormals (2**-9) and does not saturate, hence
    the clamp -- which mirrors the reference's clamp-before-cast (ours/quant_mxint8.py:203-205)."""
    assert y.dtype == torch.float32
    return torch.clamp(y, -448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)


def decode_e4m3(b: torch.Tensor) -> torch.Tensor:
    assert b.dtype == torch.uint8
    return b.view(torch.float8_e4m3fn).to(torch.float32)


def encode_e5m2(y: torch.Tensor) -> torch.Tensor:
    """float32 -> E5M2 byte: clamp to +-57344 then RNE cast.  ours/quant_mxint8.py:203-205."""
    assert y.dtype == torch.float32
    return torch.clamp(y, -57344.0, 57344.0).to(torch.float8_e5m2).view(torch.uint8)


def decode_e5m2(b: torch.Tensor) -> torch.Tensor:
    assert b.dtype == torch.uint8
    return b.view(torch.float8_e5m2).to(torch.float32)
