"""Format helper classes of the MX path -- same names and methods as the reference's ``ours/mxfp.py``.

  * MXFP4Tensor   four-bit E2M1 data, one code per byte (``SEEM`` in the low nibble)
  * MXScaleTensor eight-bit E8M0 block scale factors

Conversions and nibble packing run in HIP kernels of libmpsa (``mpsa_e2m1_encode`` ... ``mpsa_e8m0_decode``,
``mpsa_e2m1_pack`` / ``mpsa_e2m1_unpack``).  Tensors must live on the HIP device.
"""

import math

import torch

from . import _lib


def _flat_call(fn, src, out):
    src = src.contiguous()
    with torch.cuda.device(src.device):
        _lib.check(fn(_lib.ptr(src), src.numel(), _lib.ptr(out), _lib.stream_ptr(src.device)))
    return out


class MXFP4Tensor:

    def __init__(self, data=None, size=None, device=None, dtype=torch.float32):
        """E2M1 tensor (reference: ours/mxfp.py:12-34).

        data:  float32 values to encode (``dtype=torch.float32``) or ready-made uint8 codes
               (``dtype=torch.uint8``, the reference's passthrough, ours/mxfp.py:29-30, :79-82)
        size:  shape for :meth:`random`
        """
        self.device = device
        if data is not None:
            assert isinstance(data, torch.Tensor), "Parameter data must be a torch tensor"
            self.device = data.device
            assert dtype in [torch.float32, torch.uint8], "Currently only float32 and uint8 are supported for fp4e2m1"
            self.data = self._from_float(data) if dtype == torch.float32 else self._from_uint8(data)
        elif size is not None:
            self.size = size if isinstance(size, tuple) else (size, )
        else:
            raise ValueError("Either parameter data or size must be provided")

    def random(self):
        """Uniform random codes (reference: ours/mxfp.py:36-42)."""
        self.data = torch.randint(0, 16, size=self.size, dtype=torch.uint8, device=self.device)
        return self

    def to(self, dtype):
        """Decode to float32; ``0bS000`` is +-0 (reference: ours/mxfp.py:44-77)."""
        assert dtype == torch.float32, "Currently only float32 is supported for fp4e2m1 to float conversion"
        _lib.require_device(self.data)
        out = torch.empty(self.data.shape, dtype=torch.float32, device=self.data.device)
        return _flat_call(_lib.lib().mpsa_e2m1_decode, self.data, out)

    def _from_uint8(self, data):
        assert data.dtype == torch.uint8, "data must be uint8, but got {}".format(data.dtype)
        return data

    def _from_float(self, values):
        """float32 -> E2M1, round to nearest with ties to the even mantissa; NaN/Inf and overflow
        take magnitude 6, the sign is kept (reference: ours/mxfp.py:84-170)."""
        _lib.require_device(values)
        values = values.to(torch.float32)
        out = torch.empty(values.shape, dtype=torch.uint8, device=values.device)
        return _flat_call(_lib.lib().mpsa_e2m1_encode, values, out)

    def to_packed_tensor(self, dim):
        """Two codes per byte along ``dim``: element 2i in the low nibble, 2i+1 in the high one; an
        odd length is zero-padded (reference: ours/mxfp.py:172-205).  Runs ``mpsa_e2m1_pack``."""
        data = self.data
        assert 0 <= dim < data.ndim, "The dimension to pack along is not within the range of tensor dimensions"
        _lib.require_device(data)
        data = data.contiguous()
        n = data.size(dim)
        outer = math.prod(data.shape[:dim])
        inner = math.prod(data.shape[dim + 1:])
        shape = list(data.shape)
        shape[dim] = (n + 1) // 2
        out = torch.empty(shape, dtype=torch.uint8, device=data.device)
        with torch.cuda.device(data.device):
            _lib.check(_lib.lib().mpsa_e2m1_pack(_lib.ptr(data), outer, n, inner, _lib.ptr(out), _lib.stream_ptr(data.device)))
        return out

    def unpack_packed_tensor(self, packed_tensor, dim, original_shape):
        """Inverse of :meth:`to_packed_tensor` (reference: ours/mxfp.py:207-236).  Runs ``mpsa_e2m1_unpack``."""
        _lib.require_device(packed_tensor)
        packed = packed_tensor.contiguous().view(torch.uint8)
        original_shape = tuple(original_shape)
        n = original_shape[dim]
        assert packed.size(dim) == (n + 1) // 2, "packed tensor does not match the original shape"
        outer = math.prod(original_shape[:dim])
        inner = math.prod(original_shape[dim + 1:])
        out = torch.empty(original_shape, dtype=torch.uint8, device=packed.device)
        with torch.cuda.device(packed.device):
            _lib.check(_lib.lib().mpsa_e2m1_unpack(_lib.ptr(packed), outer, n, inner, _lib.ptr(out), _lib.stream_ptr(packed.device)))
        return out


class MXScaleTensor:

    def __init__(self, data=None, size=None, device=None):
        """E8M0 scale tensor (reference: ours/mxfp.py:239-258)."""
        self.device = device
        if data is not None:
            assert isinstance(data, torch.Tensor), "Parameter data must be a torch tensor"
            self.device = data.device
            self.data = self._from_float(data)
        elif size is not None:
            self.size = size if isinstance(size, tuple) else (size, )
        else:
            raise ValueError("Either parameter data or size must be provided")

    def random(self, low=None, high=None):
        """Random exponents in ``[log2(low), log2(high)]``; never the NaN code 255
        (reference: ours/mxfp.py:260-273)."""
        import math
        bias = 127
        min_exponent = 0 if low is None else max(0, int(math.log2(low)) + bias)
        max_exponent = 254 if high is None else min(254, max(0, int(math.log2(high)) + bias))
        assert min_exponent <= max_exponent, "Low must be less than or equal to high"
        self.data = torch.randint(min_exponent, max_exponent + 1, size=self.size, dtype=torch.uint8, device=self.device)
        return self

    def to(self, dtype):
        """``2**(e-127)``; 255 decodes to NaN (reference: ours/mxfp.py:275-284)."""
        assert dtype == torch.float32, "Currently only float32 is supported for f8e8m0 to float conversion"
        _lib.require_device(self.data)
        out = torch.empty(self.data.shape, dtype=torch.float32, device=self.data.device)
        return _flat_call(_lib.lib().mpsa_e8m0_decode, self.data, out)

    def _from_float(self, values):
        """Values <= 0, NaN and Inf give 255; others ``clamp(floor(log2 v) + 127, 0, 254)``
        (reference: ours/mxfp.py:286-307)."""
        _lib.require_device(values)
        values = values.to(torch.float32)
        out = torch.empty(values.shape, dtype=torch.uint8, device=values.device)
        return _flat_call(_lib.lib().mpsa_e8m0_encode, values, out)
