"""HIP format kernels behind MXFP4Tensor / MXScaleTensor against the golden vectors and the oracle (bit-exact)."""
import os

import numpy as np
import pytest
import torch

import oracle as O
from ours.mxfp import MXFP4Tensor, MXScaleTensor

pytestmark = pytest.mark.gpu
GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "mxfp_vectors.npz"))
DEV = "cuda:0"


def _f32(bits):
    return torch.from_numpy(np.ascontiguousarray(bits)).view(torch.float32)


def test_e2m1_encode_golden_and_oracle():
    x = _f32(GOLD["e2m1_in_bits"])
    got = MXFP4Tensor(data=x.to(DEV)).data.cpu()
    assert torch.equal(got, torch.from_numpy(GOLD["e2m1_codes"]))
    g = torch.Generator().manual_seed(1)
    y = torch.randn(1 << 20, generator=g) * 3
    assert torch.equal(MXFP4Tensor(data=y.to(DEV)).data.cpu(), O.encode_e2m1(y))
    bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16)
    for dt in (torch.bfloat16, torch.float16):
        z = bits.view(dt).to(torch.float32)
        assert torch.equal(MXFP4Tensor(data=z.to(DEV)).data.cpu(), O.encode_e2m1(z))


def test_e2m1_decode_pack_roundtrip():
    codes = torch.arange(16, dtype=torch.uint8, device=DEV)
    dec = MXFP4Tensor(data=codes, dtype=torch.uint8).to(torch.float32).cpu()
    assert np.array_equal(dec.view(torch.int32).numpy(), GOLD["e2m1_decode_all16_bits"])
    t = MXFP4Tensor(size=(4, 6, 64), device=DEV).random()
    assert t.data.max() < 16
    for dim in (0, 1, 2):
        p = t.to_packed_tensor(dim)
        assert torch.equal(t.unpack_packed_tensor(p, dim, t.data.shape), t.data)
    assert torch.equal(t.to_packed_tensor(2).cpu(), O.pack_fp4(t.data.cpu()))
    # literal cases: even and odd lengths, packing along the leading dimension
    e = MXFP4Tensor(data=torch.arange(16, dtype=torch.uint8, device=DEV).reshape(2, 8), dtype=torch.uint8)
    p = e.to_packed_tensor(dim=1)
    assert p.tolist() == [[0x10, 0x32, 0x54, 0x76], [0x98, 0xBA, 0xDC, 0xFE]]
    assert torch.equal(e.unpack_packed_tensor(p, 1, (2, 8)), e.data)
    odd = MXFP4Tensor(data=torch.arange(6, dtype=torch.uint8, device=DEV).reshape(2, 3), dtype=torch.uint8)
    po = odd.to_packed_tensor(dim=1)
    assert po.tolist() == [[0x10, 0x02], [0x43, 0x05]]
    assert torch.equal(odd.unpack_packed_tensor(po, 1, (2, 3)), odd.data)
    p0 = e.to_packed_tensor(dim=0)
    assert p0.shape == (1, 8) and p0[0, 3].item() == (11 << 4 | 3)
    o3 = MXFP4Tensor(size=(3, 5, 7), device=DEV).random()
    for dim in (0, 1, 2):
        p = o3.to_packed_tensor(dim)
        assert p.shape[dim] == (o3.data.shape[dim] + 1) // 2
        assert torch.equal(o3.unpack_packed_tensor(p, dim, o3.data.shape), o3.data)
    assert torch.equal(MXFP4Tensor(data=t.to(torch.float32)).data, t.data & 0xF | (t.data & 8))


def test_e8m0_golden():
    x = _f32(GOLD["e8m0_in_bits"])
    got = MXScaleTensor(data=x.to(DEV)).data.cpu()
    assert torch.equal(got, torch.from_numpy(GOLD["e8m0_codes"]))
    s = MXScaleTensor(size=(256,), device=DEV)
    s.data = torch.arange(256, dtype=torch.uint8, device=DEV)
    dec = s.to(torch.float32).cpu()
    ref = _f32(GOLD["e8m0_decode_all256_bits"])
    assert torch.equal(dec[:255], ref[:255]) and torch.isnan(dec[255])
    r = MXScaleTensor(size=(1000,), device=DEV).random(low=1 / 16, high=16)
    assert r.data.min() >= 123 and r.data.max() <= 131


@pytest.mark.parametrize("fmt,dt", [(1, torch.float8_e5m2), (0, torch.float8_e4m3fn)])
def test_fp8_elementwise_cast_equals_torch(fmt, dt):
    """mpsa_fp8_encode against torch's own float32 -> FP8 cast on the CPU (a library routine): every float16 value (all
    65536 bit patterns, NaN and infinities included), a dense sweep around the formats' largest values, subnormals."""
    from ours.block_scaled_matmul import fp8_cast
    halves = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.float16).float()
    big = torch.linspace(400.0, 70000.0, 20001)
    tiny = torch.linspace(0.0, 2.0 ** -5, 4097)
    special = torch.tensor([448.0, 464.0, 464.0001, 479.99, 480.0, 57344.0, 61440.0, 61439.9, 65536.0, float("inf"), float("nan"), -0.0])
    x = torch.cat([halves, big, -big, tiny, -tiny, special, -special])
    got = fp8_cast(x.to(DEV), fmt).cpu()
    want = x.to(dt).view(torch.uint8)
    nan = torch.isnan(want.view(dt).float())
    assert torch.equal(got[~nan], want[~nan])
    assert torch.isnan(got.view(dt).float()[nan]).all()          # NaN stays NaN (any payload)
