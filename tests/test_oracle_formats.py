"""Pins the CPU oracle's element / scale formats (no GPU needed).

Checks are independent of the oracle's own formulas: golden vectors produced by the reference's
``ours/mxfp.py`` (tests/golden/mxfp_vectors.npz), literal tables, and brute-force searches in float64.
"""
import os

import numpy as np
import pytest
import torch

import oracle as O

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "mxfp_vectors.npz"))


def _f32(bits):
    return torch.from_numpy(np.ascontiguousarray(bits)).view(torch.float32)


def test_e2m1_encode_matches_reference_vectors():
    x = _f32(GOLD["e2m1_in_bits"])
    want = torch.from_numpy(GOLD["e2m1_codes"])
    got = O.encode_e2m1(x)
    assert torch.equal(got, want)
    # the vectors really exercise the 1e-6 bias: some inputs are NOT rounded to the nearest value
    a = x.abs().double()
    grid = torch.tensor(O.E2M1_VALUES, dtype=torch.float64)
    nearest = (a.unsqueeze(1) - grid).abs().argmin(dim=1)
    finite = torch.isfinite(x) & (a <= 6)
    assert ((want & 7).long()[finite] != nearest[finite]).any()


def test_e2m1_decode_table():
    codes = torch.arange(16, dtype=torch.uint8)
    want = torch.tensor([0, .5, 1, 1.5, 2, 3, 4, 6, -0.0, -.5, -1, -1.5, -2, -3, -4, -6], dtype=torch.float32)
    got = O.decode_e2m1(codes)
    assert torch.equal(got.view(torch.int32), want.view(torch.int32))          # bit equality: -0.0 too
    assert np.array_equal(got.view(torch.int32).numpy(), GOLD["e2m1_decode_all16_bits"])


def _all_16bit(dtype):
    bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16)
    return bits.view(dtype).to(torch.float32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_e2m1_encode_is_rne_on_16bit_inputs(dtype):
    """Every bf16 / fp16 value (times a few power-of-two scalings, which is all the K path and the GEMM
    operands ever feed the encoder): brute-force nearest grid value, exact ties to the even mantissa."""
    x = _all_16bit(dtype)
    x = x[torch.isfinite(x)]
    grid = torch.tensor(O.E2M1_VALUES, dtype=torch.float64)
    even = torch.tensor([1, 0, 1, 0, 1, 0, 1, 0], dtype=torch.bool)
    for shift in (0, 3, -2):
        y = torch.ldexp(x, torch.tensor(shift)).clamp(-6, 6)
        d = (y.abs().double().unsqueeze(1) - grid).abs()
        best = d.min(dim=1, keepdim=True).values
        is_best = d == best
        # among the (one or two) nearest candidates take the even-mantissa one
        pick = torch.where(is_best & even, 2, torch.where(is_best, 1, 0)).argmax(dim=1)
        want = (torch.signbit(y).to(torch.uint8) << 3) | pick.to(torch.uint8)
        assert torch.equal(O.encode_e2m1(y), want)


def test_e2m1_roundtrip_and_specials():
    codes = torch.arange(16, dtype=torch.uint8)
    assert torch.equal(O.encode_e2m1(O.decode_e2m1(codes)), codes)
    x = torch.tensor([float("nan"), float("inf"), float("-inf"), 100.0, -100.0, -0.0, 0.0])
    got = O.encode_e2m1(x)
    assert got[1] == 7 and got[2] == 15 and got[3] == 7 and got[4] == 15 and got[5] == 8 and got[6] == 0
    assert (got[0] & 7) == 7


def test_pack_fp4():
    g = torch.Generator().manual_seed(0)
    codes = torch.randint(0, 16, (5, 3, 64), dtype=torch.uint8, generator=g)
    packed = O.pack_fp4(codes)
    assert packed.shape == (5, 3, 32)
    assert packed[1, 2, 7] == (codes[1, 2, 14] | (codes[1, 2, 15] << 4))        # low nibble = even element
    assert torch.equal(O.unpack_fp4(packed), codes)
    assert np.array_equal(O.pack_fp4(torch.from_numpy(GOLD["pack_in"])).numpy(), GOLD["pack_out"])


def test_e8m0_matches_reference_vectors_and_closed_form():
    x = _f32(GOLD["e8m0_in_bits"])
    assert torch.equal(O.encode_e8m0(x), torch.from_numpy(GOLD["e8m0_codes"]))
    dec = O.decode_e8m0(torch.arange(256, dtype=torch.uint8))
    ref = _f32(GOLD["e8m0_decode_all256_bits"])
    assert torch.equal(dec[:255], ref[:255]) and torch.isnan(dec[255]) and torch.isnan(ref[255])
    # closed form with python floats
    for e in range(0, 255):
        assert dec[e].item() == 2.0 ** (e - 127)
        if e >= 1:
            assert O.encode_e8m0(torch.tensor([2.0 ** (e - 127)], dtype=torch.float32)).item() == e
    bad = torch.tensor([0.0, -1.0, float("inf"), float("nan")])
    assert (O.encode_e8m0(bad) == 255).all()
    assert O.encode_e8m0(torch.tensor([1.5, 3.99, 4.0, 0.75])).tolist() == [127, 128, 129, 126]


def _e4m3_bruteforce(y64):
    """Independent E4M3 encoder: enumerate all 127 finite non-negative codes and round in float64."""
    vals = []
    for c in range(0x7F):
        e, m = c >> 3, c & 7
        vals.append(m * 2.0 ** -9 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7))
    grid = torch.tensor(vals, dtype=torch.float64)
    assert grid[-1] == 448.0
    a = y64.abs().clamp(max=448.0)
    d = (a.unsqueeze(1) - grid).abs()
    best = d.min(dim=1, keepdim=True).values
    is_best = d == best
    even = (torch.arange(0x7F) & 1) == 0
    pick = torch.where(is_best & even, 2, torch.where(is_best, 1, 0)).argmax(dim=1)
    return (torch.signbit(y64).to(torch.uint8) << 7) | pick.to(torch.uint8)


def test_e4m3_encode_against_bruteforce():
    g = torch.Generator().manual_seed(5)
    x16 = _all_16bit(torch.bfloat16)
    x16 = x16[torch.isfinite(x16)]
    rnd = torch.randn(50000, generator=g) * torch.exp2(torch.randint(-12, 9, (50000,), generator=g).float())
    mids = torch.tensor([2.0 ** -10, 3 * 2.0 ** -10, 2.0 ** -9, 17 / 16.0, 19 / 16.0, 440.0, 448.0, 464.0, 1e6, -1e6, 0.0, -0.0])
    for x in (x16, rnd, mids):
        assert torch.equal(O.encode_e4m3(x), _e4m3_bruteforce(x.double()))
    # decode is torch's own table; spot-check a few literals
    assert O.decode_e4m3(torch.tensor([0x38, 0x7E, 0x01, 0xB8], dtype=torch.uint8)).tolist() == [1.0, 448.0, 2.0 ** -9, -1.0]


def test_e5m2_encode_clamps_then_rounds():
    x = torch.tensor([1.0, 57344.0, 1e9, -1e9, 1.125, 1.375, 2.0 ** -16, 2.0 ** -17])
    got = O.encode_e5m2(x)
    assert got.tolist() == [0x3C, 0x7B, 0x7B, 0xFB, 0x3C, 0x3E, 0x01, 0x00]
