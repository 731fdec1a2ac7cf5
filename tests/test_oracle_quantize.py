"""Pins the CPU oracle's MX quantizer through hand-worked blocks and invariants (no GPU needed)."""
import math

import pytest
import torch

import oracle as O


def test_q_pre_scale_is_float32_of_the_double_product():
    assert O.q_pre_scale(128) == float(torch.tensor(128 ** -0.5 * 1.44269504, dtype=torch.float32))
    assert O.q_pre_scale(64) == float(torch.tensor(0.125 * 1.44269504, dtype=torch.float32))
    assert O.q_pre_scale(64, scale=0.5) == float(torch.tensor(0.5 * 1.44269504, dtype=torch.float32))


def test_hand_worked_block_e2m1():
    # amax = 5 -> floor(log2) = 2 -> shared exp 2-3 = -1 -> scale 0.5 -> y = 2x, clamp 6
    x = torch.zeros(1, 32)
    x[0, :8] = torch.tensor([5.0, -5.0, 1.0, 0.5, 0.25, 0.3, 2.9, -0.1])
    codes, scales = O.quantize_mx(x.bfloat16(), 1.0, O.FMT_E2M1)
    assert scales.tolist() == [[126]]
    c = O.unpack_fp4(codes)[0, :8].tolist()
    # y = 10 -> 6 (7); -10 -> -6 (15); 2 -> 4; 1 -> 2; .5 -> 1; bf16(.3)*2=.6015625 -> .5 (1); bf16(2.9)*2=5.8125 -> 6 (7);
    # bf16(-.1)*2 = -.2001953 -> -0 (8)
    assert c == [7, 15, 4, 2, 1, 1, 7, 8]
    assert (O.unpack_fp4(codes)[0, 8:] == 0).all()


def test_hand_worked_block_e4m3():
    # amax = 5 -> shared exp 2-7 = -5 -> y = 32x: 160, -160, 32, 16, 8
    x = torch.zeros(1, 32)
    x[0, :5] = torch.tensor([5.0, -5.0, 1.0, 0.5, 0.25])
    codes, scales = O.quantize_mx(x.bfloat16(), 1.0, O.FMT_E4M3)
    assert scales.tolist() == [[122]]
    # 160 = 1.25*2^7 -> e=14,m=2 -> 0x72; 32 = 2^5 -> e=12 -> 0x60; 16 -> 0x58; 8 -> 0x50
    assert codes[0, :5].tolist() == [0x72, 0xF2, 0x60, 0x58, 0x50]


def test_zero_block_and_padding_rule():
    x = torch.zeros(2, 64).bfloat16()
    x[1, 40] = -0.0
    x[0, 3] = 1.0
    for fmt in (O.FMT_E2M1, O.FMT_E4M3, O.FMT_E5M2):
        codes, scales = O.quantize_mx(x, 1.0, fmt)
        assert scales[0, 1] == 0 and scales[1, 0] == 0 and scales[1, 1] == 0
        assert (codes[1] == 0).all()
        assert scales[0, 0] == 127 - O.EMAX_ELEM[fmt]


@pytest.mark.parametrize("fmt", [O.FMT_E2M1, O.FMT_E4M3, O.FMT_E5M2])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_invariants(fmt, dtype):
    g = torch.Generator().manual_seed(11)
    x = (torch.randn(64, 256, generator=g) * torch.exp2(torch.randint(-6, 6, (64, 1), generator=g).float())).to(dtype)
    pre = O.q_pre_scale(128)
    codes, scales = O.quantize_mx(x, pre, fmt)
    x32 = x.float() * torch.tensor(pre, dtype=torch.float32)
    amax = x32.reshape(64, 8, 32).abs().amax(-1)
    # scale byte is exactly floor(log2(amax)) - emax + 127, computed here with python's math on doubles
    want = torch.tensor([[math.floor(math.log2(a)) - O.EMAX_ELEM[fmt] + 127 for a in row] for row in amax.double().tolist()])
    assert torch.equal(scales.long(), want)
    # scale is monotone in amax
    order = amax.flatten().argsort()
    assert (scales.flatten()[order].long().diff() >= 0).all()
    deq = O.dequantize_mx(codes, scales, fmt)
    sc = O.decode_e8m0(scales).repeat_interleave(32, dim=-1)
    y = x32 / sc
    if fmt == O.FMT_E2M1:
        # amax / scale lies in [8, 16): the block maximum always saturates to 6
        assert ((amax / O.decode_e8m0(scales)) >= 8).all() and ((amax / O.decode_e8m0(scales)) < 16).all()
        sat = y.abs() > 6
        assert (deq[sat].abs() == 6 * sc[sat]).all()
        # unsaturated elements are within half a grid step (step <= 2 at the top of the grid)
        err = (deq - x32).abs() / sc
        assert (err[~sat] <= torch.where(y[~sat].abs() >= 4, 1.0, torch.where(y[~sat].abs() >= 2, 0.5, 0.25)) + 1e-6).all()
    else:
        mant = 3 if fmt == O.FMT_E4M3 else 2
        assert ((amax / O.decode_e8m0(scales)) >= 128).all() and ((amax / O.decode_e8m0(scales)) < 256).all()
        rel = ((deq - x32).abs() / x32.abs().clamp_min(1e-30))
        normal = y.abs() >= (2.0 ** -6 if fmt == O.FMT_E4M3 else 2.0 ** -14)
        assert (rel[normal] <= 2.0 ** -(mant + 1) + 1e-7).all()
    # sign is preserved wherever the code is non-zero
    nz = deq != 0
    assert (torch.sign(deq[nz]) == torch.sign(x32[nz])).all()


def test_true_floor_of_log2_below_a_power_of_two():
    # amax one float32 ulp below 8 (reachable on the Q path only): true floor is 2, a float32 log2 says 3
    x = torch.full((1, 32), 1.0)
    pre = float(torch.nextafter(torch.tensor(8.0), torch.tensor(0.0)))
    codes, scales = O.quantize_mx(x.bfloat16(), pre, O.FMT_E2M1)
    assert scales.item() == 2 - 3 + 127


def test_tiny_and_huge_blocks_keep_scale_byte_in_range():
    x = torch.tensor([[2.0 ** -126] * 32, [2.0 ** 120] * 32]).bfloat16()
    for fmt in (O.FMT_E2M1, O.FMT_E4M3):
        codes, scales = O.quantize_mx(x, 1.0, fmt)
        assert scales[0, 0] == max(0, -126 - O.EMAX_ELEM[fmt] + 127)
        assert scales[1, 0] == 120 - O.EMAX_ELEM[fmt] + 127


def test_smooth_k():
    g = torch.Generator().manual_seed(3)
    k = (torch.randn(1, 2, 16, 32, generator=g) + 3).bfloat16()
    s = O.smooth_k(k)
    assert s.dtype == torch.bfloat16
    assert s.float().mean(dim=-2).abs().max() < 0.05


def test_seq_mean_is_the_once_rounded_mean():
    """The mean is the float32 sum times float32 1/N rounded once to the 16-bit dtype: checked against float64
    arithmetic (the two can only differ where the float64 mean sits within float32 error of a rounding
    boundary), against an exactly representable case, and the subtraction against explicit bf16 arithmetic."""
    g = torch.Generator().manual_seed(5)
    for dtype in (torch.bfloat16, torch.float16):
        k = (torch.randn(2, 3, 1000, 64, generator=g) * 2 + 1).to(dtype)
        m = O.seq_mean(k)
        assert m.dtype == dtype and m.shape == (2, 3, 1, 64)
        ref = k.double().mean(dim=-2, keepdim=True)
        ulp = torch.finfo(dtype).eps * ref.abs().clamp_min(2.0 ** -14)
        assert ((m.double() - ref).abs() <= 0.5 * ulp * (1 + 1e-3)).all()
        assert (m == ref.to(dtype)).float().mean() > 0.995
    k = torch.tensor([1.0, 2.0, 3.0, 6.0]).view(1, 1, 4, 1).expand(1, 1, 4, 32).bfloat16()
    assert (O.seq_mean(k) == 3.0).all()
    s = O.smooth_k(k)
    assert torch.equal(s[0, 0, :, 0].float(), torch.tensor([-2.0, -1.0, 0.0, 3.0]))
    # explicit mean argument: the difference is rounded to the 16-bit dtype
    k2 = torch.tensor([1.0078125, 100.0]).view(1, 1, 2, 1).expand(1, 1, 2, 32).bfloat16()
    mean = torch.full((1, 1, 32), 0.00390625).bfloat16()
    d = O.smooth_k(k2, mean)
    assert d[0, 0, 0, 0].item() == 1.0 and d[0, 0, 1, 0].item() == 100.0     # 1.00390625 and 99.996 round to bf16
