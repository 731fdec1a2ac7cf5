"""HIP MX quantizer against the CPU oracle: packed codes and E8M0 scale bytes must be bit-identical."""
import pytest
import torch

import oracle as O
from conftest import make_qkv
from ours import _lib
from ours.quant_mxint8 import seq_mean, quantize_mx, quantize_mx_dual, quant_mxfp4, quant_mxfp8, quant_mxfp8e5, pre_scale_q

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
FMTS = [O.FMT_E2M1, O.FMT_E4M3, O.FMT_E5M2]


def _check(x, pre, fmt, **kw):
    codes, scales = quantize_mx(x.to(DEV), pre, fmt, **kw)
    want_c, want_s = O.quantize_mx(x, pre, fmt)
    n = x.shape[2]
    assert torch.equal(scales[:, :, :n].cpu(), want_s), "scale bytes differ"
    bad = (codes[:, :, :n].cpu() != want_c)
    assert not bad.any(), f"{bad.sum().item()} code bytes differ (fmt {fmt})"
    return codes, scales


@pytest.mark.parametrize("fmt", FMTS)
def test_c1_shapes(fmt):
    q, k, _ = make_qkv(1, 8, 8, 1024, 64, seed=0)
    assert pre_scale_q(64) == O.q_pre_scale(64)
    _check(q, O.q_pre_scale(64), fmt)
    _check(k, 1.0, fmt)


@pytest.mark.parametrize("fmt", FMTS)
def test_c3_shapes_with_outlier_channels(fmt):
    q, k, _ = make_qkv(1, 8, 2, 8192, 128, seed=2, outliers=True)
    _check(q, O.q_pre_scale(128), fmt)
    _check(k, 1.0, fmt)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_wide_dynamic_range_zero_blocks_and_tiny_values(dtype):
    g = torch.Generator().manual_seed(9)
    x = torch.randn(2, 3, 257, 128, generator=g) * torch.exp2(torch.randint(-14, 14, (2, 3, 257, 1), generator=g).float())
    x[0, 0, 5] = 0
    x[1, 2, 100, 32:64] = 0
    x[0, 1, 7, :32] = -0.0
    x[1, 1, 9, 64:96] = 6e-8 if dtype == torch.float16 else 1e-38
    x = x.to(dtype)
    for fmt in FMTS:
        _check(x, 1.0, fmt)
        _check(x, O.q_pre_scale(128), fmt)


def test_near_tie_values_follow_the_biased_compare():
    """Q-path style inputs: bf16 values whose float32 product with the pre-scale lands within 1e-6 of a grid
    midpoint are rare, so force them: pre-scale 1 and values at midpoints +- a few float32 ulps are not bf16 --
    instead use fp16 inputs with a pre-scale that maps them next to midpoints."""
    mids = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0])
    base = torch.tensor([0.5, 1.5, 2.5, 3.5, 5.0, 7.0, 10.0])       # fp16-exact; base * 0.5 = midpoint
    rows = []
    for ulps in range(-6, 7):
        pre = float(torch.tensor(0.5).view(torch.int32).add(ulps).view(torch.float32))
        row = torch.zeros(32)
        row[:7] = base
        row[7] = 16.0                                                # pins amax: 16*pre in [4,8)*... -> scale 2^-1.. checked by oracle
        rows.append((pre, row))
    for pre, row in rows:
        x = row.reshape(1, 1, 1, 32).to(torch.float16)
        _check(x, pre, O.FMT_E2M1)
    assert mids.numel() == 7


def test_dual_equals_single_and_padding_rows_are_zero():
    q, _, _ = make_qkv(1, 4, 4, 200, 128, seed=4)
    pre = O.q_pre_scale(128)
    c4, s4, c8, s8 = quantize_mx_dual(q.to(DEV), pre, _lib.FMT_E4M3, out_rows=256)
    a4, b4 = _check(q, pre, O.FMT_E2M1, out_rows=256)
    a8, b8 = _check(q, pre, O.FMT_E4M3, out_rows=256)
    assert torch.equal(c4, a4) and torch.equal(s4, b4) and torch.equal(c8, a8) and torch.equal(s8, b8)
    for t in (c4, s4, c8, s8):
        assert t.shape[2] == 256 and (t[:, :, 200:] == 0).all()
    d4, t4, d5, t5 = quantize_mx_dual(q.to(DEV), pre, _lib.FMT_E5M2)
    w5, ws5 = O.quantize_mx(q, pre, O.FMT_E5M2)
    assert torch.equal(d5.cpu(), w5) and torch.equal(t5.cpu(), ws5) and torch.equal(d4, c4[:, :, :200])


def test_reference_style_entry_points_and_layouts():
    q, k, _ = make_qkv(2, 4, 2, 256, 64, seed=6)
    qd, kd = q.to(DEV), k.to(DEV)
    qc, qs, kc, ks = quant_mxfp4(qd, kd)
    wq, wqs = O.quantize_mx(q, O.q_pre_scale(64), O.FMT_E2M1)
    wk, wks = O.quantize_mx(k, 1.0, O.FMT_E2M1)
    assert torch.equal(qc.cpu(), wq) and torch.equal(qs.cpu(), wqs) and torch.equal(kc.cpu(), wk) and torch.equal(ks.cpu(), wks)
    # one code per byte, as the reference returns them
    qu, _, _, _ = quant_mxfp4(qd, kd, packed=False)
    assert qu.shape == q.shape and torch.equal(qu.cpu(), O.unpack_fp4(wq))
    # NHD: [B, L, H, D] input is read through its strides, outputs stay [B, H, L, *]
    qn, kn = qd.transpose(1, 2).contiguous(), kd.transpose(1, 2).contiguous()
    qc2, qs2, kc2, ks2 = quant_mxfp4(qn, kn, tensor_layout="NHD")
    assert torch.equal(qc2, qc) and torch.equal(ks2, ks)
    # custom softmax scale and the 8-bit siblings
    qc3, qs3, _, _ = quant_mxfp8(qd, kd, sm_scale=0.3)
    w3, ws3 = O.quantize_mx(q, O.q_pre_scale(64, 0.3), O.FMT_E4M3)
    assert torch.equal(qc3.cpu(), w3) and torch.equal(qs3.cpu(), ws3)
    qc5, _, kc5, ks5 = quant_mxfp8e5(qd, kd)
    assert qc5.dtype == torch.float8_e5m2
    w5, ws5 = O.quantize_mx(k, 1.0, O.FMT_E5M2)
    assert torch.equal(kc5.view(torch.uint8).cpu(), w5) and torch.equal(ks5.cpu(), ws5)
    with pytest.raises(ValueError, match="Unknown tensor layout"):
        quant_mxfp4(qd, kd, tensor_layout="DNH")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape", [(1, 8, 8192, 128), (2, 3, 1000, 64), (1, 2, 32760, 128), (1, 1, 7, 64)])
def test_smooth_k_mean_and_fused_subtraction(shape, dtype):
    """mpsa_seq_mean against the oracle's once-rounded mean (summation order may move the 16-bit result by one
    unit in the last place on rare channels: at most 1 ulp anywhere, equal on more than 99 %), and the
    quantizer's fused ``x - mean`` bit for bit against the oracle quantizing ``smooth_k(k, that mean)``."""
    B, H, N, D = shape
    g = torch.Generator().manual_seed(N + D)
    k = (torch.randn(B, H, N, D, generator=g) + torch.randn(1, H, 1, D, generator=g) * 2).to(dtype)
    got = seq_mean(k.to(DEV))
    assert got.shape == (B, H, D) and got.dtype == dtype
    want = O.seq_mean(k).squeeze(-2)
    same = (got.cpu() == want)
    assert same.float().mean().item() > 0.99
    ulp = torch.finfo(dtype).eps * want.float().abs().clamp_min(2.0 ** -14)
    assert ((got.cpu().float() - want.float()).abs() <= ulp).all()
    smoothed = O.smooth_k(k, got.cpu())
    for fmt in FMTS:
        codes, scales = quantize_mx(k.to(DEV), 1.0, fmt, sub=got)
        want_c, want_s = O.quantize_mx(smoothed, 1.0, fmt)
        assert torch.equal(scales.cpu(), want_s) and torch.equal(codes.cpu(), want_c), f"fmt {fmt}"
    c4, s4, c8, s8 = quantize_mx_dual(k.to(DEV), 1.0, O.FMT_E4M3, out_rows=N + 9, sub=got)
    w4, ws4 = O.quantize_mx(smoothed, 1.0, O.FMT_E2M1)
    w8, ws8 = O.quantize_mx(smoothed, 1.0, O.FMT_E4M3)
    assert torch.equal(c4[:, :, :N].cpu(), w4) and torch.equal(s4[:, :, :N].cpu(), ws4)
    assert torch.equal(c8[:, :, :N].cpu(), w8) and torch.equal(s8[:, :, :N].cpu(), ws8)
    assert not c4[:, :, N:].any() and not c8[:, :, N:].any() and not s4[:, :, N:].any()


def test_hardware_e2m1_conversion_agrees_with_the_explicit_rule_near_every_midpoint():
    """The quantizer's fast path (hardware FP4 conversion) must hand every value near a rounding boundary to
    the explicit rule: float32-dense sweeps around each of the seven midpoints, reached through a pre-scale
    that makes the scaled values arbitrary float32 numbers, and blocks whose scale is not a normal float32."""
    mids = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0])
    rows = []
    for m in mids.tolist():
        base = torch.tensor(m, dtype=torch.float32)
        steps = torch.arange(-24, 25, dtype=torch.float32)
        vals = base + steps * 1.25e-7 * max(m, 1.0)            # a few float32 ulps either side, +-3e-6
        for chunk in vals.split(31):
            blk = torch.full((32,), 0.0)
            blk[0] = 6.0                                        # pins the shared exponent: scale 2^(2-3)... = 0.5
            blk[1:1 + chunk.numel()] = chunk
            rows.append(blk)
            rows.append(-blk)
    x = torch.stack(rows)                                       # [R, 32] float32 targets of x*pre / 2^se with se = -1
    # choose bf16 inputs and a pre-scale so that f32(x)*pre lands on arbitrary float32 values near the targets
    pre = 0.7310585975646973
    xin = (x * 0.5 / pre).bfloat16().view(1, 1, -1, 32)
    xin = torch.cat([xin, (xin.float() * 2.0 ** -120).bfloat16()], dim=2)       # tiny blocks: scale below 2^-126
    for p in (pre, 1.0, 0.9999998807907104, 1.0000001192092896):
        codes, scales = quantize_mx(xin.to(DEV), p, O.FMT_E2M1)
        want_c, want_s = O.quantize_mx(xin, p, O.FMT_E2M1)
        assert torch.equal(scales.cpu(), want_s) and torch.equal(codes.cpu(), want_c), f"pre {p}"
    # a dense float32 sweep through the pre-scale instead of the input: the scaled value walks across each midpoint
    one = torch.zeros(1, 1, 1, 32); one[..., 0] = 6.0
    for m in mids.tolist():
        xb = one.clone(); xb[..., 1:] = m
        xb = xb.bfloat16()
        for k in range(-40, 41):
            p = float(torch.tensor(1.0 + k * 2.0 ** -23, dtype=torch.float32))
            if (xb.float().abs().max() * p) >= 8.0:
                continue
            codes, scales = quantize_mx(xb.to(DEV), p, O.FMT_E2M1)
            want_c, want_s = O.quantize_mx(xb, p, O.FMT_E2M1)
            assert torch.equal(codes.cpu(), want_c) and torch.equal(scales.cpu(), want_s), f"mid {m} pre {p}"


@pytest.mark.parametrize("fmt", [O.FMT_E2M1, O.FMT_E4M3])
def test_c2_gemm_operand_full_size(fmt):
    """The 8192 x 8192 GEMM operand of the standalone config, quantized along K: every byte against the oracle."""
    g = torch.Generator().manual_seed(1)
    a = torch.randn(8192, 8192, generator=g).bfloat16()
    codes, scales = quantize_mx(a.to(DEV)[None, None], 1.0, fmt)
    codes, scales = codes[0, 0].cpu(), scales[0, 0].cpu()
    for r0 in range(0, 8192, 2048):                       # oracle in slabs to bound host memory
        wc, ws = O.quantize_mx(a[r0:r0 + 2048], 1.0, fmt)
        assert torch.equal(codes[r0:r0 + 2048], wc) and torch.equal(scales[r0:r0 + 2048], ws)


def test_empty_and_single_row_inputs():
    """Zero heads / zero rows are accepted and write nothing; one row works."""
    for shape in [(0, 2, 16, 64), (1, 0, 16, 64), (1, 2, 0, 64)]:
        x = torch.empty(shape, dtype=torch.bfloat16, device=DEV)
        codes, scales = quantize_mx(x, 1.0, O.FMT_E2M1)
        assert codes.shape == (*shape[:3], 32) and scales.shape == (*shape[:3], 2)
    x = torch.randn(1, 1, 1, 32).bfloat16()
    _check(x, 1.0, O.FMT_E2M1)
    _check(x, 1.0, O.FMT_E4M3, out_rows=5)
