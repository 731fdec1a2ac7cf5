"""Seeded random sweeps of the attention and matmul entry points against the CPU oracle: shapes, head grouping,
ragged lengths, cross attention, every precision mode incl. routed, both 16-bit input types.  The fixed-shape tests
name their cases; this one walks combinations nobody thought of (an earlier sweep of this kind found a look-ahead
that read K scales out of bounds when a cross-attention run had more query tiles than key tiles)."""
import random

import numpy as np
import pytest
import torch

import oracle as O
from conftest import make_qkv, attention_close, check_attention
from ours.block_scaled_matmul import block_scaled_matmul, quantize_block_scaled_from_tensor
from ours.mxfp_attn_kernel import prepare_operands, route_tiles, attention_from_operands, mxfp_attn_kernel
from ours.quant_mxint8 import quantize_mx, quantize_mx_dual

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _attention_case(rnd):
    D = rnd.choice([64, 128]); tile = rnd.choice([64, 128])
    Hkv = rnd.choice([1, 2]); Hq = Hkv * rnd.choice([1, 2, 4])
    N = max(128, rnd.randint(1, 6) * tile - rnd.choice([0, 0, 1, 17, tile // 2, tile - 1]))
    mode = rnd.choice(["mxfp4", "mxfp8", "diag", "routed", "routed", "mxfp8e5", "routed_e5"])
    causal = rnd.random() < 0.5
    cross = (not causal) and mode != "diag" and rnd.random() < 0.3
    Nk = max(64, rnd.randint(1, 6) * tile - rnd.choice([0, 3, tile // 2])) if cross else N
    dt = rnd.choice([torch.bfloat16, torch.float16])
    return dict(D=D, tile=tile, Hq=Hq, Hkv=Hkv, N=N, Nk=Nk, mode=mode, causal=causal, cross=cross, dt=dt,
                seed=rnd.randint(0, 10 ** 6), hi=rnd.choice([None, 0.3, 0.6, 0.9]), lo=rnd.choice([None, 0.05, 0.3]))


@pytest.mark.parametrize("sweep_seed", [11, 12])
def test_attention_sweep(sweep_seed):
    rnd = random.Random(sweep_seed)
    for c in range(40):
        p = _attention_case(rnd)
        what = f"sweep {sweep_seed} case {c}: {p}"
        print(what, flush=True)
        q, k, v = make_qkv(1, p["Hq"], p["Hkv"], p["N"], p["D"], seed=p["seed"], dtype=p["dt"])
        if p["cross"]:
            _, k, v = make_qkv(1, p["Hq"], p["Hkv"], p["Nk"], p["D"], seed=p["seed"] + 1, dtype=p["dt"])
        g = torch.Generator().manual_seed(p["seed"] + 7)
        for t in (q, k):                                   # magnitudes that differ from tile to tile
            n = t.shape[2]
            gain = torch.exp2(torch.randint(-3, 3, (1, t.shape[1], -(-n // 64), 1), generator=g).float())
            t *= gain.repeat_interleave(64, dim=2)[:, :, :n].to(t.dtype)
        fmt8 = O.FMT_E5M2 if p["mode"].endswith("e5") else O.FMT_E4M3
        if p["mode"].startswith("routed"):
            ops = prepare_operands(q.to(DEV), k.to(DEV), v.to(DEV), p["tile"], p["mode"])
            route = route_tiles(ops, p["causal"], p["hi"], p["lo"])
            cls = route[0].cpu().numpy()
            want_cls = O.route_tiles(ops["qs4"].cpu().numpy(), ops["ks4"].cpu().numpy(), p["tile"], p["causal"], p["hi"], p["lo"])
            assert np.array_equal(cls, want_cls), what
            def run(dt):
                out = torch.empty((1, p["Hq"], p["N"], p["D"]), dtype=dt, device=DEV)
                return attention_from_operands(ops, out, p["causal"], route=route)
            want = O.attn_mx(q, k, v, tile=p["tile"], causal=p["causal"], mode="routed", route=cls, fmt8=fmt8, out_dtype=torch.float32)
        else:
            def run(dt):
                return mxfp_attn_kernel(q.to(DEV), k.to(DEV), v.to(DEV), is_causal=p["causal"], block_scale_type=p["mode"],
                                        tile=p["tile"], output_dtype=dt)
            want = O.attn_mx(q, k, v, tile=p["tile"], causal=p["causal"], mode={"mxfp8e5": "mxfp8"}.get(p["mode"], p["mode"]),
                             fmt8=fmt8, out_dtype=torch.float32)
        # the bar on the float32 outputs; the 16-bit output of the case's dtype is the rounded float32 one
        check_attention(run, want, what, p["dt"])


def _paired_tile_sweep(causal, sweep_seed, cases, any_length=False):
    rnd = random.Random(sweep_seed)
    for c in range(cases):
        Hkv = rnd.choice([1, 2]); Hq = Hkv * rnd.choice([1, 2, 4])
        if causal and any_length:
            N = 128 * rnd.randint(2, 12) - rnd.choice([0, 1, 37, 100, 127])
        elif causal:
            N = 256 * rnd.randint(1, 6)
        else:
            N = 128 * rnd.randint(6, 14) - rnd.choice([0, 0, 1, 37, 100, 127])    # the last tile ragged or not
        mode = rnd.choice(["mxfp4", "diag", "diag", "diag_e5"])
        dt = rnd.choice([torch.bfloat16, torch.float16])
        seed = rnd.randint(0, 10 ** 6)
        shape = rnd.choice(["gain", "ramp", "spikes"])
        rate = rnd.choice([0.5, 1.0, 3.0, 5.0]); height = rnd.choice([2.0, 6.0, 9.0])
        what = f"paired sweep case {c}: causal={causal} Hq={Hq} Hkv={Hkv} N={N} mode={mode} {dt} seed={seed} {shape} rate={rate} height={height}"
        print(what, flush=True)
        q, k, v = make_qkv(1, Hq, Hkv, N, 128, seed=seed, dtype=dt)
        g = torch.Generator().manual_seed(seed + 7)
        nt = (N + 127) // 128
        if shape == "gain":
            for t in (q, k):
                gain = torch.exp2(torch.randint(-3, 3, (1, t.shape[1], 2 * nt, 1), generator=g).float())
                t *= gain.repeat_interleave(64, dim=2)[:, :, :N].to(t.dtype)
        else:
            u = torch.sign(torch.randn(128, generator=g))
            if shape == "ramp":
                gk = torch.arange(N, dtype=torch.float32) / 128 * rate
            else:
                gk = ((torch.rand(nt, generator=g) < 0.3).float().repeat_interleave(128) * height)[:N]
            q = (q.float() * 0.3 + u).to(dt)
            k = (k.float() * 0.3 + gk[:, None] * u).to(dt)
        fmt8 = O.FMT_E5M2 if mode.endswith("e5") else O.FMT_E4M3
        got = mxfp_attn_kernel(q.to(DEV), k.to(DEV), v.to(DEV), is_causal=causal, block_scale_type=mode, tile=128,
                               output_dtype=torch.float32)
        want = O.attn_mx(q, k, v, tile=128, causal=causal, mode="diag" if mode.startswith("diag") else mode, fmt8=fmt8,
                         out_dtype=torch.float32)
        assert torch.isfinite(got).all(), what
        attention_close(got, want, what)


def test_paired_tile_kernel_sweep():
    """The paired-tile kernel's causal shapes (D = 128, 128x128 tiles, whole tile pairs) with score profiles that
    make its running maximum move at unpredictable places: per-64-row gains, scores climbing along the keys at
    different rates, and random tiles towering over the rest."""
    _paired_tile_sweep(True, 21, 40)


def test_paired_tile_kernel_sweep_causal_any_length():
    """The same with lengths that leave the last tile ragged or the last pair with one tile."""
    _paired_tile_sweep(True, 23, 30, any_length=True)


def test_paired_tile_kernel_sweep_without_the_mask():
    """The same score profiles on the kernel's unmasked shapes (six tiles or more, the last one ragged in most cases): the tiles are visited out of order there -- the pair's two diagonal tiles and the ragged tile last --
    so a running maximum that moves in the late straight-line steps is covered too (the ramp peaks in the last tile)."""
    _paired_tile_sweep(False, 22, 30)


def test_matmul_sweep():
    rnd = random.Random(21)
    types = {"mxfp4": O.FMT_E2M1, "mxfp8": O.FMT_E4M3, "mxfp8e5": O.FMT_E5M2}
    for c in range(16):
        M = 256 * rnd.randint(1, 3); N = 256 * rnd.randint(1, 4); K = 128 * rnd.randint(1, 20)
        bst = rnd.choice(list(types)); fmt = types[bst]
        dt = rnd.choice([torch.float32, torch.bfloat16, torch.float16])
        what = f"case {c}: M={M} N={N} K={K} {bst} out={dt}"
        print(what, flush=True)
        g = torch.Generator().manual_seed(rnd.randint(0, 10 ** 6))
        scale_a = torch.exp2(torch.randint(-4, 4, (M, K // 32), generator=g).float()).repeat_interleave(32, 1)
        a = (torch.randn(M, K, generator=g) * scale_a).bfloat16()
        b = torch.randn(N, K, generator=g).bfloat16()
        ac, asc, bc, bsc, cfg = quantize_block_scaled_from_tensor(a.to(DEV), b.to(DEV), bst)
        got = block_scaled_matmul(ac, asc, bc, bsc, dt, M, N, K, cfg).cpu()
        da = O.dequantize_mx(ac.cpu(), asc.cpu(), fmt, torch.float64)
        db = O.dequantize_mx(bc.cpu(), bsc.cpu(), fmt, torch.float64)
        want, mag = da @ db.T, da.abs() @ db.abs().T
        out_rounding = {torch.float32: 0.0, torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -10}[dt]
        err = (got.double() - want).abs()
        bound = (1e-7 * mag + out_rounding * want.abs()) if fmt == O.FMT_E2M1 else ((1e-3 + out_rounding) * want.abs() + 3e-5 * mag)
        assert not (err > bound).any(), what


def test_quantizer_sweep():
    """Codes and scale bytes bit-exact: random shapes, magnitudes over 40 binades, pre-scales, padding, strided
    ("NHD") inputs, single and dual output."""
    rnd = random.Random(31)
    for c in range(30):
        B, H = rnd.choice([1, 2]), rnd.choice([1, 3])
        N = rnd.choice([1, 31, 64, 100, 257, 640]); D = rnd.choice([64, 128, 256])
        dt = rnd.choice([torch.bfloat16, torch.float16])
        pre = rnd.choice([1.0, 0.5, O.q_pre_scale(D), 0.1275, 3.0])
        out_rows = N + rnd.choice([0, 0, 5, 128 - N % 128])
        what = f"case {c}: B={B} H={H} N={N} D={D} {dt} pre={pre} out_rows={out_rows}"
        print(what, flush=True)
        g = torch.Generator().manual_seed(rnd.randint(0, 10 ** 6))
        spread = 20 if dt == torch.bfloat16 else 6
        mag = torch.exp2(torch.randint(-spread, spread, (B, H, N, D // 32), generator=g).float()).repeat_interleave(32, 3)
        x = (torch.randn(B, H, N, D, generator=g) * mag).to(dt)
        xd = x.to(DEV)
        if rnd.random() < 0.5:                             # the same values behind "NHD" strides
            xd = xd.transpose(1, 2).contiguous().transpose(1, 2)
        for fmt in (O.FMT_E2M1, O.FMT_E4M3, O.FMT_E5M2):
            codes, scales = quantize_mx(xd, pre, fmt, out_rows=out_rows)
            want_c, want_s = O.quantize_mx(x, pre, fmt)
            assert torch.equal(scales[:, :, :N].cpu(), want_s) and torch.equal(codes[:, :, :N].cpu(), want_c), f"{what} fmt {fmt}"
            assert not scales[:, :, N:].any() and not codes[:, :, N:].any(), f"{what}: padding rows must be zero"
        c4, s4, c8, s8 = quantize_mx_dual(xd, pre, out_rows=out_rows)
        w4, ws4 = O.quantize_mx(x, pre, O.FMT_E2M1)
        w8, ws8 = O.quantize_mx(x, pre, O.FMT_E4M3)
        assert torch.equal(c4[:, :, :N].cpu(), w4) and torch.equal(s4[:, :, :N].cpu(), ws4), f"{what} dual 4-bit"
        assert torch.equal(c8[:, :, :N].cpu(), w8) and torch.equal(s8[:, :, :N].cpu(), ws8), f"{what} dual 8-bit"



def test_tile_skipping_ahead_and_inside_agree_over_shapes():
    """The rule decided ahead of the attention kernel (statistics pass + visiting lists + routed attention) against the rule
    inside the attention kernel -- which the oracle pins (test_gpu_attn.py) -- from one tile to sixteen, whole and ragged
    lengths, even and odd tile counts, with and without the mask, grouped heads: the same tiles skipped per query tile
    and the same output, at thresholds on both sides of the sink's statistic."""
    from ours.mxfp_attn_kernel import skip_routable
    cases = 0
    for N in [128, 129, 200, 256, 257, 300, 384, 385, 500, 512, 513, 640, 700, 769, 896, 1000, 1025, 1152, 1300, 1537, 2000]:
        for causal in (True, False):
            for mode in ("mxfp4", "diag", "mxfp8"):
                H, G = (4, 2) if N % 3 else (2, 1)
                g = torch.Generator().manual_seed(N * 7 + H)
                nt = -(-N // 128)
                q = (torch.randn(1, H, N, 128, generator=g) + 1.0).bfloat16().to(DEV)
                k = (torch.randn(1, H // G, N, 128, generator=g) + torch.rand(nt, generator=g).repeat_interleave(128)[:N].view(1, 1, N, 1) * 0.5).bfloat16().to(DEV)
                v = torch.randn(1, H // G, N, 128, generator=g).bfloat16().to(DEV)
                ops = prepare_operands(q, k, v, 128, mode)
                assert skip_routable(ops, causal)
                for th in (0.98, 1.02):
                    ahead = torch.full((1, H, N, 128), float("nan"), dtype=torch.float32, device=DEV)
                    inside = torch.full_like(ahead, float("nan"))
                    sk_a = torch.full((1, H, nt), -1, dtype=torch.int32, device=DEV)
                    sk_i = torch.full_like(sk_a, -1)
                    attention_from_operands(ops, ahead, causal, th, sk_a)
                    attention_from_operands(ops, inside, causal, th, sk_i, skip_in_kernel=True)
                    what = f"N={N} causal={causal} {mode} H={H} G={G} th={th}"
                    assert torch.equal(sk_a, sk_i), what
                    assert torch.equal(ahead, inside), what      # both walk the kept tiles through the same kernel code
                    cases += 1
    assert cases == 21 * 2 * 3 * 2
