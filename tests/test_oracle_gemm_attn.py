"""Pins the CPU oracle's block-scaled matmul and tiled attention (no GPU needed)."""
import pytest
import torch

import oracle as O
from conftest import make_qkv


def test_gemm_against_exact_integer_arithmetic():
    """2*E2M1 values are integers and scales are powers of two, so with every scale exponent made
    non-negative the product is an integer computable exactly in int64."""
    g = torch.Generator().manual_seed(7)
    M, N, K = 48, 40, 256
    a_codes = torch.randint(0, 16, (M, K), dtype=torch.uint8, generator=g)
    b_codes = torch.randint(0, 16, (N, K), dtype=torch.uint8, generator=g)
    sa = torch.randint(127, 131, (M, K // 32), dtype=torch.uint8, generator=g)
    sb = torch.randint(127, 131, (N, K // 32), dtype=torch.uint8, generator=g)
    table2 = torch.tensor([0, 1, 2, 3, 4, 6, 8, 12, 0, -1, -2, -3, -4, -6, -8, -12], dtype=torch.int64)
    ai = table2[a_codes.long()] * (2 ** (sa.long() - 127)).repeat_interleave(32, dim=1)
    bi = table2[b_codes.long()] * (2 ** (sb.long() - 127)).repeat_interleave(32, dim=1)
    want = (ai @ bi.T).double() / 4.0
    got = O.gemm_mx(O.pack_fp4(a_codes), sa, O.pack_fp4(b_codes), sb, O.FMT_E2M1, acc_dtype=torch.float64)
    assert torch.equal(got, want)
    got32 = O.gemm_mx(O.pack_fp4(a_codes), sa, O.pack_fp4(b_codes), sb, O.FMT_E2M1)
    assert torch.allclose(got32.double(), want, rtol=1e-5, atol=1e-3)


def test_gemm_fp8_against_float64_loop():
    g = torch.Generator().manual_seed(8)
    M, N, K = 8, 6, 64
    a = torch.randn(M, K, generator=g).bfloat16()
    b = torch.randn(N, K, generator=g).bfloat16()
    ac, asc = O.quantize_mx(a, 1.0, O.FMT_E4M3)
    bc, bsc = O.quantize_mx(b, 1.0, O.FMT_E4M3)
    got = O.gemm_mx(ac, asc, bc, bsc, O.FMT_E4M3, acc_dtype=torch.float64)
    av = O.decode_e4m3(ac).double()
    bv = O.decode_e4m3(bc).double()
    for m in range(M):
        for n in range(N):
            acc = 0.0
            for kb in range(K // 32):
                blk = sum(av[m, kb * 32 + i].item() * bv[n, kb * 32 + i].item() for i in range(32))
                acc += blk * 2.0 ** (int(asc[m, kb]) - 127) * 2.0 ** (int(bsc[n, kb]) - 127)
            assert abs(got[m, n].item() - acc) <= 1e-9 * max(1.0, abs(acc))
    # quantized product is close to the unquantized one (E4M3: 2^-4 relative per element)
    exact = a.double() @ b.double().T
    assert (got - exact).abs().max() < 0.08 * exact.abs().max() + 0.5


@pytest.mark.parametrize("mode", ["mxfp4", "mxfp8", "diag", "mixed"])
@pytest.mark.parametrize("causal", [True, False])
def test_attention_tile_loop_equals_dense_float64(mode, causal):
    q, k, v = make_qkv(1, 4, 2, 200, 64, seed=21)          # N not a multiple of the tile, GQA 2:1
    got = O.attn_mx(q, k, v, tile=64, causal=causal, mode=mode, out_dtype=torch.float32)
    want = O.attn_dense_f64(q, k, v, tile=64, causal=causal, mode=mode)
    m = O.precision_metric(got, want)
    assert m["cos"] > 0.99999 and m["max_abs"] < 1.5e-2     # only bf16 rounding of P separates the two


def test_attention_special_cases():
    q, k, v = make_qkv(1, 2, 2, 128, 64, seed=22)
    # single tile: "diag" is pure 8-bit causal attention
    a = O.attn_mx(q, k, v, tile=128, causal=True, mode="diag", out_dtype=torch.float32)
    b = O.attn_mx(q, k, v, tile=128, causal=True, mode="mxfp8", out_dtype=torch.float32)
    assert torch.equal(a, b)
    # V = 1 -> every output is 1 up to the bf16 rounding of P
    ones = torch.ones_like(v)
    o = O.attn_mx(q, k, ones, tile=64, causal=True, mode="diag", out_dtype=torch.float32)
    assert (o - 1).abs().max() < 4e-3
    # identical keys -> uniform weights -> running mean of V rows (causal)
    k_same = k[:, :, :1].expand_as(k).contiguous()
    o = O.attn_mx(q, k_same, v, tile=64, causal=True, mode="mxfp4", out_dtype=torch.float32)
    want = v.float().cumsum(dim=2) / torch.arange(1, 129).view(1, 1, -1, 1)
    assert (o - want).abs().max() < 2e-2
    # first causal row attends to key 0 only
    o = O.attn_mx(q, k, v, tile=64, causal=True, mode="diag", out_dtype=torch.float32)
    assert torch.equal(o[:, :, 0], v.float()[:, :, 0])


def test_gqa_equals_repeat_interleave_and_head_subset():
    q, k, v = make_qkv(1, 4, 2, 128, 64, seed=23)
    a = O.attn_mx(q, k, v, tile=64, causal=True, mode="diag")
    b = O.attn_mx(q, k.repeat_interleave(2, dim=1), v.repeat_interleave(2, dim=1), tile=64, causal=True, mode="diag")
    assert torch.equal(a, b)
    c = O.attn_mx(q, k, v, tile=64, causal=True, mode="diag", heads=[1, 3])
    assert torch.equal(c, a[:, [1, 3]])


def test_attention_close_to_unquantized_in_8bit():
    q, k, v = make_qkv(1, 2, 2, 256, 64, seed=24)
    got = O.attn_mx(q, k, v, tile=64, causal=True, mode="mxfp8", out_dtype=torch.float32)
    ref = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float(), is_causal=True)
    assert O.precision_metric(got, ref)["cos"] > 0.995


def test_v_fragment_order_is_a_permutation_with_zero_padding():
    v = torch.arange(1, 1 + 100 * 64, dtype=torch.float32).reshape(1, 1, 100, 64).bfloat16()
    f = O.v_fragment_order(v, 64)
    assert f.shape == (1, 1, 2, 2, 2, 2, 64, 8)
    # spot-check the index formula: tile 1, kb 0, c 1, db 1, lane 37 (h=1, r=5), t 6 -> key 64+16+8+4+2, dim 37
    assert f[0, 0, 1, 0, 1, 1, 37, 6] == v[0, 0, 64 + 16 + 8 + 4 + 2, 37]
    assert f[0, 0, 0, 1, 0, 0, 3, 1] == v[0, 0, 32 + 1, 3]
    assert f.float().sum() == v.float().sum()                # padding keys are zero
    assert (f[0, 0, 1, 1, 0, :, :32, 4:] == 0).all()          # keys 64+32+8.. >= 100


def test_tile_skipping_rule_against_a_dense_float64_restatement():
    """attn_mx(skip_thresh=...) against an independent dense formulation: dequantised operands, one float64 score
    matrix, tile statistics = mean over the tile's rows of the row maximum, decisions relative to key tile 0, then a
    float64 softmax over the kept tiles only."""
    from oracle.mx_attention import _prepare
    g = torch.Generator().manual_seed(11)
    B, H, N, D, tile = 1, 2, 320, 64, 64
    q = torch.randn(B, H, N, D, generator=g)
    k = torch.randn(B, H, N, D, generator=g)
    v = torch.randn(B, H, N, D, generator=g).bfloat16()
    nt = N // tile
    # a common direction in q and a per-tile amount of it in k spread the tile statistics out
    q = q + 1.0
    k = k + torch.rand(nt, generator=g).repeat_interleave(tile).view(1, 1, N, 1) * 0.5
    q, k = q.bfloat16(), k.bfloat16()
    for causal in (False, True):
        for th in (0.7, 0.9, 1.05):
            got, sk = O.attn_mx(q, k, v, tile=tile, causal=causal, mode="mxfp4", skip_thresh=th, return_skipped=True,
                                out_dtype=torch.float32)
            ops = _prepare(q, k, "mxfp4", None, O.FMT_E4M3)
            s = ops["q4"].double() @ ops["k4"].double().transpose(-1, -2)            # [B,H,N,N], log2 units
            if causal:
                s = s.masked_fill(torch.triu(torch.ones(N, N, dtype=torch.bool), 1), float("-inf"))
            keep = torch.ones(B, H, nt, nt, dtype=torch.bool)
            for i in range(nt):
                rows = slice(i * tile, (i + 1) * tile)
                last = i if causal else nt - 1
                stat = [s[:, :, rows, j * tile:(j + 1) * tile].amax(dim=-1).mean(dim=-1) for j in range(last + 1)]
                for j in range(1, last + 1):
                    keep[:, :, i, j] = stat[j] >= stat[0] * th
                if causal:
                    keep[:, :, i, i] = True           # the diagonal tile is exempt
                if causal:
                    keep[:, :, i, i + 1:] = True      # not visited: already -inf
            mask = keep.repeat_interleave(tile, 2).repeat_interleave(tile, 3)
            p = torch.softmax(s.masked_fill(~mask, float("-inf")) * 0.6931471805599453, dim=-1)
            want = p @ v.double()
            visited = torch.tril(torch.ones(nt, nt, dtype=torch.bool)) if causal else torch.ones(nt, nt, dtype=torch.bool)
            assert torch.equal(sk, ((~keep) & visited).sum(dim=-1).to(torch.int32))
            assert 0 < sk.sum() < visited.sum() * B * H
            assert (got.double() - want).abs().max() < 2e-2


def test_scale_5d_layout_index_formula_and_round_trip():
    rows, kb = 256, 8
    lin = torch.arange(2 * rows * kb, dtype=torch.int64).remainder(251).to(torch.uint8).view(2, rows, kb)
    pk = O.scales_to_5d(lin)
    assert pk.shape == (2, rows // 128, kb // 4, 32, 4, 4)
    for (bt, cm, ck, r32, r4, c4) in [(0, 0, 0, 0, 0, 0), (1, 1, 1, 31, 3, 3), (0, 1, 0, 7, 2, 1), (1, 0, 1, 30, 1, 2)]:
        assert pk[bt, cm, ck, r32, r4, c4] == lin[bt, cm * 128 + r4 * 32 + r32, ck * 4 + c4]
    assert torch.equal(O.scales_from_5d(pk), lin)


def test_mixed_mode_is_8bit_q_times_4bit_k():
    """The "mixed" scores are exactly dq8(Q) dq4(K)^T: with a single key (softmax weight 1) nothing else shows, so the
    check goes through a two-key softmax whose weights follow from the score difference alone."""
    torch.manual_seed(5)
    q = torch.randn(1, 1, 1, 64).bfloat16()
    k = torch.randn(1, 1, 2, 64).bfloat16()
    v = torch.tensor([[[[1.0] * 64, [0.0] * 64]]]).bfloat16()
    pre = O.q_pre_scale(64)
    q8 = O.dequantize_mx(*O.quantize_mx(q, pre, O.FMT_E4M3), O.FMT_E4M3).double()
    k4 = O.dequantize_mx(*O.quantize_mx(k, 1.0, O.FMT_E2M1), O.FMT_E2M1).double()
    s = (q8[0, 0] @ k4[0, 0].T)[0]
    want = 1.0 / (1.0 + 2.0 ** float(s[1] - s[0]))
    got = O.attn_mx(q, k, v, tile=64, causal=False, mode="mixed", out_dtype=torch.float32)
    assert abs(got[0, 0, 0, 0].item() - want) < 4e-3            # P is rounded to bf16
    other = O.attn_mx(q, k, v, tile=64, causal=False, mode="mxfp4", out_dtype=torch.float32)
    assert got[0, 0, 0, 0].item() != other[0, 0, 0, 0].item()
