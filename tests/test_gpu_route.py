"""Tile router and routed attention on the GPU against the CPU oracle.

The class map, the visiting lists and their run lengths are integer work: bit-exact.  Routed attention: cosine >= 0.999
and max-abs <= 2e-2 against the oracle's tile-by-tile attention on the same map, and bit-identical to the fixed
modes on the maps that describe them (same kernel, same visiting order)."""
import numpy as np
import pytest
import torch

import oracle as O
from conftest import make_qkv, attention_close, check_attention
from ours import _lib
from ours.mxfp_attn import mxfp_attn
from ours.mxfp_attn_kernel import prepare_operands, route_tiles, attention_from_operands, mxfp_attn_kernel

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _frames(q, k, n_frames, seed, amp):
    """Per-frame, per-channel offsets on q and k (the video-DiT input scheme): gives the tiles different magnitudes."""
    g = torch.Generator().manual_seed(seed)
    N = q.shape[2]
    per = -(-N // n_frames)
    for t in (q, k):
        off = amp * torch.randn(n_frames, 1, t.shape[-1], generator=g)
        frame = torch.arange(N) // per
        t += off[frame].reshape(1, 1, N, t.shape[-1]).to(t.dtype)
    return q, k


def _inputs(B, Hq, Hkv, N, D, seed, Nk=None):
    q, k, v = make_qkv(B, Hq, Hkv, N, D, seed=seed)
    if Nk is not None:
        _, k, v = make_qkv(B, Hq, Hkv, Nk, D, seed=seed + 1)
    g = torch.Generator().manual_seed(seed + 7)
    # magnitudes that differ from tile to tile, so that the router has something to decide
    for t in (q, k):
        n = t.shape[2]
        gain = torch.exp2(torch.randint(-3, 3, (1, t.shape[1], -(-n // 64), 1), generator=g).float())
        t *= gain.repeat_interleave(64, dim=2)[:, :, :n].to(t.dtype)
    return q, k, v


def _route_gpu(q, k, v, tile, causal, hi, lo, mode="routed"):
    ops = prepare_operands(q.to(DEV), k.to(DEV), v.to(DEV), tile, mode)
    return ops, route_tiles(ops, causal, hi, lo)


@pytest.mark.parametrize("D,tile", [(128, 128), (64, 64), (128, 64), (64, 128)])
@pytest.mark.parametrize("causal", [False, True])
def test_route_map_and_lists_bit_exact(D, tile, causal):
    N = 5 * tile + 37                                     # ragged: the last tile is cut
    q, k, v = _inputs(2, 4, 2, N, D, seed=300 + D + tile)
    ops, (cls, order, counts) = _route_gpu(q, k, v, tile, causal, 0.5, 0.01)
    qs4, ks4 = ops["qs4"].cpu().numpy(), ops["ks4"].cpu().numpy()
    want_cls = O.route_tiles(qs4, ks4, tile, causal, 0.5, 0.01)
    want_order, want_counts = O.route_order(want_cls, N, tile, causal)
    assert np.array_equal(cls.cpu().numpy(), want_cls)
    assert np.array_equal(counts.cpu().numpy(), want_counts)
    assert np.array_equal(order.cpu().numpy(), want_order)
    present = set(np.unique(want_cls).tolist())
    assert {1, 2} <= present, present                     # the case exercises both precisions


def test_route_many_key_tiles_and_thresholds():
    """More key tiles than one wave handles per pass (> 64), cross attention, each threshold alone."""
    q, k, v = _inputs(1, 2, 1, 3 * 64 + 5, 64, seed=320, Nk=70 * 64 + 11)
    for hi, lo in ((0.25, None), (None, 0.3), (0.9, 0.6), (None, None)):
        ops, (cls, order, counts) = _route_gpu(q, k, v, 64, False, hi, lo)
        want_cls = O.route_tiles(ops["qs4"].cpu().numpy(), ops["ks4"].cpu().numpy(), 64, False, hi, lo)
        want_order, want_counts = O.route_order(want_cls, k.shape[2], 64, False)
        assert np.array_equal(cls.cpu().numpy(), want_cls), (hi, lo)
        assert np.array_equal(counts.cpu().numpy(), want_counts), (hi, lo)
        assert np.array_equal(order.cpu().numpy(), want_order), (hi, lo)


def test_route_golden_vectors_on_gpu():
    """The HIP router against the committed vectors (scale bytes in, class map / lists / run lengths out)."""
    import os
    d = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "route_vectors.npz"))
    L = _lib.lib()
    for name in "abcde":
        tile, D, n_keys, causal = (int(x) for x in d[name + "_meta"])
        hi, lo = (float(x) for x in d[name + "_thresh"])
        qs, ks = torch.from_numpy(d[name + "_qs"]).to(DEV), torch.from_numpy(d[name + "_ks"]).to(DEV)
        B, Hq, nq_pad, _ = qs.shape
        Hkv, nk_pad = ks.shape[1], ks.shape[2]
        nq = n_keys if nq_pad == nk_pad else nq_pad
        ntq, ntk = nq_pad // tile, nk_pad // tile
        work = torch.empty(L.mpsa_route_workspace(B, Hq, Hkv, nq, n_keys, D, tile), dtype=torch.uint8, device=DEV)
        cls = torch.empty((B, Hq, ntq, ntk), dtype=torch.uint8, device=DEV)
        order = torch.empty((B, Hq, ntq, ntk), dtype=torch.int32, device=DEV)
        counts = torch.empty((B, Hq, ntq, 4), dtype=torch.int32, device=DEV)
        _lib.check(L.mpsa_route_tiles(_lib.ptr(qs), _lib.ptr(ks), B, Hq, Hkv, nq, n_keys, D, tile, causal, hi, lo,
                                      _lib.ptr(work), _lib.ptr(cls), _lib.ptr(order), _lib.ptr(counts), _lib.stream_ptr()))
        assert np.array_equal(cls.cpu().numpy(), d[name + "_cls"]), name
        assert np.array_equal(order.cpu().numpy(), d[name + "_order"]), name
        assert np.array_equal(counts.cpu().numpy(), d[name + "_counts"]), name


def _compare(got, want, what=""):
    return attention_close(got, want, what)


@pytest.mark.parametrize("D,tile", [(128, 128), (64, 64), (128, 64), (64, 128)])
@pytest.mark.parametrize("causal", [False, True])
def test_routed_attention_against_oracle(D, tile, causal):
    N = 4 * tile + 19
    q, k, v = _inputs(1, 4, 2, N, D, seed=340 + D + tile)
    ops, route = _route_gpu(q, k, v, tile, causal, 0.5, 0.2)
    cls = route[0].cpu().numpy()
    assert {0, 1, 2} <= set(np.unique(cls).tolist())
    def run(dt):
        out = torch.empty((1, 4, N, D), dtype=dt, device=DEV)
        return attention_from_operands(ops, out, causal, route=route)
    want = O.attn_mx(q, k, v, tile=tile, causal=causal, mode="routed", route=cls, out_dtype=torch.float32)
    check_attention(run, want, f"routed D={D} tile={tile} causal={causal}", torch.bfloat16)


def test_routed_entry_point_and_sparsity():
    q, k, v = _inputs(1, 4, 4, 640, 128, seed=360)
    run = lambda dt: mxfp_attn(q.to(DEV), k.to(DEV), v.to(DEV), is_causal=False, smooth_k=False, output_dtype=dt,
                               block_scale_type="routed", route_thresh=0.5, skip_thresh=0.2, return_sparsity=True)
    got, sparsity = run(torch.bfloat16)
    ops, route = _route_gpu(q, k, v, 128, False, 0.5, 0.2)
    cls = route[0].cpu().numpy()
    check_attention(lambda dt: run(dt)[0], O.attn_mx(q, k, v, tile=128, causal=False, mode="routed", route=cls, out_dtype=torch.float32),
                    "mxfp_attn routed", torch.bfloat16)
    assert abs(float(sparsity) - float((cls == 0).mean())) < 1e-6
    with pytest.raises(ValueError):
        mxfp_attn(q.to(DEV), k.to(DEV), v.to(DEV), block_scale_type="mxfp4", route_thresh=0.5, smooth_k=False)


def test_routed_e5m2_smooth_k_fp16_and_nhd_layout():
    """The reference's own 8-bit format (E5M2), fp16 inputs, K smoothing and the "NHD" layout through the routed path."""
    q, k, v = _inputs(1, 4, 2, 3 * 64 + 21, 64, seed=370)
    q, k, v = q.to(torch.float16), k.to(torch.float16), v.to(torch.float16)
    N = q.shape[2]
    ks = O.smooth_k(k)
    ops = prepare_operands(q.to(DEV), ks.to(DEV), v.to(DEV), 64, "routed_e5")
    cls = route_tiles(ops, True, 0.5, 0.2)[0].cpu().numpy()
    assert {1, 2} <= set(np.unique(cls).tolist())
    want = O.attn_mx(q, ks, v, tile=64, causal=True, mode="routed", route=cls, fmt8=O.FMT_E5M2, out_dtype=torch.float32)
    run = lambda dt: mxfp_attn_kernel(q.transpose(1, 2).contiguous().to(DEV), ks.transpose(1, 2).contiguous().to(DEV),
                                      v.transpose(1, 2).contiguous().to(DEV), is_causal=True, tensor_layout="NHD",
                                      output_dtype=dt, block_scale_type="routed_e5", tile=64, route_thresh=0.5, skip_thresh=0.2)
    assert run(torch.float16).shape == (1, N, 4, 64)
    check_attention(lambda dt: run(dt).transpose(1, 2), want, "routed_e5 NHD", torch.float16)
    # smoothing inside the wrapper: same map inputs up to the 16-bit mean's last place, so compare the output only
    want2 = O.attn_mx(q, k, v, tile=64, causal=True, mode="routed", smooth_k=True, fmt8=O.FMT_E5M2, out_dtype=torch.float32,
                      route=O.route_tiles(*_oracle_scales(q, O.smooth_k(k), 64), 64, True, 0.5, None))
    check_attention(lambda dt: mxfp_attn_kernel(q.to(DEV), k.to(DEV), v.to(DEV), is_causal=True, smooth_k=True, output_dtype=dt,
                                                block_scale_type="routed_e5", tile=64, route_thresh=0.5, skip_thresh=None),
                    want2, "routed_e5 smooth_k", torch.float16)


def _oracle_scales(q, k, tile):
    """Padded 4-bit scale bytes of Q (with the softmax pre-scale) and K from the oracle's quantizer."""
    def padded(x, pre):
        sc = np.asarray(O.quantize_mx(x, pre, O.FMT_E2M1)[1])
        return np.pad(sc, ((0, 0), (0, 0), (0, (-x.shape[2]) % tile), (0, 0)))
    return padded(q, O.q_pre_scale(q.shape[-1], None)), padded(k, 1.0)


@pytest.mark.parametrize("N", [512, 512 + 77])
def test_routed_reproduces_fixed_modes_bit_for_bit(N):
    """Non-causal runs of the general kernel: thresholds off = every tile 4-bit = mode mxfp4; a hand-made list with
    tile i in the 8-bit run = mode diag.  Same kernel body, same visiting order, so the outputs are identical."""
    q, k, v = make_qkv(1, 4, 2, N, 128, seed=380)
    ops, route = _route_gpu(q, k, v, 128, False, None, None)
    out = torch.empty((1, 4, N, 128), dtype=torch.bfloat16, device=DEV)
    attention_from_operands(ops, out, False, route=route)
    want4 = mxfp_attn_kernel(q.to(DEV), k.to(DEV), v.to(DEV), is_causal=False, block_scale_type="mxfp4", tile=128,
                             output_dtype=torch.bfloat16)
    assert torch.equal(out, want4)
    nt = -(-N // 128)
    cls = np.full((1, 4, nt, nt), 1, dtype=np.uint8)
    for i in range(nt):
        cls[:, :, i, i] = 2
    order, counts = O.route_order(cls, N, 128, False)
    route = (None, torch.from_numpy(order).to(DEV), torch.from_numpy(counts).to(DEV))
    attention_from_operands(ops, out, False, route=route)
    want_diag = mxfp_attn_kernel(q.to(DEV), k.to(DEV), v.to(DEV), is_causal=False, block_scale_type="diag", tile=128,
                                 output_dtype=torch.bfloat16)
    assert torch.equal(out, want_diag)


def test_routed_lists_are_clamped_and_empty_rows_give_zeros():
    q, k, v = make_qkv(1, 2, 2, 384, 64, seed=390)
    ops, (cls, order, counts) = _route_gpu(q, k, v, 64, False, None, None)
    nt = 6
    order, counts = order.clone(), counts.clone()
    counts[0, 0, 1] = 0                                    # query tile 1 of head 0: nothing to visit
    counts[0, 1, 2] = torch.tensor([1 << 30, -5, 1 << 30, 7])      # run lengths beyond the row: clamped to nt tiles
    order[0, 1, 3, 0] = 1 << 20                            # tile index beyond the sequence: clamped to the last tile
    order[0, 1, 3, 1] = -9                                 # and below it: clamped to tile 0
    out = torch.empty((1, 2, 384, 64), dtype=torch.float32, device=DEV)
    attention_from_operands(ops, out, False, route=(cls, order, counts))
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    assert (out[0, 0, 64:128] == 0).all()
    want = O.attn_mx(q, k, v, tile=64, causal=False, mode="mxfp4", out_dtype=torch.float32)
    _compare(out[:, :1, :64], want[:, :1, :64], "untouched rows")
    _compare(out[:, 1:, 256:], want[:, 1:, 256:], "untouched rows")


def test_routed_argument_errors():
    L = _lib.lib()
    q, k, v = make_qkv(1, 2, 2, 128, 64, seed=391)
    ops, (cls, order, counts) = _route_gpu(q, k, v, 64, False, None, None)
    out = torch.empty((1, 2, 128, 64), dtype=torch.bfloat16, device=DEV)
    with pytest.raises(_lib.MpsaError, match="visiting lists"):
        attention_from_operands(ops, out, False, route=(None, None, None))
    rc = L.mpsa_route_tiles(_lib.ptr(ops["qs4"]), _lib.ptr(ops["ks4"]), 1, 2, 2, 128, 192, 64, 64, 1, 0.5, 0.0,
                            _lib.ptr(cls), _lib.ptr(cls), _lib.ptr(order), _lib.ptr(counts), _lib.stream_ptr())
    assert rc == -1 and b"causal" in L.mpsa_last_error()
    rc = L.mpsa_route_tiles(_lib.ptr(ops["qs4"]), _lib.ptr(ops["ks4"]), 1, 2, 2, 128, 128, 64, 64, 0, float("nan"), 0.0,
                            _lib.ptr(cls), _lib.ptr(cls), _lib.ptr(order), _lib.ptr(counts), _lib.stream_ptr())
    assert rc == -1 and b"NaN" in L.mpsa_last_error()


def test_routed_dit_shape_thresholds_off_equals_mxfp4():
    """Size-independent property at the video-DiT sequence length (N = 32760, a ragged last tile; 4 of the 40 heads):
    with both thresholds off the routed run is the mxfp4 run, bit for bit."""
    N = 32760
    q, k, v = make_qkv(1, 4, 4, N, 128, seed=4, sigma=0.5)
    q, k = _frames(q, k, 21, seed=5, amp=0.5)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    got = mxfp_attn_kernel(qd, kd, vd, is_causal=False, block_scale_type="routed", tile=128, output_dtype=torch.bfloat16)
    want = mxfp_attn_kernel(qd, kd, vd, is_causal=False, block_scale_type="mxfp4", tile=128, output_dtype=torch.bfloat16)
    assert torch.equal(got, want)
    # with routing on, the output stays close to the all-8-bit run and the map holds both precisions
    ops = prepare_operands(qd, kd, vd, 128, "routed")
    cls, order, counts = route_tiles(ops, False, 0.9, None)
    share8 = float((cls == 2).float().mean())
    assert 0.0 < share8 < 1.0, share8
    out = torch.empty_like(got)
    attention_from_operands(ops, out, False, route=(cls, order, counts))
    ref8 = mxfp_attn_kernel(qd, kd, vd, is_causal=False, block_scale_type="mxfp8", tile=128, output_dtype=torch.bfloat16)
    cos = torch.nn.functional.cosine_similarity(out.float().flatten(), ref8.float().flatten(), dim=0).item()
    cos4 = torch.nn.functional.cosine_similarity(want.float().flatten(), ref8.float().flatten(), dim=0).item()
    assert cos >= cos4 - 1e-4, (cos, cos4)                 # 8-bit tiles do not make it worse than all-4-bit


def test_c5_video_dit_all_heads_diag_and_routed():
    """B=1 H=40 N=32760 (21 frames x 1560 tokens, a ragged last tile) D=128, bidirectional, q/k/v ~ N(0, 0.5) seed 4
    plus per-frame offsets: all 40 heads on the GPU in the diag mode and in the routed mode (route_thresh 0.9).  The
    oracle checks sampled (head, query tile) pairs -- first, middle and the ragged last tile, and one query tile of each
    of the 40 heads -- and, for the routed
    run, with its OWN class map computed from its own scale bytes (which the GPU's map must equal bit for bit)."""
    N, H = 32760, 40
    q, k, v = make_qkv(1, H, H, N, 128, seed=4, sigma=0.5)
    q, k = _frames(q, k, 21, seed=5, amp=0.5)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    samples = {0: [0, 255], 7: [100], 19: [254, 37], 39: [255, 128]}
    rows = lambda tiles: torch.cat([torch.arange(t * 128, min((t + 1) * 128, N)) for t in tiles])

    got = mxfp_attn_kernel(qd, kd, vd, is_causal=False, block_scale_type="diag", tile=128, output_dtype=torch.float32)
    assert torch.isfinite(got).all()
    for h, tiles in samples.items():
        want = O.attn_mx(q[:, h:h + 1], k[:, h:h + 1], v[:, h:h + 1], tile=128, causal=False, mode="diag", q_tiles=tiles,
                         out_dtype=torch.float32)
        _compare(got[:, h:h + 1, rows(tiles).to(DEV)], want, f"C5 diag head {h} tiles {tiles}")
    every_head = {h: [(h * 19 + 3) % 256] for h in range(H)}         # and one query tile of every head
    for h, tiles in every_head.items():
        want = O.attn_mx(q[:, h:h + 1], k[:, h:h + 1], v[:, h:h + 1], tile=128, causal=False, mode="diag", q_tiles=tiles,
                         out_dtype=torch.float32)
        _compare(got[:, h:h + 1, rows(tiles).to(DEV)], want, f"C5 diag head {h} tiles {tiles}")
    del got

    ops = prepare_operands(qd, kd, vd, 128, "routed")
    cls, order, counts = route_tiles(ops, False, 0.9, None)
    share8 = float((cls == 2).float().mean())
    assert 0.02 < share8 < 0.98, share8
    out = torch.empty((1, H, N, 128), dtype=torch.float32, device=DEV)
    attention_from_operands(ops, out, False, route=(cls, order, counts))
    assert torch.isfinite(out).all()
    pre = O.q_pre_scale(128)
    for h, tiles in list(samples.items()) + [(h, t) for h, t in every_head.items() if h not in samples]:
        _, qs4 = O.quantize_mx(q[:, h:h + 1], pre, O.FMT_E2M1)
        _, ks4 = O.quantize_mx(k[:, h:h + 1], 1.0, O.FMT_E2M1)
        pad = lambda t: torch.nn.functional.pad(t, (0, 0, 0, 256 * 128 - N)).numpy()
        own = O.route_tiles(pad(qs4), pad(ks4), 128, False, 0.9, None)
        assert np.array_equal(cls[:, h:h + 1].cpu().numpy(), own), f"class map of head {h}"
        want = O.attn_mx(q[:, h:h + 1], k[:, h:h + 1], v[:, h:h + 1], tile=128, causal=False, mode="routed", route=own, q_tiles=tiles,
                         out_dtype=torch.float32)
        _compare(out[:, h:h + 1, rows(tiles).to(DEV)], want, f"C5 routed head {h} tiles {tiles}")
