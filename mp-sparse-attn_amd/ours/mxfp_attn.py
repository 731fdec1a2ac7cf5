"""Public attention entry point -- same name, argument order and defaults as the reference's
``ours/mxfp_attn.py::mxfp_attn`` (ours/mxfp_attn.py:30-33).

The reference body stops after the Q.K^T product and returns scores; this build returns the attention
output.  ``block_scale_type`` additionally accepts ``"diag"`` (diagonal tiles MXFP8, others MXFP4);
``"routed"`` takes each tile's precision (MXFP8, MXFP4 or skipped) from the tile router with ``route_thresh`` and
``skip_thresh``; ``BLKQ`` is the score-tile edge (64 or 128).  ``compute_reference=True`` runs the reference's own
self-check first (ours/mxfp_attn.py:52-69): quantize, package with ``compute_reference``, multiply Q.K^T with the
block-scaled matmul kernel and compare the scores with the fake-quant product of the dequantized operands.
"""

import torch

from . import _lib
from .mxfp_attn_kernel import mxfp_attn_kernel, initialize_block_scaled_batched_from_tensor, _normalise
from .quant_mxint8 import quantize_mx, pre_scale_q, seq_mean, _as_bhnd


def check_scores_against_reference(q, k, block_scale_type="mxfp4", scale=None, smooth_k=False):
    """The reference's self-check of the quantized score product (ours/mxfp_attn.py:52-69) on ``[B,H,N,D]`` q and k
    (N a multiple of 128): MX-quantize, reshape the scales to the packed layout, package with
    ``compute_reference=True``, run ``block_scaled_batched_matmul`` and compare.  The bound is the reference's
    (atol = rtol = 1e-3) for every product with a 4-bit operand; a product of two 8-bit operands gets the norm-wise
    term ``3e-5 * |dq(Q)| @ |dq(K)|^T`` on top (the scaled matrix instruction aligns the 64 products of a step to the
    largest one and keeps about 16 bits).  ``"diag"`` / ``"routed"`` types check both of their products.  Returns the
    list of ``(reference, scores)`` pairs."""
    from .batched_block_scaled_matmul import block_scaled_batched_matmul
    from .block_scaled_matmul import pack_scale_5d, _expanded_scales
    from .mxfp import MXFP4Tensor
    B, H, N, D = q.shape
    Hkv, Nk = k.shape[1], k.shape[2]
    assert N % 128 == 0 and Nk % 128 == 0, "the packed scale layout needs sequence lengths that are multiples of 128"
    e5 = block_scale_type.endswith("e5")
    base = block_scale_type[:-3] if e5 else block_scale_type
    pairs = {"mxfp4": ["mxfp4"], "mxfp8": ["mxfp8"], "mixed": ["mixed"], "diag": ["mxfp4", "mxfp8"], "routed": ["mxfp4", "mxfp8"]}[base]
    sub = seq_mean(k) if smooth_k else None
    checked = []
    for bst in pairs:
        if bst != "mxfp4" and e5:
            bst = {"mxfp8": "mxfp8e5", "mixed": "mixed_e5"}[bst]
        f8 = _lib.FMT_E5M2 if e5 else _lib.FMT_E4M3
        fq = _lib.FMT_E2M1 if bst == "mxfp4" else f8
        fk = f8 if bst.startswith("mxfp8") else _lib.FMT_E2M1

        def one_code_per_byte(c, fmt):          # the form the reference's quantizers return
            return MXFP4Tensor(size=(1,)).unpack_packed_tensor(c, 3, (*c.shape[:3], c.shape[3] * 2)) if fmt == _lib.FMT_E2M1 else c

        qc, qs = quantize_mx(q, pre_scale_q(D, scale), fq)
        kc, ks = quantize_mx(k, 1.0, fk, sub=sub)
        qp, qs5, kp, ks5, configs, (reference, q_dec, k_dec) = initialize_block_scaled_batched_from_tensor(
            one_code_per_byte(qc, fq), one_code_per_byte(kc, fk), pack_scale_5d(qs), pack_scale_5d(ks), bst, compute_reference=True)
        scores = block_scaled_batched_matmul(qp, qs5, kp, ks5, torch.float32, B, H, N, Nk, D, configs)
        atol = 1e-3
        if fq != _lib.FMT_E2M1 and fk != _lib.FMT_E2M1:
            mag = torch.matmul((q_dec * _expanded_scales(qs5, D)).abs(),
                               (k_dec * _expanded_scales(ks5, D)).abs().repeat_interleave(H // Hkv, dim=1).transpose(-1, -2))
            atol = 1e-3 + 3e-5 * mag
        err = (scores - reference).abs()
        bad = err > atol + 1e-3 * reference.abs()
        if bool(bad.any()):
            raise AssertionError(f"{bst} scores differ from the fake-quant reference: {int(bad.sum())} of {bad.numel()} "
                                 f"elements, largest error {float(err.max()):.3e}")
        checked.append((reference, scores))
    return checked


@torch.compiler.disable
def mxfp_attn(q, k, v, attn_mask=None, dropout_p=0.0, is_causal=False, scale=None, smooth_k=True,
              attention_sink=False, tensor_layout="HND", output_dtype=torch.float16, return_sparsity=False, skip_thresh=None,
              block_scale_type="mxfp4", BLKQ=128, compute_reference=False, route_thresh=None):
    seq_dim = -2 if tensor_layout == "HND" else 1
    assert q.size(seq_dim) >= 128, "seq_len should be not less than 128."          # ours/mxfp_attn.py:34
    assert q.size(-1) in [64, 128], "headdim should be in [64, 96, 128]."           # ours/mxfp_attn.py:49
    if compute_reference:
        _lib.require_device(q, k, v)
        qn, kn, _ = _normalise(q, k, v)
        check_scores_against_reference(_as_bhnd(qn, tensor_layout), _as_bhnd(kn, tensor_layout), block_scale_type, scale, smooth_k)
    return mxfp_attn_kernel(q, k, v, attn_mask=attn_mask, dropout_p=dropout_p, is_causal=is_causal, scale=scale,
                            smooth_k=smooth_k, attention_sink=attention_sink, tensor_layout=tensor_layout,
                            output_dtype=output_dtype, return_sparsity=return_sparsity,
                            block_scale_type=block_scale_type, skip_thresh=skip_thresh, tile=BLKQ,
                            route_thresh=route_thresh)
