"""Public attention entry point -- same name, argument order and defaults as the reference's
``ours/mxfp_attn.py::mxfp_attn`` (ours/mxfp_attn.py:30-33).

The reference body stops after the Q.K^T product and returns scores; this build returns the attention
output.  ``block_scale_type`` additionally accepts ``"diag"`` (diagonal tiles MXFP8, others MXFP4);
``"routed"`` takes each tile's precision (MXFP8, MXFP4 or skipped) from the tile router with ``route_thresh`` and
``skip_thresh``; ``BLKQ`` is the score-tile edge (64 or 128).  ``compute_reference`` is accepted for signature
compatibility and must be False: the library carries no second implementation to compare with.
"""

import torch

from .mxfp_attn_kernel import mxfp_attn_kernel


@torch.compiler.disable
def mxfp_attn(q, k, v, attn_mask=None, dropout_p=0.0, is_causal=False, scale=None, smooth_k=True,
              attention_sink=False, tensor_layout="HND", output_dtype=torch.float16, return_sparsity=False, skip_thresh=None,
              block_scale_type="mxfp4", BLKQ=128, compute_reference=False, route_thresh=None):
    seq_dim = -2 if tensor_layout == "HND" else 1
    assert q.size(seq_dim) >= 128, "seq_len should be not less than 128."          # ours/mxfp_attn.py:34
    assert q.size(-1) in [64, 128], "headdim should be in [64, 96, 128]."           # ours/mxfp_attn.py:49
    if compute_reference:
        raise NotImplementedError("compute_reference is not available: use the test-suite's CPU oracle")
    return mxfp_attn_kernel(q, k, v, attn_mask=attn_mask, dropout_p=dropout_p, is_causal=is_causal, scale=scale,
                            smooth_k=smooth_k, attention_sink=attention_sink, tensor_layout=tensor_layout,
                            output_dtype=output_dtype, return_sparsity=return_sparsity,
                            block_scale_type=block_scale_type, skip_thresh=skip_thresh, tile=BLKQ,
                            route_thresh=route_thresh)
