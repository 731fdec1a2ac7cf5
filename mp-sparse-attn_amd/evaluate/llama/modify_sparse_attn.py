"""Llama prefill hook: route the prefill attention of a Hugging Face Llama model through the MXFP kernel.

Counterpart of the reference's ``set_spas_sage_attn_llama`` (evaluate/llama/modify_sparse_attn.py:15-136), which
replaces every layer's attention forward and sends prefill (q_len > 1) to the selected sparse kernel
(spas_sage_attn/autotune.py:143-159) and decode (q_len == 1) to SDPA.  Differences that follow from the kernel:

* K and V are handed over with their own (fewer) heads; the reference repeats them to the query head count first
  (evaluate/llama/modify_sparse_attn.py:100-101), the HIP kernel maps query heads to KV heads itself.
* The hook is an attention function registered with transformers' attention registry instead of a copy of the
  layer's forward, so projections, rotary embedding and the KV cache stay the library's own code.

As in the reference, an explicit attention mask is not supported on the prefill path.
"""

import torch

from ours._lib import require_device
from ours.mxfp_attn import mxfp_attn

ATTN_NAME = "mxfp_attn"
_registered = False


class MxfpAttnOptions:
    """Per-layer settings, the counterpart of the reference's per-layer ``SparseAttentionMeansim`` object."""

    def __init__(self, layer_idx, block_scale_type="diag", BLKQ=128, skip_thresh=None, smooth_k=False, verbose=False):
        self.layer_idx = layer_idx
        self.block_scale_type = block_scale_type
        self.BLKQ = BLKQ
        self.skip_thresh = skip_thresh
        self.smooth_k = smooth_k
        self.verbose = verbose
        self.prefill_calls = 0
        self.decode_calls = 0
        self.last_metric = None


def _precision_metric(out, ref):
    """Cosine similarity, relative L1 and RMSE as the reference reports them (spas_sage_attn/utils.py:25-36)."""
    x, y = out.float().flatten(), ref.float().flatten()
    cos = torch.nn.functional.cosine_similarity(x, y, dim=0).item()
    l1 = ((x - y).abs().sum() / y.abs().sum()).item()
    rmse = torch.sqrt(torch.mean((x - y) ** 2)).item()
    return {"Cossim": cos, "L1": l1, "RMSE": rmse}


def mxfp_attention_forward(module, query, key, value, attention_mask, dropout=0.0, scaling=None, **kwargs):
    """Attention function with transformers' interface: [B,H,N,D] in, ([B,N,H,D], None) out."""
    from transformers.integrations.sdpa_attention import sdpa_attention_forward

    opts = getattr(module, "mxfp_attn_options", None)
    q_len, kv_len = query.shape[-2], key.shape[-2]
    if opts is None or q_len == 1 or q_len != kv_len:
        # decode steps and chunked prefill against a longer cache stay on SDPA, like the reference's q_len == 1 branch
        if opts is not None:
            opts.decode_calls += 1
        return sdpa_attention_forward(module, query, key, value, attention_mask, dropout=dropout, scaling=scaling,
                                      **kwargs)
    assert attention_mask is None, "Attention mask not supported"
    assert dropout == 0.0, "dropout is not supported on the MXFP prefill path"
    require_device(query, key, value)
    out = mxfp_attn(query, key, value, is_causal=True, scale=scaling, smooth_k=opts.smooth_k,
                    output_dtype=query.dtype, skip_thresh=opts.skip_thresh,
                    block_scale_type=opts.block_scale_type, BLKQ=opts.BLKQ)
    opts.prefill_calls += 1
    if opts.verbose:
        groups = query.shape[1] // key.shape[1]
        ref = torch.nn.functional.scaled_dot_product_attention(
            query, key.repeat_interleave(groups, 1), value.repeat_interleave(groups, 1), is_causal=True,
            scale=scaling)
        opts.last_metric = _precision_metric(out, ref)
        print(f"layer {opts.layer_idx}: {opts.last_metric}")
    return out.transpose(1, 2), None


def set_mxfp_attn_llama(model, block_scale_type="diag", BLKQ=128, skip_thresh=None, smooth_k=False, verbose=False):
    """Send every layer's prefill attention through ``mxfp_attn``; returns the model.

    ``model`` is a transformers Llama model (``model.model.layers[i].self_attn``), as in the reference's
    ``set_spas_sage_attn_llama(model, ..., skip_thresh=None, kernel_name=None)``.
    """
    global _registered
    from transformers import AttentionInterface

    if not _registered:
        AttentionInterface.register(ATTN_NAME, mxfp_attention_forward)
        _registered = True
    for layer_id, layer in enumerate(model.model.layers):
        layer.self_attn.mxfp_attn_options = MxfpAttnOptions(layer_id, block_scale_type, BLKQ, skip_thresh, smooth_k,
                                                            verbose)
    model.set_attn_implementation(ATTN_NAME)
    return model


# the name the reference's evaluation scripts call (evaluate/llama/llama_main.py)
set_spas_sage_attn_llama = set_mxfp_attn_llama
