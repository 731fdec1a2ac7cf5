"""MI355X-native MXFP attention path behind the reference's Python entry points.

Modules keep the reference's names so that ``from ours.mxfp_attn import mxfp_attn`` and
``from ours.mxfp import MXFP4Tensor, MXScaleTensor`` keep working:

  ours.mxfp                  format helper classes            (reference: ours/mxfp.py)
  ours.quant_mxint8          MX quantizer entry points        (reference: ours/quant_mxint8.py)
  ours.block_scaled_matmul   block-scaled GEMM                (reference: ours/block_scaled_matmul.py)
  ours.batched_block_scaled_matmul  batched block-scaled GEMM (reference: ours/batched_block_scaled_matmul.py)
  ours.mxfp_attn_kernel      fused attention                  (reference: ours/mxfp_attn_kernel.py)
  ours.mxfp_attn             public attention entry           (reference: ours/mxfp_attn.py)

All compute runs in hand-written HIP kernels (libmpsa.so) reached through a C ABI; there is no
CPU or eager-torch fallback -- a missing library or a non-HIP tensor is an error.
"""
