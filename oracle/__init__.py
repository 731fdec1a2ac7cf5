"""CPU oracle for the diagonal-tiled MXFP attention path.

TEST INFRASTRUCTURE ONLY.  This package restates, in plain torch/numpy on the
CPU, the algorithm of the reference's MXFP path (format classes, MX quantizer,
block-scaled matmul, tile-by-tile online-softmax attention).  It exists so the
HIP kernels can be checked against it and so a CPU baseline can be timed next
to them.  Nothing in the shipped package may import it: only the test-suite,
the smoke check and the benchmark's CPU-baseline leg do.

Each function names the reference file:line it follows (paths are relative to
the reference checkout).

Parity status of each restated function:

* ``decode_e2m1``, ``pack_fp4``/``unpack_fp4``, ``encode_e8m0``/``decode_e8m0``
  -- pinned by closed forms and exhaustive enumeration (tests/test_oracle_formats.py).
* ``encode_e2m1`` -- pinned by an exhaustive brute-force nearest/ties-to-even
  search over every bf16 and fp16 value, and by golden vectors minted from the
  reference's own ``MXFP4Tensor._from_float`` for the near-tie bias
  (tests/golden/mxfp_vectors.npz).  One corner is PARITY UNPINNED: the reference
  applies the 1e-6 bias under a whole-tensor test (``if is_tie.sum() > 1``,
  ours/mxfp.py:151-158) that only a one-element tensor without an exact tie
  fails; this restatement applies the bias for every length.
* ``encode_e4m3`` -- not in the reference (which stores E5M2); pinned by an
  independent closed-form encoder and torch's own float8_e4m3fn cast.
* ``quantize_mx`` -- composition of the above; pinned by invariants and
  hand-worked blocks.  Two corners are PARITY UNPINNED against the reference's
  Triton kernel (it cannot run here): (1) ``floor(log2(amax))`` is the true
  floor (bit extraction), whereas a float32 ``log2`` may round up for an amax
  one ulp below a power of two; (2) an all-zero block gets scale byte 0 and
  codes +0.
* ``gemm_mx`` -- dequantise + matmul; pinned against exact integer arithmetic.
* ``scales_to_5d`` / ``scales_from_5d`` -- the reference's reshape/permute, pinned
  by the explicit index formula and the round trip.
* ``attn_mx`` -- pinned against dense float64 softmax attention on the same
  per-tile dequantised operands, and special cases (single tile, V = 1,
  identical keys, GQA == repeat_interleave).  Its tile-skipping rule
  (``skip_thresh``) is pinned against an independent dense float64 formulation
  of the statistic, the decisions and the restricted softmax
  (tests/test_oracle_gemm_attn.py).
* ``route_tiles`` / ``route_order`` -- this build's own integer rule (the reference has no precision router);
  pinned against an exact rational evaluation of the score bound it stands for, hand-worked maps and committed
  golden vectors (tests/test_oracle_route.py, tests/golden/route_vectors.npz); ``attn_mx(mode="routed")`` is pinned against the dense float64 attention on the
  same map and must reproduce the fixed modes on the maps that describe them.
* ``seq_mean`` / ``smooth_k`` -- the once-rounded mean is pinned against
  float64 arithmetic and exactly representable cases; the float32 summation
  order of the reference's device mean is not reproducible (PARITY UNPINNED in
  the last bit of the 16-bit mean on rare channels), everything downstream of
  the mean is exact.
"""

from .mx_formats import (  # noqa: F401
    E2M1_VALUES, decode_e2m1, encode_e2m1, pack_fp4, unpack_fp4,
    encode_e8m0, decode_e8m0, encode_e4m3, decode_e4m3, encode_e5m2, decode_e5m2,
)
from .mx_quantize import (  # noqa: F401
    FMT_E2M1, FMT_E4M3, FMT_E5M2, EMAX_ELEM, q_pre_scale, quantize_mx, dequantize_mx, smooth_k, seq_mean,
)
from .mx_gemm import gemm_mx, scales_to_5d, scales_from_5d  # noqa: F401
from .mx_route import route_tiles, route_order, tile_scale_stats  # noqa: F401
from .mx_attention import attn_mx, attn_dense_f64, precision_metric, v_fragment_order  # noqa: F401
