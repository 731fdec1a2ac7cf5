/*
 * mpsa.h -- C ABI of the MI355X (gfx950) MXFP attention path.
 *
 * One shared library, libmpsa.so, exports the functions below.  Every pointer is a plain
 * device (HBM) pointer unless stated otherwise; every function enqueues its kernels on the
 * given HIP stream and returns without synchronising.  The library keeps no reference to
 * caller memory and allocates none: inputs, outputs and intermediates are all caller-owned.
 * Return value: 0 on success, a negative MPSA_E* code otherwise; mpsa_last_error() then gives
 * a human-readable reason (thread-local).  No exception or torch type crosses this boundary.
 *
 * Citations name the reference interface each entry point replaces (paths relative to the
 * reference checkout).
 */
#ifndef MPSA_H
#define MPSA_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* hipStream_t is an opaque pointer; the ABI takes it as void* so this header needs no HIP. */
typedef void* mpsa_stream_t;

/* element dtypes of unquantized tensors */
#define MPSA_BF16 0
#define MPSA_F16  1
#define MPSA_F32  2
#define MPSA_F8E5M2 3   /* output of mpsa_gemm_mx only */

/* MX element formats; the values are the CDNA4 scaled-MFMA format selectors */
#define MPSA_FMT_E4M3 0
#define MPSA_FMT_E5M2 1
#define MPSA_FMT_E2M1 4

/* per-tile precision of the attention score product */
#define MPSA_MODE_MXFP4 0   /* every tile 4-bit */
#define MPSA_MODE_MXFP8 1   /* every tile 8-bit */
#define MPSA_MODE_DIAG  2   /* tile j == i 8-bit, all others 4-bit */
#define MPSA_MODE_ROUTED 3  /* per-tile precision from a visiting list (mpsa_route_tiles, mpsa_attn_fwd_routed) */
#define MPSA_MODE_MIXED  4  /* every tile: 8-bit Q x 4-bit K - the reference's "mixed" type (ELEM_PER_BYTE_A = 1,
                               ELEM_PER_BYTE_B = 2, ours/mxfp_attn_kernel.py:264-269, :448-449) */

#define MPSA_OK             0
#define MPSA_EINVAL        -1   /* null pointer, bad enum, bad shape */
#define MPSA_EALIGN        -2   /* pointer or stride not 16-byte aligned */
#define MPSA_EUNSUPPORTED  -3   /* shape outside the compiled variants */
#define MPSA_ELAUNCH       -4   /* the HIP runtime refused the launch */

int mpsa_version(void);
const char* mpsa_last_error(void);

/*
 * One-time set-up of the CURRENT device: raises the dynamic-LDS limit of every kernel variant that needs it and
 * resolves the address of the library's built-in device array (mpsa_seq_mean_static).  The launchers do this by
 * themselves on a device's first use; a caller that captures its very first call into a HIP graph calls mpsa_init()
 * beforehand, once per device, because function attributes cannot be set during capture.  Idempotent, thread-safe.
 * (The reference has no counterpart: Triton sets such limits when it loads a kernel.)
 */
int mpsa_init(void);

/*
 * Elementwise format conversions behind the MXFP4Tensor / MXScaleTensor helper classes; contiguous
 * arrays of n elements.
 *   mpsa_e2m1_encode  float32 -> one E2M1 code per byte (round to nearest, ties to even mantissa,
 *                     NaN/Inf/overflow -> magnitude 6).      Replaces MXFP4Tensor._from_float, ours/mxfp.py:84-170.
 *   mpsa_e2m1_decode  code byte -> float32.                  Replaces MXFP4Tensor.to, ours/mxfp.py:44-77.
 *   mpsa_e8m0_encode  float32 -> E8M0 byte (<=0, NaN, Inf -> 255; else clamp(floor(log2 v)+127, 0, 254)).
 *                                                            Replaces MXScaleTensor._from_float, ours/mxfp.py:286-307.
 *   mpsa_e8m0_decode  E8M0 byte -> float32 2^(e-127), 255 -> NaN.  Replaces MXScaleTensor.to, ours/mxfp.py:275-284.
 */
int mpsa_e2m1_encode(const float* x, int64_t n, uint8_t* codes, mpsa_stream_t stream);
int mpsa_e2m1_decode(const uint8_t* codes, int64_t n, float* out, mpsa_stream_t stream);
int mpsa_e8m0_encode(const float* x, int64_t n, uint8_t* codes, mpsa_stream_t stream);
int mpsa_e8m0_decode(const uint8_t* codes, int64_t n, float* out, mpsa_stream_t stream);

/*
 * float32 -> one FP8 byte per element, fmt MPSA_FMT_E5M2 | MPSA_FMT_E4M3: the elementwise cast the reference's operand
 * packaging applies to its 8-bit operands, a_tensor.to(torch.float8_e5m2) (ours/block_scaled_matmul.py:334-336,
 * :349-351; ours/mxfp_attn_kernel.py:467-469, :479-481): round to nearest even, no saturation (E5M2 overflows to
 * infinity, E4M3 - which has no infinity - to NaN), NaN stays NaN.  No block scale is derived here: this is not the
 * MX quantizer.
 */
int mpsa_fp8_encode(const float* x, int64_t n, int fmt, uint8_t* codes, mpsa_stream_t stream);

/*
 * Nibble packing of E2M1 codes along one dimension of a contiguous tensor seen as [outer, n, inner]:
 * packed [outer, ceil(n/2), inner], element 2i in the low nibble and 2i+1 in the high one, an odd n padded with a
 * zero code; unpack writes n codes back.  Replaces MXFP4Tensor.to_packed_tensor / unpack_packed_tensor,
 * ours/mxfp.py:172-205, :207-236 (the quantizer itself already emits packed codes; these serve code tensors that
 * arrive one code per byte, as the reference's quantizer leaves them).
 */
int mpsa_e2m1_pack(const uint8_t* codes, int64_t outer, int64_t n, int64_t inner, uint8_t* packed, mpsa_stream_t stream);
int mpsa_e2m1_unpack(const uint8_t* packed, int64_t outer, int64_t n, int64_t inner, uint8_t* codes, mpsa_stream_t stream);

/*
 * E8M0 scale re-layout between this library's linear form [batch, rows, K/32] and the 5-D packed form the
 * reference's block-scaled kernels consume, [batch, rows/128, K/128, 32, 4, 4] with
 * packed[cm][ck][r32][r4][c4] = linear[cm*128 + r4*32 + r32][ck*4 + c4].  Replaces the reshape/permute at
 * ours/mxfp_attn_kernel.py:56-57 (to the packed form) and ours/block_scaled_matmul.py:384 (back), so that scale
 * tensors can be exchanged with code written against the reference.  rows % 128 == 0, kblocks = K/32, kblocks % 4 == 0.
 */
int mpsa_scales_to_5d(const uint8_t* linear, int64_t batch, int64_t rows, int64_t kblocks, uint8_t* packed, mpsa_stream_t stream);
int mpsa_scales_from_5d(const uint8_t* packed, int64_t batch, int64_t rows, int64_t kblocks, uint8_t* linear, mpsa_stream_t stream);

/*
 * MX quantizer.  Replaces quant_mxfp4 / quant_mxfp8e5 and their Triton kernels
 * (ours/quant_mxint8.py:453-512, :276-351, :223-272, :164-219) together with the host-side
 * nibble packing MXFP4Tensor.to_packed_tensor (ours/mxfp.py:172-205).
 *
 *   x          [B,H,N,D] of x_dtype (MPSA_BF16 | MPSA_F16), element strides x_strides[4],
 *              last dim contiguous, D % 32 == 0, rows 16-byte aligned
 *   sub        NULL, or [B,H,D] of x_dtype (contiguous, 16-byte aligned): x := round_to_x_dtype(x - sub) row by
 *              row before anything else - the smooth-K step k - k.mean(dim=-2) of ours/mxfp_attn.py:44-45 and
 *              ours/mxfp_attn_kernel.py:33-34 with the mean from mpsa_seq_mean
 *   pre_scale  float32 factor multiplied in before quantizing (sm_scale*log2(e) for Q, 1 for K)
 *   fmt        MPSA_FMT_E2M1 | MPSA_FMT_E4M3 | MPSA_FMT_E5M2
 *   emax_elem  shared exponent = floor(log2(amax)) - emax_elem (reference: 3 for E2M1, 7 for 8-bit)
 *   codes      [B,H,out_rows,D/2] (E2M1, two codes per byte, even element in the low nibble)
 *              or [B,H,out_rows,D] (8-bit), contiguous
 *   scales     [B,H,out_rows,D/32] E8M0 bytes, contiguous
 *   out_rows   rows per (b,h) in the outputs, >= N; rows N..out_rows-1 are written as zero
 */
int mpsa_quantize_mx(const void* x, int x_dtype, int64_t B, int64_t H, int64_t N, int64_t D,
                     const int64_t x_strides[4], const void* sub, float pre_scale, int fmt, int emax_elem,
                     uint8_t* codes, uint8_t* scales, int64_t out_rows, mpsa_stream_t stream);

/*
 * Both precisions in one pass over x (the diagonal-tiled attention needs Q and K in E2M1 and in
 * an 8-bit format).  Same contract as two mpsa_quantize_mx calls with (E2M1, emax4) and
 * (fmt8, emax8); x is read once.  Replaces the same reference functions as above.
 */
int mpsa_quantize_mx_dual(const void* x, int x_dtype, int64_t B, int64_t H, int64_t N, int64_t D,
                          const int64_t x_strides[4], const void* sub, float pre_scale, int emax4, int fmt8, int emax8,
                          uint8_t* codes4, uint8_t* scales4, uint8_t* codes8, uint8_t* scales8,
                          int64_t out_rows, mpsa_stream_t stream);

/*
 * Mean over the sequence dim, per (batch, head, channel): mean[b,h,d] = round_to_x_dtype(float32 sum over n of
 * x[b,h,n,d] * float32(1/N)).  Replaces the k.mean(dim=-2, keepdim=True) of the smooth-K prologue
 * (ours/mxfp_attn.py:44-45, ours/mxfp_attn_kernel.py:33-34); the subtraction itself happens inside the quantizer
 * (its sub argument).  The float32 additions run in a fixed order (256-row partial sums, then those in order), so the
 * result is reproducible; it can differ from another summation order in the last bit of the 16-bit mean.
 *
 *   x          as for mpsa_quantize_mx, D in {64,128}
 *   workspace  mpsa_seq_mean_workspace(B,H,N,D) bytes of device memory (float32 partial sums), caller-owned
 *   mean       [B,H,D] of x_dtype
 */
int64_t mpsa_seq_mean_workspace(int64_t B, int64_t H, int64_t N, int64_t D);
int mpsa_seq_mean(const void* x, int x_dtype, int64_t B, int64_t H, int64_t N, int64_t D,
                  const int64_t x_strides[4], float* workspace, void* mean, mpsa_stream_t stream);

/*
 * mpsa_seq_mean without a workspace argument, for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid allocation).  It has no counterpart in the reference.  The
 * float32 partial sums go to a device array built into the library (MPSA_SEQ_MEAN_STATIC_BYTES per GPU, held until
 * the process ends); the call allocates and frees nothing.  Same kernels, same bits as mpsa_seq_mean.
 *   - mpsa_seq_mean_workspace(B,H,N,D) must not exceed MPSA_SEQ_MEAN_STATIC_BYTES (e.g. B*H = 8 heads of D = 128 up to
 *     N = 262144), else MPSA_EUNSUPPORTED;
 *   - all calls on one GPU share the array: calls that overlap on one GPU (different streams or host threads) race;
 *     calls ordered on one stream are safe.  Nothing needs clearing between calls (every partial sum read was
 *     written by the same call).
 */
#define MPSA_SEQ_MEAN_STATIC_BYTES 4194304
int mpsa_seq_mean_static(const void* x, int x_dtype, int64_t B, int64_t H, int64_t N, int64_t D,
                         const int64_t x_strides[4], void* mean, mpsa_stream_t stream);

/*
 * Block-scaled matmul  C[M,N] = (A o 2^(sa-127)) (B o 2^(sb-127))^T.  Replaces block_scaled_matmul
 * and its Triton kernel (ours/block_scaled_matmul.py:271-296, :154-267).
 *
 *   a, b     packed codes [M,K/2] / [N,K/2] (E2M1) or [M,K] / [N,K] (8-bit), row-major, contiguous
 *   sa, sb   E8M0 bytes [M,K/32] / [N,K/32], row-major (the linear layout; mpsa_gemm_mx_packed below takes the 5-D packed one)
 *   fmt_a, fmt_b   element format of each operand (MPSA_FMT_*); they may differ - the reference's "mixed" type is an
 *            8-bit A with a 4-bit B (ELEM_PER_BYTE_A / ELEM_PER_BYTE_B, ours/block_scaled_matmul.py:318-324, :252-257)
 *   c        [M,N] of c_dtype (MPSA_BF16 | MPSA_F16 | MPSA_F32 | MPSA_F8E5M2: one E5M2 byte per element, round to
 *            nearest even, overflow to infinity - the reference's output dtypes are f32, f16 and e5m2,
 *            ours/block_scaled_matmul.py:185-190, :273-280), leading dimension ldc elements
 *   M, N >= 1 (edge tiles are masked, as in the reference's kernel), K % 64 == 0.  Equal formats with M % 256 == 0,
 *   N % 256 == 0 and K % 128 == 0, and an 8-bit A against a 4-bit B with K % 256 == 0 besides, run on the LDS-staged
 *   256 x 256 kernel; every other case on a 128 x 128 kernel with masked edge tiles, LDS-staged too (two buffers,
 *   direct-to-LDS loads).  Same results either way; MPSA_GEMM_GENERAL=1 in the environment forces the second.
 *   Accumulation: E2M1 x E2M1 products are added exactly (the float32 result is the correctly rounded sum).  With an
 *   8-bit operand the matrix cores add the products of 8 consecutive K elements together first and cut every product of
 *   such a group to 13 bits below the group's largest exponent (toward zero); group sums are then added to float32
 *   accuracy.  A product more than 2^13 times smaller than a neighbour in its group is lost in part or whole.
 */
int mpsa_gemm_mx(const uint8_t* a, const uint8_t* sa, int fmt_a, const uint8_t* b, const uint8_t* sb, int fmt_b,
                 int64_t M, int64_t N, int64_t K, void* c, int c_dtype, int64_t ldc, mpsa_stream_t stream);

/*
 * The same product for every (batch, head): a [batch,heads_a,M,K'] and sa [batch,heads_a,M,K/32], b
 * [batch,heads_b,N,K'] and sb likewise, c [batch,heads_a,M,ldc], all contiguous; head h of a multiplies head
 * h / (heads_a/heads_b) of b (grouped heads; heads_a % heads_b == 0).  Replaces block_scaled_batched_matmul and its
 * Triton kernel (ours/batched_block_scaled_matmul.py:183-236, :43-180) - the batched Q.K^T of the reference's
 * mxfp_attn (ours/mxfp_attn.py:64-66) - with the 2-D kernel's semantics.
 */
int mpsa_gemm_mx_batched(const uint8_t* a, const uint8_t* sa, int fmt_a, const uint8_t* b, const uint8_t* sb, int fmt_b,
                         int64_t batch, int64_t heads_a, int64_t heads_b, int64_t M, int64_t N, int64_t K,
                         void* c, int c_dtype, int64_t ldc, mpsa_stream_t stream);

/*
 * Both products with the scales in the reference's packed form [rows/128, K/128, 32, 4, 4] - what its wrappers build
 * before calling the Triton kernel (ours/mxfp_attn_kernel.py:56-57, consumed at ours/block_scaled_matmul.py:207-216)
 * and what mpsa_scales_to_5d produces: byte (r%32)*16 + (r/32 % 4)*4 + k of chunk (r/128, kb/4) is the scale of row r,
 * K block kb = 4*(kb/4) + k.  The kernel fetches a 128-row x 128-element chunk as 512 contiguous bytes (a quarter of
 * the cache lines the row-major layout costs) and reads a lane's scale words for four row blocks with one 128-bit
 * LDS read.  Same results as the row-major entry points, bit for bit.  sa5, sb5: 16-byte aligned; M, N and K in
 * multiples of 128 (the layout's chunk).
 */
int mpsa_gemm_mx_packed(const uint8_t* a, const uint8_t* sa5, int fmt_a, const uint8_t* b, const uint8_t* sb5, int fmt_b,
                        int64_t M, int64_t N, int64_t K, void* c, int c_dtype, int64_t ldc, mpsa_stream_t stream);
int mpsa_gemm_mx_batched_packed(const uint8_t* a, const uint8_t* sa5, int fmt_a, const uint8_t* b, const uint8_t* sb5, int fmt_b,
                                int64_t batch, int64_t heads_a, int64_t heads_b, int64_t M, int64_t N, int64_t K,
                                void* c, int c_dtype, int64_t ldc, mpsa_stream_t stream);

/*
 * Value-tile repack: v [B,H,N,D] (bf16 | f16, strided, last dim contiguous) -> v_tiles
 * [B,H,ceil(N/tile),tile*D] of the same dtype in matrix-core operand order, keys past N zero.
 * Replaces the dtype normalisation / .contiguous() of V in the reference wrapper
 * (ours/mxfp_attn_kernel.py:27-31); the layout is this library's own.
 */
int mpsa_v_tiles(const void* v, int v_dtype, int64_t B, int64_t H, int64_t N, int64_t D,
                 const int64_t v_strides[4], int tile, void* v_tiles, mpsa_stream_t stream);

/*
 * All operands of one attention call in ONE launch: Q quantized with pre_scale_q folded in, K quantized (minus
 * k_sub if given, see mpsa_quantize_mx), V repacked - the results are bit-identical to the separate calls
 * mpsa_quantize_mx(_dual) on q and k (emax 3 for E2M1, 7 for the 8-bit format) and mpsa_v_tiles on v, rows padded to
 * ceil(Nq/tile)*tile and ceil(Nk/tile)*tile.  Replaces the prologue of the reference's wrapper, ours/mxfp_attn_kernel.py:27-57.
 *
 *   q [B,Hq,Nq,D], k and v [B,Hkv,Nk,D] of dtype (MPSA_BF16 | MPSA_F16), element strides as for mpsa_quantize_mx;
 *              q == NULL leaves Q out (its outputs are not touched): for mpsa_attn_fwd_q16, which quantizes Q itself
 *   mode       MPSA_MODE_MXFP4: only the 4-bit outputs are written (8-bit pointers may be null),
 *              MPSA_MODE_MXFP8: only the 8-bit ones, MPSA_MODE_DIAG / MPSA_MODE_ROUTED / MPSA_MODE_MIXED: both
 *   k_sub      NULL or [B,Hkv,D] (smooth-K mean from mpsa_seq_mean)
 *   outputs    as the inputs of mpsa_attn_fwd
 */
int mpsa_attn_prepare(const void* q, const int64_t q_strides[4], const void* k, const int64_t k_strides[4],
                      const void* v, const int64_t v_strides[4], int dtype,
                      int64_t B, int64_t Hq, int64_t Hkv, int64_t Nq, int64_t Nk, int64_t D, int tile, int mode, int fmt8,
                      float pre_scale_q, const void* k_sub,
                      uint8_t* q4, uint8_t* qs4, uint8_t* q8, uint8_t* qs8,
                      uint8_t* k4, uint8_t* ks4, uint8_t* k8, uint8_t* ks8, void* v_tiles, mpsa_stream_t stream);

/*
 * Fused attention forward.  Replaces block_scaled_batched_attn and its Triton kernel
 * (ours/mxfp_attn_kernel.py:362-423, :103-359), with the causal tile structure and grouped-query
 * head mapping of ours/online_routing.py:68-77, :113-118, :160-171.
 *
 *   q4,qs4 / q8,qs8   Q codes + scales from the quantizer, rows padded to nq_pad per head:
 *                     [B,Hq,nq_pad,D/2],[B,Hq,nq_pad,D/32] and [B,Hq,nq_pad,D],[B,Hq,nq_pad,D/32]
 *   k4,ks4 / k8,ks8   same for K with Hkv heads and nk_pad rows
 *                     (the 4-bit set may be null in MPSA_MODE_MXFP8, the 8-bit set in MPSA_MODE_MXFP4;
 *                     MPSA_MODE_MIXED reads q8, qs8, k4, ks4 only)
 *   fmt8              MPSA_FMT_E4M3 | MPSA_FMT_E5M2
 *   v_tiles           output of mpsa_v_tiles for the same tile, pv_dtype (MPSA_BF16 | MPSA_F16);
 *                     P is rounded to that dtype before P.V
 *   o                 [B,Hq,nq,D] of o_dtype (MPSA_BF16 | MPSA_F16 | MPSA_F32), element strides o_strides[4],
 *                     last dim contiguous
 *   nq, nk            valid query and key/value counts, each padded to ceil(count/tile)*tile rows; the reference takes them
 *                     separately as well (M and N of block_scaled_batched_attn, ours/mxfp_attn_kernel.py:362-371);
 *                     causal masking and MPSA_MODE_DIAG need nq == nk
 *   tile              64 | 128 (score tile edge = precision granularity), D in {64,128}
 */
int mpsa_attn_fwd(const uint8_t* q4, const uint8_t* qs4, const uint8_t* q8, const uint8_t* qs8,
                  const uint8_t* k4, const uint8_t* ks4, const uint8_t* k8, const uint8_t* ks8, int fmt8,
                  const void* v_tiles, int pv_dtype, void* o, int o_dtype, const int64_t o_strides[4],
                  int64_t B, int64_t Hq, int64_t Hkv, int64_t nq, int64_t nk, int64_t D, int tile, int causal, int mode,
                  mpsa_stream_t stream);

/*
 * Fused attention forward that takes Q UNQUANTIZED and MX-quantizes it inside the kernel, in registers: the quantizer
 * call for Q of the reference's wrapper (quant_mxfp4 / quant_mxfp8e5 on q, ours/mxfp_attn_kernel.py:43-50,
 * ours/quant_mxint8.py:479-494) and the attention launch (ours/mxfp_attn_kernel.py:66-70) in one; Q's codes and scales
 * never travel through HBM (at the B1 Hq32 N8192 shape that is 52 MB written and read back).  Same bits as
 * mpsa_attn_prepare + mpsa_attn_fwd.  Built for the paired-tile kernel's shapes only: D = 128, tile = 128, any mode but
 * MPSA_MODE_ROUTED (MPSA_MODE_MIXED and MPSA_MODE_MXFP8 quantize Q to 8 bits only, MPSA_MODE_MXFP4 to 4 bits only, and
 * the K operands a mode does not multiply may be NULL); causal with at least two key tiles (n >= 129), or unmasked with at least six
 * (n >= 641); n need not be a multiple of the tile -- mpsa_attn_fwd_q16_supported() says whether a shape qualifies (1)
 * or not (0); other shapes return MPSA_EUNSUPPORTED and go through mpsa_attn_prepare + mpsa_attn_fwd.
 *   q            [B,Hq,n,D] of q_dtype == pv_dtype (MPSA_BF16 | MPSA_F16), element strides q_strides[4], last dim
 *                contiguous, rows 16-byte aligned
 *   pre_scale_q  float32 factor folded in before quantizing (sm_scale * log2(e))
 *   k4 .. v_tiles, o   as for mpsa_attn_fwd; mpsa_attn_prepare with q == NULL prepares just these (K and V)
 */
int mpsa_attn_fwd_q16(const void* q, const int64_t q_strides[4], int q_dtype, float pre_scale_q,
                      const uint8_t* k4, const uint8_t* ks4, const uint8_t* k8, const uint8_t* ks8, int fmt8,
                      const void* v_tiles, int pv_dtype, void* o, int o_dtype, const int64_t o_strides[4],
                      int64_t B, int64_t Hq, int64_t Hkv, int64_t n, int64_t D, int tile, int causal, int mode,
                      mpsa_stream_t stream);
int mpsa_attn_fwd_q16_supported(int64_t B, int64_t Hq, int64_t Hkv, int64_t n, int64_t D, int tile, int causal, int mode);

/*
 * Fused attention forward with the reference's tile-skipping rule (the skip_thresh argument of mxfp_attn /
 * mxfp_attn_kernel, ours/mxfp_attn.py:32, ours/mxfp_attn_kernel.py:272-297, with the key/value pointers advancing
 * past a skipped tile, which the reference's loop forgets): for query tile i, the statistic of key tile j is the mean
 * over the tile's valid query rows of the row maximum of S (after masking); tile 0 is always kept and sets the
 * reference value; tile j > 0 is kept iff stat(j) >= stat(0) * skip_thresh, and the diagonal tile of a causal run is
 * always kept (ours/online_routing.py:68-77: its stage starts a loop of its own); a skipped tile contributes nothing.
 * Arguments as mpsa_attn_fwd; mode MPSA_MODE_MXFP4, MPSA_MODE_MXFP8, MPSA_MODE_MIXED or MPSA_MODE_DIAG (each tile's
 * statistic is that of the precision the tile runs in), plus
 *   skip_thresh   the factor above (scores are in log2 units with sm_scale folded in, as in the reference)
 *   skipped       NULL, or int32 [B,Hq,ceil(n/tile)]: number of key tiles skipped for each query tile
 */
int mpsa_attn_fwd_skip(const uint8_t* q4, const uint8_t* qs4, const uint8_t* q8, const uint8_t* qs8,
                       const uint8_t* k4, const uint8_t* ks4, const uint8_t* k8, const uint8_t* ks8, int fmt8,
                       const void* v_tiles, int pv_dtype, void* o, int o_dtype, const int64_t o_strides[4],
                       int64_t B, int64_t Hq, int64_t Hkv, int64_t nq, int64_t nk, int64_t D, int tile, int causal, int mode,
                       float skip_thresh, int32_t* skipped, mpsa_stream_t stream);

/*
 * Tile router: precision class of every (query tile, key tile) pair from the 4-bit E8M0 scale bytes of Q and K.
 * The reference's online routing keeps or skips a tile by comparing a tile statistic with the first tile's
 * (ours/online_routing.py:87-112, the skip_thresh of ours/mxfp_attn.py:32); this router extends that to a precision
 * choice and takes the statistic from the quantizer's own output.  Per tile and 32-wide block c of the head
 * dimension, over the tile's rows r (e = scale byte): M[c] = max_r e[r][c], F[c] = sum_r 2^(10 - (M[c] - e[r][c]))
 * with terms below 1 dropped.  For query tile I and key tile J: s[c] = Mq[I][c] + Mk[J][c], w[c] = Fq[I][c] * Fk[J][c],
 * smax[I] the largest s[c] over the visited key tiles, T[I][J] = (sum_c (w[c] >> (smax[I] - s[c]))) >> 13 (shifts
 * above 40 give 0) and Tmax[I] the largest T[I][J]:
 *     8-bit    if (float)T >= hi_thresh * (float)Tmax
 *     skipped  else if (float)T < skip_thresh * (float)Tmax and J != 0 and not (causal and J == I)
 *     4-bit    otherwise;                         a threshold <= 0 switches its class off.
 * T is proportional to the summed magnitude bound of the tile's scores, i.e. to the absolute error of a 4-bit product.
 *   qs4, ks4   [B,Hq,nq_pad,D/32], [B,Hkv,nk_pad,D/32] from the quantizer (padding rows zero)
 *   work       mpsa_route_workspace(...) bytes of device memory (the per-tile statistics), 4-byte aligned
 *   cls        out, uint8 [B,Hq,ntq,ntk]: 0 skipped, 1 4-bit, 2 8-bit, 255 not visited (causal, J > I)
 *   order      out, int32 [B,Hq,ntq,ntk]: per query tile the key tiles to visit -- 4-bit ones that need no mask
 *              (ascending), 4-bit ones that do (the diagonal tile of a causal run, the tile holding a ragged sequence
 *              end), then the 8-bit ones likewise; the rest is -1
 *   counts     out, int32 [B,Hq,ntq,4]: lengths of those four runs
 */
int64_t mpsa_route_workspace(int64_t B, int64_t Hq, int64_t Hkv, int64_t nq, int64_t nk, int64_t D, int tile);
int mpsa_route_tiles(const uint8_t* qs4, const uint8_t* ks4, int64_t B, int64_t Hq, int64_t Hkv, int64_t nq, int64_t nk,
                     int64_t D, int tile, int causal, float hi_thresh, float skip_thresh, void* work,
                     uint8_t* cls, int32_t* order, int32_t* counts, mpsa_stream_t stream);

/*
 * Tile skipping decided ahead of the attention kernel: the reference's rule (ours/mxfp_attn_kernel.py:272-297 -- the
 * statistic of a score tile is the mean over its query rows of the row maximum of S; key tile 0 is always kept and sets
 * the reference value, tile j > 0 is kept iff stat(j) >= stat(0) * skip_thresh; the diagonal tile of a causal run is
 * kept, ours/online_routing.py:68-77) applied to the statistics of ALL tiles, which a score-product-only kernel takes
 * first, and written out as the visiting lists of mpsa_attn_fwd_routed.  Same decisions as mpsa_attn_fwd_skip (which
 * applies the rule inside the attention kernel, tile by tile); the attention call that follows visits the kept tiles
 * only, so that skipped tiles cost a fifth of a tile's matrix work and nothing else.
 * D = 128, tile = 128, mode MPSA_MODE_MXFP4 | MPSA_MODE_MXFP8 | MPSA_MODE_DIAG, at most MPSA_SKIP_ROUTE_MAX_TILES key
 * tiles: mpsa_skip_route_supported() says whether a shape qualifies (1) or not (0).
 *   q4 .. ks8, fmt8   the quantized operands of mpsa_attn_prepare (the sets the mode multiplies)
 *   work       mpsa_skip_route_workspace(...) bytes of device memory (the statistics, float32 [B,Hq,ntq,ntk]), 4-byte aligned
 *   cls        out, optional (may be NULL), uint8 [B,Hq,ntq,ntk]: 0 skipped, 1 4-bit, 2 8-bit, 255 not visited
 *   order, counts   out, as mpsa_route_tiles writes them
 *   skipped    out, optional, int32 [B,Hq,ntq]: number of skipped key tiles per query tile
 */
#define MPSA_SKIP_ROUTE_MAX_TILES 2048
int mpsa_skip_route_supported(int64_t nq, int64_t nk, int64_t D, int tile, int causal, int mode);
int64_t mpsa_skip_route_workspace(int64_t B, int64_t Hq, int64_t nq, int64_t nk, int tile);
int mpsa_skip_route(const uint8_t* q4, const uint8_t* qs4, const uint8_t* q8, const uint8_t* qs8,
                    const uint8_t* k4, const uint8_t* ks4, const uint8_t* k8, const uint8_t* ks8, int fmt8,
                    int64_t B, int64_t Hq, int64_t Hkv, int64_t nq, int64_t nk, int64_t D, int tile, int causal, int mode,
                    float skip_thresh, void* work, uint8_t* cls, int32_t* order, int32_t* counts, int32_t* skipped,
                    mpsa_stream_t stream);

/*
 * Fused attention forward over visiting lists (per-tile precision; BLKQ x BLKQ granularity as in mpsa_attn_fwd).
 * Arguments as mpsa_attn_fwd without mode, plus order / counts as written by mpsa_route_tiles or mpsa_skip_route -- or
 * by the caller: any list of distinct key tiles works, as long as every tile that needs a mask sits in a masked run.
 * Both operand sets are needed unless the lists name tiles of one precision only: then the other set (q and k codes and
 * scales of that width) may be NULL.  Key tiles not on a query tile's list contribute nothing; a query tile with an
 * empty list returns zeros.  Out-of-range list entries and run lengths are clamped, never followed.
 */
int mpsa_attn_fwd_routed(const uint8_t* q4, const uint8_t* qs4, const uint8_t* q8, const uint8_t* qs8,
                         const uint8_t* k4, const uint8_t* ks4, const uint8_t* k8, const uint8_t* ks8, int fmt8,
                         const void* v_tiles, int pv_dtype, void* o, int o_dtype, const int64_t o_strides[4],
                         int64_t B, int64_t Hq, int64_t Hkv, int64_t nq, int64_t nk, int64_t D, int tile, int causal,
                         const int32_t* order, const int32_t* counts, mpsa_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MPSA_H */
