// Elementwise format kernels behind the MXFP4Tensor / MXScaleTensor helper classes (gfx950).
//
//   E2M1 encode  -- MXFP4Tensor._from_float   (ours/mxfp.py:84-170), one code per byte
//   E2M1 decode  -- MXFP4Tensor.to(float32)   (ours/mxfp.py:44-77)
//   E8M0 encode  -- MXScaleTensor._from_float (ours/mxfp.py:286-307)
//   E8M0 decode  -- MXScaleTensor.to(float32) (ours/mxfp.py:275-284)
// All four stream contiguous arrays: HBM-bound.
#include "mpsa_common.h"
#include "mx_codec.h"

namespace {

// Literal form of the reference encoder: float32 distance to all eight magnitudes, 1e-6f off the
// even-mantissa ones, first minimum wins.  (For magnitudes beyond 2^24 float32 cancellation makes several
// distances equal and the reference then returns a smaller code, down to zero; this keeps that behaviour,
// which the two-candidate form used inside the quantizer -- inputs clamped to 6 -- need not.)
__global__ __launch_bounds__(256) void e2m1_encode_kernel(const float* x, int64_t n, uint8_t* out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float v = x[i];
    const uint32_t u = mpsa_f2u(v);
    const uint32_t mag = u & 0x7FFFFFFFu;
    const float a = mag >= 0x7F800000u ? 6.0f : mpsa_u2f(mag);      // NaN and Inf take the largest magnitude
    const float cand[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
    uint32_t best = 0;
    float best_err = __builtin_fabsf(a - cand[0]) - 1e-6f;
#pragma unroll
    for (uint32_t c = 1; c < 8; ++c) {
        const float err = __builtin_fabsf(a - cand[c]) - ((c & 1u) ? 0.0f : 1e-6f);
        if (err < best_err) { best_err = err; best = c; }
    }
    if (mag == 0u) best = 0;
    out[i] = (uint8_t)(((u >> 31) << 3) | best);
}

__global__ __launch_bounds__(256) void e2m1_decode_kernel(const uint8_t* c, int64_t n, float* out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = e2m1_decode(c[i]);
}

__global__ __launch_bounds__(256) void e8m0_encode_kernel(const float* x, int64_t n, uint8_t* out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const uint32_t u = mpsa_f2u(x[i]);
    uint32_t code;
    if ((u >> 31) || u == 0u || u >= 0x7F800000u) {
        code = 255u;                                   // <= 0, NaN, Inf
    } else {
        const uint32_t ef = u >> 23;                   // biased exponent = floor(log2 v) + 127 for normals
        code = ef > 254u ? 254u : ef;                  // subnormals: ef == 0, i.e. clamp(.., 0, 254)
    }
    out[i] = (uint8_t)code;
}

__global__ __launch_bounds__(256) void e8m0_decode_kernel(const uint8_t* c, int64_t n, float* out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const uint32_t e = c[i];
    // 2^(e-127): e == 0 is the subnormal 2^-127, e == 255 is NaN
    out[i] = e == 255u ? mpsa_u2f(0x7FC00000u) : (e == 0u ? mpsa_u2f(0x00400000u) : mpsa_u2f(e << 23));
}

// float32 -> one FP8 byte, the cast torch performs for x.to(torch.float8_e5m2) / x.to(torch.float8_e4m3fn): round to
// nearest even, no saturation.  E5M2 overflows to infinity (0x7C) and keeps NaN (0x7F); E4M3 ("fn": no infinities)
// turns everything that rounds beyond 448 into NaN (0x7F).  The reference's operand packaging casts its 8-bit
// operands this way (ours/block_scaled_matmul.py:334-336, :349-351).
template <int FMT>
__global__ __launch_bounds__(256) void fp8_encode_kernel(const float* x, int64_t n, uint8_t* out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const uint32_t u = mpsa_f2u(x[i]);
    const uint32_t sign = (u >> 24) & 0x80u;
    uint32_t a = u & 0x7FFFFFFFu;
    uint32_t code;
    if (a > 0x7F800000u) {
        code = 0x7Fu;
    } else if constexpr (FMT == MPSA_FMT_E5M2) {
        if (a >= 0x38800000u) {                       // |x| >= 2^-14: normal
            a += 0xFFFFFu + ((a >> 21) & 1u);
            code = (a >> 21) - (112u << 2);
            code = code > 0x7Cu ? 0x7Cu : code;
        } else {                                      // subnormal, unit 2^-16
            code = mpsa_f2u(mpsa_u2f(a) + 128.0f) - 0x43000000u;
        }
    } else {
        if (a >= 0x43F00000u) {                       // |x| >= 480 (incl. infinity)
            code = 0x7Fu;
        } else if (a >= 0x3C800000u) {                // |x| >= 2^-6: normal
            a += 0x7FFFFu + ((a >> 20) & 1u);
            code = (a >> 20) - (120u << 3);
            code = code > 0x7Fu ? 0x7Fu : code;
        } else {                                      // subnormal, unit 2^-9
            code = mpsa_f2u(mpsa_u2f(a) + 16384.0f) - 0x46800000u;
        }
    }
    out[i] = (uint8_t)(sign | code);
}

template <typename K, typename... A>
int run(const char* what, K kern, int64_t n, hipStream_t st, A... args) {
    if (n < 0) return mpsa_fail(MPSA_EINVAL, "%s: negative length", what);
    if (n == 0) return MPSA_OK;
    if ((n + 255) / 256 >= (int64_t(1) << 31)) return mpsa_fail(MPSA_EUNSUPPORTED, "%s: too many elements", what);
    hipLaunchKernelGGL(kern, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, args...);
    MPSA_CHECK_LAUNCH(what);
    return MPSA_OK;
}

// Scale re-layout between the linear [rows, K/32] form and the 5-D packed form of the reference's block-scaled
// kernels, [rows/128, K/128, 32, 4, 4] with packed[cm][ck][r32][r4][c4] = linear[cm*128 + r4*32 + r32][ck*4 + c4]
// (ours/mxfp_attn_kernel.py:56-57, ours/block_scaled_matmul.py:384 for the way back).  The innermost c4 group is four
// consecutive bytes in both forms, so a thread moves one 32-bit word; `w` runs over the packed form's words.
template <bool TO_PACKED>
__global__ __launch_bounds__(256) void scale_layout_kernel(const uint32_t* src, uint32_t* dst, int64_t words_per_batch, int kc) {
    const int64_t w = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (w >= words_per_batch) return;
    const int64_t boff = (int64_t)blockIdx.y * words_per_batch;
    const int r4 = (int)(w & 3), r32 = (int)((w >> 2) & 31);
    const int64_t t = w >> 7;                      // cm * kc + ck
    const int64_t cm = t / kc;
    const int ck = (int)(t - cm * kc);
    const int64_t lin = (cm * 128 + r4 * 32 + r32) * kc + ck;
    if (TO_PACKED) dst[boff + w] = src[boff + lin];
    else           dst[boff + lin] = src[boff + w];
}

// Nibble packing along one dimension of a contiguous code tensor seen as [outer, n, inner]:
// packed[o][i][x] = codes[o][2i][x] | codes[o][2i+1][x] << 4, an odd n padded with a zero code
// (MXFP4Tensor.to_packed_tensor / unpack_packed_tensor, ours/mxfp.py:172-236).  One thread per packed byte.
template <bool PACK>
__global__ __launch_bounds__(256) void nibble_kernel(const uint8_t* src, uint8_t* dst, int64_t outer, int64_t n, int64_t inner) {
    const int64_t np = (n + 1) / 2;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= outer * np * inner) return;
    const int64_t x = idx % inner, i = (idx / inner) % np, o = idx / (inner * np);
    const int64_t lo = (o * n + 2 * i) * inner + x, hi = lo + inner;
    const bool has_hi = 2 * i + 1 < n;
    if (PACK) {
        dst[idx] = (uint8_t)((src[lo] & 0xF) | (has_hi ? (src[hi] & 0xF) << 4 : 0));
    } else {
        const uint8_t b = src[idx];
        dst[lo] = b & 0xF;
        if (has_hi) dst[hi] = b >> 4;
    }
}

int nibble_run(const char* what, const uint8_t* src, int64_t outer, int64_t n, int64_t inner, uint8_t* dst, bool pack, hipStream_t st) {
    if (outer < 0 || n < 0 || inner < 0) return mpsa_fail(MPSA_EINVAL, "%s: bad shape", what);
    const int64_t total = outer * ((n + 1) / 2) * inner;
    if (total == 0) return MPSA_OK;
    if (!src || !dst) return mpsa_fail(MPSA_EINVAL, "%s: null pointer", what);
    if (total >= (int64_t(1) << 39)) return mpsa_fail(MPSA_EUNSUPPORTED, "%s: tensor too large", what);
    const dim3 grid((unsigned)((total + 255) / 256));
    if (pack) hipLaunchKernelGGL(nibble_kernel<true>, grid, dim3(256), 0, st, src, dst, outer, n, inner);
    else      hipLaunchKernelGGL(nibble_kernel<false>, grid, dim3(256), 0, st, src, dst, outer, n, inner);
    MPSA_CHECK_LAUNCH(what);
    return MPSA_OK;
}

int scale_layout(const char* what, const uint8_t* src, int64_t batch, int64_t rows, int64_t kblocks, uint8_t* dst,
                 bool to_packed, hipStream_t st) {
    if (batch <= 0 || rows <= 0 || kblocks <= 0) return mpsa_fail(MPSA_EINVAL, "%s: bad shape", what);
    if (rows % 128 || kblocks % 4) return mpsa_fail(MPSA_EUNSUPPORTED, "%s: rows must be a multiple of 128 and K of 128 (got rows=%lld, K/32=%lld)", what, (long long)rows, (long long)kblocks);
    if (!src || !dst) return mpsa_fail(MPSA_EINVAL, "%s: null pointer", what);
    if ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 3) return mpsa_fail(MPSA_EALIGN, "%s: pointers must be 4-byte aligned", what);
    const int64_t words = rows * (kblocks / 4);
    if (batch > 65535 || words >= (int64_t(1) << 38)) return mpsa_fail(MPSA_EUNSUPPORTED, "%s: shape too large", what);
    dim3 grid((unsigned)((words + 255) / 256), (unsigned)batch);
    if (to_packed) hipLaunchKernelGGL(scale_layout_kernel<true>, grid, dim3(256), 0, st, reinterpret_cast<const uint32_t*>(src), reinterpret_cast<uint32_t*>(dst), words, (int)(kblocks / 4));
    else           hipLaunchKernelGGL(scale_layout_kernel<false>, grid, dim3(256), 0, st, reinterpret_cast<const uint32_t*>(src), reinterpret_cast<uint32_t*>(dst), words, (int)(kblocks / 4));
    MPSA_CHECK_LAUNCH(what);
    return MPSA_OK;
}

}  // namespace

extern "C" int mpsa_e2m1_pack(const uint8_t* codes, int64_t outer, int64_t n, int64_t inner, uint8_t* packed, mpsa_stream_t stream) {
    return nibble_run("e2m1_pack", codes, outer, n, inner, packed, true, (hipStream_t)stream);
}
extern "C" int mpsa_e2m1_unpack(const uint8_t* packed, int64_t outer, int64_t n, int64_t inner, uint8_t* codes, mpsa_stream_t stream) {
    return nibble_run("e2m1_unpack", packed, outer, n, inner, codes, false, (hipStream_t)stream);
}

extern "C" int mpsa_scales_to_5d(const uint8_t* linear, int64_t batch, int64_t rows, int64_t kblocks, uint8_t* packed, mpsa_stream_t stream) {
    return scale_layout("scales_to_5d", linear, batch, rows, kblocks, packed, true, (hipStream_t)stream);
}
extern "C" int mpsa_scales_from_5d(const uint8_t* packed, int64_t batch, int64_t rows, int64_t kblocks, uint8_t* linear, mpsa_stream_t stream) {
    return scale_layout("scales_from_5d", packed, batch, rows, kblocks, linear, false, (hipStream_t)stream);
}

extern "C" int mpsa_e2m1_encode(const float* x, int64_t n, uint8_t* codes, mpsa_stream_t stream) {
    if (n > 0 && (!x || !codes)) return mpsa_fail(MPSA_EINVAL, "e2m1_encode: null pointer");
    return run("e2m1_encode", e2m1_encode_kernel, n, (hipStream_t)stream, x, n, codes);
}
extern "C" int mpsa_e2m1_decode(const uint8_t* codes, int64_t n, float* out, mpsa_stream_t stream) {
    if (n > 0 && (!codes || !out)) return mpsa_fail(MPSA_EINVAL, "e2m1_decode: null pointer");
    return run("e2m1_decode", e2m1_decode_kernel, n, (hipStream_t)stream, codes, n, out);
}
extern "C" int mpsa_e8m0_encode(const float* x, int64_t n, uint8_t* codes, mpsa_stream_t stream) {
    if (n > 0 && (!x || !codes)) return mpsa_fail(MPSA_EINVAL, "e8m0_encode: null pointer");
    return run("e8m0_encode", e8m0_encode_kernel, n, (hipStream_t)stream, x, n, codes);
}
extern "C" int mpsa_e8m0_decode(const uint8_t* codes, int64_t n, float* out, mpsa_stream_t stream) {
    if (n > 0 && (!codes || !out)) return mpsa_fail(MPSA_EINVAL, "e8m0_decode: null pointer");
    return run("e8m0_decode", e8m0_decode_kernel, n, (hipStream_t)stream, codes, n, out);
}
extern "C" int mpsa_fp8_encode(const float* x, int64_t n, int fmt, uint8_t* codes, mpsa_stream_t stream) {
    if (fmt != MPSA_FMT_E4M3 && fmt != MPSA_FMT_E5M2) return mpsa_fail(MPSA_EINVAL, "fp8_encode: format must be E4M3 or E5M2");
    if (n > 0 && (!x || !codes)) return mpsa_fail(MPSA_EINVAL, "fp8_encode: null pointer");
    if (fmt == MPSA_FMT_E5M2) return run("fp8_encode", fp8_encode_kernel<MPSA_FMT_E5M2>, n, (hipStream_t)stream, x, n, codes);
    return run("fp8_encode", fp8_encode_kernel<MPSA_FMT_E4M3>, n, (hipStream_t)stream, x, n, codes);
}
