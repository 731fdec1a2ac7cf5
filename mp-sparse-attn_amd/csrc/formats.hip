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

template <typename K, typename... A>
int run(const char* what, K kern, int64_t n, hipStream_t st, A... args) {
    if (n < 0) return mpsa_fail(MPSA_EINVAL, "%s: negative length", what);
    if (n == 0) return MPSA_OK;
    if ((n + 255) / 256 >= (int64_t(1) << 31)) return mpsa_fail(MPSA_EUNSUPPORTED, "%s: too many elements", what);
    hipLaunchKernelGGL(kern, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, args...);
    MPSA_CHECK_LAUNCH(what);
    return MPSA_OK;
}

}  // namespace

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
