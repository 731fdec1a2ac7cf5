// MX quantizer for gfx950: bf16/f16 rows -> E2M1 / E4M3 / E5M2 codes + one E8M0 scale per 32 elements.
//
// Semantics follow the reference's quantizer (ours/quant_mxint8.py:276-351 for E2M1, :164-219 for the
// 8-bit format): x32 = f32(x) * pre; amax per 32 elements of the last dim; shared exponent
// floor(log2(amax)) - emax_elem; divide by that power of two; clamp; encode; scale byte
// clamp(shared_exp + 127, 0, 254).  The E2M1 encoder reproduces MXFP4Tensor._from_float
// (ours/mxfp.py:84-170) bit for bit, including its float32 1e-6 tie-break bias; codes leave the
// kernel already nibble-packed (ours/mxfp.py:196-205: even element in the low nibble).
//
// Smooth-K (ours/mxfp_attn.py:44-45, ours/mxfp_attn_kernel.py:33-34: k = k - k.mean(dim=-2, keepdim=True) in k's
// 16-bit dtype) is folded in: seq_mean_kernel + seq_mean_finish_kernel produce the per-(batch, head, channel) mean
// over the sequence, rounded to the input dtype, and the quantizer subtracts it - rounding the difference to the
// input dtype again, as the elementwise torch op would - before it does anything else.
//
// Work mapping: one lane owns 8 consecutive elements (one 128-bit load), four neighbouring lanes
// own one MX block, so the block maximum is two DPP quad exchanges.  The kernel is HBM-bound:
// 2 B/element in, 0.5 (+1) B/element of codes and 1/32 (x2) B/element of scales out.
#include "mpsa_common.h"
#include <cstring>
#include "mx_codec.h"

namespace {

struct QuantArgs {
    const void* x;
    const void* sub;           // optional [B,H,D] of x's dtype, subtracted (and the difference rounded to that dtype) first
    int64_t sb, sh, sn;        // element strides of x
    int n, d;                  // valid rows, row length
    int out_rows;              // rows per (b,h) in the outputs
    float pre;
    int exact16;               // pre is a power of two: scaled values keep the inputs' 16-bit significands
    int emax4, emax8;
    uint8_t *codes4, *scales4, *codes8, *scales8;
};

template <int DPP_CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), DPP_CTRL, 0xf, 0xf, false));
}

template <int FMT8, bool SW8>
__device__ __forceinline__ uint32_t fp8_pack4(float y0, float y1, float y2, float y3) {
    if constexpr (SW8) {
        if constexpr (FMT8 == MPSA_FMT_E4M3)
            return e4m3_encode_sw(y0) | (e4m3_encode_sw(y1) << 8) | (e4m3_encode_sw(y2) << 16) | (e4m3_encode_sw(y3) << 24);
        else
            return e5m2_encode_sw(y0) | (e5m2_encode_sw(y1) << 8) | (e5m2_encode_sw(y2) << 16) | (e5m2_encode_sw(y3) << 24);
    } else {
        int w = 0;
        if constexpr (FMT8 == MPSA_FMT_E4M3) {
            w = __builtin_amdgcn_cvt_pk_fp8_f32(y0, y1, w, false);
            w = __builtin_amdgcn_cvt_pk_fp8_f32(y2, y3, w, true);
        } else {
            w = __builtin_amdgcn_cvt_pk_bf8_f32(y0, y1, w, false);
            w = __builtin_amdgcn_cvt_pk_bf8_f32(y2, y3, w, true);
        }
        return (uint32_t)w;
    }
}

template <int XDT>
__device__ __forceinline__ void load8(const void* p, float (&x)[8]) {
    const uint4 raw = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if constexpr (XDT == MPSA_BF16) {
            x[2 * i] = mpsa_u2f(w[i] << 16);
            x[2 * i + 1] = mpsa_u2f(w[i] & 0xFFFF0000u);
        } else {
            x[2 * i] = (float)__builtin_bit_cast(_Float16, (unsigned short)(w[i] & 0xFFFFu));
            x[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (unsigned short)(w[i] >> 16));
        }
    }
}

// round a float32 to the 16-bit dtype XDT (nearest even) and back
template <int XDT>
__device__ __forceinline__ float round16(float v) {
    if constexpr (XDT == MPSA_BF16) {
        const uint32_t u = mpsa_f2u(v);
        return mpsa_u2f((u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u);
    } else {
        return (float)(_Float16)v;
    }
}

// Eight E2M1 codes (one packed word, element i in nibble i) of x[0..7] / 2^se.
// Fast path: v_cvt_scalef32_pk_fp4_f32 divides by the power of two and rounds to nearest, ties to even.  The
// reference's rule (argmin of float32 distances with 1e-6 taken off the even-mantissa candidate, e2m1_index in
// mx_codec.h) differs from that only for a value within about 1e-6 of the midpoint between two E2M1 values.  Such
// a value is found by converting the inputs nudged down and up by 2^-17 of themselves: if the two conversions
// differ anywhere in the word, the lane falls back to the explicit rule.  (2^-17 of a value near a midpoint - the
// smallest is 0.25 - is at least 1.9e-6.)  Scales too small for a normal float32 take the explicit rule as well.
// When the pre-scale is a power of two the scaled values are 16-bit inputs times a power of two, at most 11
// significant bits: such a value is either exactly a midpoint - where the two rules agree (both take the even
// mantissa) - or at least 2^-12 away from one, so the check is skipped (`exact16`); it would otherwise fire on every
// exact tie, which 16-bit data hits all the time.
template <bool HW4>
__device__ __forceinline__ uint32_t e2m1_pack8(const float (&x)[8], int se, bool exact16) {
    if constexpr (HW4) {
        if (se >= -126) {
            const float sc = mpsa_u2f((uint32_t)(se + 127) << 23);
            const float dn = 1.0f - 0x1p-17f, up = 1.0f + 0x1p-17f;
            uint32_t w = 0, wd = 0, wu = 0;
            w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, x[0], x[1], sc, 0);
            w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, x[2], x[3], sc, 1);
            w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, x[4], x[5], sc, 2);
            w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, x[6], x[7], sc, 3);
            if (exact16) return w;
            wd = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(wd, x[0] * dn, x[1] * dn, sc, 0);
            wd = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(wd, x[2] * dn, x[3] * dn, sc, 1);
            wd = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(wd, x[4] * dn, x[5] * dn, sc, 2);
            wd = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(wd, x[6] * dn, x[7] * dn, sc, 3);
            wu = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(wu, x[0] * up, x[1] * up, sc, 0);
            wu = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(wu, x[2] * up, x[3] * up, sc, 1);
            wu = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(wu, x[4] * up, x[5] * up, sc, 2);
            wu = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(wu, x[6] * up, x[7] * up, sc, 3);
            if (wd == wu) return w;
        }
    }
    uint32_t word = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) word |= e2m1_encode(ldexpf(x[i], -se)) << (4 * i);
    return word;
}

template <int XDT, bool DO4, bool DO8, int FMT8, bool SW8>
__global__ __launch_bounds__(256) void quantize_kernel(QuantArgs a) {
    const uint32_t cpr = (uint32_t)a.d >> 3;                              // 16-byte chunks per row
    const uint32_t chunks = (uint32_t)a.out_rows * cpr;                   // per (b,h)
    const uint32_t c = blockIdx.x * 256u + threadIdx.x;
    if (c >= chunks) return;                                              // whole quads leave together (cpr % 4 == 0)
    const uint32_t row = c / cpr;
    const uint32_t col8 = c - row * cpr;
    const int64_t head = (int64_t)blockIdx.z * gridDim.y + blockIdx.y;    // flat (b,h)

    float x[8];
    if (row < (uint32_t)a.n) {
        const char* base = static_cast<const char*>(a.x) +
                           2 * ((int64_t)blockIdx.z * a.sb + (int64_t)blockIdx.y * a.sh + (int64_t)row * a.sn + 8 * (int64_t)col8);
        load8<XDT>(base, x);
        if (a.sub) {
            float m[8];
            load8<XDT>(static_cast<const char*>(a.sub) + 2 * (head * a.d + 8 * (int64_t)col8), m);
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] = round16<XDT>(x[i] - m[i]);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = 0.0f;
    }
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        x[i] = x[i] * a.pre;
        amax = __builtin_fmaxf(amax, __builtin_fabsf(x[i]));
    }
    amax = __builtin_fmaxf(amax, dpp_f32<0xB1>(amax));   // quad_perm [1,0,3,2]
    amax = __builtin_fmaxf(amax, dpp_f32<0x4E>(amax));   // quad_perm [2,3,0,1]

    const uint32_t ab = mpsa_f2u(amax);
    const bool zero = (ab == 0u);
    const uint32_t ef = ab >> 23;
    const int e = ef ? (int)ef - 127 : (31 - __builtin_clz(ab | 1u)) - 149;   // floor(log2(amax)), subnormals included

    const int64_t oc = head * chunks + c;                                 // flat output chunk
    const bool quad_leader = (threadIdx.x & 3u) == 0u;

    if constexpr (DO4) {
        const int se = e - a.emax4;
        const uint32_t word = zero ? 0u : e2m1_pack8<!SW8>(x, se, a.exact16 != 0);
        reinterpret_cast<uint32_t*>(a.codes4)[oc] = word;
        const int sbyte = zero ? 0 : min(max(se + 127, 0), 254);
        if (quad_leader) a.scales4[oc >> 2] = (uint8_t)sbyte;
    }
    if constexpr (DO8) {
        const int se = e - a.emax8;
        const float lim = (FMT8 == MPSA_FMT_E4M3) ? 448.0f : 57344.0f;
        uint2 w = make_uint2(0u, 0u);
        if (!zero) {
            float y[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) y[i] = __builtin_fminf(__builtin_fmaxf(ldexpf(x[i], -se), -lim), lim);
            w.x = fp8_pack4<FMT8, SW8>(y[0], y[1], y[2], y[3]);
            w.y = fp8_pack4<FMT8, SW8>(y[4], y[5], y[6], y[7]);
        }
        reinterpret_cast<uint2*>(a.codes8)[oc] = w;
        const int sbyte = zero ? 0 : min(max(se + 127, 0), 254);
        if (quad_leader) a.scales8[oc >> 2] = (uint8_t)sbyte;
    }
}

// ---- mean over the sequence, per (batch, head, channel) ----
constexpr int MEAN_ROWS = 256;     // rows per partial sum

struct MeanArgs {
    const void* x;
    int64_t sb, sh, sn;
    int n, d, nchunk;
    float* partial;            // [B,H,nchunk,D]
    void* mean;                // [B,H,D] of x's dtype
    float inv_n;
};

// One workgroup sums MEAN_ROWS rows of one head: a thread owns 8 channels of every (256*8/D)-th row; the row
// groups are then added in a fixed order through LDS, so the result does not depend on timing.
template <int XDT>
__global__ __launch_bounds__(256) void seq_mean_kernel(MeanArgs a) {
    __shared__ float part[256][9];
    const int cpr = a.d >> 3;                    // 8-channel groups per row (8 or 16)
    const int rthreads = 256 / cpr;
    const int cg = threadIdx.x % cpr, rt = threadIdx.x / cpr;
    const int chunk = blockIdx.x;
    const int row0 = chunk * MEAN_ROWS;
    const int row1 = min(row0 + MEAN_ROWS, a.n);
    const char* base = static_cast<const char*>(a.x) + 2 * ((int64_t)blockIdx.z * a.sb + (int64_t)blockIdx.y * a.sh + 8 * (int64_t)cg);
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int row = row0 + rt; row < row1; row += rthreads) {
        float x[8];
        load8<XDT>(base + 2 * (int64_t)row * a.sn, x);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] += x[i];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) part[threadIdx.x][i] = acc[i];
    __syncthreads();
    if (threadIdx.x < a.d) {
        const int c = threadIdx.x;               // channel
        float s = 0.0f;
        for (int t = 0; t < rthreads; ++t) s += part[t * cpr + (c >> 3)][c & 7];
        const int64_t head = (int64_t)blockIdx.z * gridDim.y + blockIdx.y;
        a.partial[(head * a.nchunk + chunk) * a.d + c] = s;
    }
}

// adds a head's partial sums in chunk order, multiplies by 1/N (float32) and rounds to the 16-bit dtype
template <int XDT>
__global__ __launch_bounds__(128) void seq_mean_finish_kernel(MeanArgs a) {
    const int c = threadIdx.x;
    if (c >= a.d) return;
    const int64_t head = blockIdx.x;
    float s = 0.0f;
    for (int k = 0; k < a.nchunk; ++k) s += a.partial[(head * a.nchunk + k) * a.d + c];
    const float m = s * a.inv_n;
    if constexpr (XDT == MPSA_BF16) {
        const uint32_t u = mpsa_f2u(m);
        static_cast<uint16_t*>(a.mean)[head * a.d + c] = (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
    } else {
        static_cast<_Float16*>(a.mean)[head * a.d + c] = (_Float16)m;
    }
}

// MPSA_FP8_ENCODE=sw or MPSA_FP4_ENCODE=sw in the environment selects the kernels that encode with explicit
// integer/float arithmetic only (no hardware conversion instructions), for cross-checking
bool use_sw_fp8() {
    static const bool sw = [] {
        const char* v = getenv("MPSA_FP8_ENCODE");
        const char* w = getenv("MPSA_FP4_ENCODE");
        return (v && v[0] == 's') || (w && w[0] == 's');
    }();
    return sw;
}

template <int XDT, bool DO4, bool DO8>
void launch(const QuantArgs& a, int fmt8, dim3 grid, hipStream_t st) {
    const bool sw = use_sw_fp8();
    if (!DO8 || fmt8 == MPSA_FMT_E4M3) {
        if (sw) hipLaunchKernelGGL((quantize_kernel<XDT, DO4, DO8, MPSA_FMT_E4M3, true>), grid, dim3(256), 0, st, a);
        else    hipLaunchKernelGGL((quantize_kernel<XDT, DO4, DO8, MPSA_FMT_E4M3, false>), grid, dim3(256), 0, st, a);
    } else {
        if (sw) hipLaunchKernelGGL((quantize_kernel<XDT, DO4, DO8, MPSA_FMT_E5M2, true>), grid, dim3(256), 0, st, a);
        else    hipLaunchKernelGGL((quantize_kernel<XDT, DO4, DO8, MPSA_FMT_E5M2, false>), grid, dim3(256), 0, st, a);
    }
}

int quantize_common(const void* x, int x_dtype, int64_t B, int64_t H, int64_t N, int64_t D, const int64_t* xs,
                    const void* sub, float pre, bool do4, int emax4, bool do8, int fmt8, int emax8,
                    uint8_t* c4, uint8_t* s4, uint8_t* c8, uint8_t* s8, int64_t out_rows, hipStream_t st) {
    if (!x || !xs) return mpsa_fail(MPSA_EINVAL, "quantize: null input");
    if ((do4 && (!c4 || !s4)) || (do8 && (!c8 || !s8))) return mpsa_fail(MPSA_EINVAL, "quantize: null output");
    if (x_dtype != MPSA_BF16 && x_dtype != MPSA_F16) return mpsa_fail(MPSA_EINVAL, "quantize: x_dtype must be bf16 or f16");
    if (do8 && fmt8 != MPSA_FMT_E4M3 && fmt8 != MPSA_FMT_E5M2) return mpsa_fail(MPSA_EINVAL, "quantize: 8-bit format must be E4M3 or E5M2");
    if (B < 0 || H < 0 || N < 0 || D <= 0 || out_rows < N) return mpsa_fail(MPSA_EINVAL, "quantize: bad shape");
    if (D % 32) return mpsa_fail(MPSA_EINVAL, "quantize: D=%lld is not a multiple of 32", (long long)D);
    if (xs[3] != 1) return mpsa_fail(MPSA_EINVAL, "quantize: last dim of x must be contiguous");
    if (!mpsa_aligned16(x) || (xs[0] % 8) || (xs[1] % 8) || (xs[2] % 8)) return mpsa_fail(MPSA_EALIGN, "quantize: x rows must be 16-byte aligned");
    if ((do4 && !mpsa_aligned16(c4)) || (do8 && !mpsa_aligned16(c8))) return mpsa_fail(MPSA_EALIGN, "quantize: outputs must be 16-byte aligned");
    if (sub && !mpsa_aligned16(sub)) return mpsa_fail(MPSA_EALIGN, "quantize: sub must be 16-byte aligned");
    if (B == 0 || H == 0 || out_rows == 0) return MPSA_OK;
    const int64_t chunks = out_rows * (D / 8);
    if (chunks >= (int64_t(1) << 31) || H > 65535 || B > 65535) return mpsa_fail(MPSA_EUNSUPPORTED, "quantize: a head has too many elements, or too many heads");
    QuantArgs a;
    a.x = x; a.sub = sub; a.sb = xs[0]; a.sh = xs[1]; a.sn = xs[2];
    a.n = (int)N; a.d = (int)D; a.out_rows = (int)out_rows; a.pre = pre;
    {
        uint32_t pb;
        memcpy(&pb, &pre, 4);
        a.exact16 = ((pb & 0x007FFFFFu) == 0u && (pb & 0x7F800000u) != 0u && (pb & 0x7F800000u) != 0x7F800000u) ? 1 : 0;
    }
    a.emax4 = emax4; a.emax8 = emax8;
    a.codes4 = c4; a.scales4 = s4; a.codes8 = c8; a.scales8 = s8;
    dim3 grid((unsigned)((chunks + 255) / 256), (unsigned)H, (unsigned)B);
    if (x_dtype == MPSA_BF16) {
        if (do4 && do8) launch<MPSA_BF16, true, true>(a, fmt8, grid, st);
        else if (do4)   launch<MPSA_BF16, true, false>(a, fmt8, grid, st);
        else            launch<MPSA_BF16, false, true>(a, fmt8, grid, st);
    } else {
        if (do4 && do8) launch<MPSA_F16, true, true>(a, fmt8, grid, st);
        else if (do4)   launch<MPSA_F16, true, false>(a, fmt8, grid, st);
        else            launch<MPSA_F16, false, true>(a, fmt8, grid, st);
    }
    MPSA_CHECK_LAUNCH("quantize");
    return MPSA_OK;
}

}  // namespace

extern "C" int mpsa_quantize_mx(const void* x, int x_dtype, int64_t B, int64_t H, int64_t N, int64_t D,
                                const int64_t x_strides[4], const void* sub, float pre_scale, int fmt, int emax_elem,
                                uint8_t* codes, uint8_t* scales, int64_t out_rows, mpsa_stream_t stream) {
    if (fmt == MPSA_FMT_E2M1)
        return quantize_common(x, x_dtype, B, H, N, D, x_strides, sub, pre_scale, true, emax_elem, false, 0, 0,
                               codes, scales, nullptr, nullptr, out_rows, (hipStream_t)stream);
    if (fmt == MPSA_FMT_E4M3 || fmt == MPSA_FMT_E5M2)
        return quantize_common(x, x_dtype, B, H, N, D, x_strides, sub, pre_scale, false, 0, true, fmt, emax_elem,
                               nullptr, nullptr, codes, scales, out_rows, (hipStream_t)stream);
    return mpsa_fail(MPSA_EINVAL, "quantize: unknown format %d", fmt);
}

extern "C" int mpsa_quantize_mx_dual(const void* x, int x_dtype, int64_t B, int64_t H, int64_t N, int64_t D,
                                     const int64_t x_strides[4], const void* sub, float pre_scale, int emax4, int fmt8, int emax8,
                                     uint8_t* codes4, uint8_t* scales4, uint8_t* codes8, uint8_t* scales8,
                                     int64_t out_rows, mpsa_stream_t stream) {
    return quantize_common(x, x_dtype, B, H, N, D, x_strides, sub, pre_scale, true, emax4, true, fmt8, emax8,
                           codes4, scales4, codes8, scales8, out_rows, (hipStream_t)stream);
}

extern "C" int64_t mpsa_seq_mean_workspace(int64_t B, int64_t H, int64_t N, int64_t D) {
    if (B < 0 || H < 0 || N < 0 || D < 0) return 0;
    return B * H * ((N + MEAN_ROWS - 1) / MEAN_ROWS) * D * (int64_t)sizeof(float);
}

extern "C" int mpsa_seq_mean(const void* x, int x_dtype, int64_t B, int64_t H, int64_t N, int64_t D,
                             const int64_t x_strides[4], float* workspace, void* mean, mpsa_stream_t stream) {
    if (!x || !x_strides || !workspace || !mean) return mpsa_fail(MPSA_EINVAL, "seq_mean: null pointer");
    if (x_dtype != MPSA_BF16 && x_dtype != MPSA_F16) return mpsa_fail(MPSA_EINVAL, "seq_mean: x_dtype must be bf16 or f16");
    if (B <= 0 || H <= 0 || N <= 0) return mpsa_fail(MPSA_EINVAL, "seq_mean: bad shape");
    if (D != 64 && D != 128) return mpsa_fail(MPSA_EUNSUPPORTED, "seq_mean: D must be 64 or 128 (got %lld)", (long long)D);
    if (x_strides[3] != 1) return mpsa_fail(MPSA_EINVAL, "seq_mean: last dim of x must be contiguous");
    if (!mpsa_aligned16(x) || (x_strides[0] % 8) || (x_strides[1] % 8) || (x_strides[2] % 8)) return mpsa_fail(MPSA_EALIGN, "seq_mean: x rows must be 16-byte aligned");
    if (H > 65535 || B > 65535 || N >= (int64_t(1) << 31)) return mpsa_fail(MPSA_EUNSUPPORTED, "seq_mean: shape too large");
    MeanArgs a;
    a.x = x; a.sb = x_strides[0]; a.sh = x_strides[1]; a.sn = x_strides[2];
    a.n = (int)N; a.d = (int)D; a.nchunk = (int)((N + MEAN_ROWS - 1) / MEAN_ROWS);
    a.partial = workspace; a.mean = mean; a.inv_n = 1.0f / (float)N;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid((unsigned)a.nchunk, (unsigned)H, (unsigned)B);
    if (x_dtype == MPSA_BF16) {
        hipLaunchKernelGGL(seq_mean_kernel<MPSA_BF16>, grid, dim3(256), 0, st, a);
        hipLaunchKernelGGL(seq_mean_finish_kernel<MPSA_BF16>, dim3((unsigned)(B * H)), dim3(128), 0, st, a);
    } else {
        hipLaunchKernelGGL(seq_mean_kernel<MPSA_F16>, grid, dim3(256), 0, st, a);
        hipLaunchKernelGGL(seq_mean_finish_kernel<MPSA_F16>, dim3((unsigned)(B * H)), dim3(128), 0, st, a);
    }
    MPSA_CHECK_LAUNCH("seq_mean");
    return MPSA_OK;
}
