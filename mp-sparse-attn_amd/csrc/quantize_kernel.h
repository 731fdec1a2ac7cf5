// The MX quantizer's per-workgroup body and its argument block, shared by quantize.hip (the stand-alone entry
// points) and prepare.hip (the one-launch operand preparation of the attention path).  The scheme is described at
// the top of quantize.hip.
#pragma once
#include "mpsa_common.h"
#include "mx_codec.h"


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

// host side, defined in quantize.hip
int mpsa_quantize_setup(const void* x, int x_dtype, int64_t B, int64_t H, int64_t N, int64_t D, const int64_t* xs,
                        const void* sub, float pre, bool do4, int emax4, bool do8, int fmt8, int emax8,
                        uint8_t* c4, uint8_t* s4, uint8_t* c8, uint8_t* s8, int64_t out_rows, QuantArgs* out, unsigned* blocks);
bool mpsa_quantize_sw_encoders();

namespace {


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
// agree, no rounding boundary lies between them and that word is the result; if they differ anywhere in the word,
// the lane falls back to the explicit rule.  (2^-17 of a value near a midpoint - the
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
            if (exact16) {
                uint32_t w = 0;
                w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, x[0], x[1], sc, 0);
                w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, x[2], x[3], sc, 1);
                w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, x[4], x[5], sc, 2);
                w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, x[6], x[7], sc, 3);
                return w;
            }
            // no boundary between the two nudged values: the value itself converts to the same codes
            uint32_t wd = 0, wu = 0;
            wd = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(wd, x[0] * dn, x[1] * dn, sc, 0);
            wd = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(wd, x[2] * dn, x[3] * dn, sc, 1);
            wd = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(wd, x[4] * dn, x[5] * dn, sc, 2);
            wd = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(wd, x[6] * dn, x[7] * dn, sc, 3);
            wu = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(wu, x[0] * up, x[1] * up, sc, 0);
            wu = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(wu, x[2] * up, x[3] * up, sc, 1);
            wu = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(wu, x[4] * up, x[5] * up, sc, 2);
            wu = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(wu, x[6] * up, x[7] * up, sc, 3);
            if (wd == wu) return wd;
        }
    }
    uint32_t word = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) word |= e2m1_encode(ldexpf(x[i], -se)) << (4 * i);
    return word;
}

// One workgroup's share: 256 consecutive 16-byte chunks, starting at chunk 256*bx, of head hh of batch bb (nh heads).
template <int XDT, bool DO4, bool DO8, int FMT8, bool SW8>
__device__ __forceinline__ void quantize_block(const QuantArgs& a, uint32_t bx, uint32_t hh, uint32_t bb, uint32_t nh) {
    const uint32_t cpr = (uint32_t)a.d >> 3;                              // 16-byte chunks per row
    const uint32_t chunks = (uint32_t)a.out_rows * cpr;                   // per (b,h)
    const uint32_t c = bx * 256u + threadIdx.x;
    if (c >= chunks) return;                                              // whole quads leave together (cpr % 4 == 0)
    const uint32_t row = c / cpr;
    const uint32_t col8 = c - row * cpr;
    const int64_t head = (int64_t)bb * nh + hh;                           // flat (b,h)

    float x[8];
    if (row < (uint32_t)a.n) {
        const char* base = static_cast<const char*>(a.x) +
                           2 * ((int64_t)bb * a.sb + (int64_t)hh * a.sh + (int64_t)row * a.sn + 8 * (int64_t)col8);
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

template <int XDT, bool DO4, bool DO8, int FMT8, bool SW8>
__global__ __launch_bounds__(256) void quantize_kernel(QuantArgs a) {
    // two 256-chunk blocks per workgroup: both loads are in flight before either block is converted
    quantize_block<XDT, DO4, DO8, FMT8, SW8>(a, 2 * blockIdx.x, blockIdx.y, blockIdx.z, gridDim.y);
    quantize_block<XDT, DO4, DO8, FMT8, SW8>(a, 2 * blockIdx.x + 1, blockIdx.y, blockIdx.z, gridDim.y);
}

}  // namespace
