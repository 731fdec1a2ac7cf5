// Element encoders / decoders shared by the quantizer and the elementwise format kernels (device only).
#pragma once
#include "mpsa_common.h"

// E2M1 magnitude index of a in [0, 6]: nearest of {0,.5,1,1.5,2,3,4,6}; the candidate with the even
// mantissa bit has 1e-6f subtracted from its float32 distance and the lower index wins an exact tie
// of the biased distances -- exactly what an argmin over all eight biased distances returns, since
// every other candidate is at least 0.5 further away.
__device__ __forceinline__ uint32_t e2m1_index(float a) {
    const uint32_t u = mpsa_f2u(a);
    uint32_t lo;
    float clo, chi;
    if (a < 1.0f) {
        const bool half = a >= 0.5f;
        lo = half ? 1u : 0u;
        clo = half ? 0.5f : 0.0f;
        chi = half ? 1.0f : 0.5f;
    } else {
        const uint32_t mbit = (u >> 22) & 1u;
        lo = 2u + 2u * ((u >> 23) - 127u) + mbit;
        clo = mpsa_u2f(u & 0xFFC00000u);
        chi = mbit ? mpsa_u2f((u & 0xFF800000u) + 0x00800000u) : mpsa_u2f((u & 0xFF800000u) | 0x00400000u);
    }
    const bool lo_even = (lo & 1u) == 0u;
    const float elo = __builtin_fabsf(a - clo) - (lo_even ? 1e-6f : 0.0f);
    const float ehi = __builtin_fabsf(a - chi) - (lo_even ? 0.0f : 1e-6f);
    const uint32_t idx = (ehi < elo) ? lo + 1u : lo;
    return lo >= 7u ? 7u : idx;
}

__device__ __forceinline__ uint32_t e2m1_encode(float y) {
    const uint32_t u = mpsa_f2u(y);
    const float a = __builtin_fminf(__builtin_fabsf(y), 6.0f);
    return ((u >> 31) << 3) | e2m1_index(a);
}

// software round-to-nearest-even encoders (|y| already clamped to the format's maximum)
__device__ __forceinline__ uint32_t e4m3_encode_sw(float y) {
    const uint32_t u = mpsa_f2u(y);
    const uint32_t sign = (u >> 24) & 0x80u;
    uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return sign | 0x7Fu;
    uint32_t code;
    if (a >= 0x3C800000u) {                       // |y| >= 2^-6: normal
        a += 0x7FFFFu + ((a >> 20) & 1u);
        code = (a >> 20) - (120u << 3);
        code = code > 0x7Eu ? 0x7Eu : code;
    } else {                                      // subnormal, unit 2^-9
        code = mpsa_f2u(mpsa_u2f(a) + 16384.0f) - 0x46800000u;
    }
    return sign | code;
}

__device__ __forceinline__ uint32_t e5m2_encode_sw(float y) {
    const uint32_t u = mpsa_f2u(y);
    const uint32_t sign = (u >> 24) & 0x80u;
    uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return sign | 0x7Fu;
    uint32_t code;
    if (a >= 0x38800000u) {                       // |y| >= 2^-14: normal
        a += 0xFFFFFu + ((a >> 21) & 1u);
        code = (a >> 21) - (112u << 2);
        code = code > 0x7Bu ? 0x7Bu : code;
    } else {                                      // subnormal, unit 2^-16
        code = mpsa_f2u(mpsa_u2f(a) + 128.0f) - 0x43000000u;
    }
    return sign | code;
}

// E2M1 code (low nibble SEEM) -> float32; 0bS000 is +-0.  ours/mxfp.py:44-77.
__device__ __forceinline__ float e2m1_decode(uint32_t code) {
    const uint32_t idx = code & 7u;
    // magnitudes 0, .5, 1, 1.5, 2, 3, 4, 6: subnormal for idx < 2, else (1 + M/2) * 2^(E-1)
    const float mag = idx < 2u ? 0.5f * (float)idx : mpsa_u2f(((126u + (idx >> 1)) << 23) | ((idx & 1u) << 22));
    return (code & 8u) ? -mag : mag;
}
