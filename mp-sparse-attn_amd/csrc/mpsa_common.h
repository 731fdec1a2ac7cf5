// Shared host/device helpers of libmpsa (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include "../../include/mpsa.h"

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef unsigned short v8us __attribute__((ext_vector_type(8)));

// thread-local error text, filled by mpsa_fail()
int mpsa_fail(int code, const char* fmt, ...);

static inline bool mpsa_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Kernels that need more dynamic LDS than the default limit carry a function attribute, which is per device and
// cannot be set while a stream is being captured.  Every such kernel instantiation registers itself at library load
// (LdsKernel<...>::registered, a static initialiser); mpsa_init() sets the attribute of all of them on the current
// device, and the launchers call mpsa_ensure_init(), which does that on a device's first use if the caller has not.
#define MPSA_MAX_DEVICES 64
bool mpsa_register_lds_kernel(const void* kern, int bytes);      // api.hip; always returns true
int mpsa_ensure_init();                                          // api.hip; MPSA_OK or the failure of mpsa_init()
int mpsa_seq_mean_static_resolve();                              // quantize.hip; address of the built-in partial-sum array

#define MPSA_CHECK_LAUNCH(what)                                                        \
    do {                                                                               \
        hipError_t e__ = hipGetLastError();                                            \
        if (e__ != hipSuccess) return mpsa_fail(MPSA_ELAUNCH, "%s: %s", what, hipGetErrorString(e__)); \
    } while (0)

__device__ __forceinline__ float mpsa_u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t mpsa_f2u(float f) { return __builtin_bit_cast(uint32_t, f); }

// A wave-uniform pointer as a 64-bit value the compiler knows to be uniform (scalar registers).
__device__ __forceinline__ uint64_t uniform_bits(const void* p) {
    // the broadcast builtin returns a signed int: widen through uint32_t, or the low half sign-extends
    const uint64_t v = (uint64_t)(uintptr_t)p;
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(v >> 32));
    return (uint64_t)lo | ((uint64_t)hi << 32);
}
