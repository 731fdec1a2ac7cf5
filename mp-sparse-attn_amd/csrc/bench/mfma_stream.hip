// Measurement aid: a register-resident stream of matrix instructions, to read the rate the matrix cores SUSTAIN on this
// chip -- the practical ceiling next to the datasheet peaks that the rooflines are quoted against.  MI355X manages its
// clock by power: the same instruction stream runs near 2.4 GHz on constant operands and several hundred MHz lower on
// operands with random bits, so a kernel's distance from the datasheet peak is partly not the kernel's.  No counterpart in
// the reference.  Built into its own shared object (lib/libmpsa_bench.so), which only bench.py loads: it is a
// measurement, not part of the library's interface.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

namespace {

// kind: 0 = v_mfma_f32_32x32x16_bf16, 1 = v_mfma_scale_f32_32x32x64_f8f6f4 with E2M1 operands, 2 = the same with E4M3
template <int KIND>
__global__ __launch_bounds__(512, 1) void mfma_stream_kernel(float* sink, int iters, int random_bits) {
    const uint32_t lane = threadIdx.x;
    // operand registers: a hash of (lane, register) or one constant; exponent bits kept away from Inf/NaN patterns
    uint32_t seed = random_bits ? lane * 2654435761u + blockIdx.x * 40503u + 12345u : 0u;
    auto next = [&]() {
        seed = seed * 1664525u + 1013904223u;
        return random_bits ? (int)(seed & 0xbf7fbf7fu) : 0x3c003c00;
    };
    v8i a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) { a[i] = next(); b[i] = next(); }
    v16f acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[j][e] = 0.0f;
    const int sa = 0x7f7f7f7f, sb = 0x7f7f7f7f;           // E8M0 scale 2^0
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if constexpr (KIND == 0) {
                    const v4i a4 = {a[0], a[1], a[2], a[3]}, b4 = {b[0], b[1], b[2], b[3]};
                    acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a4), __builtin_bit_cast(v8bf, b4), acc[j], 0, 0, 0);
                } else if constexpr (KIND == 1) {
                    acc[j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[j], 4, 4, 0, sa, 0, sb);
                } else {
                    acc[j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[j], 0, 0, 0, sa, 0, sb);
                }
            }
    }
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) s += acc[j][e];
    if (s == 123.456f) sink[0] = s;                        // keeps the accumulators alive; never true in practice
}

}  // namespace

// Launches `blocks` workgroups of 8 waves (two per SIMD); every wave issues iters x 16 matrix instructions.
// Returns 0, -1 for a bad argument or -4 for a failed launch, and the FLOP of the launch through *flop
// (2 x 32 x 32 x K per instruction).
extern "C" int bench_mfma_stream(int kind, int random_bits, int iters, int blocks, float* sink, double* flop, void* stream) {
    if (kind < 0 || kind > 2 || iters <= 0 || blocks <= 0 || !sink) return -1;
    hipStream_t st = (hipStream_t)stream;
    if (kind == 0)      hipLaunchKernelGGL(mfma_stream_kernel<0>, dim3(blocks), dim3(512), 0, st, sink, iters, random_bits);
    else if (kind == 1) hipLaunchKernelGGL(mfma_stream_kernel<1>, dim3(blocks), dim3(512), 0, st, sink, iters, random_bits);
    else                hipLaunchKernelGGL(mfma_stream_kernel<2>, dim3(blocks), dim3(512), 0, st, sink, iters, random_bits);
    if (hipGetLastError() != hipSuccess) return -4;
    if (flop) *flop = (double)blocks * 8.0 * iters * 16.0 * 2.0 * 32 * 32 * (kind == 0 ? 16 : 64);
    return 0;
}
