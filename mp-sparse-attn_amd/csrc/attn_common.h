// Pieces shared by the attention kernels (device helpers, argument block).
#pragma once
#include "mpsa_common.h"
#include <type_traits>

struct AttnArgs {
    const uint8_t *q4, *qs4, *q8, *qs8, *k4, *ks4, *k8, *ks8;
    const void* v;
    void* o;
    int64_t o_sb, o_sh, o_sn;
    int B, Hq, Hkv, n, n_pad, nt;        // n, n_pad, nt: keys/values
    int nq, nq_pad, ntq;                 // queries (equal to the above for self-attention)
    int causal, mode, fmt8, o_dtype;
    int d, tile;
    float skip_thresh;         // tile-skipping variants only
    int32_t* skipped;          // optional [B,Hq,nt] count of skipped key tiles per query tile
    const int32_t* order;      // routed runs only: [B,Hq,ntq,nt] visiting lists and [B,Hq,ntq,4] run lengths
    const int32_t* counts;
    // paired-tile kernel with the Q quantizer fused in: unquantized Q (16-bit, element strides, last dim contiguous)
    // and the factor folded in before quantizing; q4 / qs4 / q8 / qs8 are unused then
    const void* q_raw;
    int64_t q_sb, q_sh, q_sn;
    float q_pre;
};

template <int PVT> struct PV;
template <> struct PV<MPSA_BF16> {
    typedef v8bf vec;
    typedef __bf16 v2 __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ v16f mfma(vec a, vec b, v16f c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
    static __device__ __forceinline__ v2 pack(float x, float y) { return (v2){(__bf16)x, (__bf16)y}; }
    // c + p.x + p.y with the 16-bit values the P.V product will see
    static __device__ __forceinline__ float add2(v2 p, float c) { return __builtin_amdgcn_fdot2_f32_bf16(p, (v2){(__bf16)1.0f, (__bf16)1.0f}, c, false); }
    // P = exp2(S - m_run) may grow to 2^REBASE before the running maximum is moved: bf16 has float32's range
    static constexpr float REBASE = 60.0f;
    // a lane's row sum of one tile at which a kernel that takes the exponentials first and looks afterwards does
    // the tile again with the maximum pass (2^REBASE)
    static constexpr float OPTIMISTIC_LIMIT = 1152921504606846976.0f;
};
template <> struct PV<MPSA_F16> {
    typedef v8h vec;
    typedef _Float16 v2 __attribute__((ext_vector_type(2)));
    static __device__ __forceinline__ v16f mfma(vec a, vec b, v16f c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
    static __device__ __forceinline__ v2 pack(float x, float y) { return (v2){(_Float16)x, (_Float16)y}; }
    static __device__ __forceinline__ float add2(v2 p, float c) { return __builtin_amdgcn_fdot2(p, (v2){(_Float16)1.0f, (_Float16)1.0f}, c, false); }
    static constexpr float REBASE = 12.0f;      // fp16 P must stay below 65504
    static constexpr float OPTIMISTIC_LIMIT = 4096.0f;
};

// Exchange between the two lanes (l, l^32) that share one query.  v_permlane32_swap swaps lanes 32-63 of its first
// register with lanes 0-31 of its second; fed two copies of x, every lane ends up holding both halves' values.
// Written as inline assembly because both registers are outputs (the compiler builtin of this toolchain returns
// the first register for both results); the s_nop's cover the instruction's read/write wait states.
__device__ __forceinline__ void lane_pair(float x, float& a, float& b) {
    a = x;
    b = x;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ float max_lane_pair(float x) {
    float a, b;
    lane_pair(x, a, b);
    return __builtin_fmaxf(a, b);
}
__device__ __forceinline__ float sum_lane_pair(float x) {
    float a, b;
    lane_pair(x, a, b);
    return a + b;
}

template <int FMT8>
__device__ __forceinline__ v16f score_mfma8(v8i k, v8i q, v16f c, int sel, int ks, int qs) {
    if (sel == 0) return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(k, q, c, FMT8, FMT8, 0, ks, 0, qs);
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(k, q, c, FMT8, FMT8, 2, ks, 2, qs);
}
// 4-bit K operand x 8-bit Q operand ("mixed"): each operand's registers follow its own format's layout
template <int FMT8>
__device__ __forceinline__ v16f score_mfma48(v8i k, v8i q, v16f c, int sel, int ks, int qs) {
    if (sel == 0) return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(k, q, c, 4, FMT8, 0, ks, 0, qs);
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(k, q, c, 4, FMT8, 2, ks, 2, qs);
}
__device__ __forceinline__ v16f score_mfma4(v8i k, v8i q, v16f c, int sel, int ks, int qs) {
    if (sel == 0) return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(k, q, c, 4, 4, 0, ks, 0, qs);
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(k, q, c, 4, 4, 2, ks, 2, qs);
}

// One wave-wide direct-to-LDS load: lane l copies 16 bytes from its own global address to lds_wave_base + 16*l.
__device__ __forceinline__ void load16_to_lds(const uint8_t* gsrc, uint8_t* lds_wave_base) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)gsrc,
                                     (__attribute__((address_space(3))) void*)lds_wave_base, 16, 0, 0);
}

// The same load with the address split into a wave-uniform 64-bit base (scalar registers) and the lane's unsigned
// 32-bit byte offset: no per-lane 64-bit pointers to keep or to compute.  Written as assembly (the builtin only
// takes a full per-lane pointer); the compiler does not count these loads, so the kernel waits for them itself
// (s_waitcnt vmcnt(0) before the barrier that publishes the data).
__device__ __forceinline__ void load16_to_lds_sv(uint32_t lane_off, const uint8_t* wave_base, uint8_t* lds_wave_base) {
    // the low 32 bits of a generic pointer into LDS are the LDS byte address (the aperture base has none set)
    const uint32_t base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds_wave_base);
    const uint64_t gb = uniform_bits(wave_base);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(base), "v"(lane_off), "s"(gb) : "memory", "m0");
}

// A scalar load of one list entry.  The compiler turns a plain load that follows a workgroup barrier into a vector
// load plus a broadcast; as assembly it stays a scalar load.  The wait is part of the same statement (a register
// that is still being loaded must not be visible to the compiler as holding a value), so callers place it where
// a short stall costs nothing.
__device__ __forceinline__ int scalar_load(const int32_t* uniform_ptr) {
    int x;
    asm volatile("s_load_dword %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(x) : "s"(uniform_bits(uniform_ptr)) : "memory");
    return x;
}

// Tile-skipping variants of the general kernel (modes mxfp4 / mxfp8): attn_fwd_skip.hip
int attn_skip_launch(const AttnArgs& a, int pv_dtype, hipStream_t st);

// Routed variants of the general kernel (per-tile precision from a visiting list): attn_fwd_routed.hip
int attn_routed_launch(const AttnArgs& a, int pv_dtype, hipStream_t st);

// Paired-tile ("ping-pong") kernel for self-attention with D = 128, tile = 128 in the diag / mxfp4 / mixed / mxfp8 modes: attn_fwd_pp.hip
bool attn_pp_supported(const AttnArgs& a, int pv_dtype);
int attn_pp_launch(const AttnArgs& a, int pv_dtype, hipStream_t st);       // a.q_raw != nullptr: the fused-quantizer variants
