// Block-scaled NT matmul on the CDNA4 scaled matrix cores (gfx950).
//
//   C[m][n] = sum over 32-wide K blocks kb of  2^(sa[m][kb]-127) * 2^(sb[n][kb]-127) * sum_{k in kb} a[m][k] * b[n][k]
//
// the computation of the reference's block_scaled_matmul_kernel (ours/block_scaled_matmul.py:154-267)
// whose torch statement is ours/block_scaled_matmul.py:382-392.  Operands arrive as the quantizer
// leaves them: row-major packed codes and row-major E8M0 bytes (one per 32 elements of K).
//
// Mapping.  A workgroup of four waves owns a 256x256 tile of C; each wave owns 128x128 as a 4x4 grid of
// v_mfma_scale_f32_32x32x64_f8f6f4 accumulators (256 accumulator registers).  For that instruction
// lane (h = lane/32, r = lane%32) supplies 32 K elements of row r of its operand and the E8M0 byte of MX
// block h of the 64-element step.  With 4-bit elements the lane's four registers are exactly block h;
// with 8-bit elements registers 0-3 of the two lane halves together are block 0 and registers 4-7 block 1
// (each half holds 16 bytes of either block).  Either way fragments are plain 16-byte pieces of the
// row-major HBM layout.  K advances 64 bytes of codes per row per stage (128 E2M1 or 64 8-bit elements).
// Stages are double-buffered in LDS with rows padded from 64 to 80 bytes: the 16 lanes of a 128-bit
// LDS access phase then fall into 16 distinct 4-bank groups.  Wave tiles of 128x128 keep LDS reads at
// 8 operand fragments per 16 matrix instructions.
#include "mpsa_common.h"

namespace {

constexpr int BM = 256, BN = 256;       // workgroup tile
constexpr int ROWB = 64;                // code bytes per row per stage
constexpr int PITCH = 80;               // LDS row pitch

struct GemmArgs {
    const uint8_t *a, *sa, *b, *sb;
    void* c;
    int64_t ldc;
    int M, N, K;
};

template <typename T> __device__ __forceinline__ T cvt_out(float v);
template <> __device__ __forceinline__ float cvt_out<float>(float v) { return v; }
template <> __device__ __forceinline__ __bf16 cvt_out<__bf16>(float v) { return (__bf16)v; }
template <> __device__ __forceinline__ _Float16 cvt_out<_Float16>(float v) { return (_Float16)v; }

template <int FMT, typename OutT>
__global__ __launch_bounds__(256, 1) void gemm_mx_kernel(GemmArgs g) {
    constexpr bool FP4 = (FMT == MPSA_FMT_E2M1);
    constexpr int STEPS = FP4 ? 2 : 1;                 // matrix instructions along K per stage
    constexpr int SCB = FP4 ? 4 : 2;                   // scale bytes per row per stage
    const int row_bytes = FP4 ? g.K / 2 : g.K;         // code bytes per matrix row
    const int srow_bytes = g.K / 32;
    const int KT = row_bytes / ROWB;

    __shared__ __attribute__((aligned(16))) uint8_t lds_a[2][BM * PITCH];
    __shared__ __attribute__((aligned(16))) uint8_t lds_b[2][BN * PITCH];
    __shared__ uint32_t lds_sa[2][BM];
    __shared__ uint32_t lds_sb[2][BN];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int h = lane >> 5, r = lane & 31;

    // XCD-aware tile order: consecutive workgroup ids go to different XCDs (8 of them), so give each
    // XCD a contiguous band of tile rows; tiles of one band share their A rows in that XCD's L2.
    const int tiles_n = g.N / BN;
    const int ntiles = (g.M / BM) * tiles_n;
    int wg = blockIdx.x;
    if (ntiles % 8 == 0) wg = (wg & 7) * (ntiles >> 3) + (wg >> 3);
    const int m0 = (wg / tiles_n) * BM;
    const int n0 = (wg % tiles_n) * BN;

    // global -> register staging: thread t moves 16-byte chunk (row t/4 + 64 i, column chunk t%4)
    const int crow = tid >> 2, ccol = tid & 3;
    const uint8_t* ga = g.a + (int64_t)(m0 + crow) * row_bytes + ccol * 16;
    const uint8_t* gb = g.b + (int64_t)(n0 + crow) * row_bytes + ccol * 16;
    const uint8_t* gsa = g.sa + (int64_t)(m0 + tid) * srow_bytes;
    const uint8_t* gsb = g.sb + (int64_t)(n0 + tid) * srow_bytes;
    const int64_t rstep = (int64_t)64 * row_bytes;

    uint4 ra[4], rb[4];
    uint32_t rsa, rsb;
    auto load_stage = [&](int kt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            ra[i] = *reinterpret_cast<const uint4*>(ga + i * rstep + (int64_t)kt * ROWB);
            rb[i] = *reinterpret_cast<const uint4*>(gb + i * rstep + (int64_t)kt * ROWB);
        }
        if constexpr (FP4) {
            rsa = *reinterpret_cast<const uint32_t*>(gsa + kt * SCB);
            rsb = *reinterpret_cast<const uint32_t*>(gsb + kt * SCB);
        } else {
            rsa = *reinterpret_cast<const uint16_t*>(gsa + kt * SCB);
            rsb = *reinterpret_cast<const uint16_t*>(gsb + kt * SCB);
        }
    };
    auto store_stage = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            *reinterpret_cast<uint4*>(&lds_a[buf][(crow + 64 * i) * PITCH + ccol * 16]) = ra[i];
            *reinterpret_cast<uint4*>(&lds_b[buf][(crow + 64 * i) * PITCH + ccol * 16]) = rb[i];
        }
        lds_sa[buf][tid] = rsa;
        lds_sb[buf][tid] = rsb;
    };

    v16f acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    load_stage(0);
    store_stage(0);
    __syncthreads();

    for (int kt = 0; kt < KT; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < KT) load_stage(kt + 1);

        int sca[4], scb[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            sca[i] = (int)(lds_sa[buf][wm * 128 + i * 32 + r] >> (8 * h));
            scb[i] = (int)(lds_sb[buf][wn * 128 + i * 32 + r] >> (8 * h));
        }
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            v8i fa[4], fb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint8_t* pa = &lds_a[buf][(wm * 128 + i * 32 + r) * PITCH];
                const uint8_t* pb = &lds_b[buf][(wn * 128 + i * 32 + r) * PITCH];
                if constexpr (FP4) {
                    const v4i xa = *reinterpret_cast<const v4i*>(pa + (2 * s + h) * 16);
                    const v4i xb = *reinterpret_cast<const v4i*>(pb + (2 * s + h) * 16);
                    fa[i] = (v8i){xa[0], xa[1], xa[2], xa[3], 0, 0, 0, 0};
                    fb[i] = (v8i){xb[0], xb[1], xb[2], xb[3], 0, 0, 0, 0};
                } else {
                    // 8-bit operands: registers 0-3 of both lane halves form MX block 0 (scaled by the byte
                    // lane half 0 supplies), registers 4-7 form block 1 (scaled by lane half 1's byte)
                    const v4i xa0 = *reinterpret_cast<const v4i*>(pa + h * 16);
                    const v4i xa1 = *reinterpret_cast<const v4i*>(pa + h * 16 + 32);
                    const v4i xb0 = *reinterpret_cast<const v4i*>(pb + h * 16);
                    const v4i xb1 = *reinterpret_cast<const v4i*>(pb + h * 16 + 32);
                    fa[i] = (v8i){xa0[0], xa0[1], xa0[2], xa0[3], xa1[0], xa1[1], xa1[2], xa1[3]};
                    fb[i] = (v8i){xb0[0], xb0[1], xb0[2], xb0[3], xb1[0], xb1[1], xb1[2], xb1[3]};
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (s == 0)
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[j], acc[i][j], FMT, FMT, 0, sca[i], 0, scb[j]);
                    else
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[j], acc[i][j], FMT, FMT, 2, sca[i], 2, scb[j]);
                }
        }
        if (kt + 1 < KT) store_stage(buf ^ 1);
        __syncthreads();
    }

    // epilogue: accumulator register e of lane (h, r) is C[8*(e/4) + 4*h + e%4][r] of its 32x32 block
    OutT* c = static_cast<OutT*>(g.c);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = n0 + wn * 128 + j * 32 + r;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int row = m0 + wm * 128 + i * 32 + 8 * (e >> 2) + 4 * h + (e & 3);
                c[(int64_t)row * g.ldc + col] = cvt_out<OutT>(acc[i][j][e]);
            }
        }
}

template <int FMT>
void launch_fmt(const GemmArgs& g, int c_dtype, dim3 grid, hipStream_t st) {
    if (c_dtype == MPSA_BF16)      hipLaunchKernelGGL((gemm_mx_kernel<FMT, __bf16>), grid, dim3(256), 0, st, g);
    else if (c_dtype == MPSA_F16)  hipLaunchKernelGGL((gemm_mx_kernel<FMT, _Float16>), grid, dim3(256), 0, st, g);
    else                           hipLaunchKernelGGL((gemm_mx_kernel<FMT, float>), grid, dim3(256), 0, st, g);
}

}  // namespace

extern "C" int mpsa_gemm_mx(const uint8_t* a, const uint8_t* sa, const uint8_t* b, const uint8_t* sb, int fmt,
                            int64_t M, int64_t N, int64_t K, void* c, int c_dtype, int64_t ldc, mpsa_stream_t stream) {
    if (!a || !sa || !b || !sb || !c) return mpsa_fail(MPSA_EINVAL, "gemm: null pointer");
    if (fmt != MPSA_FMT_E2M1 && fmt != MPSA_FMT_E4M3 && fmt != MPSA_FMT_E5M2) return mpsa_fail(MPSA_EINVAL, "gemm: unknown format %d", fmt);
    if (c_dtype != MPSA_BF16 && c_dtype != MPSA_F16 && c_dtype != MPSA_F32) return mpsa_fail(MPSA_EINVAL, "gemm: unsupported output dtype %d", c_dtype);
    if (M <= 0 || N <= 0 || K <= 0 || ldc < N) return mpsa_fail(MPSA_EINVAL, "gemm: bad shape");
    if (M % BM || N % BN || K % 128) return mpsa_fail(MPSA_EUNSUPPORTED, "gemm: M,N must be multiples of 256 and K of 128 (got %lld,%lld,%lld)", (long long)M, (long long)N, (long long)K);
    if (M > (1 << 30) || N > (1 << 30) || K > (1 << 30) || (M / BM) * (N / BN) > (int64_t(1) << 30)) return mpsa_fail(MPSA_EUNSUPPORTED, "gemm: shape too large");
    if (!mpsa_aligned16(a) || !mpsa_aligned16(b) || (reinterpret_cast<uintptr_t>(sa) & 3) || (reinterpret_cast<uintptr_t>(sb) & 3))
        return mpsa_fail(MPSA_EALIGN, "gemm: codes must be 16-byte and scales 4-byte aligned");
    GemmArgs g;
    g.a = a; g.sa = sa; g.b = b; g.sb = sb; g.c = c; g.ldc = ldc;
    g.M = (int)M; g.N = (int)N; g.K = (int)K;
    dim3 grid((unsigned)((M / BM) * (N / BN)));
    hipStream_t st = (hipStream_t)stream;
    if (fmt == MPSA_FMT_E2M1)      launch_fmt<MPSA_FMT_E2M1>(g, c_dtype, grid, st);
    else if (fmt == MPSA_FMT_E4M3) launch_fmt<MPSA_FMT_E4M3>(g, c_dtype, grid, st);
    else                           launch_fmt<MPSA_FMT_E5M2>(g, c_dtype, grid, st);
    MPSA_CHECK_LAUNCH("gemm");
    return MPSA_OK;
}
