// One-launch operand preparation for the fused attention kernel (gfx950): the MX quantization of Q (with
// sm_scale*log2(e) folded in) and of K (optionally minus its sequence mean) and the value-tile repack of V run as
// three groups of workgroups of ONE kernel instead of three launches - at the benchmark shape the three kernels take
// about 45 us together and the gaps between their launches another 20.  The work per workgroup is exactly that of
// quantize_kernel / v_tiles_kernel (quantize_kernel.h, v_tiles_kernel.h); this file only routes workgroup ids.
// Replaces the prologue of the reference's wrapper, ours/mxfp_attn_kernel.py:27-57 (dtype normalisation, quant_mxfp4 /
// quant_mxfp8e5 calls, operand packaging).
#include "quantize_kernel.h"
#include "v_tiles_kernel.h"

namespace {

struct PrepArgs {
    QuantArgs q, k;
    VTArgs v;
    uint32_t bq, bk, bv;          // workgroups per (batch, head) of each job
    uint32_t hq, hkv;
    uint32_t q_total, k_total, v_total;    // blocks of the Q job, of the K job, of the V job
};

template <int XDT, bool DO4, bool DO8, int FMT8, int TILE, int D>
__device__ __forceinline__ void prepare_block(const PrepArgs& p, uint32_t blk) {
    if (blk < p.q_total) {
        const uint32_t head = blk / p.bq;
        quantize_block<XDT, DO4, DO8, FMT8, false>(p.q, blk - head * p.bq, head % p.hq, head / p.hq, p.hq);
        return;
    }
    blk -= p.q_total;
    if (blk < p.k_total) {
        const uint32_t head = blk / p.bk;
        quantize_block<XDT, DO4, DO8, FMT8, false>(p.k, blk - head * p.bk, head % p.hkv, head / p.hkv, p.hkv);
        return;
    }
    blk -= p.k_total;
    if (blk >= p.v_total) return;
    const uint32_t head = blk / p.bv;
    v_tiles_block<TILE, D>(p.v, blk - head * p.bv, head % p.hkv, head / p.hkv, p.hkv);
}

// two blocks of work per workgroup (measured on the stand-alone quantizer: 8-13 % more bandwidth than one)
template <int XDT, bool DO4, bool DO8, int FMT8, int TILE, int D>
__global__ __launch_bounds__(256) void prepare_kernel(PrepArgs p) {
    prepare_block<XDT, DO4, DO8, FMT8, TILE, D>(p, 2 * blockIdx.x);
    prepare_block<XDT, DO4, DO8, FMT8, TILE, D>(p, 2 * blockIdx.x + 1);
}

template <int XDT, bool DO4, bool DO8, int FMT8>
void launch_td(const PrepArgs& p, int tile, int d, unsigned grid, hipStream_t st) {
    if (tile == 128 && d == 128)      hipLaunchKernelGGL((prepare_kernel<XDT, DO4, DO8, FMT8, 128, 128>), dim3(grid), dim3(256), 0, st, p);
    else if (tile == 128 && d == 64)  hipLaunchKernelGGL((prepare_kernel<XDT, DO4, DO8, FMT8, 128, 64>), dim3(grid), dim3(256), 0, st, p);
    else if (tile == 64 && d == 128)  hipLaunchKernelGGL((prepare_kernel<XDT, DO4, DO8, FMT8, 64, 128>), dim3(grid), dim3(256), 0, st, p);
    else                              hipLaunchKernelGGL((prepare_kernel<XDT, DO4, DO8, FMT8, 64, 64>), dim3(grid), dim3(256), 0, st, p);
}

template <int XDT>
void launch_mode(const PrepArgs& p, int mode, int fmt8, int tile, int d, unsigned grid, hipStream_t st) {
    if (mode == MPSA_MODE_MXFP4) launch_td<XDT, true, false, MPSA_FMT_E4M3>(p, tile, d, grid, st);
    else if (mode == MPSA_MODE_MXFP8) {
        if (fmt8 == MPSA_FMT_E5M2) launch_td<XDT, false, true, MPSA_FMT_E5M2>(p, tile, d, grid, st);
        else                       launch_td<XDT, false, true, MPSA_FMT_E4M3>(p, tile, d, grid, st);
    } else {
        if (fmt8 == MPSA_FMT_E5M2) launch_td<XDT, true, true, MPSA_FMT_E5M2>(p, tile, d, grid, st);
        else                       launch_td<XDT, true, true, MPSA_FMT_E4M3>(p, tile, d, grid, st);
    }
}

}  // namespace

extern "C" int mpsa_attn_prepare(const void* q, const int64_t q_strides[4], const void* k, const int64_t k_strides[4],
                                 const void* v, const int64_t v_strides[4], int dtype,
                                 int64_t B, int64_t Hq, int64_t Hkv, int64_t Nq, int64_t Nk, int64_t D, int tile, int mode, int fmt8,
                                 float pre_scale_q, const void* k_sub,
                                 uint8_t* q4, uint8_t* qs4, uint8_t* q8, uint8_t* qs8,
                                 uint8_t* k4, uint8_t* ks4, uint8_t* k8, uint8_t* ks8, void* v_tiles, mpsa_stream_t stream) {
    if (mode == MPSA_MODE_ROUTED || mode == MPSA_MODE_MIXED) mode = MPSA_MODE_DIAG;   // both operand sets, like a diag run
    if (mode != MPSA_MODE_MXFP4 && mode != MPSA_MODE_MXFP8 && mode != MPSA_MODE_DIAG) return mpsa_fail(MPSA_EINVAL, "prepare: unknown mode %d", mode);
    if (tile != 64 && tile != 128) return mpsa_fail(MPSA_EUNSUPPORTED, "prepare: tile must be 64 or 128 (got %d)", tile);
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || Nq <= 0 || Nk <= 0 || Hq % Hkv) return mpsa_fail(MPSA_EINVAL, "prepare: bad shape (B=%lld Hq=%lld Hkv=%lld Nq=%lld Nk=%lld)", (long long)B, (long long)Hq, (long long)Hkv, (long long)Nq, (long long)Nk);
    const bool do4 = mode != MPSA_MODE_MXFP8, do8 = mode != MPSA_MODE_MXFP4;
    const int64_t nq_pad = (Nq + tile - 1) / tile * tile, nk_pad = (Nk + tile - 1) / tile * tile;
    constexpr int EMAX4 = 3, EMAX8 = 7;            // ours/quant_mxint8.py:303, :191
    if (mpsa_quantize_sw_encoders() && q) {
        // the cross-checking encoders exist only as stand-alone kernels
        int rc = do4 && do8 ? mpsa_quantize_mx_dual(q, dtype, B, Hq, Nq, D, q_strides, nullptr, pre_scale_q, EMAX4, fmt8, EMAX8, q4, qs4, q8, qs8, nq_pad, stream)
                            : mpsa_quantize_mx(q, dtype, B, Hq, Nq, D, q_strides, nullptr, pre_scale_q, do4 ? MPSA_FMT_E2M1 : fmt8, do4 ? EMAX4 : EMAX8, do4 ? q4 : q8, do4 ? qs4 : qs8, nq_pad, stream);
        if (rc != MPSA_OK) return rc;
        rc = do4 && do8 ? mpsa_quantize_mx_dual(k, dtype, B, Hkv, Nk, D, k_strides, k_sub, 1.0f, EMAX4, fmt8, EMAX8, k4, ks4, k8, ks8, nk_pad, stream)
                        : mpsa_quantize_mx(k, dtype, B, Hkv, Nk, D, k_strides, k_sub, 1.0f, do4 ? MPSA_FMT_E2M1 : fmt8, do4 ? EMAX4 : EMAX8, do4 ? k4 : k8, do4 ? ks4 : ks8, nk_pad, stream);
        if (rc != MPSA_OK) return rc;
        return mpsa_v_tiles(v, dtype, B, Hkv, Nk, D, v_strides, tile, v_tiles, stream);
    }
    PrepArgs p;
    unsigned bq = 0, bk = 0, bv = 0;
    int rc = MPSA_OK;
    if (q) {
        rc = mpsa_quantize_setup(q, dtype, B, Hq, Nq, D, q_strides, nullptr, pre_scale_q, do4, EMAX4, do8, fmt8, EMAX8, q4, qs4, q8, qs8, nq_pad, &p.q, &bq);
        if (rc != MPSA_OK) return rc;
    } else {
        p.q = QuantArgs{};                       // no Q job: the attention kernel quantizes Q itself (mpsa_attn_fwd_q16)
    }
    rc = mpsa_quantize_setup(k, dtype, B, Hkv, Nk, D, k_strides, k_sub, 1.0f, do4, EMAX4, do8, fmt8, EMAX8, k4, ks4, k8, ks8, nk_pad, &p.k, &bk);
    if (rc != MPSA_OK) return rc;
    rc = mpsa_v_tiles_setup(v, dtype, B, Hkv, Nk, D, v_strides, tile, v_tiles, &p.v, &bv);
    if (rc != MPSA_OK) return rc;
    const int64_t total = (int64_t)bq * Hq * B + (int64_t)(bk + bv) * Hkv * B;
    if (total >= (int64_t(1) << 31)) return mpsa_fail(MPSA_EUNSUPPORTED, "prepare: problem too large for one launch");
    p.bq = bq; p.bk = bk; p.bv = bv; p.hq = (uint32_t)Hq; p.hkv = (uint32_t)Hkv;
    p.q_total = (uint32_t)((int64_t)bq * Hq * B); p.k_total = (uint32_t)((int64_t)bk * Hkv * B);
    p.v_total = (uint32_t)((int64_t)bv * Hkv * B);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == MPSA_BF16) launch_mode<MPSA_BF16>(p, mode, fmt8, tile, (int)D, (unsigned)((total + 1) / 2), st);
    else                    launch_mode<MPSA_F16>(p, mode, fmt8, tile, (int)D, (unsigned)((total + 1) / 2), st);
    MPSA_CHECK_LAUNCH("prepare");
    return MPSA_OK;
}
