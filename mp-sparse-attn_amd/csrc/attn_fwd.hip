// Fused diagonal-tiled MXFP attention forward for gfx950.
//
// Per query tile i of one head: for every visited key tile j, S = Q_i K_j^T on the scaled matrix cores
// (8-bit operands when the tile's precision is 8-bit, 4-bit otherwise), base-2 online softmax with
// float32 running max / sum, P rounded to 16 bits, O += P V_j, and O / l at the end -- the loop of the
// reference's block_scaled_batched_attn_kernel (ours/mxfp_attn_kernel.py:216-359).  Causal runs visit
// tiles j <= i and mask only tile j == i (ours/online_routing.py:68-77, :113-118); query head hq reads
// key/value head hq / (Hq/Hkv) (ours/online_routing.py:160-171).  Q already carries sm_scale*log2(e)
// (folded in by the quantizer, ours/quant_mxint8.py:494), so scores are in log2 units.
//
// Mapping.  A workgroup owns one TILE-query tile; each of its TILE/32 waves owns 32 queries and walks all
// keys of every tile.  Both products are computed transposed so that a lane always owns ONE query:
//   S^T = K Q^T   on v_mfma_scale_f32_32x32x64_f8f6f4: lane (h = lane/32, r = lane%32) of the K operand
//                 supplies 32 elements of key row r and the E8M0 byte of MX block h of the 64-wide step
//                 (4-bit: the lane's registers are block h; 8-bit: registers 0-3 of both lane halves are
//                 block 0, registers 4-7 block 1), the Q operand the same for query r; the result leaves query r's scores for 16 keys per 32-key block in
//                 that lane's registers, so the row maximum is a register reduction plus one exchange
//                 with lane^32, and running max / sum / rescale factors are plain per-lane scalars.
//   O^T += V^T P^T on v_mfma_f32_32x32x16_{bf16,f16}: the P^T operand of lane (h, r) is exactly the eight
//                 scores that lane already holds (keys are contracted in the order the score MFMA left
//                 them); V is pre-arranged by mpsa_v_tiles to match, one 16-byte LDS read per operand.
// Staging.  4-bit K codes and the V tile travel HBM/L2 -> LDS with direct-to-LDS loads (global_load_lds_dwordx4:
// each lane names a 16-byte global source, the wave's 64 pieces land contiguously in LDS), so they cost neither
// registers nor LDS-write instructions.  The V tile is already in operand order (a flat copy); K rows keep their
// row-major order but the 16-byte chunks of a row are XOR-swizzled with the row index, which makes the 128-bit
// operand reads of 16 consecutive rows hit 16 distinct 4-bank groups.  Both are double-buffered and the loop
// needs ONE barrier per tile: after the barrier of step t a wave issues the loads of V(t+1) and K(t+2), pulls the
// K(t+1) fragments from LDS into registers and runs P.V of step t; the next step's score MFMAs then start from
// registers.  The single 8-bit K tile of a "diag" run bypasses LDS (each lane reads its fragments from global memory);
// runs with many 8-bit tiles ("mxfp8", routed) stage them through the same LDS area, one buffer plus the fragment
// registers (see attn_fwd_kernel.h).  K scales are read from global memory one step ahead.  80 KiB of LDS and at most 256 registers per workgroup let two workgroups share a CU, so one's matrix
// instructions overlap the other's softmax VALU work.
#include "attn_fwd_kernel.h"

namespace {

template <int D, int TILE, int PVT>
int launch_mode(const AttnArgs& a, hipStream_t st) {
    if (a.mode == MPSA_MODE_MXFP4) return launch_one<D, TILE, PVT, MPSA_FMT_E4M3, MPSA_MODE_MXFP4>(a, st);
    if (a.mode == MPSA_MODE_MIXED)
        return a.fmt8 == MPSA_FMT_E5M2 ? launch_one<D, TILE, PVT, MPSA_FMT_E5M2, MPSA_MODE_MIXED>(a, st)
                                       : launch_one<D, TILE, PVT, MPSA_FMT_E4M3, MPSA_MODE_MIXED>(a, st);
    if (a.mode == MPSA_MODE_MXFP8)
        return a.fmt8 == MPSA_FMT_E5M2 ? launch_one<D, TILE, PVT, MPSA_FMT_E5M2, MPSA_MODE_MXFP8>(a, st)
                                       : launch_one<D, TILE, PVT, MPSA_FMT_E4M3, MPSA_MODE_MXFP8>(a, st);
    return a.fmt8 == MPSA_FMT_E5M2 ? launch_one<D, TILE, PVT, MPSA_FMT_E5M2, MPSA_MODE_DIAG>(a, st)
                                   : launch_one<D, TILE, PVT, MPSA_FMT_E4M3, MPSA_MODE_DIAG>(a, st);
}

template <int D, int TILE>
int launch_dt(const AttnArgs& a, int pv_dtype, hipStream_t st) {
    if (pv_dtype == MPSA_BF16) return launch_mode<D, TILE, MPSA_BF16>(a, st);
    return launch_mode<D, TILE, MPSA_F16>(a, st);
}

}  // namespace

struct RawQ { const void* q; const int64_t* strides; int dtype; float pre; };

static int attn_entry(const RawQ* rq, const uint8_t* q4, const uint8_t* qs4, const uint8_t* q8, const uint8_t* qs8,
                      const uint8_t* k4, const uint8_t* ks4, const uint8_t* k8, const uint8_t* ks8, int fmt8,
                      const void* v_tiles, int pv_dtype, void* o, int o_dtype, const int64_t o_strides[4],
                      int64_t B, int64_t Hq, int64_t Hkv, int64_t nq, int64_t n, int64_t D, int tile, int causal, int mode,
                      bool skip, float skip_thresh, int32_t* skipped, const int32_t* order, const int32_t* counts,
                      mpsa_stream_t stream) {
    if (mode != MPSA_MODE_MXFP4 && mode != MPSA_MODE_MXFP8 && mode != MPSA_MODE_DIAG && mode != MPSA_MODE_ROUTED && mode != MPSA_MODE_MIXED) return mpsa_fail(MPSA_EINVAL, "attn: unknown mode %d", mode);
    const bool routed = mode == MPSA_MODE_ROUTED;
    if (routed && (!order || !counts)) return mpsa_fail(MPSA_EINVAL, "attn: a routed run needs the visiting lists (order, counts)");
    if (routed && ((reinterpret_cast<uintptr_t>(order) | reinterpret_cast<uintptr_t>(counts)) & 3)) return mpsa_fail(MPSA_EALIGN, "attn: order and counts must be 4-byte aligned");
    const bool mixed = mode == MPSA_MODE_MIXED;
    const bool need4 = mode != MPSA_MODE_MXFP8, need8 = mode != MPSA_MODE_MXFP4;
    if (rq) {
        if (!rq->q || !rq->strides) return mpsa_fail(MPSA_EINVAL, "attn: null q");
        if (rq->dtype != pv_dtype) return mpsa_fail(MPSA_EINVAL, "attn: unquantized q must have the P.V dtype (the dtype of v)");
        if (rq->strides[3] != 1 || !mpsa_aligned16(rq->q) || (rq->strides[0] % 8) || (rq->strides[1] % 8) || (rq->strides[2] % 8))
            return mpsa_fail(MPSA_EALIGN, "attn: q rows must be contiguous and 16-byte aligned");
        if (mode == MPSA_MODE_ROUTED) return mpsa_fail(MPSA_EUNSUPPORTED, "attn: unquantized q is not taken in the routed mode (the router reads Q's scale bytes)");
        const bool k8_read = mode == MPSA_MODE_DIAG || mode == MPSA_MODE_MXFP8;       // the mixed mode multiplies 4-bit K only
        if ((need4 && (!k4 || !ks4)) || (k8_read && (!k8 || !ks8))) return mpsa_fail(MPSA_EINVAL, "attn: K operands missing");
    } else if (mixed) {
        if (!q8 || !qs8 || !k4 || !ks4) return mpsa_fail(MPSA_EINVAL, "attn: the mixed mode needs 8-bit Q and 4-bit K operands");
    } else if (routed) {
        // lists that name tiles of one precision only need that operand set only (the caller's promise); a set is whole or absent
        const bool has4 = q4 && qs4 && k4 && ks4, has8 = q8 && qs8 && k8 && ks8;
        const bool none4 = !q4 && !qs4 && !k4 && !ks4, none8 = !q8 && !qs8 && !k8 && !ks8;
        if (!(has4 || none4) || !(has8 || none8) || (none4 && none8)) return mpsa_fail(MPSA_EINVAL, "attn: a routed run needs the whole 4-bit operand set, the whole 8-bit one, or both");
    } else {
        if (need4 && (!q4 || !qs4 || !k4 || !ks4)) return mpsa_fail(MPSA_EINVAL, "attn: 4-bit operands missing");
        if (need8 && (!q8 || !qs8 || !k8 || !ks8)) return mpsa_fail(MPSA_EINVAL, "attn: 8-bit operands missing");
    }
    if (!v_tiles || !o || !o_strides) return mpsa_fail(MPSA_EINVAL, "attn: null pointer");
    if (need8 && (!routed || q8) && fmt8 != MPSA_FMT_E4M3 && fmt8 != MPSA_FMT_E5M2) return mpsa_fail(MPSA_EINVAL, "attn: 8-bit format must be E4M3 or E5M2");
    if (pv_dtype != MPSA_BF16 && pv_dtype != MPSA_F16) return mpsa_fail(MPSA_EINVAL, "attn: pv_dtype must be bf16 or f16");
    if (o_dtype != MPSA_BF16 && o_dtype != MPSA_F16 && o_dtype != MPSA_F32) return mpsa_fail(MPSA_EINVAL, "attn: bad output dtype");
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || n <= 0 || nq <= 0 || Hq % Hkv) return mpsa_fail(MPSA_EINVAL, "attn: bad shape (B=%lld Hq=%lld Hkv=%lld nq=%lld nk=%lld)", (long long)B, (long long)Hq, (long long)Hkv, (long long)nq, (long long)n);
    if (nq != n && (causal || mode == MPSA_MODE_DIAG)) return mpsa_fail(MPSA_EINVAL, "attn: causal masking and the diag mode need as many queries as keys (nq=%lld nk=%lld)", (long long)nq, (long long)n);
    if ((D != 64 && D != 128) || (tile != 64 && tile != 128)) return mpsa_fail(MPSA_EUNSUPPORTED, "attn: D=%lld tile=%d (both must be 64 or 128)", (long long)D, tile);
    if (o_strides[3] != 1 || (o_strides[0] % 4) || (o_strides[1] % 4) || (o_strides[2] % 4)) return mpsa_fail(MPSA_EALIGN, "attn: output rows must be contiguous and 8-byte aligned");
    const uintptr_t al = reinterpret_cast<uintptr_t>(q4) | reinterpret_cast<uintptr_t>(q8) | reinterpret_cast<uintptr_t>(k4) |
                         reinterpret_cast<uintptr_t>(k8) | reinterpret_cast<uintptr_t>(v_tiles) | reinterpret_cast<uintptr_t>(o);
    const uintptr_t al4 = reinterpret_cast<uintptr_t>(qs4) | reinterpret_cast<uintptr_t>(qs8) | reinterpret_cast<uintptr_t>(ks4) | reinterpret_cast<uintptr_t>(ks8);
    if ((al & 15) || (al4 & 3)) return mpsa_fail(MPSA_EALIGN, "attn: operands must be 16-byte (codes, v, o) / 4-byte (scales) aligned");
    const int64_t nt = (n + tile - 1) / tile, ntq = (nq + tile - 1) / tile;
    if (B * Hq * ntq >= (int64_t(1) << 31) || nt * tile >= (int64_t(1) << 30) || ntq * tile >= (int64_t(1) << 30)) return mpsa_fail(MPSA_EUNSUPPORTED, "attn: problem too large");
    AttnArgs a;
    a.q4 = q4; a.qs4 = qs4; a.q8 = q8; a.qs8 = qs8; a.k4 = k4; a.ks4 = ks4; a.k8 = k8; a.ks8 = ks8;
    a.v = v_tiles; a.o = o;
    a.o_sb = o_strides[0]; a.o_sh = o_strides[1]; a.o_sn = o_strides[2];
    a.B = (int)B; a.Hq = (int)Hq; a.Hkv = (int)Hkv; a.n = (int)n; a.nt = (int)nt; a.n_pad = (int)(nt * tile);
    a.nq = (int)nq; a.ntq = (int)ntq; a.nq_pad = (int)(ntq * tile);
    a.causal = causal ? 1 : 0; a.mode = mode; a.fmt8 = fmt8; a.o_dtype = o_dtype;
    a.d = (int)D; a.tile = tile;
    a.skip_thresh = skip_thresh; a.skipped = skipped;
    a.order = order; a.counts = counts;
    a.q_raw = nullptr; a.q_sb = a.q_sh = a.q_sn = 0; a.q_pre = 1.0f;
    hipStream_t st = (hipStream_t)stream;
    if (rq) {
        a.q_raw = rq->q; a.q_sb = rq->strides[0]; a.q_sh = rq->strides[1]; a.q_sn = rq->strides[2]; a.q_pre = rq->pre;
        if (!attn_pp_supported(a, pv_dtype))
            return mpsa_fail(MPSA_EUNSUPPORTED, "attn: unquantized q needs the paired-tile kernel's shape (D = 128, tile = 128; "
                                                "causal: at least two tiles, unmasked: at least six); quantize q with mpsa_attn_prepare and call mpsa_attn_fwd");
        return attn_pp_launch(a, pv_dtype, st);
    }
    if (routed) return attn_routed_launch(a, pv_dtype, st);
    if (skip) {
        if (!(skip_thresh == skip_thresh)) return mpsa_fail(MPSA_EINVAL, "attn: skip_thresh is NaN");
        if (skipped && (reinterpret_cast<uintptr_t>(skipped) & 3)) return mpsa_fail(MPSA_EALIGN, "attn: skipped must be 4-byte aligned");
        return attn_skip_launch(a, pv_dtype, st);
    }
    if (attn_pp_supported(a, pv_dtype)) return attn_pp_launch(a, pv_dtype, st);
    if (D == 128 && tile == 128) return launch_dt<128, 128>(a, pv_dtype, st);
    if (D == 64 && tile == 64)   return launch_dt<64, 64>(a, pv_dtype, st);
    if (D == 128 && tile == 64)  return launch_dt<128, 64>(a, pv_dtype, st);
    return launch_dt<64, 128>(a, pv_dtype, st);
}

extern "C" int mpsa_attn_fwd(const uint8_t* q4, const uint8_t* qs4, const uint8_t* q8, const uint8_t* qs8,
                             const uint8_t* k4, const uint8_t* ks4, const uint8_t* k8, const uint8_t* ks8, int fmt8,
                             const void* v_tiles, int pv_dtype, void* o, int o_dtype, const int64_t o_strides[4],
                             int64_t B, int64_t Hq, int64_t Hkv, int64_t nq, int64_t n, int64_t D, int tile, int causal, int mode,
                             mpsa_stream_t stream) {
    return attn_entry(nullptr, q4, qs4, q8, qs8, k4, ks4, k8, ks8, fmt8, v_tiles, pv_dtype, o, o_dtype, o_strides,
                      B, Hq, Hkv, nq, n, D, tile, causal, mode, false, 0.0f, nullptr, nullptr, nullptr, stream);
}

extern "C" int mpsa_attn_fwd_skip(const uint8_t* q4, const uint8_t* qs4, const uint8_t* q8, const uint8_t* qs8,
                                  const uint8_t* k4, const uint8_t* ks4, const uint8_t* k8, const uint8_t* ks8, int fmt8,
                                  const void* v_tiles, int pv_dtype, void* o, int o_dtype, const int64_t o_strides[4],
                                  int64_t B, int64_t Hq, int64_t Hkv, int64_t nq, int64_t n, int64_t D, int tile, int causal, int mode,
                                  float skip_thresh, int32_t* skipped, mpsa_stream_t stream) {
    return attn_entry(nullptr, q4, qs4, q8, qs8, k4, ks4, k8, ks8, fmt8, v_tiles, pv_dtype, o, o_dtype, o_strides,
                      B, Hq, Hkv, nq, n, D, tile, causal, mode, true, skip_thresh, skipped, nullptr, nullptr, stream);
}

extern "C" int mpsa_attn_fwd_routed(const uint8_t* q4, const uint8_t* qs4, const uint8_t* q8, const uint8_t* qs8,
                                    const uint8_t* k4, const uint8_t* ks4, const uint8_t* k8, const uint8_t* ks8, int fmt8,
                                    const void* v_tiles, int pv_dtype, void* o, int o_dtype, const int64_t o_strides[4],
                                    int64_t B, int64_t Hq, int64_t Hkv, int64_t nq, int64_t n, int64_t D, int tile, int causal,
                                    const int32_t* order, const int32_t* counts, mpsa_stream_t stream) {
    return attn_entry(nullptr, q4, qs4, q8, qs8, k4, ks4, k8, ks8, fmt8, v_tiles, pv_dtype, o, o_dtype, o_strides,
                      B, Hq, Hkv, nq, n, D, tile, causal, MPSA_MODE_ROUTED, false, 0.0f, nullptr, order, counts, stream);
}

extern "C" int mpsa_attn_fwd_q16(const void* q, const int64_t q_strides[4], int q_dtype, float pre_scale_q,
                                 const uint8_t* k4, const uint8_t* ks4, const uint8_t* k8, const uint8_t* ks8, int fmt8,
                                 const void* v_tiles, int pv_dtype, void* o, int o_dtype, const int64_t o_strides[4],
                                 int64_t B, int64_t Hq, int64_t Hkv, int64_t n, int64_t D, int tile, int causal, int mode,
                                 mpsa_stream_t stream) {
    const RawQ rq = {q, q_strides, q_dtype, pre_scale_q};
    return attn_entry(&rq, nullptr, nullptr, nullptr, nullptr, k4, ks4, k8, ks8, fmt8, v_tiles, pv_dtype, o, o_dtype, o_strides,
                      B, Hq, Hkv, n, n, D, tile, causal, mode, false, 0.0f, nullptr, nullptr, nullptr, stream);
}

extern "C" int mpsa_attn_fwd_q16_supported(int64_t B, int64_t Hq, int64_t Hkv, int64_t n, int64_t D, int tile, int causal, int mode) {
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || n <= 0 || Hq % Hkv || B * Hq * (n / 256 + 1) >= (int64_t(1) << 31)) return 0;
    if (mode != MPSA_MODE_DIAG && mode != MPSA_MODE_MXFP4 && mode != MPSA_MODE_MIXED && mode != MPSA_MODE_MXFP8) return 0;
    AttnArgs a = {};
    a.B = (int)B; a.Hq = (int)Hq; a.Hkv = (int)Hkv; a.n = (int)n; a.d = (int)D; a.tile = tile; a.causal = causal ? 1 : 0; a.mode = mode;
    a.nt = (int)((n + tile - 1) / (tile > 0 ? tile : 1)); a.n_pad = a.nt * tile;
    a.nq = a.n; a.ntq = a.nt; a.nq_pad = a.n_pad;
    return (tile == 64 || tile == 128) && attn_pp_supported(a, MPSA_BF16) ? 1 : 0;
}
