// Tile-skipping variants of the general fused attention kernel (see attn_fwd_kernel.h for the rule, which is the
// reference's, ours/mxfp_attn_kernel.py:272-297).  Fixed-precision modes (mxfp4, mxfp8, mixed) and the diag mode.  The rule's reference
// tile is key tile 0; every walk starts there except query tile 0 of a non-causal diag run, whose diagonal tile
// (= key tile 0) comes last -- that workgroup takes the tile's statistic ahead of its walk.
#include "attn_fwd_kernel.h"

namespace {

template <int D, int TILE, int PVT>
int launch_mode(const AttnArgs& a, hipStream_t st) {
    if (a.mode == MPSA_MODE_MXFP4) return launch_one<D, TILE, PVT, MPSA_FMT_E4M3, MPSA_MODE_MXFP4, true>(a, st);
    if (a.mode == MPSA_MODE_DIAG)
        return a.fmt8 == MPSA_FMT_E5M2 ? launch_one<D, TILE, PVT, MPSA_FMT_E5M2, MPSA_MODE_DIAG, true>(a, st)
                                       : launch_one<D, TILE, PVT, MPSA_FMT_E4M3, MPSA_MODE_DIAG, true>(a, st);
    if (a.mode == MPSA_MODE_MIXED)
        return a.fmt8 == MPSA_FMT_E5M2 ? launch_one<D, TILE, PVT, MPSA_FMT_E5M2, MPSA_MODE_MIXED, true>(a, st)
                                       : launch_one<D, TILE, PVT, MPSA_FMT_E4M3, MPSA_MODE_MIXED, true>(a, st);
    return a.fmt8 == MPSA_FMT_E5M2 ? launch_one<D, TILE, PVT, MPSA_FMT_E5M2, MPSA_MODE_MXFP8, true>(a, st)
                                   : launch_one<D, TILE, PVT, MPSA_FMT_E4M3, MPSA_MODE_MXFP8, true>(a, st);
}

template <int D, int TILE>
int launch_dt(const AttnArgs& a, int pv_dtype, hipStream_t st) {
    if (pv_dtype == MPSA_BF16) return launch_mode<D, TILE, MPSA_BF16>(a, st);
    return launch_mode<D, TILE, MPSA_F16>(a, st);
}

}  // namespace

int attn_skip_launch(const AttnArgs& a, int pv_dtype, hipStream_t st) {
    if (a.mode != MPSA_MODE_MXFP4 && a.mode != MPSA_MODE_MXFP8 && a.mode != MPSA_MODE_DIAG && a.mode != MPSA_MODE_MIXED)
        return mpsa_fail(MPSA_EUNSUPPORTED, "attn: tile skipping needs mode mxfp4, mxfp8, diag or mixed");
    if (a.d == 128 && a.tile == 128) return launch_dt<128, 128>(a, pv_dtype, st);
    if (a.d == 64 && a.tile == 64)   return launch_dt<64, 64>(a, pv_dtype, st);
    if (a.d == 128 && a.tile == 64)  return launch_dt<128, 64>(a, pv_dtype, st);
    return launch_dt<64, 128>(a, pv_dtype, st);
}
