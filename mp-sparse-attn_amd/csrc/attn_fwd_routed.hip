// Routed variants of the general fused attention kernel: every (query tile, key tile) pair runs at the precision the
// visiting list names (see attn_fwd_kernel.h and route.hip); pairs that are not on the list are skipped.
#include "attn_fwd_kernel.h"

namespace {

template <int D, int TILE>
int launch_dt(const AttnArgs& a, int pv_dtype, hipStream_t st) {
    if (pv_dtype == MPSA_BF16)
        return a.fmt8 == MPSA_FMT_E5M2 ? launch_one<D, TILE, MPSA_BF16, MPSA_FMT_E5M2, MPSA_MODE_ROUTED>(a, st)
                                       : launch_one<D, TILE, MPSA_BF16, MPSA_FMT_E4M3, MPSA_MODE_ROUTED>(a, st);
    return a.fmt8 == MPSA_FMT_E5M2 ? launch_one<D, TILE, MPSA_F16, MPSA_FMT_E5M2, MPSA_MODE_ROUTED>(a, st)
                                   : launch_one<D, TILE, MPSA_F16, MPSA_FMT_E4M3, MPSA_MODE_ROUTED>(a, st);
}

}  // namespace

int attn_routed_launch(const AttnArgs& a, int pv_dtype, hipStream_t st) {
    if (a.d == 128 && a.tile == 128) return launch_dt<128, 128>(a, pv_dtype, st);
    if (a.d == 64 && a.tile == 64)   return launch_dt<64, 64>(a, pv_dtype, st);
    if (a.d == 128 && a.tile == 64)  return launch_dt<128, 64>(a, pv_dtype, st);
    return launch_dt<64, 128>(a, pv_dtype, st);
}
