// Per-tile precision routing from the E8M0 scale bytes the MX quantizer has already written.
//
// The reference's online routing keeps or skips a score tile by comparing a statistic of the tile with the first
// tile's (ours/online_routing.py:87-112).  This router extends the idea to a precision choice and takes its
// statistic from data that costs nothing to get: the 4-bit scale byte e of a 32-wide block is
// floor(log2(amax)) - 2 + 127, so 6 * 2^(e-127) bounds every element of the block.  Per tile and block c, over the
// tile's rows r:   M[c] = max_r e[r][c],   F[c] = sum_r 2^(10 - (M[c] - e[r][c]))   (terms below 1 dropped),
// so 2^(M-10) * F is the sum of the rows' 2^e.  For query tile I and key tile J, with s[c] = Mq[I][c] + Mk[J][c],
// w[c] = Fq[I][c] * Fk[J][c] and smax[I] the largest s[c] over the visited key tiles:
//   T[I][J] = (sum_c (w[c] >> (smax[I] - s[c]))) >> 13                       (shifts above 40 give 0; T < 2^24)
// is proportional to the summed magnitude bound of the tile's scores -- and so to the absolute error its 4-bit
// product makes.  With Tmax[I] the largest T over the visited key tiles:
//   8-bit   if float(T) >= hi_thresh * float(Tmax)
//   skipped if float(T) <  skip_thresh * float(Tmax), unless J == 0 (the reference's always-kept first tile) or the
//           diagonal tile of a causal run
//   4-bit   otherwise.
// Integer work on a few bytes per tile: two small launches (tile statistics, then one wave per query tile that
// classifies its key tiles and compacts them into the visiting lists the attention kernel walks).
#include "mpsa_common.h"

namespace {

constexpr int ROW_BITS = 10, OUT_SHIFT = 13, MAX_SHIFT = 40;
enum : uint8_t { CLS_SKIP = 0, CLS_FP4 = 1, CLS_FP8 = 2, CLS_NOT_VISITED = 255 };

__device__ __forceinline__ int wave_max(int x) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) x = max(x, __shfl_xor(x, o));
    return x;
}
__device__ __forceinline__ int wave_sum(int x) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) x += __shfl_xor(x, o);
    return x;
}

// One wave per tile.  Blocks [0, q_tiles) work on Q's scales, the rest on K's.  Output per tile: NB pairs (M, F).
template <int NB>
__global__ __launch_bounds__(64) void tile_scale_stats_kernel(const uint8_t* qs, const uint8_t* ks, int64_t q_tiles, int tile,
                                                             int32_t* qstat, int32_t* kstat) {
    const int64_t t = blockIdx.x;
    const bool is_q = t < q_tiles;
    const int64_t local = is_q ? t : t - q_tiles;
    const uint8_t* src = (is_q ? qs : ks) + local * tile * NB;
    // tile is 64 or 128: a lane holds one or two rows
    uint32_t w[2];
#pragma unroll
    for (int x = 0; x < 2; ++x) {
        const int row = threadIdx.x + 64 * x;
        w[x] = row < tile ? (NB == 4 ? *reinterpret_cast<const uint32_t*>(src + row * 4)
                                     : (uint32_t)*reinterpret_cast<const uint16_t*>(src + row * 2))
                          : 0u;
    }
    int32_t* dst = (is_q ? qstat : kstat) + local * NB * 2;
#pragma unroll
    for (int c = 0; c < NB; ++c) {
        const int e0 = (int)((w[0] >> (8 * c)) & 255u), e1 = (int)((w[1] >> (8 * c)) & 255u);
        const int m = wave_max(max(e0, e1));
        int f = m - e0 <= ROW_BITS ? 1 << (ROW_BITS - (m - e0)) : 0;
        if (tile > 64) f += m - e1 <= ROW_BITS ? 1 << (ROW_BITS - (m - e1)) : 0;
        f = wave_sum(f);
        if (threadIdx.x == 0) {
            dst[2 * c] = m;
            dst[2 * c + 1] = f;
        }
    }
}

struct RouteArgs {
    const int32_t *qstat, *kstat;
    int Hq, Hkv, ntq, nt, causal, ragged;
    float hi, lo;
    uint8_t* cls;
    int32_t *order, *counts;
};

// One wave per (batch, query head, query tile).
template <int NB>
__global__ __launch_bounds__(64) void route_kernel(RouteArgs a) {
    const int64_t row = blockIdx.x;
    const int lane = threadIdx.x;
    const int i = (int)(row % a.ntq);
    const int64_t bh = row / a.ntq;
    const int hq = (int)(bh % a.Hq);
    const int64_t b = bh / a.Hq;
    const int kvh = hq / (a.Hq / a.Hkv);
    const int32_t* kst = a.kstat + (b * a.Hkv + kvh) * (int64_t)a.nt * NB * 2;
    int mq[NB];
    uint64_t fq[NB];
#pragma unroll
    for (int c = 0; c < NB; ++c) {
        mq[c] = a.qstat[(row * NB + c) * 2];
        fq[c] = (uint64_t)a.qstat[(row * NB + c) * 2 + 1];
    }
    const int last = a.causal ? min(i, a.nt - 1) : a.nt - 1;

    auto sums = [&](int j, int (&s)[NB]) {
#pragma unroll
        for (int c = 0; c < NB; ++c) s[c] = mq[c] + kst[((int64_t)j * NB + c) * 2];
    };
    int smax = 0;
    for (int j = lane; j <= last; j += 64) {
        int s[NB];
        sums(j, s);
#pragma unroll
        for (int c = 0; c < NB; ++c) smax = max(smax, s[c]);
    }
    smax = wave_max(smax);
    auto stat = [&](int j) {
        int s[NB];
        sums(j, s);
        uint64_t t = 0;
#pragma unroll
        for (int c = 0; c < NB; ++c) {
            const int d = smax - s[c];
            const uint64_t w = fq[c] * (uint64_t)kst[((int64_t)j * NB + c) * 2 + 1];
            t += d <= MAX_SHIFT ? w >> d : 0ull;
        }
        return (int)(t >> OUT_SHIFT);
    };
    int tmax = 0;
    for (int j = lane; j <= last; j += 64) tmax = max(tmax, stat(j));
    tmax = wave_max(tmax);
    const float tmaxf = (float)tmax;
    const float hi_cut = a.hi * tmaxf, lo_cut = a.lo * tmaxf;

    // run k of the visiting list: 0 = 4-bit plain, 1 = 4-bit masked, 2 = 8-bit plain, 3 = 8-bit masked
    auto classify = [&](int j, int& run) {
        run = -1;
        if (j > last) return (uint8_t)CLS_NOT_VISITED;
        const float tf = (float)stat(j);
        uint8_t c = CLS_FP4;
        if (a.lo > 0.0f && tf < lo_cut && j != 0 && !(a.causal && j == i)) c = CLS_SKIP;
        if (a.hi > 0.0f && tf >= hi_cut) c = CLS_FP8;
        if (c != CLS_SKIP) {
            const bool masked = (a.causal && j == i) || (a.ragged && j == a.nt - 1);
            run = (c == CLS_FP8 ? 2 : 0) + (masked ? 1 : 0);
        }
        return c;
    };
    int cnt[4] = {0, 0, 0, 0};
    const int chunks = (a.nt + 63) / 64;
    for (int ch = 0; ch < chunks; ++ch) {
        const int j = ch * 64 + lane;
        int run = -1;
        if (j < a.nt) a.cls[row * a.nt + j] = classify(j, run);
#pragma unroll
        for (int k = 0; k < 4; ++k) cnt[k] += __popcll(__ballot(run == k));
    }
    int base[4] = {0, cnt[0], cnt[0] + cnt[1], cnt[0] + cnt[1] + cnt[2]};
    const int total = base[3] + cnt[3];
    if (lane < 4) a.counts[row * 4 + lane] = cnt[lane];
    const uint64_t below = (1ull << lane) - 1ull;
    for (int ch = 0; ch < chunks; ++ch) {
        const int j = ch * 64 + lane;
        int run = -1;
        if (j < a.nt) classify(j, run);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const uint64_t mask = __ballot(run == k);
            if (run == k) a.order[row * a.nt + base[k] + __popcll(mask & below)] = j;
            base[k] += __popcll(mask);
        }
    }
    for (int t = total + lane; t < a.nt; t += 64) a.order[row * a.nt + t] = -1;
}

int64_t ceil_div(int64_t x, int64_t y) { return (x + y - 1) / y; }

}  // namespace

extern "C" int64_t mpsa_route_workspace(int64_t B, int64_t Hq, int64_t Hkv, int64_t nq, int64_t nk, int64_t D, int tile) {
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || nq <= 0 || nk <= 0 || D <= 0 || tile <= 0) return 0;
    return (B * Hq * ceil_div(nq, tile) + B * Hkv * ceil_div(nk, tile)) * (D / 32) * 2 * (int64_t)sizeof(int32_t);
}

extern "C" int mpsa_route_tiles(const uint8_t* qs4, const uint8_t* ks4, int64_t B, int64_t Hq, int64_t Hkv, int64_t nq,
                                int64_t nk, int64_t D, int tile, int causal, float hi_thresh, float skip_thresh, void* work,
                                uint8_t* cls, int32_t* order, int32_t* counts, mpsa_stream_t stream) {
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || nq <= 0 || nk <= 0 || Hq % Hkv) return mpsa_fail(MPSA_EINVAL, "route: bad shape (B=%lld Hq=%lld Hkv=%lld nq=%lld nk=%lld)", (long long)B, (long long)Hq, (long long)Hkv, (long long)nq, (long long)nk);
    if ((D != 64 && D != 128) || (tile != 64 && tile != 128)) return mpsa_fail(MPSA_EUNSUPPORTED, "route: D=%lld tile=%d (both must be 64 or 128)", (long long)D, tile);
    if (causal && nq != nk) return mpsa_fail(MPSA_EINVAL, "route: causal masking needs as many queries as keys (nq=%lld nk=%lld)", (long long)nq, (long long)nk);
    if (!(hi_thresh == hi_thresh) || !(skip_thresh == skip_thresh)) return mpsa_fail(MPSA_EINVAL, "route: a threshold is NaN");
    if (!qs4 || !ks4 || !work || !cls || !order || !counts) return mpsa_fail(MPSA_EINVAL, "route: null pointer");
    const uintptr_t al4 = reinterpret_cast<uintptr_t>(qs4) | reinterpret_cast<uintptr_t>(ks4) | reinterpret_cast<uintptr_t>(order) |
                          reinterpret_cast<uintptr_t>(counts) | reinterpret_cast<uintptr_t>(work);
    if (al4 & 3) return mpsa_fail(MPSA_EALIGN, "route: scales, workspace, order and counts must be 4-byte aligned");
    const int64_t ntq = ceil_div(nq, tile), nt = ceil_div(nk, tile);
    const int64_t q_tiles = B * Hq * ntq, k_tiles = B * Hkv * nt;
    if (q_tiles + k_tiles >= (int64_t(1) << 31) || nt >= (int64_t(1) << 24)) return mpsa_fail(MPSA_EUNSUPPORTED, "route: problem too large");
    const int nb = (int)(D / 32);
    int32_t* qstat = static_cast<int32_t*>(work);
    int32_t* kstat = qstat + q_tiles * nb * 2;
    hipStream_t st = (hipStream_t)stream;
    RouteArgs a;
    a.qstat = qstat; a.kstat = kstat;
    a.Hq = (int)Hq; a.Hkv = (int)Hkv; a.ntq = (int)ntq; a.nt = (int)nt; a.causal = causal ? 1 : 0; a.ragged = (nk % tile) != 0;
    a.hi = hi_thresh; a.lo = skip_thresh;
    a.cls = cls; a.order = order; a.counts = counts;
    if (nb == 4) {
        hipLaunchKernelGGL(tile_scale_stats_kernel<4>, dim3((unsigned)(q_tiles + k_tiles)), dim3(64), 0, st, qs4, ks4, q_tiles, tile, qstat, kstat);
        hipLaunchKernelGGL(route_kernel<4>, dim3((unsigned)q_tiles), dim3(64), 0, st, a);
    } else {
        hipLaunchKernelGGL(tile_scale_stats_kernel<2>, dim3((unsigned)(q_tiles + k_tiles)), dim3(64), 0, st, qs4, ks4, q_tiles, tile, qstat, kstat);
        hipLaunchKernelGGL(route_kernel<2>, dim3((unsigned)q_tiles), dim3(64), 0, st, a);
    }
    MPSA_CHECK_LAUNCH("route");
    return MPSA_OK;
}
