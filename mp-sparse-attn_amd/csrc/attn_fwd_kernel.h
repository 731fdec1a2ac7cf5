// The general fused attention kernel (template) and its launcher; included by attn_fwd.hip (all modes) and
// attn_fwd_skip.hip (the tile-skipping variants).  The design is described at the top of attn_fwd.hip.
#pragma once
#include "attn_common.h"

namespace {

template <int D, int TILE>
struct Geom {
    static constexpr int NW = TILE / 32;          // waves per workgroup
    static constexpr int NT = NW * 64;            // threads
    static constexpr int KB = TILE / 32;          // 32-key blocks per tile
    static constexpr int SST = D / 64;            // score matrix instructions along D
    static constexpr int NDB = D / 32;            // 32-wide output dim blocks
    static constexpr int ROW4 = D / 2, ROW8 = D;  // bytes per K row
    static constexpr int CPR4 = ROW4 / 16;        // 16-byte chunks per 4-bit K row (2 | 4)
    static constexpr int SH4 = CPR4 == 2 ? 3 : 2; // log2(rows per 256 bytes)
    static constexpr int K_BYTES = TILE * ROW4;   // one 4-bit K tile
    static constexpr int V_BYTES = TILE * D * 2;
    static constexpr int SMEM = 2 * K_BYTES + 2 * V_BYTES;
    static constexpr int CPR8 = ROW8 / 16;        // 16-byte chunks per 8-bit K row (4 | 8)
    static constexpr int SH8 = CPR8 == 4 ? 2 : 1; // log2(rows per 256 bytes)
    static constexpr int K8_BYTES = TILE * ROW8;  // one 8-bit K tile: exactly the two 4-bit buffers
    static constexpr int KI8 = K8_BYTES / 1024 / NW;
    static constexpr int KI4 = K_BYTES / 1024 / NW;                   // direct-load instructions per wave
    static constexpr int VI = V_BYTES / 1024 / NW;
    static constexpr int NV = KB * 2 * NDB;       // V fragments (= P.V matrix instructions) per tile
};

// MODE is compile-time: an all-4-bit run carries no 8-bit code, and a "diag" run pipelines 4-bit tiles through
// LDS and fetches its single 8-bit tile straight from global memory when it gets there.  Runs with many 8-bit tiles
// (all-8-bit, routed) stage them through LDS as well: an 8-bit K tile is as large as the two 4-bit buffers together,
// so it has ONE buffer, and the registers that hold the coming step's fragments are its second one.  That takes a
// second barrier per 8-bit step: barrier A publishes V(t) and K8(t+1); every wave pulls the K8(t+1) fragments into
// registers; barrier B says that everyone has, and only then the loads of K8(t+2) go out.
//
// A "routed" run (MPSA_MODE_ROUTED) walks a visiting list made by the tile router (route.hip): the 4-bit tiles through
// the LDS pipeline, then the 8-bit tiles with their K fragments prefetched from global memory; inside each precision
// the tiles that need a mask come last, so the two long loops keep the single-variant body.
//
// SKIP adds the reference's tile-skipping rule (ours/mxfp_attn_kernel.py:272-297): the statistic of a score tile
// is the mean over its query rows of the row maximum; the first key tile (the "sink") is always kept and sets the
// reference value, any later tile is kept only if its statistic is at least skip_thresh times the sink's (the
// diagonal tile of a causal run is always kept as well).  A skipped tile contributes nothing (no softmax, no P.V).  The statistic needs all rows of the tile, i.e. all
// waves: one extra workgroup barrier per tile, through a few floats of LDS behind the K/V buffers.
template <int D, int TILE, int PVT, int FMT8, int MODE, bool SKIP>
__global__ __launch_bounds__(TILE * 2, 2) void attn_fwd_kernel(AttnArgs a) {
    typedef Geom<D, TILE> G;
    typedef PV<PVT> P;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63, w = tid >> 6;
    const int h = lane >> 5, r = lane & 31;

    // ---- which (batch, kv head, query head, query tile) -- XCD-aware, heavy causal tiles first ----
    const int group = a.Hq / a.Hkv;
    const int total = a.B * a.Hq * a.ntq;
    int L = blockIdx.x;
    if ((total & 7) == 0) L = (L & 7) * (total >> 3) + (L >> 3);      // XCD x gets one contiguous logical range
    const int per_unit = group * a.ntq;
    const int unit = L / per_unit;
    const int rem = L - unit * per_unit;
    const int rank = rem / group;
    const int hq = (unit % a.Hkv) * group + (rem - rank * group);
    const int b = unit / a.Hkv;
    const int kvh = unit % a.Hkv;
    const int i = a.causal ? a.ntq - 1 - rank : rank;

    const int64_t qhead_row = ((int64_t)b * a.Hq + hq) * a.nq_pad;
    const int64_t khead_row = ((int64_t)b * a.Hkv + kvh) * a.n_pad;
    const int q_local = 32 * w + r;
    const int64_t q_row = qhead_row + (int64_t)i * TILE + q_local;

    uint8_t* const kbuf0 = smem;
    uint8_t* const vbuf0 = smem + 2 * G::K_BYTES;
    float* const stat_lds = reinterpret_cast<float*>(smem + G::SMEM);     // SKIP: [2][NW] partial statistics
    float sink_stat = 0.0f;
    bool sink_preset = false;   // SKIP, non-causal diag run, query tile 0: the sink's statistic was taken ahead of the walk
    bool started = false;       // SKIP: a kept tile has set the running maximum
    int n_skipped = 0;
    // Visiting order.  The order of key tiles does not matter to the softmax, so the tiles that need special
    // treatment go LAST: first every plain tile (main precision, no mask) in one tight loop, then the tile that
    // holds the sequence tail (masked) if there is one, then the diagonal tile i (causal mask and / or 8-bit).
    constexpr bool ROUTED = MODE == MPSA_MODE_ROUTED;
    constexpr bool MIXED = MODE == MPSA_MODE_MIXED;       // every tile: 8-bit Q against 4-bit K
    constexpr bool HAS4 = MODE != MPSA_MODE_MXFP8;        // 4-bit tiles exist (LDS pipeline in use)
    constexpr bool PRE8 = MODE == MPSA_MODE_MXFP8 || ROUTED;   // 8-bit K fragments are prefetched one step ahead
    const bool tail = a.n < a.n_pad;
    const bool diag_special = a.causal || MODE == MPSA_MODE_DIAG;
    const bool tail_special = tail && !a.causal && !(MODE == MPSA_MODE_DIAG && i == a.nt - 1);
    // routed: lengths of the list's four runs (4-bit plain, 4-bit masked, 8-bit plain, 8-bit masked), clamped so
    // that a malformed list cannot take the kernel outside its buffers
    const int64_t route_row = ((int64_t)b * a.Hq + hq) * a.ntq + i;
    const int32_t* const ord = ROUTED ? a.order + route_row * a.nt : nullptr;
    int r4p = 0, r4 = 0, r8p = 0;
    int nsteps = a.causal ? i + 1 : a.nt;
    if constexpr (ROUTED) {
        const int32_t* cn = a.counts + route_row * 4;
        const int c0 = min(max(cn[0], 0), a.nt);
        const int c1 = min(max(cn[1], 0), a.nt - c0);
        const int c2 = min(max(cn[2], 0), a.nt - c0 - c1);
        const int c3 = min(max(cn[3], 0), a.nt - c0 - c1 - c2);
        r4p = c0; r4 = c0 + c1; r8p = r4 + c2; nsteps = r8p + c3;
    }
    const int n_plain = nsteps - (diag_special ? 1 : 0) - (tail_special ? 1 : 0);
    const int skip = (MODE == MPSA_MODE_DIAG && !a.causal) ? i : 0x7fffffff;   // plain steps jump over tile i
    const int n_k4 = ROUTED ? r4 : nsteps;                // steps whose K tile travels through LDS
    auto tile_at = [&](int t) {
        if constexpr (ROUTED) return t < nsteps ? min(max(ord[t], 0), a.nt - 1) : 0;
        if (t < n_plain) return t + (t >= skip ? 1 : 0);
        if (tail_special && t == n_plain) return a.nt - 1;
        // the diagonal tile (runs that have one have as many key tiles as query tiles) -- and, past the last step,
        // any valid key tile: with more query tiles than key tiles (cross attention) i itself is not one
        return min(i, a.nt - 1);
    };
    // routed: the key tiles of steps t, t+1, t+2 are kept in scalar registers and the list entry of step t+3 is
    // fetched a whole step before its first use -- a scalar load that is waited for in the middle of a step would
    // also wait for the step's outstanding LDS reads (they share a counter)
    int jq0 = 0, jq1 = 0, jq2 = 0;
    if constexpr (ROUTED) {
        jq0 = tile_at(0); jq1 = tile_at(1); jq2 = tile_at(2);
    }
    auto tile_rel = [&](int t, auto k_c) {               // key tile of step t + K, t being the step in progress
        constexpr int K = decltype(k_c)::value;
        if constexpr (ROUTED) return K == 0 ? jq0 : (K == 1 ? jq1 : jq2);
        else return tile_at(t + K);
    };
    typedef std::integral_constant<int, 0> R0;
    typedef std::integral_constant<int, 1> R1;
    typedef std::integral_constant<int, 2> R2;
    auto step_is8 = [&](int t) {
        if constexpr (ROUTED) return t >= r4;
        return MODE == MPSA_MODE_MXFP8 || (MODE == MPSA_MODE_DIAG && t == nsteps - 1);
    };

    // ---- Q fragments of the current precision stay in registers; re-read when the precision changes ----
    v8i qf[G::SST];
    int qsc = 0;
    auto load_q = [&](bool is8) __attribute__((always_inline)) {
        if (is8) {
#pragma unroll
            for (int s = 0; s < G::SST; ++s) {
                // 8-bit operand: registers 0-3 hold 16 bytes of MX block 2s, registers 4-7 of block 2s+1
                const v4i x0 = *reinterpret_cast<const v4i*>(a.q8 + q_row * D + s * 64 + h * 16);
                const v4i x1 = *reinterpret_cast<const v4i*>(a.q8 + q_row * D + s * 64 + h * 16 + 32);
                qf[s] = (v8i){x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
            }
        } else {
#pragma unroll
            for (int s = 0; s < G::SST; ++s) {
                const v4i x = *reinterpret_cast<const v4i*>(a.q4 + q_row * (D / 2) + (2 * s + h) * 16);
                qf[s] = (v8i){x[0], x[1], x[2], x[3], 0, 0, 0, 0};
            }
        }
        const uint8_t* qs = (is8 ? a.qs8 : a.qs4) + q_row * (D / 32);
        const uint32_t sw = (D == 128) ? *reinterpret_cast<const uint32_t*>(qs) : (uint32_t)*reinterpret_cast<const uint16_t*>(qs);
        qsc = (int)(sw >> (8 * h));
    };

    // ---- staging ----
    const int wu = __builtin_amdgcn_readfirstlane(w);    // the wave index, known to be uniform
    // Lane offsets of the staging loads are recomputed where they are used (a handful of integer instructions)
    // from a lane index the compiler cannot see through in the variants that are short of registers: kept there
    // across the loops they get spilled, and a reload in front of a load instruction costs a memory round trip per step.
    auto opaque_lane = [&]() __attribute__((always_inline)) {
        int ln = lane;
        if constexpr (ROUTED || SKIP || MODE == MPSA_MODE_MXFP8) asm volatile("" : "+v"(ln));
        return ln;
    };
    auto issue_k4 = [&](int t, int j) __attribute__((always_inline)) {    // 4-bit K tile j (step t) -> kbuf[t & 1], swizzled rows
        const uint8_t* src = a.k4 + (khead_row + (int64_t)j * TILE) * G::ROW4;
        uint8_t* dst = kbuf0 + (t & 1) * G::K_BYTES;
        const int ln = opaque_lane();
#pragma unroll
        for (int c = 0; c < G::KI4; ++c) {
            const int p = (wu * G::KI4 + c) * 64 + ln;
            const int row = p / G::CPR4, slot = p % G::CPR4;
            const int cb = slot ^ ((row >> G::SH4) & (G::CPR4 - 1));
            load16_to_lds_sv((uint32_t)(row * G::ROW4 + cb * 16), src, dst + (wu * G::KI4 + c) * 1024);
        }
    };
    auto issue_k8 = [&](int j) __attribute__((always_inline)) {           // 8-bit K tile j -> the K area (one buffer), swizzled rows
        const uint8_t* src = a.k8 + (khead_row + (int64_t)j * TILE) * G::ROW8;
        const int ln = opaque_lane();
#pragma unroll
        for (int c = 0; c < (PRE8 ? G::KI8 : 0); ++c) {
            const int p = (wu * G::KI8 + c) * 64 + ln;
            const int row = p / G::CPR8, slot = p % G::CPR8;
            const int cb = slot ^ ((row >> G::SH8) & (G::CPR8 - 1));
            load16_to_lds_sv((uint32_t)(row * G::ROW8 + cb * 16), src, kbuf0 + (wu * G::KI8 + c) * 1024);
        }
    };
    auto issue_v = [&](int t, int j) __attribute__((always_inline)) {     // V tile j (step t) -> vbuf[t & 1], flat
        const uint8_t* src = static_cast<const uint8_t*>(a.v) + (khead_row + (int64_t)j * TILE) * (D * 2);
        uint8_t* dst = vbuf0 + (t & 1) * G::V_BYTES;
        const uint32_t lo = (uint32_t)opaque_lane() * 16u;
#pragma unroll
        for (int c = 0; c < G::VI; ++c) {
            const int ci = wu * G::VI + c;
            load16_to_lds_sv(lo, src + ci * 1024, dst + ci * 1024);
        }
    };
    // K operand of the coming step, in registers: 4-bit fragments come from LDS, 8-bit ones straight from global
    v4i kf4[HAS4 ? G::KB : 1][G::SST];
    v8i kf8[PRE8 ? G::KB : 1][G::SST];
    int ksc[G::KB];             // E8M0 bytes of this lane's key rows, shifted so bytes 0 / 2 belong to MX block h / 2+h
    auto load_kscales = [&](int j, bool is8) __attribute__((always_inline)) {
        const uint8_t* sp = (is8 ? a.ks8 : a.ks4) + (khead_row + (int64_t)j * TILE + r) * (D / 32);
#pragma unroll
        for (int kb = 0; kb < G::KB; ++kb) {
            const uint32_t sw = (D == 128) ? *reinterpret_cast<const uint32_t*>(sp + kb * 32 * (D / 32))
                                           : (uint32_t)*reinterpret_cast<const uint16_t*>(sp + kb * 32 * (D / 32));
            ksc[kb] = (int)(sw >> (8 * h));
        }
    };
    auto read_kf4 = [&](int t) __attribute__((always_inline)) {
        const uint8_t* kl = kbuf0 + (t & 1) * G::K_BYTES;
#pragma unroll
        for (int kb = 0; kb < G::KB; ++kb) {
            const int krow = 32 * kb + r;
            const int f = (krow >> G::SH4) & (G::CPR4 - 1);
#pragma unroll
            for (int s = 0; s < G::SST; ++s)
                kf4[kb][s] = *reinterpret_cast<const v4i*>(kl + krow * G::ROW4 + (((2 * s + h) ^ f) * 16));
        }
    };
    auto read_kf8 = [&]() __attribute__((always_inline)) {                // the staged 8-bit K tile -> fragments
#pragma unroll
        for (int kb = 0; kb < (PRE8 ? G::KB : 0); ++kb) {
            const int krow = 32 * kb + r;
            const int f = (krow >> G::SH8) & (G::CPR8 - 1);
#pragma unroll
            for (int s = 0; s < G::SST; ++s) {
                // 8-bit operand: registers 0-3 hold 16 bytes of MX block 2s, registers 4-7 of block 2s+1
                const v4i x0 = *reinterpret_cast<const v4i*>(kbuf0 + krow * G::ROW8 + (((4 * s + h) ^ f) * 16));
                const v4i x1 = *reinterpret_cast<const v4i*>(kbuf0 + krow * G::ROW8 + (((4 * s + h + 2) ^ f) * 16));
                kf8[kb][s] = (v8i){x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
            }
        }
    };
    // barrier B of an 8-bit step (and of the switch to 8-bit tiles): every wave has the staged tile's fragments in
    // registers, so the one buffer may take the next tile
    auto k8_handover = [&](bool more, int j_next) __attribute__((always_inline)) {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0xC07F);            // lgkmcnt(0): the fragment reads have arrived
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        if (more) issue_k8(j_next);
    };

    v16f acc[G::NDB];
#pragma unroll
    for (int d = 0; d < G::NDB; ++d)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[d][e] = 0.0f;
    // Running reference maximum of this lane's query, kept LAZILY: it moves only when a tile's maximum exceeds
    // it by more than REBASE (so P stays below 2^REBASE, far inside the range of P's 16-bit type and of the float32
    // accumulators), and -m_run rides into the score MFMA as its C operand,
    // which makes the matrix core deliver S - m_run: the softmax costs no subtract and (almost) no rescale.
    constexpr float REBASE = P::REBASE;
    float m_run = 0.0f;
    float l_run = 0.0f;
    v16f negm;
#pragma unroll
    for (int e = 0; e < 16; ++e) negm[e] = 0.0f;

    // ---- prologue: V(0), K(0), K(1) on their way; operands of step 0 into registers ----
    const bool first8 = step_is8(0);
    issue_v(0, tile_rel(0, R0{}));
    if constexpr (HAS4) {
        if (n_k4 > 0) issue_k4(0, tile_rel(0, R0{}));
        if (n_k4 > 1) issue_k4(1, tile_rel(0, R1{}));
    }
    if constexpr (PRE8) {
        if (!ROUTED || first8) issue_k8(tile_rel(0, R0{}));
    }
    load_kscales(tile_rel(0, R0{}), first8);
    load_q(first8 || MIXED);
    __builtin_amdgcn_s_waitcnt(0x0F70);                // vmcnt(0)
    __syncthreads();
    if constexpr (HAS4) read_kf4(0);
    if constexpr (PRE8) {
        if (!ROUTED || first8) {
            read_kf8();
            k8_handover(nsteps > 1, tile_rel(0, R1{}));
        }
    }

    // SKIP in a non-causal diag run: the rule's reference tile, key tile 0, is query tile 0's diagonal tile, which
    // the walk visits last.  That one workgroup takes the tile's statistic (8-bit scores, no softmax, no P.V) first.
    if constexpr (SKIP && MODE == MPSA_MODE_DIAG) {
        if (!a.causal && i == 0 && nsteps > 1) {
            load_kscales(0, true);
            load_q(true);
            float mx = -__builtin_inff();
#pragma unroll
            for (int kb = 0; kb < G::KB; ++kb) {
                const uint8_t* src = a.k8 + (khead_row + 32 * kb + r) * G::ROW8 + h * 16;
                v16f sk;
#pragma unroll
                for (int e = 0; e < 16; ++e) sk[e] = 0.0f;
#pragma unroll
                for (int s = 0; s < G::SST; ++s) {
                    const v4i x0 = *reinterpret_cast<const v4i*>(src + s * 64);
                    const v4i x1 = *reinterpret_cast<const v4i*>(src + s * 64 + 32);
                    const v8i kd = (v8i){x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
                    sk = score_mfma8<FMT8>(kd, qf[s], sk, s, ksc[kb], qsc);
                }
#pragma unroll
                for (int e = 0; e < 16; ++e) mx = __builtin_fmaxf(mx, sk[e]);     // more than one key tile: tile 0 is full
            }
            mx = max_lane_pair(mx);
            float sv = (q_local < a.nq) ? mx : 0.0f;
#pragma unroll
            for (int o = 1; o < 32; o <<= 1) sv += __shfl_xor(sv, o);
            float* sl = stat_lds + G::NW;                  // the slot of odd steps: step 1 writes it after step 0's barrier
            if (lane == 0) sl[w] = sv;
            __syncthreads();
            float tot = 0.0f;
#pragma unroll
            for (int x = 0; x < G::NW; ++x) tot += sl[x];
            sink_stat = tot / (float)min(TILE, a.nq);
            sink_preset = true;
            load_kscales(tile_rel(0, R0{}), false);        // back to the operands of step 0
            load_q(false);
        }
    }

    // One step = one key tile.  IS8 / MASKED are compile-time so the common step (4-bit, unmasked) carries no
    // branches or mask arithmetic.
    //   PREP: also pull the next step's K operand (same precision as the run's plain tiles) into registers.
    auto step = [&](int t, auto is8_c, auto masked_c, auto prep_c) __attribute__((always_inline)) {
        constexpr bool IS8 = decltype(is8_c)::value;
        constexpr bool MASKED = decltype(masked_c)::value;
        constexpr bool PREP = decltype(prep_c)::value;
        const int j = tile_rel(t, R0{});                   // key tile of this step
        int jq3 = 0;

        // ---- S^T - m_run = K Q^T + (-m_run) ----
        v16f st[G::KB];
#pragma unroll
        for (int kb = 0; kb < G::KB; ++kb) {
            if constexpr (IS8 && PRE8) {
                st[kb] = score_mfma8<FMT8>(kf8[kb][0], qf[0], negm, 0, ksc[kb], qsc);
#pragma unroll
                for (int s = 1; s < G::SST; ++s) st[kb] = score_mfma8<FMT8>(kf8[kb][s], qf[s], st[kb], s, ksc[kb], qsc);
            } else if constexpr (IS8) {
                // "diag" run: the single 8-bit tile's fragments come straight from global memory, block by block
                const uint8_t* src = a.k8 + (khead_row + (int64_t)j * TILE + 32 * kb + r) * G::ROW8 + h * 16;
#pragma unroll
                for (int s = 0; s < G::SST; ++s) {
                    const v4i x0 = *reinterpret_cast<const v4i*>(src + s * 64);
                    const v4i x1 = *reinterpret_cast<const v4i*>(src + s * 64 + 32);
                    const v8i kd = (v8i){x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
                    st[kb] = score_mfma8<FMT8>(kd, qf[s], s == 0 ? negm : st[kb], s, ksc[kb], qsc);
                }
            } else {
#pragma unroll
                for (int s = 0; s < G::SST; ++s) {
                    const v4i x = kf4[kb][s];
                    const v8i k8v = (v8i){x[0], x[1], x[2], x[3], 0, 0, 0, 0};
                    if constexpr (MIXED) st[kb] = score_mfma48<FMT8>(k8v, qf[s], s == 0 ? negm : st[kb], s, ksc[kb], qsc);
                    else                 st[kb] = score_mfma4(k8v, qf[s], s == 0 ? negm : st[kb], s, ksc[kb], qsc);
                }
            }
        }

        // routed: fetch the list entry of step t + 3 while the matrix cores work on the scores (the operand reads
        // from LDS are complete at this point, so the scalar load's wait holds up nothing else)
        if constexpr (ROUTED) {
            if (t + 3 < nsteps) jq3 = min(max(scalar_load(ord + t + 3), 0), a.nt - 1);
        }

        // ---- masks: causal on the diagonal tile, key tail on the last tile ----
        if constexpr (MASKED) {
            const bool diag_mask = a.causal && j == i;
            const int kmax = (j == a.nt - 1) ? a.n - j * TILE : TILE;   // keys >= kmax are padding
#pragma unroll
            for (int kb = 0; kb < G::KB; ++kb)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int key = 32 * kb + 8 * (e >> 2) + 4 * h + (e & 3);
                    const bool dead = (diag_mask && key > q_local) || key >= kmax;
                    if (dead) st[kb][e] = -__builtin_inff();
                }
        }

        // ---- online softmax (per lane = per query): st holds S - m_run ----
        float mx = st[0][0];
#pragma unroll
        for (int kb = 0; kb < G::KB; ++kb)
#pragma unroll
            for (int e = 0; e < 16; ++e) mx = __builtin_fmaxf(mx, st[kb][e]);
        mx = max_lane_pair(mx);
        bool keep = true;
        if constexpr (SKIP) {
            // row maximum of S itself (st holds S - m_run), summed over the wave's valid queries, then over the waves
            float sv = (i * TILE + q_local < a.nq) ? mx + m_run : 0.0f;
#pragma unroll
            for (int o = 1; o < 32; o <<= 1) sv += __shfl_xor(sv, o);
            float* sl = stat_lds + (t & 1) * G::NW;
            if (lane == 0) sl[w] = sv;
            __syncthreads();
            float tot = 0.0f;
#pragma unroll
            for (int x = 0; x < G::NW; ++x) tot += sl[x];
            const float stat = tot / (float)min(TILE, a.nq - i * TILE);
            // the diagonal tile of a causal run is exempt like the sink: the reference walks it in a stage of its
            // own, whose first tile is always kept (ours/online_routing.py:68-77, :87-112)
            if (t == 0 && !sink_preset) sink_stat = stat;
            else keep = j == 0 || (a.causal && j == i) || stat >= sink_stat * a.skip_thresh;
            if (!keep) ++n_skipped;
        }
        // the first tile that counts sets the running maximum (with a sink taken ahead, step 0 may be skipped)
        const bool first = SKIP ? !started : (t == 0);
        v4i pk[G::KB][2];                               // 8 packed 16-bit values = one P^T operand
        if (keep) {
        if constexpr (SKIP) started = true;
        if (first || __any(mx > REBASE)) {
            // move the reference maximum up to this tile's maximum (first tile: set it)
            const float delta = first ? mx : __builtin_fmaxf(mx, 0.0f);
            const float alpha = first ? 1.0f : __builtin_amdgcn_exp2f(-delta);
            m_run += delta;
#pragma unroll
            for (int e = 0; e < 16; ++e) negm[e] = -m_run;
#pragma unroll
            for (int kb = 0; kb < G::KB; ++kb)
#pragma unroll
                for (int e = 0; e < 16; ++e) st[kb][e] -= delta;
            l_run *= alpha;
#pragma unroll
            for (int d = 0; d < G::NDB; ++d)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[d][e] *= alpha;
        }
        // P = exp2(S - m_run), rounded to 16 bits for the P.V product; the row sum adds those 16-bit values
        float ps0 = 0.0f, ps1 = 0.0f;
#pragma unroll
        for (int kb = 0; kb < G::KB; ++kb)
#pragma unroll
            for (int c = 0; c < 2; ++c)
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    const float p0 = __builtin_amdgcn_exp2f(st[kb][8 * c + e]);
                    const float p1 = __builtin_amdgcn_exp2f(st[kb][8 * c + e + 1]);
                    const typename P::v2 pp = P::pack(p0, p1);
                    pk[kb][c][e >> 1] = __builtin_bit_cast(int, pp);
                    // float32 additions (ours/mxfp_attn_kernel.py:324-327 sums P before the down-cast); the
                    // dot-product instructions share the matrix pipe and stall the other waves' matrix work
                    ps0 += p0;
                    ps1 += p1;
                }
        l_run += ps0 + ps1;
        }

        // this wave's pieces of V(t) and K(t+1) have landed; after the barrier everybody's have, and everybody
        // is done reading V(t-1) and the K(t) fragments
        __builtin_amdgcn_sched_barrier(0);             // keep the softmax above and the loads below: register lifetimes
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);

        if (t + 1 < nsteps) issue_v(t + 1, tile_rel(t, R1{}));
        if constexpr (HAS4) {
            if (t + 2 < n_k4) issue_k4(t + 2, tile_rel(t, R2{}));
        }

        // 8-bit steps: the K8(t+1) fragments, published by this step's barrier, go into registers first (before the
        // V fragments are fetched, so that the two sets are not in flight together); then barrier B and K8(t+2)
        if constexpr (PREP && PRE8) {
            if constexpr (IS8) {
                read_kf8();
                k8_handover(t + 2 < nsteps, tile_rel(t, R2{}));
            }
        }

        // ---- O^T += V^T P^T, V fragments prefetched PRE instructions ahead ----
        constexpr int PRE = 8;
        const uint8_t* vl = vbuf0 + (t & 1) * G::V_BYTES + opaque_lane() * 16;
        typename P::vec vf[PRE];
        if (keep) {
#pragma unroll
            for (int x = 0; x < PRE; ++x) vf[x] = *reinterpret_cast<const typename P::vec*>(vl + x * 1024);
        }
        // operands of the next step: scales (and 8-bit K) from global memory, 4-bit K from LDS.  Past the last
        // step this reads a valid but unused tile.
        if constexpr (PREP) {
            load_kscales(tile_rel(t, R1{}), IS8);
            if constexpr (HAS4) {
                if constexpr (!IS8) read_kf4(t + 1);
            }
        }
        if (keep) {
#pragma unroll
            for (int idx = 0; idx < G::NV; ++idx) {
                const int d = idx % G::NDB, kc = idx / G::NDB;
                const typename P::vec cur = vf[idx % PRE];
                if (idx + PRE < G::NV) vf[idx % PRE] = *reinterpret_cast<const typename P::vec*>(vl + (idx + PRE) * 1024);
                acc[d] = P::mfma(cur, __builtin_bit_cast(typename P::vec, pk[kc >> 1][kc & 1]), acc[d]);
            }
        }
        if constexpr (ROUTED) {
            jq0 = jq1; jq1 = jq2; jq2 = jq3;
        }
    };

    // ---- plain tiles: one tight single-variant loop ----
    if constexpr (!ROUTED) {
        for (int t = 0; t < n_plain; ++t) step(t, std::integral_constant<bool, PRE8>{}, std::false_type{}, std::true_type{});
    }
    // ---- the (at most two) special tiles: the sequence-tail tile, then the diagonal tile; both run the masked
    //      variant (a mask that hides nothing is harmless).  The step before has already fetched their K operand
    //      unless the precision changes. ----
    if constexpr (ROUTED) {
        // (the first loop above is empty: n_plain is not used by routed runs)
        for (int t = 0; t < r4p; ++t) step(t, std::false_type{}, std::false_type{}, std::true_type{});
        for (int t = r4p; t < r4; ++t) step(t, std::false_type{}, std::true_type{}, std::true_type{});
        if (r4 > 0 && r4 < nsteps) {                   // otherwise the prologue already loaded the 8-bit operands
            // the 4-bit buffers become the 8-bit tile's single buffer: nothing that matters is read from them any
            // more (a slower wave may still fetch fragments of a 4-bit step that does not exist)
            issue_k8(jq0);
            load_kscales(jq0, true);
            load_q(true);
            __builtin_amdgcn_s_waitcnt(0x0F70);
            __syncthreads();
            read_kf8();
            k8_handover(r4 + 1 < nsteps, jq1);
        }
        for (int t = r4; t < r8p; ++t) step(t, std::true_type{}, std::false_type{}, std::true_type{});
        for (int t = r8p; t < nsteps; ++t) step(t, std::true_type{}, std::true_type{}, std::true_type{});
    } else if constexpr (MODE == MPSA_MODE_DIAG) {
        if (tail_special) step(n_plain, std::false_type{}, std::true_type{}, std::true_type{});
        if (nsteps > 1) {                              // otherwise the prologue already loaded 8-bit Q and scales
            load_kscales(tile_at(nsteps - 1), true);
            load_q(true);
        }
        step(nsteps - 1, std::true_type{}, std::true_type{}, std::false_type{});
    } else {
        for (int t = n_plain; t < nsteps; ++t) step(t, std::integral_constant<bool, PRE8>{}, std::true_type{}, std::true_type{});
    }
    (void)r4p; (void)r8p;
    __builtin_amdgcn_s_waitcnt(0x0F70);                // no direct-to-LDS load may outlive the workgroup

    if constexpr (SKIP) {
        if (a.skipped && tid == 0) a.skipped[((int64_t)b * a.Hq + hq) * a.ntq + i] = n_skipped;
    }
    // ---- epilogue: O = acc / l ; register e of lane (h, r): dim 32*db + 8*(e/4) + 4*h + e%4 of query r ----
    const float l_tot = sum_lane_pair(l_run);
    const float inv = (ROUTED && !(l_tot > 0.0f)) ? 0.0f : 1.0f / l_tot;   // routed: a row with every tile skipped gives zeros
    const int q_global = i * TILE + q_local;
    uint8_t* orow = static_cast<uint8_t*>(a.o);
    const int64_t off = (int64_t)b * a.o_sb + (int64_t)hq * a.o_sh + (int64_t)q_global * a.o_sn;
    if (a.o_dtype != MPSA_F32 && ((a.o_sn | a.o_sh | a.o_sb) & 7) == 0 && (reinterpret_cast<uintptr_t>(a.o) & 15) == 0) {
        // 16-bit output: the two lanes of a query trade register groups (lane half 0 hands over dims 8..11 of every
        // 16 and receives dims 4..7), so that each lane owns 8 consecutive dims and stores 16 bytes at a time.
        // Every lane takes part in the exchange; only queries inside the sequence are stored.
#pragma unroll
        for (int d = 0; d < G::NDB; ++d)
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                int x[2], y[2];                           // packed dims 16u+4h .. +3 (x) and 16u+8+4h .. +3 (y)
#pragma unroll
                for (int c = 0; c < 2; ++c) {
                    const float x0 = acc[d][8 * u + 2 * c] * inv, x1 = acc[d][8 * u + 2 * c + 1] * inv;
                    const float y0 = acc[d][8 * u + 4 + 2 * c] * inv, y1 = acc[d][8 * u + 4 + 2 * c + 1] * inv;
                    if (a.o_dtype == MPSA_BF16) {
                        typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
                        x[c] = __builtin_bit_cast(int, (v2bf){(__bf16)x0, (__bf16)x1});
                        y[c] = __builtin_bit_cast(int, (v2bf){(__bf16)y0, (__bf16)y1});
                    } else {
                        typedef _Float16 v2hh __attribute__((ext_vector_type(2)));
                        x[c] = __builtin_bit_cast(int, (v2hh){(_Float16)x0, (_Float16)x1});
                        y[c] = __builtin_bit_cast(int, (v2hh){(_Float16)y0, (_Float16)y1});
                    }
                    // swap x of lanes 32-63 with y of lanes 0-31: half 0 ends with dims 16u .. 16u+7 in (x, y),
                    // half 1 with dims 16u+8 .. 16u+15
                    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(x[c]), "+v"(y[c]));
                }
                const int dim = 32 * d + 16 * u + 8 * h;
                const v4i pk8 = {x[0], x[1], y[0], y[1]};
                if (q_global < a.nq) *reinterpret_cast<v4i*>(orow + (off + dim) * 2) = pk8;
            }
    } else if (q_global < a.nq) {
#pragma unroll
        for (int d = 0; d < G::NDB; ++d)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const int dim = 32 * d + 8 * g4 + 4 * h;
                const float o0 = acc[d][4 * g4 + 0] * inv, o1 = acc[d][4 * g4 + 1] * inv;
                const float o2 = acc[d][4 * g4 + 2] * inv, o3 = acc[d][4 * g4 + 3] * inv;
                if (a.o_dtype == MPSA_BF16) {
                    typedef __bf16 v4bf __attribute__((ext_vector_type(4)));
                    const v4bf pk4 = {(__bf16)o0, (__bf16)o1, (__bf16)o2, (__bf16)o3};
                    *reinterpret_cast<v4bf*>(orow + (off + dim) * 2) = pk4;
                } else if (a.o_dtype == MPSA_F16) {
                    typedef _Float16 v4hh __attribute__((ext_vector_type(4)));
                    const v4hh pk4 = {(_Float16)o0, (_Float16)o1, (_Float16)o2, (_Float16)o3};
                    *reinterpret_cast<v4hh*>(orow + (off + dim) * 2) = pk4;
                } else {
                    const v4f pk4 = {o0, o1, o2, o3};
                    *reinterpret_cast<v4f*>(orow + (off + dim) * 4) = pk4;
                }
            }
    }
}

template <int D, int TILE, int PVT, int FMT8, int MODE, bool SKIP>
struct AttnLds {
    static constexpr int smem = Geom<D, TILE>::SMEM + (SKIP ? 2 * Geom<D, TILE>::NW * (int)sizeof(float) : 0);
    static inline const bool registered =
        mpsa_register_lds_kernel(reinterpret_cast<const void*>(attn_fwd_kernel<D, TILE, PVT, FMT8, MODE, SKIP>), smem);
};

template <int D, int TILE, int PVT, int FMT8, int MODE, bool SKIP = false>
int launch_one(const AttnArgs& a, hipStream_t st) {
    typedef Geom<D, TILE> G;
    typedef AttnLds<D, TILE, PVT, FMT8, MODE, SKIP> L;
    if (!L::registered) return mpsa_fail(MPSA_ELAUNCH, "attn: kernel not registered");
    const int rc = mpsa_ensure_init();
    if (rc != MPSA_OK) return rc;
    dim3 grid((unsigned)(a.B * a.Hq * a.ntq));
    hipLaunchKernelGGL((attn_fwd_kernel<D, TILE, PVT, FMT8, MODE, SKIP>), grid, dim3(G::NT), L::smem, st, a);
    MPSA_CHECK_LAUNCH("attn");
    return MPSA_OK;
}

}  // namespace
