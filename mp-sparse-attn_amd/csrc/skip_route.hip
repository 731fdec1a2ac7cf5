// Tile skipping ahead of the attention kernel (gfx950): the reference's rule (ours/mxfp_attn_kernel.py:272-297, with the
// causal stage structure of ours/online_routing.py:68-77) decides from a statistic of every score tile -- the mean over
// the tile's query rows of the row maximum of S -- whether the tile is kept: key tile 0 is always kept and sets the
// reference value, tile j > 0 is kept iff stat(j) >= stat(0) * skip_thresh, the diagonal tile of a causal run is kept.
//
// Inside the attention kernel the rule costs a workgroup-wide exchange between a tile's scores and its softmax in every
// step (mpsa_attn_fwd_skip: attn_fwd_kernel.h), and a skipped tile still pays for staging, barriers and that exchange.
// Here the statistic of ALL tiles of a query tile is taken first, by a kernel that does nothing but the score products
// (a fifth of attention's matrix work, no exponentials, no P.V), one workgroup barrier per key tile; a second, small
// kernel applies the rule and compacts the kept tiles into the visiting lists of mpsa_attn_fwd_routed, which then walks
// the kept tiles only.  D = 128, 128-key tiles; modes mxfp4, mxfp8 and diag.
#include <type_traits>
#include "attn_common.h"

namespace {

constexpr int D = 128, TILE = 128;
constexpr int KB = TILE / 32, SST = D / 64;
constexpr int ROW4 = D / 2, ROW8 = D;
constexpr int CPR4 = ROW4 / 16, CPR8 = ROW8 / 16;
constexpr int K4_BYTES = TILE * ROW4, K8_BYTES = TILE * ROW8;
constexpr int NK = 3;                      // K tiles in LDS: the one being multiplied and two on their way (a deeper ring was no faster:
                                           // its LDS costs resident workgroups, which hide more latency than it does)
// s_waitcnt immediate: at most v vector-memory operations outstanding, the other counters unconstrained
constexpr int vm_imm(int v) { return (v & 15) | ((v >> 4) << 14) | 0x0F70; }
constexpr int NW = 4;
enum : uint8_t { CLS_SKIP = 0, CLS_FP4 = 1, CLS_FP8 = 2, CLS_NOT_VISITED = 255 };

template <int CTRL>
__device__ __forceinline__ float lane_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}

__device__ __forceinline__ float max3f(float a, float b, float c) { return __builtin_fmaxf(__builtin_fmaxf(a, b), c); }
__device__ __forceinline__ float tree_max16(const v16f& v) {
    const float m0 = max3f(v[0], v[1], v[2]), m1 = max3f(v[3], v[4], v[5]), m2 = max3f(v[6], v[7], v[8]);
    const float m3 = max3f(v[9], v[10], v[11]), m4 = max3f(v[12], v[13], v[14]);
    return __builtin_fmaxf(max3f(m0, m1, m2), max3f(m3, m4, v[15]));
}

struct StatArgs {
    const uint8_t *q4, *qs4, *q8, *qs8, *k4, *ks4, *k8, *ks8;
    float* stats;                          // [B,Hq,ntq,nt]
    int B, Hq, Hkv, n, n_pad, nt, nq, nq_pad, ntq, causal;
};

constexpr int KS_BYTES = TILE * (D / 32);  // a K tile's scale bytes travel with it
constexpr int QT = 2;                      // query tiles per workgroup: they share the staged K tiles
constexpr int stat_lds_bytes(int mode, int nt) { return NK * ((mode == MPSA_MODE_MXFP8 ? K8_BYTES : K4_BYTES) + KS_BYTES) + QT * nt * NW * 4 + NW * 64 * 4; }

// One workgroup of four waves per (batch, query head, pair of query tiles 2P, 2P+1); wave w owns queries 32w .. 32w+31 of
// both tiles, a lane pair one query of each (the score instruction's layout, see attn_fwd_kernel.h).  Key tiles in
// ascending order; K tiles travel through a ring of LDS buffers as in the attention kernels (4-bit tiles, or 8-bit ones in
// the mxfp8 mode; the one 8-bit tile of a diag run's query tile -- the diagonal one -- is read straight from global
// memory) and are multiplied with both query tiles.  A tile's scale bytes ride along into LDS: the loop then holds no
// global load the compiler counts, so that its waits never fall on the tiles in flight.
// What bounds it (C5, 8 heads: 1.05 M wave-steps, measured): a wave issues in order and a SIMD holds two of them (the two
// tiles of scores take half the registers), so a step costs what the wave's own instruction stream costs -- the matrix
// pipe was busy 41 % of the cycles and the vector unit 50 % when the step did one thing after the other, and the two
// workgroups of a CU did not fill each other's gaps.  Hence, in the steps that need no mask (nearly all): one query
// tile's row maxima sit between the other tile's score instructions, both tiles' sums are taken by one chain of lane
// moves, the fetch pointers and ring slots are running values and the wait for a tile is a constant.  That is 150
// instructions per wave and step instead of 220, 31 % fewer cycles (matrix pipe busy 60 % of them) and 20 % less time;
// most of what is left over the 0.23 ms of the matrix instructions is clock, which falls as the matrix work gets denser: with every operand element the same the pass takes 0.39 ms, with random ones 0.50 (the
// matrix instructions' power draw, as in the attention kernel).
template <int FMT8, int MODE>
__global__ __launch_bounds__(256, 2) void skip_stats_kernel(StatArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    constexpr bool ALL8 = MODE == MPSA_MODE_MXFP8;
    constexpr bool HAS4 = !ALL8;
    constexpr int KT_BYTES = ALL8 ? K8_BYTES : K4_BYTES;
    constexpr int PIECES = KT_BYTES / 1024 / NW;          // direct-to-LDS instructions per wave and tile (plus one for the scales)
    constexpr int SLOT = KT_BYTES + KS_BYTES;
    constexpr int G = PIECES + 1;                         // loads per wave and tile

    const int tid = threadIdx.x;
    const int lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = lane >> 5, r = lane & 31;
    // heavy pairs first (causal runs)
    const int npairs = (a.ntq + 1) >> 1;
    // consecutive workgroup ids go to different XCDs: give each XCD a contiguous eighth of the (head-major) list, so that a
    // head's K tiles stay in one L2
    const int64_t total = (int64_t)gridDim.x;
    int64_t row_id = blockIdx.x;
    if ((total & 7) == 0) row_id = (row_id & 7) * (total >> 3) + (row_id >> 3);
    const int rank = (int)(row_id % npairs);
    const int pair = a.causal ? npairs - 1 - rank : rank;
    const int64_t bh = row_id / npairs;
    const int hq = (int)(bh % a.Hq);
    const int b = (int)(bh / a.Hq);
    const int kvh = hq / (a.Hq / a.Hkv);
    const int i_hi = min(2 * pair + 1, a.ntq - 1);                         // the pair's last query tile
    const int nsteps = a.causal ? min(i_hi, a.nt - 1) + 1 : a.nt;
    const int64_t khead_row = ((int64_t)b * a.Hkv + kvh) * a.n_pad;
    const int q_local = 32 * w + r;
    float* part = reinterpret_cast<float*>(smem + NK * SLOT);              // [QT][nt][NW]
    float* spare = part + QT * a.nt * NW;                                  // [NW][64]

    // Q fragments of both query tiles, in the widths the mode multiplies
    v8i qf4[QT][SST], qf8[QT][SST];
    int qsc4[QT] = {0, 0}, qsc8[QT] = {0, 0};
#pragma unroll
    for (int x = 0; x < QT; ++x) {
        const int i = 2 * pair + x;
        if (i >= a.ntq) continue;                                          // an odd tile count: the last pair has one tile
        const int64_t q_row = ((int64_t)b * a.Hq + hq) * a.nq_pad + (int64_t)i * TILE + q_local;
        if constexpr (HAS4) {
#pragma unroll
            for (int s = 0; s < SST; ++s) {
                const v4i v = *reinterpret_cast<const v4i*>(a.q4 + q_row * ROW4 + (2 * s + h) * 16);
                qf4[x][s] = (v8i){v[0], v[1], v[2], v[3], 0, 0, 0, 0};
            }
            qsc4[x] = (int)(*reinterpret_cast<const uint32_t*>(a.qs4 + q_row * (D / 32)) >> (8 * h));
        }
        if constexpr (MODE != MPSA_MODE_MXFP4) {
#pragma unroll
            for (int s = 0; s < SST; ++s) {
                const v4i x0 = *reinterpret_cast<const v4i*>(a.q8 + q_row * ROW8 + s * 64 + h * 16);
                const v4i x1 = *reinterpret_cast<const v4i*>(a.q8 + q_row * ROW8 + s * 64 + h * 16 + 32);
                qf8[x][s] = (v8i){x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
            }
            qsc8[x] = (int)(*reinterpret_cast<const uint32_t*>(a.qs8 + q_row * (D / 32)) >> (8 * h));
        }
    }

    // this lane's offsets into a K tile for the wave's pieces (rows XOR-swizzled, as in attn_fwd_pp.hip)
    uint32_t koff[PIECES];
#pragma unroll
    for (int c = 0; c < PIECES; ++c) {
        const int p = (w * PIECES + c) * 64 + lane;
        if constexpr (ALL8) {
            const int row = p / CPR8, slot = p % CPR8;
            koff[c] = (uint32_t)(row * ROW8 + (slot ^ ((row >> 1) & (CPR8 - 1))) * 16);
        } else {
            const int row = p / CPR4, slot = p % CPR4;
            koff[c] = (uint32_t)(row * ROW4 + (slot ^ ((row >> 2) & (CPR4 - 1))) * 16);
        }
    }
    // The next K tile to fetch and the ring slot it goes to, kept as running values (a pointer and an offset that move by one
    // tile) rather than worked out from the step number at every step.  Past the last tile the last one is fetched again, into
    // a slot nobody reads any more: every step then finds the same number of loads in flight, and its wait is a constant.
    const uint8_t* ksrc = ALL8 ? a.k8 + khead_row * ROW8 : a.k4 + khead_row * ROW4;
    const uint8_t* ssrc = (ALL8 ? a.ks8 : a.ks4) + khead_row * (D / 32) + w * (KS_BYTES / NW);
    uint32_t islot = 0, rslot = 0;
    int issued = 0;
    auto issue_next = [&]() __attribute__((always_inline)) {
        uint8_t* slot = smem + islot;
#pragma unroll
        for (int c = 0; c < PIECES; ++c) load16_to_lds_sv(koff[c], ksrc, slot + (w * PIECES + c) * 1024);
        // the tile's 512 scale bytes, a quarter per wave (eight lanes of 16 bytes)
        if (lane < KS_BYTES / NW / 16) load16_to_lds_sv((uint32_t)lane * 16u, ssrc, slot + KT_BYTES + w * (KS_BYTES / NW));
        ++issued;
        const bool more = issued < nsteps;
        ksrc += more ? KT_BYTES : 0;
        ssrc += more ? KS_BYTES : 0;
        islot = islot == (NK - 1) * SLOT ? 0u : islot + SLOT;
    };

    const int i0 = 2 * pair, i1 = 2 * pair + 1;
    const bool has1 = i1 < a.ntq;
    v4i kf[KB][SST][ALL8 ? 2 : 1];
    int ksc[KB];
    v16f st0[KB], st1[KB];
    // A step begins: its K tile has landed (its loads are older than those of the NK - 2 tiles fetched after it), everybody is
    // past the tile before, whose slot takes the next fetch; then the staged tile's fragments and scales, once for both query tiles
    auto begin_step = [&]() __attribute__((always_inline)) {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(vm_imm((NK - 2) * G));
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        issue_next();
        // one address per step for the fragments of each half of the head dimension and one for the scales: the key blocks are
        // constant offsets from them (the swizzle depends on the row inside a block only), which the opaque values keep
        // in the instructions' offset fields instead of a vector addition per read
        const uint32_t slot = rslot;
        rslot = rslot == (NK - 1) * SLOT ? 0u : rslot + SLOT;
        uint32_t fa[SST], sa = slot + KT_BYTES + r * (D / 32);
        asm volatile("" : "+v"(sa));
#pragma unroll
        for (int s = 0; s < SST; ++s) {
            fa[s] = slot + (ALL8 ? r * ROW8 + (((4 * s + h) ^ ((r >> 1) & (CPR8 - 1))) * 16) : r * ROW4 + (((2 * s + h) ^ ((r >> 2) & (CPR4 - 1))) * 16));
            asm volatile("" : "+v"(fa[s]));
        }
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
            ksc[kb] = (int)(*reinterpret_cast<const uint32_t*>(smem + sa + 32 * kb * (D / 32)) >> (8 * h));
#pragma unroll
            for (int s = 0; s < SST; ++s) {
                if constexpr (ALL8) {
                    // the second half's 16 bytes sit two chunks on: bit 1 of the chunk index, which the swizzle leaves to 4*s+h
                    kf[kb][s][0] = *reinterpret_cast<const v4i*>(smem + fa[s] + 32 * kb * ROW8);
                    kf[kb][s][1] = *reinterpret_cast<const v4i*>(smem + (fa[s] ^ 32u) + 32 * kb * ROW8);
                } else {
                    kf[kb][s][0] = *reinterpret_cast<const v4i*>(smem + fa[s] + 32 * kb * ROW4);
                }
            }
        }
    };
    // the eight score instructions of query tile x on the staged K tile
    auto scores = [&](v16f (&st)[KB], int x) __attribute__((always_inline)) {
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
            for (int e = 0; e < 16; ++e) st[kb][e] = 0.0f;
        // the four key blocks of one half of the head dimension, then of the other: no instruction waits for the one before it
#pragma unroll
        for (int s = 0; s < SST; ++s) {
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                if constexpr (ALL8) {
                    const v4i x0 = kf[kb][s][0], x1 = kf[kb][s][1];
                    const v8i kd = (v8i){x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
                    st[kb] = score_mfma8<FMT8>(kd, qf8[x][s], st[kb], s, ksc[kb], qsc8[x]);
                } else {
                    const v4i v = kf[kb][s][0];
                    const v8i kd = (v8i){v[0], v[1], v[2], v[3], 0, 0, 0, 0};
                    st[kb] = score_mfma4(kd, qf4[x][s], st[kb], s, ksc[kb], qsc4[x]);
                }
            }
        }
    };
    // a diag run's one 8-bit tile of query tile x (key tile j == its own index), operands straight from global memory
    auto scores_diag = [&](v16f (&st)[KB], int x, int j) __attribute__((always_inline)) {
        if constexpr (MODE == MPSA_MODE_DIAG) {
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                const int krow = 32 * kb + r;
                const int ks = (int)(*reinterpret_cast<const uint32_t*>(a.ks8 + (khead_row + (int64_t)j * TILE + krow) * (D / 32)) >> (8 * h));
                const uint8_t* src = a.k8 + (khead_row + (int64_t)j * TILE + krow) * ROW8 + h * 16;
#pragma unroll
                for (int e = 0; e < 16; ++e) st[kb][e] = 0.0f;
#pragma unroll
                for (int s = 0; s < SST; ++s) {
                    const v4i x0 = *reinterpret_cast<const v4i*>(src + s * 64);
                    const v4i x1 = *reinterpret_cast<const v4i*>(src + s * 64 + 32);
                    const v8i kd = (v8i){x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
                    st[kb] = score_mfma8<FMT8>(kd, qf8[x][s], st[kb], s, ks, qsc8[x]);
                }
            }
        }
    };
    // this lane's maximum over its 64 scores of a tile: 26 three-input maxima, which go into the gaps of the other query
    // tile's score instructions in the plain steps
    auto row_max = [&](const v16f (&st)[KB]) __attribute__((always_inline)) {
        float mk[KB];
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) mk[kb] = tree_max16(st[kb]);
        return max3f(mk[0], mk[1], __builtin_fmaxf(mk[2], mk[3]));
    };
    auto interleave = [&](auto per) __attribute__((always_inline)) {
#pragma unroll
        for (int g = 0; g < KB * SST; ++g) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);        // one matrix instruction
            __builtin_amdgcn_sched_group_barrier(0x002, decltype(per)::value, 0);      // some vector instructions
        }
    };
    // this wave's share of the statistic of (query tile x, step t): the row maxima of its valid queries summed in the order
    // the attention kernel adds them (attn_fwd_kernel.h: a butterfly over lanes 0-31; written with lane-permuting moves
    // instead of the LDS shuffles of __shfl_xor, whose five dependent round trips cost more than the score instructions:
    // lanes 1, 2 apart inside a quad, then -- every lane of a group holding the group's sum by then -- the mirrored lane
    // of the 8- and the 16-lane group, then lane 0 + lane 16; float addition commutes, so lane 0 ends with the butterfly's bits)
    auto finish = [&](float rm, int x, int t) __attribute__((always_inline)) {
        const float mx = max_lane_pair(rm);
        float sv = ((2 * pair + x) * TILE + q_local < a.nq) ? mx : 0.0f;
        sv += lane_move<0xB1>(sv);                     // quad_perm [1,0,3,2]
        sv += lane_move<0x4E>(sv);                     // quad_perm [2,3,0,1]
        sv += lane_move<0x141>(sv);                    // row_half_mirror
        sv += lane_move<0x140>(sv);                    // row_mirror
        const float s0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, sv), 0));
        const float s16 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, sv), 16));
        // lane 0 writes the sum; the other lanes write it to a spare word each, because a branch around the store would
        // split the step into basic blocks and the score instructions would be moved out of the vector work they are to hide
        float* dst = lane == 0 ? part + (x * a.nt + t) * NW + w : spare + 64 * w + lane;
        *dst = s0 + s16;
    };
    // A step that needs a mask, an 8-bit tile from global memory, or has one of the two query tiles only: one thing after the other.
    auto slow_step = [&](int t) __attribute__((always_inline)) {
        begin_step();
        const int j = t;
#pragma unroll
        for (int x = 0; x < QT; ++x) {
            const int i = 2 * pair + x;
            if (i >= a.ntq || (a.causal && j > i)) continue;               // no such query tile, or a tile it does not visit
            if (MODE == MPSA_MODE_DIAG && j == i) scores_diag(st0, x, j);
            else scores(st0, x);
            // the masks the attention kernel applies before it takes the statistic: the causal diagonal, the keys past the end
            const bool diag_mask = a.causal && j == i;
            const int kmax = (j == a.nt - 1) ? a.n - j * TILE : TILE;
            if (diag_mask || kmax < TILE) {
                // first dead key of this lane's query; opaque, or the 64 comparisons are taken out of the loop and their
                // results kept in scalar registers across every step
                int limit = diag_mask ? min(q_local + 1, kmax) : kmax;
                asm volatile("" : "+v"(limit));
#pragma unroll
                for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int key = 32 * kb + 8 * (e >> 2) + 4 * h + (e & 3);
                        if (key >= limit) st0[kb][e] = -__builtin_inff();
                    }
            }
            finish(row_max(st0), x, t);
        }
    };
    // The same sums for both query tiles of a plain step at once.  One exchange of the upper and lower 32 lanes of the two
    // tiles' lane maxima and one maximum leave tile 0's row maxima in lanes 0-31 and tile 1's in lanes 32-63; the lane moves
    // above sum each row of 16 lanes; lane 15 of a row broadcast into the next row adds rows 0 + 1 and rows 2 + 3 (the
    // operands of "lane 0 + lane 16", so the same bits).  Lanes 16 and 48 store: 12 vector instructions for two tiles.
    const bool pair_valid = (2 * pair + h) * TILE + q_local < a.nq;
    const uint32_t pair_step = r == 16 ? NW * 4u : 0u;
    const uint32_t pair_dst = (uint32_t)(NK * SLOT) + (r == 16 ? (uint32_t)(h * a.nt * NW + w) * 4u : (uint32_t)(QT * a.nt * NW + 64 * w + lane) * 4u);
    auto finish_pair = [&](float rm0, float rm1, int t) __attribute__((always_inline)) {
        int x0 = __builtin_bit_cast(int, rm0), x1 = __builtin_bit_cast(int, rm1);
        asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(x0), "+v"(x1));
        const float mx = __builtin_fmaxf(__builtin_bit_cast(float, x0), __builtin_bit_cast(float, x1));
        float sv = pair_valid ? mx : 0.0f;
        sv += lane_move<0xB1>(sv);
        sv += lane_move<0x4E>(sv);
        sv += lane_move<0x141>(sv);
        sv += lane_move<0x140>(sv);
        // row_bcast:15 into rows 1 and 3
        sv += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, sv), 0x142, 0xA, 0xF, false));
        *reinterpret_cast<float*>(smem + pair_dst + (uint32_t)t * pair_step) = sv;
    };
    // Plain steps ta .. tb-1 (both query tiles, 4-bit tiles from LDS, no mask).  Vector instructions run under a wave's own
    // matrix instructions but hardly under the other wave's, and a wave issues in order: what counts is the length of the
    // wave's own instruction stream and how much of it sits between its matrix instructions.  Query tile 0's row maxima go
    // into the gaps of tile 1's score instructions, tile 1's and the step's sums into those of tile 0 in the next step.
    auto plain_steps = [&](int ta, int tb) __attribute__((always_inline)) {
        if (ta >= tb) return;
        begin_step();
        scores(st0, 0);
        for (int t = ta;; ++t) {
            scores(st1, 1);
            const float rm0 = row_max(st0);
            interleave(std::integral_constant<int, 4>{});
            if (t + 1 >= tb) {
                finish_pair(rm0, row_max(st1), t);
                break;
            }
            begin_step();
            scores(st0, 0);
            finish_pair(rm0, row_max(st1), t);
            interleave(std::integral_constant<int, 6>{});
        }
    };
    // steps that are not plain, in ascending order: (causal) everything from tile 0's diagonal on; (diag mode) the two diagonal
    // tiles; the ragged last tile; and every step of a pair that has one query tile only.  (The mxfp8 mode's plain steps fit
    // the registers with nothing to spare: twice the K fragments beside the two tiles of scores.)
    auto next_special = [&](int t) __attribute__((always_inline)) {
        if (!has1) return t;
        int e = nsteps;
        if (a.n < a.n_pad) e = a.nt - 1;
        if (a.causal) return max(t, min(e, i0));
        if constexpr (MODE == MPSA_MODE_DIAG) {
            if (t <= i0) e = min(e, i0);
            else if (t <= i1) e = min(e, i1);
        }
        return max(t, e);
    };

#pragma unroll
    for (int t = 0; t < NK - 1; ++t) issue_next();
    for (int t = 0; t < nsteps;) {
        const int te = min(next_special(t), nsteps);
        plain_steps(t, te);
        if (te < nsteps) slow_step(te);
        t = te + 1;
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
#pragma unroll
    for (int x = 0; x < QT; ++x) {
        const int i = 2 * pair + x;
        if (i >= a.ntq) continue;
        const int visited = a.causal ? min(i, a.nt - 1) + 1 : a.nt;
        const float rows = (float)min(TILE, a.nq - i * TILE);
        float* out = a.stats + (((int64_t)b * a.Hq + hq) * a.ntq + i) * a.nt;
        for (int t = tid; t < visited; t += 256) {
            float tot = 0.0f;
#pragma unroll
            for (int y = 0; y < NW; ++y) tot += part[(x * a.nt + t) * NW + y];
            out[t] = tot / rows;
        }
    }
}

template <int FMT8, int MODE>
struct StatLds {
    static inline const bool registered = mpsa_register_lds_kernel(reinterpret_cast<const void*>(skip_stats_kernel<FMT8, MODE>), stat_lds_bytes(MODE, MPSA_SKIP_ROUTE_MAX_TILES));
};

struct ListArgs {
    const float* stats;
    int Hq, ntq, nt, causal, ragged, mode;
    float thresh;
    uint8_t* cls;
    int32_t *order, *counts, *skipped;
};

// One wave per (batch, query head, query tile): the rule, the class of every key tile and the visiting lists in the order
// mpsa_attn_fwd_routed walks them (4-bit plain, 4-bit masked, 8-bit plain, 8-bit masked).
__global__ __launch_bounds__(64) void skip_lists_kernel(ListArgs a) {
    const int64_t row = blockIdx.x;
    const int lane = threadIdx.x;
    const int i = (int)(row % a.ntq);
    const float* st = a.stats + row * a.nt;
    const int last = a.causal ? min(i, a.nt - 1) : a.nt - 1;
    const float cut = st[0] * a.thresh;
    auto classify = [&](int j, int& run) {
        run = -1;
        if (j > last) return (uint8_t)CLS_NOT_VISITED;
        const bool keep = j == 0 || (a.causal && j == i) || st[j] >= cut;
        if (!keep) return (uint8_t)CLS_SKIP;
        const bool is8 = a.mode == MPSA_MODE_MXFP8 || (a.mode == MPSA_MODE_DIAG && j == i);
        const bool masked = (a.causal && j == i) || (a.ragged && j == a.nt - 1);
        run = (is8 ? 2 : 0) + (masked ? 1 : 0);
        return (uint8_t)(is8 ? CLS_FP8 : CLS_FP4);
    };
    int cnt[4] = {0, 0, 0, 0};
    int nskip = 0;
    const int chunks = (a.nt + 63) / 64;
    for (int ch = 0; ch < chunks; ++ch) {
        const int j = ch * 64 + lane;
        int run = -1;
        uint8_t c = CLS_NOT_VISITED;
        if (j < a.nt) {
            c = classify(j, run);
            if (a.cls) a.cls[row * a.nt + j] = c;
        }
        nskip += __popcll(__ballot(c == CLS_SKIP));
#pragma unroll
        for (int k = 0; k < 4; ++k) cnt[k] += __popcll(__ballot(run == k));
    }
    int base[4] = {0, cnt[0], cnt[0] + cnt[1], cnt[0] + cnt[1] + cnt[2]};
    const int total = base[3] + cnt[3];
    if (lane < 4) a.counts[row * 4 + lane] = cnt[lane];
    if (lane == 0 && a.skipped) a.skipped[row] = nskip;
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

template <int FMT8, int MODE>
int launch_stats(const StatArgs& a, unsigned grid, hipStream_t st) {
    if (!StatLds<FMT8, MODE>::registered) return mpsa_fail(MPSA_ELAUNCH, "skip route: kernel not registered");
    hipLaunchKernelGGL((skip_stats_kernel<FMT8, MODE>), dim3(grid), dim3(256), stat_lds_bytes(MODE, a.nt), st, a);
    return MPSA_OK;
}

int64_t ceil_div(int64_t x, int64_t y) { return (x + y - 1) / y; }

}  // namespace

extern "C" int mpsa_skip_route_supported(int64_t nq, int64_t nk, int64_t D, int tile, int causal, int mode) {
    if (D != 128 || tile != 128 || nq <= 0 || nk <= 0) return 0;
    if (mode != MPSA_MODE_MXFP4 && mode != MPSA_MODE_MXFP8 && mode != MPSA_MODE_DIAG) return 0;
    if (nq != nk && (causal || mode == MPSA_MODE_DIAG)) return 0;
    return ceil_div(nk, tile) <= MPSA_SKIP_ROUTE_MAX_TILES ? 1 : 0;
}

extern "C" int64_t mpsa_skip_route_workspace(int64_t B, int64_t Hq, int64_t nq, int64_t nk, int tile) {
    if (B <= 0 || Hq <= 0 || nq <= 0 || nk <= 0 || tile <= 0) return 0;
    return B * Hq * ceil_div(nq, tile) * ceil_div(nk, tile) * (int64_t)sizeof(float);
}

extern "C" int mpsa_skip_route(const uint8_t* q4, const uint8_t* qs4, const uint8_t* q8, const uint8_t* qs8,
                               const uint8_t* k4, const uint8_t* ks4, const uint8_t* k8, const uint8_t* ks8, int fmt8,
                               int64_t B, int64_t Hq, int64_t Hkv, int64_t nq, int64_t nk, int64_t D, int tile, int causal, int mode,
                               float skip_thresh, void* work, uint8_t* cls, int32_t* order, int32_t* counts, int32_t* skipped,
                               mpsa_stream_t stream) {
    if (B <= 0 || Hq <= 0 || Hkv <= 0 || nq <= 0 || nk <= 0 || Hq % Hkv) return mpsa_fail(MPSA_EINVAL, "skip route: bad shape (B=%lld Hq=%lld Hkv=%lld nq=%lld nk=%lld)", (long long)B, (long long)Hq, (long long)Hkv, (long long)nq, (long long)nk);
    if (!mpsa_skip_route_supported(nq, nk, D, tile, causal, mode))
        return mpsa_fail(MPSA_EUNSUPPORTED, "skip route: needs D = 128, tile = 128, mode mxfp4, mxfp8 or diag, at most %d key tiles (and nq == nk for causal or diag runs); use mpsa_attn_fwd_skip", MPSA_SKIP_ROUTE_MAX_TILES);
    if (!(skip_thresh == skip_thresh)) return mpsa_fail(MPSA_EINVAL, "skip route: skip_thresh is NaN");
    const bool need4 = mode != MPSA_MODE_MXFP8, need8 = mode != MPSA_MODE_MXFP4;
    if (need4 && (!q4 || !qs4 || !k4 || !ks4)) return mpsa_fail(MPSA_EINVAL, "skip route: 4-bit operands missing");
    if (need8 && (!q8 || !qs8 || !k8 || !ks8)) return mpsa_fail(MPSA_EINVAL, "skip route: 8-bit operands missing");
    if (need8 && fmt8 != MPSA_FMT_E4M3 && fmt8 != MPSA_FMT_E5M2) return mpsa_fail(MPSA_EINVAL, "skip route: 8-bit format must be E4M3 or E5M2");
    if (!work || !order || !counts) return mpsa_fail(MPSA_EINVAL, "skip route: null pointer");
    const uintptr_t al = reinterpret_cast<uintptr_t>(q4) | reinterpret_cast<uintptr_t>(q8) | reinterpret_cast<uintptr_t>(k4) | reinterpret_cast<uintptr_t>(k8);
    const uintptr_t al4 = reinterpret_cast<uintptr_t>(qs4) | reinterpret_cast<uintptr_t>(qs8) | reinterpret_cast<uintptr_t>(ks4) | reinterpret_cast<uintptr_t>(ks8) |
                          reinterpret_cast<uintptr_t>(work) | reinterpret_cast<uintptr_t>(order) | reinterpret_cast<uintptr_t>(counts) | reinterpret_cast<uintptr_t>(skipped);
    if ((al & 15) || (al4 & 3)) return mpsa_fail(MPSA_EALIGN, "skip route: operands must be 16-byte (codes) / 4-byte (scales, workspace, lists) aligned");
    const int64_t ntq = ceil_div(nq, tile), nt = ceil_div(nk, tile);
    if (B * Hq * ntq >= (int64_t(1) << 31)) return mpsa_fail(MPSA_EUNSUPPORTED, "skip route: problem too large");
    const int rc = mpsa_ensure_init();
    if (rc != MPSA_OK) return rc;
    StatArgs a;
    a.q4 = q4; a.qs4 = qs4; a.q8 = q8; a.qs8 = qs8; a.k4 = k4; a.ks4 = ks4; a.k8 = k8; a.ks8 = ks8;
    a.stats = static_cast<float*>(work);
    a.B = (int)B; a.Hq = (int)Hq; a.Hkv = (int)Hkv; a.n = (int)nk; a.nt = (int)nt; a.n_pad = (int)(nt * tile);
    a.nq = (int)nq; a.ntq = (int)ntq; a.nq_pad = (int)(ntq * tile); a.causal = causal ? 1 : 0;
    hipStream_t st = (hipStream_t)stream;
    const unsigned grid = (unsigned)(B * Hq * ntq);
    const unsigned grid_pairs = (unsigned)(B * Hq * ((ntq + 1) / 2));
    int lrc;
    if (mode == MPSA_MODE_MXFP4) lrc = launch_stats<MPSA_FMT_E4M3, MPSA_MODE_MXFP4>(a, grid_pairs, st);
    else if (mode == MPSA_MODE_MXFP8) lrc = fmt8 == MPSA_FMT_E5M2 ? launch_stats<MPSA_FMT_E5M2, MPSA_MODE_MXFP8>(a, grid_pairs, st) : launch_stats<MPSA_FMT_E4M3, MPSA_MODE_MXFP8>(a, grid_pairs, st);
    else lrc = fmt8 == MPSA_FMT_E5M2 ? launch_stats<MPSA_FMT_E5M2, MPSA_MODE_DIAG>(a, grid_pairs, st) : launch_stats<MPSA_FMT_E4M3, MPSA_MODE_DIAG>(a, grid_pairs, st);
    if (lrc != MPSA_OK) return lrc;
    MPSA_CHECK_LAUNCH("skip route (statistics)");
    ListArgs l;
    l.stats = a.stats; l.Hq = (int)Hq; l.ntq = (int)ntq; l.nt = (int)nt; l.causal = a.causal; l.ragged = (nk % tile) != 0; l.mode = mode;
    l.thresh = skip_thresh; l.cls = cls; l.order = order; l.counts = counts; l.skipped = skipped;
    hipLaunchKernelGGL(skip_lists_kernel, dim3(grid), dim3(64), 0, st, l);
    MPSA_CHECK_LAUNCH("skip route (lists)");
    return MPSA_OK;
}
