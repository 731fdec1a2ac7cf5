// Paired-tile ("ping-pong") fused MXFP attention forward for gfx950: D = 128, 128x128 tiles, causal or (self-attention of
// six tiles or more) unmasked.
//
// Same arithmetic as attn_fwd.hip (see there for the operand layouts and the reference citations:
// ours/mxfp_attn_kernel.py:216-359 for the loop, ours/online_routing.py:68-77, :113-118, :160-171 for the causal
// tile structure and the grouped-query head mapping).  What differs is the work split.  A workgroup of EIGHT waves
// owns TWO adjacent query tiles: waves 0-3 ("X", tile 2I+1) and waves 4-7 ("Y", tile 2I); wave w and wave w+4 sit
// on the same SIMD.  Both groups read the same K and V tiles from LDS, which halves the L2 -> LDS traffic per query
// and the number of direct-to-LDS loads per CU.
//
// Step t of a wave (between workgroup barriers t and t+1) is software-pipelined inside the wave: first the score
// instructions S(t+1), then the 32 matrix instructions of P.V(t) with the softmax of tile t+1 placed in the gaps
// between them -- measured on MI355X, vector instructions of the *other* wave of a SIMD get almost no issue slots
// while a wave streams matrix instructions, but a few vector instructions between a wave's own matrix instructions
// are free.  The exponentials run in place over the score registers, one pair per gap from the first matrix instruction
// on; the registers of a 16-key group of P(t) take the new P(t+1) as soon as the four instructions that consume the
// group have been issued.  The exponentials are taken without a maximum pass: the (lazy) running maximum
// only has to move when a score exceeds it by more than a threshold, which the tile's row sum then shows; the wave
// does such a tile again the careful way (scores from the K tile still in LDS, maximum, rebase of row sum and output
// accumulators -- P.V(t), relative to the old maximum, is through by then -- and exponentials).
// The wave's diagonal tile runs as straight-line code after the loop; in a causal run Y, one tile short of X, idles in
// the last step.
//
// Staging is the one of attn_fwd.hip: 4-bit K tiles (XOR-swizzled rows) and V tiles (operand order) arrive by
// direct-to-LDS loads, one barrier per key tile; K has three buffers (the tile whose fragments are being pulled into
// registers is two steps ahead of the P.V tile), V two; the two 8-bit (diagonal) K tiles of a "diag" run's pair are staged
// once, in the prologue, into an LDS area of their own (read straight from global memory at the diagonal step their
// latency sat on the wave's critical path).  The running maximum rides in the score MFMA's C operand.  The "mixed" mode
// (8-bit Q, 4-bit K) differs in the score instruction's operand formats only; the "mxfp8" mode's K ring holds 8-bit tiles.
#include "attn_common.h"
#include "quantize_kernel.h"

namespace {

constexpr int D = 128, TILE = 128;
constexpr int KB = TILE / 32, SST = D / 64, NDB = D / 32;
constexpr int ROW4 = D / 2, ROW8 = D;
constexpr int CPR4 = ROW4 / 16, SH4 = 2;
constexpr int K_BYTES = TILE * ROW4, V_BYTES = TILE * D * 2;
constexpr int NKBUF = 3;                        // K tiles in LDS: one being multiplied, two ahead
constexpr int SMEM = NKBUF * K_BYTES + 2 * V_BYTES;
constexpr int Q8_BYTES = 512 * 64;              // fused-quantizer variants: every lane's 8-bit Q fragments (64 bytes), parked until the diagonal tile
constexpr int SMEM_QRAW = SMEM + Q8_BYTES;
constexpr int K8_BYTES = TILE * ROW8;           // "diag" runs: the two 8-bit diagonal K tiles of the pair (X's, then Y's), staged in the prologue
constexpr int CPR8 = ROW8 / 16;
constexpr int Q4_BYTES = 256 * 32;              // fused-quantizer "diag" runs without the causal mask: Y's 4-bit Q fragments, parked while the 8-bit ones are in use
constexpr int smem_bytes(bool qraw, int mode, bool causal) {
    if (mode == MPSA_MODE_MXFP8) return NKBUF * K8_BYTES + 2 * V_BYTES;      // every K tile in 8 bits: a ring of 16 KB tiles
    const bool diag = mode == MPSA_MODE_DIAG;                                 // the parked Q fragments and staged diagonal tiles are a diag run's
    return (qraw && diag ? SMEM_QRAW : SMEM) + (diag ? 2 * K8_BYTES : 0) + (qraw && diag && !causal ? Q4_BYTES : 0);
}
static_assert(smem_bytes(true, MPSA_MODE_DIAG, false) <= 160 * 1024, "LDS of a CU");
constexpr int NWAVES = 8;
constexpr int VI = V_BYTES / 1024 / NWAVES;     // direct-load instructions per wave for one V tile (4)
constexpr int NV = KB * 2 * NDB;                // P.V matrix instructions per tile (32)
static_assert(K_BYTES / 1024 == NWAVES, "one K direct-load instruction per wave");

// QRAW: Q arrives unquantized (in the P.V dtype) and is MX-quantized here, in registers, with the quantizer's own device
// functions -- the bits are those mpsa_quantize_mx would have written (ours/quant_mxint8.py:276-351, :164-219 with
// sm_scale*log2(e) folded in, :479-494), but the codes and scales never travel through HBM.
//
// CAUSAL = false: every query tile visits every key tile.  The steps then walk the key tiles in an order of the
// workgroup's own: first the tiles both groups take in 4 bits, pipelined as above; then, as straight-line steps, the
// ragged last tile (keys beyond the sequence masked) and the pair's two diagonal tiles 2I (8 bits for Y) and 2I+1
// (8 bits for X).  Softmax does not care about the order of the keys.
template <int PVT, int FMT8, int MODE, bool QRAW, bool CAUSAL>
__global__ __launch_bounds__(512, 1) void attn_pp_kernel(AttnArgs a) {
    typedef PV<PVT> P;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63, w = tid >> 6;
    const int h = lane >> 5, r = lane & 31;
    const int wu = __builtin_amdgcn_readfirstlane(w);    // the wave index, known to be uniform
    const int role = wu >> 2;                    // 0 = X (tile 2I+1), 1 = Y (tile 2I); uniform, so the loops below are scalar
    const int wq = wu & 3;

    // ---- which (batch, kv head, query head, query-tile pair) -- XCD-aware, heavy pairs first ----
    const int npairs = (a.nt + 1) >> 1;          // an odd tile count leaves the last pair with its lower tile only
    const int group = a.Hq / a.Hkv;
    const int total = a.B * a.Hq * npairs;
    int L = blockIdx.x;
    if ((total & 7) == 0) L = (L & 7) * (total >> 3) + (L >> 3);
    const int per_unit = group * npairs;
    const int unit = L / per_unit;
    const int rem = L - unit * per_unit;
    const int rank = rem / group;
    const int hq = (unit % a.Hkv) * group + (rem - rank * group);
    const int b = unit / a.Hkv;
    const int kvh = unit % a.Hkv;
    const int pair = CAUSAL ? npairs - 1 - rank : rank;
    const int i = 2 * pair + (1 - role);         // this wave's query tile
    const bool lone = 2 * pair + 1 >= a.nt;      // the pair without an upper tile: X has no queries and only helps with the staging
    const bool inactive = lone && role == 0;
    const int nsteps = CAUSAL ? 2 * pair + (lone ? 1 : 2) : a.nt;      // causal: key tiles 0 .. 2*pair+1, step t visits tile t
    // Without the mask: steps 0 .. n_plain-1 visit the tiles everybody takes in 4 bits and unmasked, in ascending order; the
    // remaining steps visit [the ragged last tile, unless the pair holds it,] tile 2I, tile 2I+1 (a run in 4 bits throughout
    // keeps the natural order and has only its last tile there).
    const int d0 = 2 * pair, d1 = 2 * pair + 1;
    const bool ragged = !CAUSAL && a.n < a.n_pad;
    const int n_plain = CAUSAL ? i
                        : lone ? a.nt - 1
                        : MODE == MPSA_MODE_DIAG ? a.nt - 2 - ((ragged && d1 != a.nt - 1) ? 1 : 0)
                                                 : a.nt - 1;       // the last tile, ragged or not, gets the straight-line step
    auto tile_at = [&](int t) __attribute__((always_inline)) {
        if constexpr (CAUSAL || MODE != MPSA_MODE_DIAG) {
            return t;
        } else {
            if (t < n_plain) return t + (t >= d0 ? 2 : 0);
            if (lone) return d0;
            return t == a.nt - 1 ? d1 : t == a.nt - 2 ? d0 : a.nt - 1;
        }
    };

    const int64_t qhead_row = ((int64_t)b * a.Hq + hq) * a.n_pad;
    const int64_t khead_row = ((int64_t)b * a.Hkv + kvh) * a.n_pad;
    const int q_local = 32 * wq + r;
    const int64_t q_row = qhead_row + (int64_t)i * TILE + q_local;

    // MODE_MXFP8: every K tile is an 8-bit one (16 KB, 128-byte rows swizzled like the staged diagonal tiles); the fragment
    // registers hold two of a tile's four key blocks at a time (the 4-bit tiles': all four)
    constexpr bool K8ALL = MODE == MPSA_MODE_MXFP8;
    constexpr int KT_BYTES = K8ALL ? K8_BYTES : K_BYTES;
    uint8_t* const kbuf0 = smem;
    uint8_t* const vbuf0 = smem + NKBUF * KT_BYTES;
    uint8_t* const k8d0 = smem + (QRAW ? SMEM_QRAW : SMEM);     // the pair's two 8-bit diagonal K tiles: tile 2I+1, tile 2I

    // ---- operands in registers ----
    v8i qf[SST];
    int qsc = 0;                                 // Q's scale bytes (bytes 0 and 2 of the word; the fused-quantizer variants keep
                                                 // those of the parked 8-bit fragments in bytes 1 and 3)
    v4i kf4[KB][SST];
    int ksc[KB];
    // shared exponent of an MX block from its largest magnitude, as the quantizer takes it (quantize_kernel.h)
    auto block_exponent = [&](float amax) __attribute__((always_inline)) {
        const uint32_t ab = mpsa_f2u(amax);
        const uint32_t ef = ab >> 23;
        return ef ? (int)ef - 127 : (31 - __builtin_clz(ab | 1u)) - 149;
    };
    // Both precisions from one pass over the lane's query row: lane half h owns MX blocks h and 2 + h of the row's four
    // (the 4-bit operand layout), so a block's maximum and shared exponent are lane-local and serve both formats (the
    // element exponent limits differ: 3 and 7).  The 8-bit operand wants 16 bytes of EVERY block in each lane half
    // (registers 0-3: block 2s, 4-7: block 2s + 1), so the two lanes of a query trade halves of their blocks afterwards:
    // one v_permlane32_swap per register pair.  q8f receives the 8-bit fragments when WANT8 is set.
    auto load_q_raw = [&](auto want8_c, v8i (&q8f)[SST]) __attribute__((always_inline)) {
#pragma clang fp contract(off)        // the quantizer's arithmetic, operation by operation
        constexpr bool WANT8 = decltype(want8_c)::value;
        constexpr bool WANT4 = MODE != MPSA_MODE_MIXED && MODE != MPSA_MODE_MXFP8;   // those two multiply 8-bit Q everywhere
        // rows beyond the sequence (ragged last tile) read the last row instead and are zeroed below
        const bool row_ok = i * TILE + q_local < a.nq;
        const int64_t row_idx = row_ok ? (int64_t)i * TILE + q_local : (int64_t)a.nq - 1;
        const char* row = static_cast<const char*>(a.q_raw) +
                          2 * ((int64_t)b * a.q_sb + (int64_t)hq * a.q_sh + row_idx * a.q_sn);
        uint32_t sbytes = 0, sbytes8 = 0;
#pragma unroll
        for (int s = 0; s < SST; ++s) {
            float x[4][8];
            float amax = 0.0f;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                load8<PVT>(row + 2 * (32 * (2 * s + h) + 8 * c), x[c]);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    x[c][e] = x[c][e] * a.q_pre;
                    amax = __builtin_fmaxf(amax, __builtin_fabsf(x[c][e]));
                }
            }
            const bool zero = mpsa_f2u(amax) == 0u;
            const int ex = block_exponent(amax);
            if constexpr (WANT4) {
                const int se = ex - 3;                                         // emax of E2M1: ours/quant_mxint8.py:303
                int w[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) w[c] = zero ? 0 : (int)e2m1_pack8<true>(x[c], se, false);
                qf[s] = (v8i){w[0], w[1], w[2], w[3], 0, 0, 0, 0};
                sbytes |= (uint32_t)(zero ? 0 : min(max(se + 127, 0), 254)) << (16 * s);
            }
            if constexpr (WANT8) {
                const int se8 = ex - 7;                                        // emax of the 8-bit formats: ours/quant_mxint8.py:191
                // the quantizer's clamp to the format's maximum (quantize_kernel.h): finite blocks scale into
                // [128, 256) and never meet it, a block with an infinity saturates there instead of giving NaN codes
                const float lim = (FMT8 == MPSA_FMT_E4M3) ? 448.0f : 57344.0f;
                int w8[8];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    float y[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) y[e] = __builtin_fminf(__builtin_fmaxf(ldexpf(x[c][e], -se8), -lim), lim);
                    w8[2 * c] = zero ? 0 : (int)fp8_pack4<FMT8, false>(y[0], y[1], y[2], y[3]);
                    w8[2 * c + 1] = zero ? 0 : (int)fp8_pack4<FMT8, false>(y[4], y[5], y[6], y[7]);
                }
                // w8[0..3] = bytes 0-15, w8[4..7] = bytes 16-31 of block 2s + h.  Lane half 0 keeps its low half in
                // registers 0-3 and takes block 2s + 1's low half from its partner into 4-7; lane half 1 keeps its high
                // half in 4-7 and takes block 2s's high half into 0-3: swap (lanes 32-63 of register i) with (lanes 0-31 of
                // register 4 + i).
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(w8[q]), "+v"(w8[4 + q]));
                q8f[s] = (v8i){w8[0], w8[1], w8[2], w8[3], w8[4], w8[5], w8[6], w8[7]};
                // lane half h hands the matrix core the scale byte of block 2s + h: its own
                sbytes8 |= (uint32_t)(zero ? 0 : min(max(se8 + 127, 0), 254)) << (16 * s);
            }
        }
        if constexpr (WANT4) {
            qsc = (int)(sbytes | (sbytes8 << 8));
        } else {
#pragma unroll
            for (int s = 0; s < SST; ++s) qf[s] = q8f[s];
            qsc = (int)sbytes8;
        }
        if (i * TILE + 32 * wq + 31 >= a.nq) {            // a wave of the ragged last tile: zero codes and scales for its padding
#pragma unroll                                            // rows, as the standalone quantizer pads them
            for (int s = 0; s < SST; ++s)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    qf[s][e] = row_ok ? qf[s][e] : 0;
                    if constexpr (WANT8) q8f[s][e] = row_ok ? q8f[s][e] : 0;
                }
            qsc = row_ok ? qsc : 0;
        }
    };
    auto load_q = [&](bool is8) __attribute__((always_inline)) {
        if constexpr (QRAW) return;                   // the fused-quantizer variants fill the fragments in the prologue
        if (is8) {
#pragma unroll
            for (int s = 0; s < SST; ++s) {
                // 8-bit operand: registers 0-3 hold 16 bytes of MX block 2s, registers 4-7 of block 2s+1
                const v4i x0 = *reinterpret_cast<const v4i*>(a.q8 + q_row * D + s * 64 + h * 16);
                const v4i x1 = *reinterpret_cast<const v4i*>(a.q8 + q_row * D + s * 64 + h * 16 + 32);
                qf[s] = (v8i){x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
            }
        } else {
#pragma unroll
            for (int s = 0; s < SST; ++s) {
                const v4i x = *reinterpret_cast<const v4i*>(a.q4 + q_row * (D / 2) + (2 * s + h) * 16);
                qf[s] = (v8i){x[0], x[1], x[2], x[3], 0, 0, 0, 0};
            }
        }
        const uint8_t* qs = (is8 ? a.qs8 : a.qs4) + q_row * (D / 32);
        qsc = (int)(*reinterpret_cast<const uint32_t*>(qs) >> (8 * h));
    };
    auto load_kscales = [&](int tile, bool is8) __attribute__((always_inline)) {
        const uint8_t* sp = (is8 ? a.ks8 : a.ks4) + (khead_row + (int64_t)tile * TILE + r) * (D / 32);
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
            ksc[kb] = (int)(*reinterpret_cast<const uint32_t*>(sp + kb * 32 * (D / 32)) >> (8 * h));
    };
    // 8-bit tiles: fragment (key block kb0 + kbl, step s) = registers kf4[2 kbl][s] (bytes of MX block 2s) and kf4[2 kbl + 1][s]
    // (of block 2s + 1)
    auto read_kf8_pair = [&](int t, int kb0) __attribute__((always_inline)) {
        const uint8_t* kl = kbuf0 + (t % NKBUF) * K8_BYTES;
#pragma unroll
        for (int kbl = 0; kbl < 2; ++kbl) {
            const int krow = 32 * (kb0 + kbl) + r;
            const int f = (krow >> 1) & (CPR8 - 1);
#pragma unroll
            for (int s = 0; s < SST; ++s) {
                kf4[2 * kbl][s] = *reinterpret_cast<const v4i*>(kl + krow * ROW8 + (((4 * s + h) ^ f) * 16));
                kf4[2 * kbl + 1][s] = *reinterpret_cast<const v4i*>(kl + krow * ROW8 + (((4 * s + h + 2) ^ f) * 16));
            }
        }
    };
    auto read_kf4 = [&](int t) __attribute__((always_inline)) {
        if constexpr (K8ALL) {
            read_kf8_pair(t, 0);
            return;
        }
        const uint8_t* kl = kbuf0 + (t % NKBUF) * K_BYTES;
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
            const int krow = 32 * kb + r;
            const int f = (krow >> SH4) & (CPR4 - 1);
#pragma unroll
            for (int s = 0; s < SST; ++s)
                kf4[kb][s] = *reinterpret_cast<const v4i*>(kl + krow * ROW4 + (((2 * s + h) ^ f) * 16));
        }
    };

    // ---- staging: every wave issues its share of each tile ----
    uint32_t koff;                                        // this lane's byte offset into a 4-bit K tile (swizzled rows)
    {
        const int p = w * 64 + lane;
        const int row = p / CPR4, slot = p % CPR4;
        const int cb = slot ^ ((row >> SH4) & (CPR4 - 1));
        koff = (uint32_t)(row * ROW4 + cb * 16);
    }
    uint32_t koff8[2];                                    // the same for an 8-bit tile's two pieces per wave
#pragma unroll
    for (int c = 0; c < 2; ++c) {
        const int p = (w * 2 + c) * 64 + lane;
        const int row = p / CPR8, slot = p % CPR8;
        koff8[c] = (uint32_t)(row * ROW8 + (slot ^ ((row >> 1) & (CPR8 - 1))) * 16);
    }
    auto issue_k4 = [&](int t) __attribute__((always_inline)) {           // step t's K tile, in the width the mode multiplies
        if constexpr (K8ALL) {
            const uint8_t* src = a.k8 + (khead_row + (int64_t)tile_at(t) * TILE) * ROW8;
#pragma unroll
            for (int c = 0; c < 2; ++c) load16_to_lds_sv(koff8[c], src, kbuf0 + (t % NKBUF) * K8_BYTES + (wu * 2 + c) * 1024);
        } else {
            const uint8_t* src = a.k4 + (khead_row + (int64_t)tile_at(t) * TILE) * ROW4;
            load16_to_lds_sv(koff, src, kbuf0 + (t % NKBUF) * K_BYTES + wu * 1024);
        }
    };
    auto issue_v = [&](int t) __attribute__((always_inline)) {
        const uint8_t* src = static_cast<const uint8_t*>(a.v) + (khead_row + (int64_t)tile_at(t) * TILE) * (D * 2);
        uint8_t* dst = vbuf0 + (t & 1) * V_BYTES;
#pragma unroll
        for (int c = 0; c < VI; ++c) {
            const int ci = wu * VI + c;
            load16_to_lds_sv((uint32_t)lane * 16u, src + ci * 1024, dst + ci * 1024);
        }
    };
    // barrier of step t: this wave's pieces of V(t) and K(t+1) have landed, after it everybody's have and everybody
    // is done with V(t-1) and the K(t) fragments; then the next loads go out
    auto sync_issue = [&](int t) __attribute__((always_inline)) {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        if (t + 1 < nsteps) issue_v(t + 1);
        if (t + 3 < nsteps) issue_k4(t + 3);
    };

    // ---- per-query state ----
    v16f acc[NDB];
#pragma unroll
    for (int d = 0; d < NDB; ++d)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[d][e] = 0.0f;
    constexpr float REBASE = P::REBASE;          // lazy running maximum, see attn_fwd.hip
    float m_run = 0.0f, l_run = 0.0f;
    v16f negm;
#pragma unroll
    for (int e = 0; e < 16; ++e) negm[e] = 0.0f;
    v16f st[KB];
    v4i pk[KB][2];

    auto prep_plain = [&](int t) __attribute__((always_inline)) {       // step t's tile in the mode's plain width
        load_kscales(tile_at(t), K8ALL);
        read_kf4(t);
    };
    auto prep_special = [&](int t) __attribute__((always_inline)) {      // this wave's diagonal tile (key tile i) at step t
        if constexpr (MODE == MPSA_MODE_DIAG) {
            load_kscales(i, true);
            if constexpr (QRAW) {
                const uint8_t* park = smem + SMEM + tid * 16;
#pragma unroll
                for (int s = 0; s < SST; ++s) {
                    const v4i x0 = *reinterpret_cast<const v4i*>(park + (2 * s) * 8192);
                    const v4i x1 = *reinterpret_cast<const v4i*>(park + (2 * s + 1) * 8192);
                    qf[s] = (v8i){x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
                }
            } else {
                load_q(true);
            }
        } else {
            prep_plain(t);
        }
    };
    // Y without the causal mask takes a 4-bit tile (2I+1) after its 8-bit one (2I): back to the 4-bit Q fragments
    auto restore_q4 = [&]() __attribute__((always_inline)) {
        if constexpr (QRAW) {
            const uint8_t* park4 = k8d0 + 2 * K8_BYTES + (tid & 255) * 16;
#pragma unroll
            for (int s = 0; s < SST; ++s) {
                const v4i x = *reinterpret_cast<const v4i*>(park4 + s * 4096);
                qf[s] = (v8i){x[0], x[1], x[2], x[3], 0, 0, 0, 0};
            }
        } else {
            load_q(false);
        }
    };
    auto s_plain = [&](int ts) __attribute__((always_inline)) {          // scores of step ts's tile
        if constexpr (K8ALL) {
            // key blocks 0, 1 are in the fragment registers; blocks 2, 3 follow into the same registers while the first
            // four matrix instructions run
#pragma unroll
            for (int half = 0; half < 2; ++half) {
#pragma unroll
                for (int kbl = 0; kbl < 2; ++kbl) {
                    const int kb = 2 * half + kbl;
#pragma unroll
                    for (int s = 0; s < SST; ++s) {
                        const v4i x0 = kf4[2 * kbl][s], x1 = kf4[2 * kbl + 1][s];
                        const v8i kd = (v8i){x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
                        st[kb] = score_mfma8<FMT8>(kd, qf[s], s == 0 ? negm : st[kb], s, ksc[kb], qsc);
                    }
                }
                if (half == 0) read_kf8_pair(ts, 2);
            }
            return;
        }
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
            for (int s = 0; s < SST; ++s) {
                const v4i x = kf4[kb][s];
                const v8i k8v = (v8i){x[0], x[1], x[2], x[3], 0, 0, 0, 0};
                if constexpr (MODE == MPSA_MODE_MIXED) st[kb] = score_mfma48<FMT8>(k8v, qf[s], s == 0 ? negm : st[kb], s, ksc[kb], qsc);
                else st[kb] = score_mfma4(k8v, qf[s], s == 0 ? negm : st[kb], s, ksc[kb], qsc);
            }
    };
    auto s_special = [&](int t) __attribute__((always_inline)) {
        if constexpr (MODE == MPSA_MODE_DIAG) {
            // this wave's 8-bit diagonal K tile has been in LDS since the prologue (rows XOR-swizzled like the 4-bit ones)
            const uint8_t* kl = k8d0 + role * K8_BYTES;
            const int qs8 = QRAW ? (int)((uint32_t)qsc >> 8) : qsc;
#pragma unroll
            for (int kb = 0; kb < KB; ++kb) {
                const int krow = 32 * kb + r;
                const int f = (krow >> 1) & (CPR8 - 1);
#pragma unroll
                for (int s = 0; s < SST; ++s) {
                    // 8-bit operand: registers 0-3 hold 16 bytes of MX block 2s, registers 4-7 of block 2s+1
                    const v4i x0 = *reinterpret_cast<const v4i*>(kl + krow * ROW8 + (((4 * s + h) ^ f) * 16));
                    const v4i x1 = *reinterpret_cast<const v4i*>(kl + krow * ROW8 + (((4 * s + h + 2) ^ f) * 16));
                    const v8i kd = (v8i){x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
                    st[kb] = score_mfma8<FMT8>(kd, qf[s], s == 0 ? negm : st[kb], s, ksc[kb], qs8);
                }
            }
        } else {
            s_plain(t);
        }
    };
    // masked: keys from `limit` on are dead (the causal diagonal tile: the keys after the query; the ragged last tile:
    // the keys beyond the sequence)
    auto softmax = [&](bool first, auto masked_c, int limit) __attribute__((always_inline)) {
        __builtin_amdgcn_s_setprio(0);
        if constexpr (decltype(masked_c)::value) {
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int key = 32 * kb + 8 * (e >> 2) + 4 * h + (e & 3);
                    if (key >= limit) st[kb][e] = -__builtin_inff();
                }
        }
        float mx = st[0][0];
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
            for (int e = 0; e < 16; ++e) mx = __builtin_fmaxf(mx, st[kb][e]);
        mx = max_lane_pair(mx);
        if (first || __any(mx > REBASE)) {
            const float delta = first ? mx : __builtin_fmaxf(mx, 0.0f);
            const float alpha = first ? 1.0f : __builtin_amdgcn_exp2f(-delta);
            m_run += delta;
#pragma unroll
            for (int e = 0; e < 16; ++e) negm[e] = -m_run;
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                for (int e = 0; e < 16; ++e) st[kb][e] -= delta;
            l_run *= alpha;
#pragma unroll
            for (int d = 0; d < NDB; ++d)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[d][e] *= alpha;
        }
        float ps0 = 0.0f, ps1 = 0.0f;
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
            for (int c = 0; c < 2; ++c)
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                    const float p0 = __builtin_amdgcn_exp2f(st[kb][8 * c + e]);
                    const float p1 = __builtin_amdgcn_exp2f(st[kb][8 * c + e + 1]);
                    const typename P::v2 pp = P::pack(p0, p1);
                    pk[kb][c][e >> 1] = __builtin_bit_cast(int, pp);
                    ps0 += p0;
                    ps1 += p1;
                }
        l_run += ps0 + ps1;
        __builtin_amdgcn_s_setprio(2);
    };
    auto pv = [&](int t) __attribute__((always_inline)) {
        constexpr int PRE = 8;
        const uint8_t* vl = vbuf0 + (t & 1) * V_BYTES + lane * 16;
        typename P::vec vf[PRE];
#pragma unroll
        for (int x = 0; x < PRE; ++x) vf[x] = *reinterpret_cast<const typename P::vec*>(vl + x * 1024);
#pragma unroll
        for (int idx = 0; idx < NV; ++idx) {
            const int d = idx % NDB, kc = idx / NDB;
            const typename P::vec cur = vf[idx % PRE];
            if (idx + PRE < NV) vf[idx % PRE] = *reinterpret_cast<const typename P::vec*>(vl + (idx + PRE) * 1024);
            acc[d] = P::mfma(cur, __builtin_bit_cast(typename P::vec, pk[kc >> 1][kc & 1]), acc[d]);
        }
    };

    // One pair of exponentials of the coming tile: P = exp2(S - m), rounded to 16 bits for P.V; the row sum adds the
    // float32 values, as the reference does (ours/mxfp_attn_kernel.py:324-327), with plain additions (the dot-product
    // instructions share the matrix pipe and stall the P.V stream).
    auto ex = [&](int g, int j, float& ps0, float& ps1) __attribute__((always_inline)) {
        const int kb = g >> 1, c = g & 1;
        const float p0 = __builtin_amdgcn_exp2f(st[kb][8 * c + 2 * j]);
        const float p1 = __builtin_amdgcn_exp2f(st[kb][8 * c + 2 * j + 1]);
        const typename P::v2 pp = P::pack(p0, p1);
        int word = __builtin_bit_cast(int, pp);
        // pin the conversion here, between the matrix instructions: the redo path overwrites pk, so the compiler
        // would otherwise sink all 32 conversions behind the check, where nothing overlaps them
        asm volatile("" : "+v"(word));
        pk[kb][c][j] = word;
        ps0 += p0;
        ps1 += p1;
    };
    // The exponentials of tile t+1 were taken optimistically, without looking for the tile's maximum first: the running
    // maximum only has to move when a score exceeds it by more than REBASE, and then the row sum shows it (it exceeds
    // 2^REBASE or is not finite).  In that rare case the tile is done again the careful way, from its K fragments,
    // which are still in LDS: scores again, maximum, rebase (P.V(t) is through, the accumulators can be rescaled now).
    auto finish_tile = [&](int t, float ps0, float ps1) __attribute__((always_inline)) {
        float tot = ps0 + ps1;
        if (__any(!(tot < P::OPTIMISTIC_LIMIT))) {
            prep_plain(t + 1);
            s_plain(t + 1);
            float mx = st[0][0];
#pragma unroll
            for (int kb = 0; kb < KB; ++kb)
#pragma unroll
                for (int e = 0; e < 16; ++e) mx = __builtin_fmaxf(mx, st[kb][e]);
            mx = max_lane_pair(mx);
            const float delta = __builtin_fmaxf(mx, 0.0f);
            const float alpha = __builtin_amdgcn_exp2f(-delta);
            m_run += delta;
#pragma unroll
            for (int e = 0; e < 16; ++e) negm[e] = -m_run;
            l_run *= alpha;
#pragma unroll
            for (int d = 0; d < NDB; ++d)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[d][e] *= alpha;
            ps0 = 0.0f;
            ps1 = 0.0f;
#pragma unroll
            for (int g = 0; g < 2 * KB; ++g) {
#pragma unroll
                for (int e = 0; e < 8; ++e) st[g >> 1][8 * (g & 1) + e] -= delta;
#pragma unroll
                for (int j = 0; j < 4; ++j) ex(g, j, ps0, ps1);
            }
            tot = ps0 + ps1;
            prep_plain(t + 2);                             // back to the operands of the next step
        }
        l_run += tot;
    };

    // P.V(t) with the softmax of tile t+1 (whose scores are in st) in the gaps between its matrix instructions.  The work
    // of score pair e (two of a lane's 64 scores) is spread over three gaps so that no instruction waits for the one
    // before it: the exponentials are taken in place in the gap of matrix instruction e; the row-sum additions follow one
    // gap later (the exponential unit's latency is over by then); the conversion into the P registers follows four gaps
    // later -- the four matrix instructions that consume a 16-key group of P(t) are out, so the group's registers take
    // the new P(t+1).  Only the last addition and the last group's four conversions are left behind the last matrix
    // instruction (with exponentials, additions and conversions of a pair all in one gap, the wave stalled on the
    // exponentials' results in every gap and a whole group's softmax ran after the last matrix instruction: 6 % more
    // cycles per step at a fixed clock).
    auto pv_exp = [&](int t) __attribute__((always_inline)) {
        constexpr int PRE = 8;
        const uint8_t* vl = vbuf0 + (t & 1) * V_BYTES + lane * 16;
        typename P::vec vf[PRE];
#pragma unroll
        for (int x = 0; x < PRE; ++x) vf[x] = *reinterpret_cast<const typename P::vec*>(vl + x * 1024);
        auto mm = [&](int idx) __attribute__((always_inline)) {
            const int d = idx % NDB, kc = idx / NDB;
            const typename P::vec cur = vf[idx % PRE];
            if (idx + PRE < NV) vf[idx % PRE] = *reinterpret_cast<const typename P::vec*>(vl + (idx + PRE) * 1024);
            acc[d] = P::mfma(cur, __builtin_bit_cast(typename P::vec, pk[kc >> 1][kc & 1]), acc[d]);
        };
        float ps0 = 0.0f, ps1 = 0.0f;
        const uint8_t* kl = kbuf0 + ((t + 2) % NKBUF) * KT_BYTES;
        auto kfrag = [&](int kb, int s) __attribute__((always_inline)) {
            if constexpr (K8ALL) {                       // register kf4[kb][s] of the 8-bit layout: key block kb / 2, half kb % 2
                const int krow = 32 * (kb >> 1) + r;
                const int f = (krow >> 1) & (CPR8 - 1);
                kf4[kb][s] = *reinterpret_cast<const v4i*>(kl + krow * ROW8 + (((4 * s + h + 2 * (kb & 1)) ^ f) * 16));
            } else {
                const int krow = 32 * kb + r;
                const int f = (krow >> SH4) & (CPR4 - 1);
                kf4[kb][s] = *reinterpret_cast<const v4i*>(kl + krow * ROW4 + (((2 * s + h) ^ f) * 16));
            }
        };
        // score pair e = 4 g + j: registers 8c + 2j, 8c + 2j + 1 of key block kb, with g = 2 kb + c the 16-key group
        auto do_exp = [&](int e) __attribute__((always_inline)) {
            const int g = e >> 2, j = e & 3, kb = g >> 1, c = g & 1;
            st[kb][8 * c + 2 * j] = __builtin_amdgcn_exp2f(st[kb][8 * c + 2 * j]);
            st[kb][8 * c + 2 * j + 1] = __builtin_amdgcn_exp2f(st[kb][8 * c + 2 * j + 1]);
        };
        auto do_add = [&](int e) __attribute__((always_inline)) {
            const int g = e >> 2, j = e & 3, kb = g >> 1, c = g & 1;
            ps0 += st[kb][8 * c + 2 * j];
            ps1 += st[kb][8 * c + 2 * j + 1];
        };
        auto do_cvt = [&](int e) __attribute__((always_inline)) {
            const int g = e >> 2, j = e & 3, kb = g >> 1, c = g & 1;
            const typename P::v2 pp = P::pack(st[kb][8 * c + 2 * j], st[kb][8 * c + 2 * j + 1]);
            int word = __builtin_bit_cast(int, pp);
            // pin the conversion here, between the matrix instructions: the redo path overwrites pk, so the compiler
            // would otherwise sink all 32 conversions behind the check, where nothing overlaps them
            asm volatile("" : "+v"(word));
            pk[kb][c][j] = word;
        };
#pragma unroll
        for (int idx = 0; idx < NV; ++idx) {
            const int d = idx % NDB, kc = idx / NDB;
            mm(idx);
            do_exp(idx);
            if (idx >= 1) do_add(idx - 1);
            if (idx >= NDB) do_cvt(idx - NDB);
            if (kc >= KB && d < SST) kfrag(kc - KB, d);   // K fragments of tile t+2 (the score MFMAs are long gone)
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x400, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
        }
        do_add(NV - 1);
#pragma unroll
        for (int e = NV - NDB; e < NV; ++e) do_cvt(e);
        finish_tile(t, ps0, ps1);
    };

    // ---- prologue (all waves): V(0), K(0..2) on their way; Q into registers ----
    issue_v(0);
    issue_k4(0);
    if (nsteps > 1) issue_k4(1);
    if (nsteps > 2) issue_k4(2);
    if constexpr (MODE == MPSA_MODE_DIAG) {
        // the pair's two diagonal tiles in 8 bits (X's: key tile 2I+1, Y's: 2I), 16 one-KiB pieces each, two per wave:
        // piece position p = 8 row + slot holds the row's 16-byte chunk slot ^ ((row >> 1) & 7)
#pragma unroll
        for (int x = 0; x < 2; ++x) {
            if (lone && x == 0) continue;
            const uint8_t* src = a.k8 + (khead_row + (int64_t)(2 * pair + 1 - x) * TILE) * ROW8;
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const int p = (w * 2 + c) * 64 + lane;
                const int row = p / CPR8, slot = p % CPR8;
                const int cb = slot ^ ((row >> 1) & (CPR8 - 1));
                load16_to_lds_sv((uint32_t)(row * ROW8 + cb * 16), src, k8d0 + x * K8_BYTES + (wu * 2 + c) * 1024);
            }
        }
    }
    if (inactive) {
        // no queries here: this wave only issues its share of the staging loads and keeps the barriers' count
    } else if constexpr (QRAW) {
        // Q is quantized now, while the first K/V tiles are on their way.  The diagonal tile's 8-bit fragments come out
        // of the same pass and are parked in LDS (each lane reads back only what it wrote itself): at the diagonal tile
        // the loads and the conversion would sit on the wave's critical path.
        v8i q8f[SST];
        if constexpr (MODE == MPSA_MODE_DIAG) {
            load_q_raw(std::true_type{}, q8f);
            if constexpr (!CAUSAL) {
                if (role == 1) {
                    uint8_t* park4 = k8d0 + 2 * K8_BYTES + (tid & 255) * 16;
#pragma unroll
                    for (int s = 0; s < SST; ++s)
                        *reinterpret_cast<v4i*>(park4 + s * 4096) = (v4i){qf[s][0], qf[s][1], qf[s][2], qf[s][3]};
                }
            }
            uint8_t* park = smem + SMEM + tid * 16;
#pragma unroll
            for (int s = 0; s < SST; ++s) {
                *reinterpret_cast<v4i*>(park + (2 * s) * 8192) = (v4i){q8f[s][0], q8f[s][1], q8f[s][2], q8f[s][3]};
                *reinterpret_cast<v4i*>(park + (2 * s + 1) * 8192) = (v4i){q8f[s][4], q8f[s][5], q8f[s][6], q8f[s][7]};
            }
        } else if constexpr (MODE == MPSA_MODE_MIXED || K8ALL) {
            load_q_raw(std::true_type{}, q8f);
        } else {
            load_q_raw(std::false_type{}, q8f);
        }
    } else {
        load_q(MODE == MPSA_MODE_MIXED || K8ALL);  // "mixed" and "mxfp8": 8-bit Q fragments for the whole run
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    if (inactive) {
        const int nsync = CAUSAL ? nsteps + 1 : nsteps;
        for (int t = 0; t < nsync; ++t) sync_issue(t);
        __builtin_amdgcn_s_waitcnt(0x0F70);
        return;
    }

    // Step t (between barriers t and t+1): S(t+1), then P.V(t) with the softmax of t+1 in its gaps.  The first `last`
    // steps take plain tiles; the tiles after them get straight-line code.
    const int last = n_plain;
    if constexpr (CAUSAL) {
        // the wave's last key tile is the diagonal one (index i); Y, one tile short of X, idles through the last step
        if (last == 0) {
            prep_special(0);
            s_special(0);
            softmax(true, std::true_type{}, q_local + 1);
        } else {
            prep_plain(0);
            s_plain(0);
            softmax(true, std::false_type{}, 0);
            if (last >= 2) prep_plain(1);
        }
    } else {
        prep_plain(0);
        s_plain(0);
        softmax(true, std::false_type{}, 0);
        if (last >= 2) prep_plain(1);
    }
    for (int t = 0; t + 2 <= last; ++t) {
        sync_issue(t);
        s_plain(t + 1);
        load_kscales(tile_at(t + 2), K8ALL);
        pv_exp(t);
    }
    if constexpr (CAUSAL) {
        if (last >= 1) {
            const int t = last - 1;
            sync_issue(t);
            prep_special(t + 1);
            pv(t);
            s_special(t + 1);
            softmax(false, std::true_type{}, q_local + 1);
        }
        sync_issue(last);
        pv(last);
        if (role == 1) sync_issue(last + 1);
    } else {
        bool q_is8 = false;
#pragma nounroll
        for (int t = last - 1; t + 1 < nsteps; ++t) {          // P.V(t) is pending; step t+1's tile comes next
            const int j = tile_at(t + 1);
            const bool is8 = MODE == MPSA_MODE_DIAG && j == i;
            const int limit = (ragged && j == a.nt - 1) ? a.n - j * TILE : TILE;
            sync_issue(t);
            if (is8) {
                prep_special(t + 1);
                q_is8 = true;
            } else {
                prep_plain(t + 1);
                if (q_is8) restore_q4();
                q_is8 = false;
            }
            pv(t);
            if (is8) s_special(t + 1);
            else s_plain(t + 1);
            softmax(false, std::true_type{}, limit);
        }
        sync_issue(nsteps - 1);
        pv(nsteps - 1);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);                // no direct-to-LDS load may outlive the workgroup

    // ---- epilogue: O = acc / l ; register e of lane (h, r): dim 32*db + 8*(e/4) + 4*h + e%4 of query r ----
    const float l_tot = sum_lane_pair(l_run);
    const float inv = 1.0f / l_tot;
    const int q_global = i * TILE + q_local;
    if (q_global >= a.nq) return;                       // a row of the ragged last tile's padding (both lanes of a query leave together)
    uint8_t* orow = static_cast<uint8_t*>(a.o);
    const int64_t off = (int64_t)b * a.o_sb + (int64_t)hq * a.o_sh + (int64_t)q_global * a.o_sn;
    if (a.o_dtype != MPSA_F32 && ((a.o_sn | a.o_sh | a.o_sb) & 7) == 0 && (reinterpret_cast<uintptr_t>(a.o) & 15) == 0) {
        // 16-bit output: the two lanes of a query trade register groups (lane half 0 hands over dims 8..11 of every
        // 16 and receives dims 4..7), so that each lane owns 8 consecutive dims and stores 16 bytes at a time
#pragma unroll
        for (int d = 0; d < NDB; ++d)
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
                *reinterpret_cast<v4i*>(orow + (off + dim) * 2) = pk8;
            }
        return;
    }
#pragma unroll
    for (int d = 0; d < NDB; ++d)
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

template <int PVT, int FMT8, int MODE, bool QRAW, bool CAUSAL>
struct PpLds {
    static inline const bool registered = mpsa_register_lds_kernel(reinterpret_cast<const void*>(attn_pp_kernel<PVT, FMT8, MODE, QRAW, CAUSAL>), smem_bytes(QRAW, MODE, CAUSAL));
};

template <int PVT, int FMT8, int MODE, bool QRAW, bool CAUSAL>
int launch_pp_c(const AttnArgs& a, hipStream_t st) {
    if (!PpLds<PVT, FMT8, MODE, QRAW, CAUSAL>::registered) return mpsa_fail(MPSA_ELAUNCH, "attn: kernel not registered");
    const int rc = mpsa_ensure_init();
    if (rc != MPSA_OK) return rc;
    dim3 grid((unsigned)(a.B * a.Hq * ((a.nt + 1) / 2)));
    hipLaunchKernelGGL((attn_pp_kernel<PVT, FMT8, MODE, QRAW, CAUSAL>), grid, dim3(512), smem_bytes(QRAW, MODE, CAUSAL), st, a);
    MPSA_CHECK_LAUNCH("attn(pp)");
    return MPSA_OK;
}

template <int PVT, int FMT8, int MODE, bool QRAW>
int launch_pp(const AttnArgs& a, hipStream_t st) {
    return a.causal ? launch_pp_c<PVT, FMT8, MODE, QRAW, true>(a, st) : launch_pp_c<PVT, FMT8, MODE, QRAW, false>(a, st);
}

template <int PVT, bool QRAW>
int launch_pp_mode(const AttnArgs& a, hipStream_t st) {
    if (a.mode == MPSA_MODE_MXFP4) return launch_pp<PVT, MPSA_FMT_E4M3, MPSA_MODE_MXFP4, QRAW>(a, st);
    if (a.mode == MPSA_MODE_MIXED)
        return a.fmt8 == MPSA_FMT_E5M2 ? launch_pp<PVT, MPSA_FMT_E5M2, MPSA_MODE_MIXED, QRAW>(a, st)
                                       : launch_pp<PVT, MPSA_FMT_E4M3, MPSA_MODE_MIXED, QRAW>(a, st);
    if (a.mode == MPSA_MODE_MXFP8)
        return a.fmt8 == MPSA_FMT_E5M2 ? launch_pp<PVT, MPSA_FMT_E5M2, MPSA_MODE_MXFP8, QRAW>(a, st)
                                       : launch_pp<PVT, MPSA_FMT_E4M3, MPSA_MODE_MXFP8, QRAW>(a, st);
    return a.fmt8 == MPSA_FMT_E5M2 ? launch_pp<PVT, MPSA_FMT_E5M2, MPSA_MODE_DIAG, QRAW>(a, st)
                                   : launch_pp<PVT, MPSA_FMT_E4M3, MPSA_MODE_DIAG, QRAW>(a, st);
}

}  // namespace

// The paired-tile kernel covers self-attention with D = 128 and 128-key tiles in the diag, mxfp4, mixed and mxfp8 modes: causal
// runs from two tiles on, runs without the mask from six tiles on; the last tile may be ragged, and with an odd number of
// tiles the last workgroup of a head works on its one tile with half of its waves.
// MPSA_ATTN_PP=0 in the environment switches it off (the general kernel then runs everything).
bool attn_pp_supported(const AttnArgs& a, int pv_dtype) {
    static const bool enabled = [] {
        const char* v = getenv("MPSA_ATTN_PP");
        return !(v && v[0] == '0');
    }();
    (void)pv_dtype;
    const bool mode_ok = a.mode == MPSA_MODE_DIAG || a.mode == MPSA_MODE_MXFP4 || a.mode == MPSA_MODE_MIXED || a.mode == MPSA_MODE_MXFP8;
    if (!enabled || a.d != 128 || a.tile != 128 || a.nq != a.n || !mode_ok) return false;
    return a.nt >= (a.causal ? 2 : 6);
}

int attn_pp_launch(const AttnArgs& a, int pv_dtype, hipStream_t st) {
    if (a.q_raw) {
        if (pv_dtype == MPSA_BF16) return launch_pp_mode<MPSA_BF16, true>(a, st);
        return launch_pp_mode<MPSA_F16, true>(a, st);
    }
    if (pv_dtype == MPSA_BF16) return launch_pp_mode<MPSA_BF16, false>(a, st);
    return launch_pp_mode<MPSA_F16, false>(a, st);
}
