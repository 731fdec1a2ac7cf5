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
//
// Staging.  Codes go HBM/L2 -> LDS with direct-to-LDS loads (no registers, no LDS-write instructions) into a
// ring of four stages.  The vector memory path moves cache lines: a wave instruction that takes 64 bytes from each
// of 16 rows uses half of every 128-byte line it touches and runs at half the rate of one that takes 128 bytes
// from each of 8 rows (measured L2 -> LDS: 17 against 31 TB/s chip-wide).  So whenever the number of stages is
// even (PAIR) the ring is refilled two stages -- one "unit" of 128 bytes per row -- at a time: the unit's LDS image
// has a 128-byte row pitch, one workgroup barrier per unit, one unit in flight while the other is multiplied.
// Runs with an odd number of stages (4-bit codes, K % 256 == 128) keep the stage-by-stage ring, three stages in
// flight while one is multiplied.  Either way the 16-byte pieces of a row are XOR-swizzled with the row index so
// that the 128-bit operand reads of 16 consecutive rows hit 16 distinct 4-bank groups, and wave tiles of
// 128x128 keep LDS reads at 8 operand fragments per 16 matrix instructions.
//
// Scale bytes.  A row's scale bytes for one stage are 4 (or 2) bytes in a line of their own, so fetching them
// stage by stage costs the vector memory path one cache-line access per row per stage - as many accesses as
// the codes themselves.  When K is a multiple of 512 the kernel instead fetches 16 scale bytes per row at a
// time (a "group" of 4 stages of 4-bit codes, 8 stages of 8-bit codes) into a double-buffered LDS area, one
// group ahead.  Other K fall back to one 4-byte scale load per row per stage.
// With the scales in the reference's packed form [rows/128, K/128, 32, 4, 4] (ours/mxfp_attn_kernel.py:56-57) the
// scale bytes of 128 rows x 128 elements of K are one contiguous 512-byte chunk: a stage's scales are four chunks,
// one 32-lane load per wave, and a lane reads its scale words for all four row blocks with one 128-bit LDS read.
#include "mpsa_common.h"

namespace {

constexpr int BM = 256, BN = 256;       // workgroup tile
constexpr int ROWB = 64;                // code bytes per row per stage
constexpr int NSTAGE = 4;               // LDS ring depth
constexpr int OP_BYTES = BM * ROWB;     // one operand's codes per stage (16 KiB)
constexpr int SC_BYTES = BM * 4;        // narrow path: one operand's scale bytes per stage (4 per row)
constexpr int SCG_BYTES = BM * 16;      // wide path: one operand's scale bytes per group (16 per row)
constexpr int CODE_LOADS = 2 * (OP_BYTES / 1024 / 4);   // direct-to-LDS code instructions per wave per stage (8)

template <bool WIDE> constexpr int stage_bytes() { return WIDE ? 2 * OP_BYTES : 2 * OP_BYTES + 2 * SC_BYTES; }
template <bool WIDE> constexpr int smem_bytes() { return NSTAGE * stage_bytes<WIDE>() + (WIDE ? 4 * SCG_BYTES : 0); }

// s_waitcnt immediate: vmcnt(vm), lgkmcnt(0), expcnt untouched
constexpr int wait_imm(int vm) { return 0x0070 | (vm & 15) | ((vm >> 4) << 14); }

struct GemmArgs {
    const uint8_t *a, *sa, *b, *sb;
    void* c;
    int64_t ldc;
    int M, N, K;
    int packed;                // scales in the packed [rows/128, K/128, 32, 4, 4] form instead of [rows, K/32]
    int heads_a, heads_b;      // batched runs: blockIdx.y = batch * heads_a + head; B's head is head / (heads_a / heads_b)
};

template <typename T> __device__ __forceinline__ T cvt_out(float v);
template <> __device__ __forceinline__ float cvt_out<float>(float v) { return v; }
template <> __device__ __forceinline__ __bf16 cvt_out<__bf16>(float v) { return (__bf16)v; }
template <> __device__ __forceinline__ _Float16 cvt_out<_Float16>(float v) { return (_Float16)v; }
// E5M2 output byte, round to nearest even, overflow to infinity (what a float32 -> float8_e5m2 cast does in torch;
// the reference's kernel casts with c.to(tl.float8e5), ours/block_scaled_matmul.py:185-190)
struct OutE5M2 { uint8_t b; };
template <> __device__ __forceinline__ OutE5M2 cvt_out<OutE5M2>(float v) {
    const uint32_t u = mpsa_f2u(v);
    const uint32_t a = u & 0x7FFFFFFFu;
    // 61440 = the largest finite E5M2 value plus half a step: from there on the cast gives infinity (or keeps NaN)
    if (a >= 0x47700000u) return OutE5M2{(uint8_t)(((u >> 24) & 0x80u) | (a > 0x7F800000u ? 0x7Fu : 0x7Cu))};
    // below that the conversion instruction rounds to nearest even, subnormals included
    return OutE5M2{(uint8_t)(__builtin_amdgcn_cvt_pk_bf8_f32(v, v, 0, false) & 0xFF)};
}

// Direct-to-LDS load written as inline assembly: lane L's BYTES bytes at wave_base + lane_off land at
// lds_wave_base + L*BYTES (M0 carries the wave-uniform LDS base; the global address is a scalar base plus a
// 32-bit lane offset, so advancing along K costs scalar additions only).  The compiler's own builtin for this instruction makes it wait for
// every outstanding load (vmcnt(0)) before the next barrier or LDS read, which would drain the ring each stage;
// as assembly the loads are invisible to that bookkeeping and the kernel's explicit partial waits stand.
template <int BYTES>
__device__ __forceinline__ void load_to_lds(uint32_t lane_off, const uint8_t* wave_base, uint8_t* lds_wave_base) {
    // address = wave-uniform base (scalar registers) + the lane's unsigned 32-bit byte offset
    // the low 32 bits of a generic pointer into LDS are the LDS byte address (a cast to the LDS address space
    // would add a null check per load)
    const uint32_t base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds_wave_base);
    const uint64_t gb = (uint64_t)(uintptr_t)wave_base;
    if constexpr (BYTES == 16)
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(base), "v"(lane_off), "s"(gb) : "memory", "m0");
    else
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(base), "v"(lane_off), "s"(gb) : "memory", "m0");
}

// FMT: element format of A (and of B, unless FMTB says otherwise).  FMTB == E2M1 under an 8-bit FMT is the reference's
// "mixed" type (ours/block_scaled_matmul.py:318-324): everything follows the 8-bit geometry -- a stage is 64 elements
// of K, a unit 128 -- except B's codes, which are half as wide: 32 bytes per row and stage, a unit's image 64-byte rows.
template <int FMT, int FMTB, typename OutT, bool WIDE, bool PK, bool PAIR>
__global__ __launch_bounds__(256, 1) void gemm_mx_kernel(GemmArgs g) {
    static_assert(!(WIDE && PK), "packed scales use the per-stage scale area");
    static_assert(NSTAGE == 4, "PAIR: the ring is two units of two stages");
    constexpr bool FP4 = (FMT == MPSA_FMT_E2M1);
    constexpr bool B4 = !FP4 && (FMTB == MPSA_FMT_E2M1);       // 8-bit A against 4-bit B
    static_assert(FMT == FMTB || B4, "the operands share a format, or A is 8-bit and B is E2M1");
    static_assert(!B4 || PAIR, "mixed formats: K % 128 == 0, so the stage count is even");
    constexpr int STAGE_BYTES = stage_bytes<WIDE>();
    constexpr int GROUP = FP4 ? 4 : 8;                 // stages covered by 16 scale bytes of a row
    const int row_bytes = FP4 ? g.K / 2 : g.K;         // code bytes per matrix row (of A)
    const int row_bytes_b = B4 ? g.K / 2 : row_bytes;  // and of B
    const int srow_bytes = g.K / 32;
    const int KT = row_bytes / ROWB;

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* const scg = smem + NSTAGE * STAGE_BYTES;  // wide path: [group parity][operand][row][16]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // the wave index, known to be uniform
    const int wm = wave >> 1, wn = wave & 1;
    const int h = lane >> 5, r = lane & 31;

    // XCD-aware tile order.  Consecutive workgroup ids go to different XCDs (8 of them, each with its own L2) and
    // an XCD starts its workgroups in id order.  Give XCD x one block of a 2 x 4 split of the tile grid and walk
    // that block in panels four tile rows high, column by column: the workgroups running together on an XCD
    // then cover a few tile rows by a few tile columns and share both operands' K-slices in that L2.
    const int tiles_m = g.M / BM, tiles_n = g.N / BN;
    int tm, tn;
    if (tiles_m % 2 == 0 && tiles_n % 4 == 0) {
        const int x = blockIdx.x & 7, j = blockIdx.x >> 3;
        const int rm = tiles_m / 2, rn = tiles_n / 4;
        const int ph = rm % 4 == 0 ? 4 : (rm % 2 == 0 ? 2 : 1);
        const int panel = j / (ph * rn), jj = j % (ph * rn);
        tm = (x >> 2) * rm + panel * ph + jj % ph;
        tn = (x & 3) * rn + jj / ph;
    } else {
        tm = blockIdx.x / tiles_n;
        tn = blockIdx.x % tiles_n;
    }
    const int m0 = tm * BM;
    const int n0 = tn * BN;

    // ---- direct-to-LDS staging: wave w moves chunks [4w, 4w+4) x 1 KiB of either operand and the scale bytes
    //      of rows [64w, 64w+64); chunk position p = row*4 + slot holds row's 16-byte piece slot ^ ((row>>2)&3)
    // batched runs (blockIdx.y): operands of this batch entry; grouped heads share a B operand
    const int bz = blockIdx.y;
    const int bb = bz / g.heads_a, ha = bz - bb * g.heads_a;
    const int64_t zb = (int64_t)bb * g.heads_b + ha / (g.heads_a / g.heads_b);
    g.a += (int64_t)bz * g.M * row_bytes;
    g.sa += (int64_t)bz * g.M * srow_bytes;
    g.b += zb * g.N * row_bytes_b;
    g.sb += zb * g.N * srow_bytes;
    // lane offsets inside a tile's operand (the same for A and B) and inside its scale rows; tile bases are scalar
    // PAIR: a unit = two consecutive stages = 128 code bytes per row, fetched as whole cache lines: an instruction
    // of a wave covers 8 rows x 128 B (half-used lines move at half the rate through the vector memory path).  The
    // unit's LDS image has a 128-byte row pitch; row's 16-byte piece c sits at slot c ^ ((row >> 1) & 7), so that
    // 16 consecutive rows' reads of one piece fall into 16 distinct 4-bank groups.  Instruction x of the unit
    // (wave * 8 + c2, c2 = 0..7) covers rows 8x .. 8x+7: only the parity of c2 enters the lane's swizzle.
    uint32_t lo[4];
    if constexpr (PAIR) {
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const int cb = (lane & 7) ^ (4 * e + ((lane >> 4) & 3));
            lo[e] = (uint32_t)(lane >> 3) * (uint32_t)row_bytes + cb * 16;
        }
        lo[2] = lo[3] = 0;
    } else {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int p = (wave * 4 + c) * 64 + lane;
            const int row = p >> 2, slot = p & 3;
            const int cb = slot ^ ((row >> 2) & 3);
            lo[c] = (uint32_t)row * (uint32_t)row_bytes + cb * 16;
        }
    }
    // mixed formats: a unit of B is 64 bytes per row, fetched like a stage of the stage-by-stage ring (four
    // instructions per wave, row's piece c at slot c ^ ((row >> 2) & 3))
    uint32_t lob[4] = {0, 0, 0, 0};
    if constexpr (B4) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int p = (wave * 4 + c) * 64 + lane;
            const int row = p >> 2, slot = p & 3;
            lob[c] = (uint32_t)row * (uint32_t)row_bytes_b + (slot ^ ((row >> 2) & 3)) * 16;
        }
    }
    const uint32_t los = (uint32_t)(wave * 64 + lane) * (uint32_t)srow_bytes;
    const uint8_t* const a_base = g.a + (int64_t)m0 * row_bytes;
    const uint8_t* const b_base = g.b + (int64_t)n0 * row_bytes_b;
    const uint8_t* const sa_base = g.sa + (int64_t)m0 * srow_bytes;
    const uint8_t* const sb_base = g.sb + (int64_t)n0 * srow_bytes;
    // packed scales (the reference's [rows/128, K/128, 32, 4, 4] form, ours/mxfp_attn_kernel.py:56-57): the scale bytes
    // of 128 rows x 128 elements of K are one 512-byte chunk, byte (row%32)*16 + (row/32)*4 + k.  A stage needs two
    // chunks per operand: waves 0, 1 bring A's, waves 2, 3 B's, each with its first 32 lanes.
    const int kchunks = g.K / 128;
    const uint32_t pko = (uint32_t)((lane & 31) * 16);
    const uint8_t* const s_pk = (wave < 2 ? g.sa + (int64_t)(m0 / 128) * kchunks * 512 : g.sb + (int64_t)(n0 / 128) * kchunks * 512) +
                                (int64_t)(wave & 1) * kchunks * 512;
    // a stage's loads go out in four parts (two code instructions each, the narrow path's scale words with the
    // last) so that they can be spread between the matrix instructions of a step
    // PAIR: part `part` of unit u's loads (four code instructions: two per operand; the scale bytes with the last).
    // Unit u lives in ring half u & 1: [A codes 32 KiB][B codes 32 KiB][scale bytes of its two stages]
    auto unit_base = [&](int u) __attribute__((always_inline)) { return smem + (u & 1) * 2 * STAGE_BYTES; };
    auto issue_unit_part = [&](int u, int part) __attribute__((always_inline)) {
        const int NU = KT / 2;
        const int uc = u < NU ? u : NU - 1;               // past the end: re-load the last unit
        uint8_t* ub = unit_base(u);
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const int c2 = part * 2 + q, x = wave * 8 + c2;
            const int64_t go = (int64_t)uc * (2 * ROWB) + (int64_t)x * 8 * row_bytes;
            load_to_lds<16>(lo[q], a_base + go, ub + x * 1024);
            if constexpr (!B4) load_to_lds<16>(lo[q], b_base + go, ub + 2 * OP_BYTES + x * 1024);
        }
        if constexpr (B4) load_to_lds<16>(lob[part], b_base + (int64_t)uc * ROWB, ub + 2 * OP_BYTES + (wave * 4 + part) * 1024);
        if (part != 3) return;
        uint8_t* sc = ub + 4 * OP_BYTES;
        if constexpr (PK) {
            // 4-bit codes: the unit's two stages are two consecutive 512-byte chunks -- one 64-lane load; 8-bit
            // codes: one chunk covers the unit, the odd stage takes its scale words from the even stage's registers
            if constexpr (FP4) load_to_lds<16>((uint32_t)lane * 16u, s_pk + (int64_t)uc * 1024, sc + wave * 1024);
            else if (lane < 32) load_to_lds<16>(pko, s_pk + (int64_t)uc * 512, sc + wave * 1024);
        } else if constexpr (!WIDE) {
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
                const int sco = FP4 ? (2 * uc + hh) * 4 : uc * 4;
                load_to_lds<4>(los, sa_base + sco, sc + hh * 2 * SC_BYTES + wave * 256);
                load_to_lds<4>(los, sb_base + sco, sc + hh * 2 * SC_BYTES + SC_BYTES + wave * 256);
            }
        }
    };
    auto issue_part = [&](int kt, int part) __attribute__((always_inline)) {
        const int kc = kt < KT ? kt : KT - 1;             // past the end: re-load the last stage (keeps the count uniform)
        uint8_t* st = smem + (kt % NSTAGE) * STAGE_BYTES;
        load_to_lds<16>(lo[part], a_base + (int64_t)kc * ROWB, st + (wave * 4 + part) * 1024);
        load_to_lds<16>(lo[part], b_base + (int64_t)kc * ROWB, st + OP_BYTES + (wave * 4 + part) * 1024);
        if constexpr (PK) {
            // with 8-bit codes a chunk covers two stages and the odd stage's step takes its scale words from the
            // even step's registers, so only even stages fetch (any two consecutive stages still issue the same
            // number of loads, which is what the partial waits count)
            if (part == 3 && (FP4 || (kt & 1) == 0)) {
                const int64_t kb = FP4 ? kc : (kc >> 1);
                if (lane < 32) load_to_lds<16>(pko, s_pk + kb * 512, st + 2 * OP_BYTES + wave * 512);
            }
        } else if constexpr (!WIDE) {
            if (part == 3) {
                // four scale bytes per row: the stage's own with 4-bit codes; with 8-bit codes the aligned word
                // that holds this stage's two bytes (the stage count is even, so the word is inside the row)
                const int sco = FP4 ? kc * 4 : (kc >> 1) * 4;
                load_to_lds<4>(los, sa_base + sco, st + 2 * OP_BYTES + wave * 256);
                load_to_lds<4>(los, sb_base + sco, st + 2 * OP_BYTES + SC_BYTES + wave * 256);
            }
        }
    };
    auto issue_stage = [&](int kt) __attribute__((always_inline)) {
#pragma unroll
        for (int part = 0; part < 4; ++part) issue_part(kt, part);
    };
    auto issue_unit = [&](int u) __attribute__((always_inline)) {
#pragma unroll
        for (int part = 0; part < 4; ++part) issue_unit_part(u, part);
    };
    // wide path: the 16 scale bytes per row of group grp (two instructions per wave)
    auto issue_scales = [&](int grp) __attribute__((always_inline)) {
        const int ng = KT / GROUP;
        const int gc = grp < ng ? grp : ng - 1;
        uint8_t* dst = scg + (grp & 1) * 2 * SCG_BYTES + wave * 1024;
        load_to_lds<16>(los, sa_base + gc * 16, dst);
        load_to_lds<16>(los, sb_base + gc * 16, dst + SCG_BYTES);
    };

    v16f acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    if constexpr (WIDE) issue_scales(0);
    if constexpr (PAIR) {
        issue_unit(0);
        issue_unit(1);
    } else {
#pragma unroll
        for (int s = 0; s < NSTAGE; ++s) issue_stage(s);
    }

    // LDS offsets of this lane's operand rows (row-major 64-byte rows -- PAIR: 128-byte rows --, swizzled chunks)
    int offa[4], offb[4], swz_a[4], swz_b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int ra_ = wm * 128 + i * 32 + r, rb_ = wn * 128 + i * 32 + r;
        if constexpr (B4) {
            offa[i] = ra_ * 2 * ROWB; swz_a[i] = (ra_ >> 1) & 7;
            offb[i] = rb_ * ROWB; swz_b[i] = (rb_ >> 2) & 3;
        } else if constexpr (PAIR) {
            offa[i] = ra_ * 2 * ROWB; swz_a[i] = (ra_ >> 1) & 7;
            offb[i] = rb_ * 2 * ROWB; swz_b[i] = (rb_ >> 1) & 7;
        } else {
            offa[i] = ra_ * ROWB; swz_a[i] = (ra_ >> 2) & 3;
            offb[i] = rb_ * ROWB; swz_b[i] = (rb_ >> 2) & 3;
        }
    }

    // One matrix-instruction step's operands: 4 + 4 fragments and their scale bytes.  Two sets alternate: while
    // the 16 instructions of one set run, the LDS reads of the next set are in flight.
    // Scale bytes: the four bytes of a row's aligned scale word cover an even step and the odd step after it
    // (bytes h and 2+h of the lane half h).  The word is read once, with the even step's operands, shifted right by
    // 8h when that step starts, and handed on to the odd step's set, whose instructions select byte 2.
    struct Frag { v8i a[4], b[4]; int sa[4], sb[4]; uint32_t ra[4], rb[4]; };
    // Wide path, 4-bit codes: a row's 16 scale bytes of the current group are read from LDS ONCE per group with one
    // 128-bit read per row (16 consecutive rows x 16 bytes are conflict-free; a 32-bit read per step pair at this
    // 16-byte row pitch is a four-way bank conflict, and those conflicts were 38 % of the kernel's LDS cycles).
    // Dword k of a row covers step pair k of the group.  With 8-bit codes the operand sets fill the register file:
    // 32 (or, reading half a group at a time, 16) more registers spill and the kernel gets slower, so that path
    // keeps the 32-bit read per step pair.
    constexpr bool GREAD = WIDE && FP4;
    v4i w_a[4], w_b[4];

    // reads operands of step s of stage kt out of the ring: part 0 the B fragments and their scale bytes,
    // part 1 the A fragments and theirs.  grp >= 0 (wide path): also this part's scale rows of group grp.
    auto read_part = [&](Frag& f, const Frag& even, int kt, int s, int part, bool fresh, int grp) __attribute__((always_inline)) {
        const bool isb = part == 0;
        const int hh = kt & 1;                             // PAIR: which stage of its unit
        const uint8_t* st = PAIR ? unit_base(kt >> 1) : smem + (kt % NSTAGE) * STAGE_BYTES;
        const uint8_t* lx = PAIR ? (isb ? st + 2 * OP_BYTES : st) : (isb ? st + OP_BYTES : st);
        const int c0 = PAIR ? 4 * hh : 0;                  // first 16-byte piece of this stage inside the LDS row
        // the row's scale word of this step pair (paths without the per-group read)
        const uint8_t* sc = WIDE ? scg + ((kt / GROUP) & 1) * 2 * SCG_BYTES + 4 * (FP4 ? kt % GROUP : (kt % GROUP) >> 1) + (isb ? SCG_BYTES : 0)
                          : PAIR ? (PK ? st + 4 * OP_BYTES + hh * 512 + (isb ? 2048 : 0)
                                       : st + 4 * OP_BYTES + hh * 2 * SC_BYTES + (isb ? SC_BYTES : 0))
                                 : st + 2 * OP_BYTES + (isb ? SC_BYTES : 0);
        constexpr int sstride = WIDE ? 16 : 4;
        const uint8_t* sg = scg + (grp & 1) * 2 * SCG_BYTES + (isb ? SCG_BYTES : 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = (isb ? wn : wm) * 128 + i * 32 + r;
            const int off = isb ? offb[i] : offa[i], swz = isb ? swz_b[i] : swz_a[i];
            v8i& fx = isb ? f.b[i] : f.a[i];
            if constexpr (GREAD) {
                if (grp >= 0) (isb ? w_b[i] : w_a[i]) = *reinterpret_cast<const v4i*>(sg + row * 16);
                if (!fresh) {
                    if (isb) f.sb[i] = even.sb[i]; else f.sa[i] = even.sa[i];
                }
            } else if (fresh) {
                if constexpr (PK) {
                    // one conflict-free 128-bit read: the scale words of this lane's row in all four row blocks
                    if (i == 0) {
                        const v4i wsc = *reinterpret_cast<const v4i*>(sc + (isb ? wn : wm) * (PAIR ? 1024 : 512) + r * 16);
#pragma unroll
                        for (int q = 0; q < 4; ++q) (isb ? f.rb[q] : f.ra[q]) = (uint32_t)wsc[q];
                    }
                } else {
                    (isb ? f.rb[i] : f.ra[i]) = *reinterpret_cast<const uint32_t*>(sc + row * sstride);
                }
            } else {
                if (isb) f.sb[i] = even.sb[i]; else f.sa[i] = even.sa[i];
            }
            if constexpr (FP4) {
                const v4i x = *reinterpret_cast<const v4i*>(lx + off + (((c0 + 2 * s + h) ^ swz) * 16));
                fx = (v8i){x[0], x[1], x[2], x[3], 0, 0, 0, 0};
            } else if (B4 && isb) {
                // the 4-bit operand of a mixed product: stage hh of the unit is pieces 2hh, 2hh + 1 of the 64-byte row
                const v4i x = *reinterpret_cast<const v4i*>(lx + off + (((2 * hh + h) ^ swz) * 16));
                fx = (v8i){x[0], x[1], x[2], x[3], 0, 0, 0, 0};
            } else {
                // 8-bit operands: registers 0-3 of both lane halves form MX block 0 (scaled by the byte
                // lane half 0 supplies), registers 4-7 form block 1 (scaled by lane half 1's byte)
                const v4i x0 = *reinterpret_cast<const v4i*>(lx + off + (((c0 + h) ^ swz) * 16));
                const v4i x1 = *reinterpret_cast<const v4i*>(lx + off + (((c0 + h + 2) ^ swz) * 16));
                fx = (v8i){x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
            }
        }
    };
    // the four matrix instructions of accumulator row i
    auto multiply_row = [&](const Frag& f, int i, bool odd) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (odd) acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(f.a[i], f.b[j], acc[i][j], FMT, FMTB, 2, f.sa[i], 2, f.sb[j]);
            else     acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(f.a[i], f.b[j], acc[i][j], FMT, FMTB, 0, f.sa[i], 0, f.sb[j]);
        }
    };
    // One step: the 16 matrix instructions on operand set `cur`, in four rows.  Between them go the LDS reads
    // that fill the other set `nxt` with step ns of stage nkt (rows 0 and 1) and, when `refill` is set, the
    // loads of stage lkt into the buffer of stage lkt-NSTAGE (two per row; on the wide path the first stage of
    // a group also brings the next group's scale bytes), so that the matrix pipe keeps running while they issue.
    // `odd`: cur is the odd step of its pair (its scale words were handed on by the even step's set)
    // wide path: `kd` = which dword of the group's scale rows an even step uses; `fetch_grp` >= 0: the refill also
    // fetches that group's scale bytes; `read_grp` >= 0: the operand reads also bring that group's scale rows into
    // registers (the step after the group's last even step, so the registers are free)
    auto step = [&](Frag& cur, Frag& nxt, int nkt, int ns, bool refill, int lkt, bool odd, int kd, int fetch_grp, int read_grp) __attribute__((always_inline)) {
        constexpr int PER = FP4 ? 2 : 3;                   // LDS reads issued behind each matrix instruction
        if (!odd) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if constexpr (GREAD) {
                    cur.sa[i] = (int)((uint32_t)w_a[i][kd] >> (8 * h));
                    cur.sb[i] = (int)((uint32_t)w_b[i][kd] >> (8 * h));
                } else {
                    cur.sa[i] = (int)(cur.ra[i] >> (8 * h));
                    cur.sb[i] = (int)(cur.rb[i] >> (8 * h));
                }
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (refill) {
                if constexpr (PAIR) issue_unit_part(lkt >> 1, i);     // lkt: first stage of the unit to fetch
                else issue_part(lkt, i);
                if constexpr (WIDE) {
                    if (i == 3 && fetch_grp >= 0) issue_scales(fetch_grp);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (i < 2) read_part(nxt, cur, nkt, ns, i, odd, read_grp);   // the step after an odd one starts a new pair
            multiply_row(cur, i, odd);
            if (i < 2) {
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);      // one matrix instruction
                    __builtin_amdgcn_sched_group_barrier(0x100, PER, 0);    // PER LDS reads
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // Every wave has read stage kt into registers.  Wait until stage kt+1 has landed - everything but the loads
    // of the two stages issued last - and meet the other waves; after that stage kt's buffer may be refilled.
    // The next group's scale bytes, fetched with the first stage of a group, land like that stage's codes three
    // stages later, before the next group's first stage is read.  (The wait leaves 16 loads in flight on the
    // wide path although the two stages after a scale fetch amount to 18: waiting for two loads more than
    // needed is harmless and keeps the count a constant.)
    // PAIR: called once per unit, after its second stage has been read: the only loads in flight are the next
    // unit's (and possibly a scale group's), all of which must have landed before that unit is read.
    auto publish = [&]() __attribute__((always_inline)) {
        constexpr int KEEP = PAIR ? 0 : WIDE ? 2 * CODE_LOADS : PK ? (FP4 ? 2 * (CODE_LOADS + 1) : 2 * CODE_LOADS + 1) : 2 * (CODE_LOADS + 2);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(wait_imm(KEEP));
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
    };

    Frag f0, f1;
    {
        // stages 1 .. NSTAGE-1 stay in flight (packed 8-bit: only stage 2 of them carries scale loads)
        // PAIR: unit 1 stays in flight (16 code loads and its scale loads: none, one, or four)
        constexpr int KEEP = PAIR ? (B4 ? CODE_LOADS + CODE_LOADS / 2 : 2 * CODE_LOADS) + (WIDE ? 0 : PK ? 1 : 4)
                           : WIDE ? (NSTAGE - 1) * CODE_LOADS : PK ? (FP4 ? (NSTAGE - 1) * (CODE_LOADS + 1) : (NSTAGE - 1) * CODE_LOADS + 1) : (NSTAGE - 1) * (CODE_LOADS + 2);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(wait_imm(KEEP));
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
    }
    read_part(f0, f0, 0, 0, 0, true, GREAD ? 0 : -1);
    read_part(f0, f0, 0, 0, 1, true, GREAD ? 0 : -1);
    // wide path without the per-group read: the group whose scale bytes the refill of stage kt also fetches
    auto fetch_at = [&](int kt) { return (WIDE && kt % GROUP == (PAIR ? 1 : 0)) ? kt / GROUP + 1 : -1; };
    if constexpr (PAIR && GREAD) {
        // as below, with the ring refilled unit by unit: barrier and refill after a unit's second stage only
        for (int grp = 0; grp < KT / GROUP; ++grp) {
#pragma unroll
            for (int u = 0; u < GROUP; ++u) {
                const int kt = grp * GROUP + u;            // written so that the stage's parity is a constant
                step(f0, f1, kt, 1, false, 0, false, u, -1, -1);
                if (u & 1) publish();
                step(f1, f0, kt + 1, 0, (u & 1) != 0, kt + 3, true, 0, u == 1 ? grp + 1 : -1, u == GROUP - 1 ? grp + 1 : -1);
            }
        }
    } else if constexpr (PAIR && FP4) {
        for (int u2 = 0; u2 < KT / 2; ++u2) {
            const int kt = 2 * u2;
            step(f0, f1, kt, 1, false, 0, false, 0, -1, -1);
            step(f1, f0, kt + 1, 0, false, 0, true, 0, -1, -1);
            step(f0, f1, kt + 1, 1, false, 0, false, 0, -1, -1);
            publish();
            step(f1, f0, kt + 2, 0, true, kt + 4, true, 0, fetch_at(kt + 1), -1);
        }
    } else if constexpr (PAIR) {
        for (int u2 = 0; u2 < KT / 2; ++u2) {
            const int kt = 2 * u2;
            step(f0, f1, kt + 1, 0, false, 0, false, 0, -1, -1);
            publish();
            step(f1, f0, kt + 2, 0, true, kt + 4, true, 0, fetch_at(kt + 1), -1);
        }
    } else if constexpr (GREAD) {
        // one trip = one scale group (4 stages = four step pairs), unrolled so that the dword a pair takes from the
        // group's scale rows, the refill that fetches the next group's scale bytes and the step that reads them
        // into registers are all fixed at compile time
        for (int kt0 = 0; kt0 < KT; kt0 += GROUP) {
            const int grp = kt0 / GROUP;
#pragma unroll
            for (int u = 0; u < GROUP; ++u) {
                const int kt = kt0 + u;
                step(f0, f1, kt, 1, false, 0, false, u, -1, -1);
                publish();
                step(f1, f0, kt + 1, 0, true, kt + NSTAGE, true, 0, u == 0 ? grp + 1 : -1, u == GROUP - 1 ? grp + 1 : -1);
            }
        }
    } else if constexpr (FP4) {
        // a stage is two steps: the second step's operands load under the first step's instructions, and the
        // next stage's first operands (after the barrier that publishes it) under the second step's
        for (int kt = 0; kt < KT; ++kt) {
            step(f0, f1, kt, 1, false, 0, false, 0, -1, -1);
            publish();
            step(f1, f0, kt + 1, 0, true, kt + NSTAGE, true, 0, fetch_at(kt), -1);
        }
    } else {
        // a stage is one step; two stages per trip so that the two operand sets keep their registers
        for (int kt = 0; kt < KT; kt += 2) {
            publish();
            step(f0, f1, kt + 1, 0, true, kt + NSTAGE, false, 0, fetch_at(kt), -1);
            publish();
            step(f1, f0, kt + 2, 0, true, kt + 1 + NSTAGE, true, 0, fetch_at(kt + 1), -1);
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);                // no direct-to-LDS load may outlive the workgroup

    // epilogue: accumulator register e of lane (h, r) is C[8*(e/4) + 4*h + e%4][r] of its 32x32 block
    OutT* c = static_cast<OutT*>(g.c) + (int64_t)bz * g.M * g.ldc;
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

// ---- general kernel: any M and N (edge tiles masked), operands of different element formats ----
// The reference's kernel tiles 128 x 256 with masked edges (ours/block_scaled_matmul.py:154-267) and takes the two
// operands' element widths separately (ELEM_PER_BYTE_A / ELEM_PER_BYTE_B, "mixed" = 8-bit A x 4-bit B,
// ours/block_scaled_matmul.py:318-324).  This kernel covers what the 256 x 256 kernel above does not: a workgroup of
// four waves owns a 128 x 128 tile, a wave 64 x 64 (2 x 2 accumulators), two workgroups share a CU.  K advances
// 128 elements per stage (two matrix-instruction steps; 64 code bytes per row of a 4-bit operand, 128 of an 8-bit
// one): the stage's codes travel L2 -> LDS with direct-to-LDS loads into one of two buffers while the other is
// multiplied, rows XOR-swizzled as in the kernel above; rows past M or N are fetched from the last valid row and
// never stored.  The four scale bytes a row has per stage come straight from global memory as one word, a stage
// ahead (byte by byte when K is not a multiple of 128: the last stage is then half a stage).  Each operand's
// registers follow its own format's layout (4-bit: the lane half's registers are MX block h of the step; 8-bit:
// registers 0-3 of both halves are block 0, 4-7 block 1).
template <int FMT> struct EdgeOp {
    static constexpr bool FP4 = FMT == MPSA_FMT_E2M1;
    static constexpr int ROW = FP4 ? 64 : 128;           // code bytes per row per stage
    static constexpr int CPR = ROW / 16;                 // 16-byte pieces per row
    static constexpr int BYTES = 128 * ROW;              // the operand's codes of one stage
    static constexpr int IPW = BYTES / 1024 / 4;         // direct-to-LDS instructions per wave and stage
    __device__ static __forceinline__ int swz(int row) { return FP4 ? (row >> 2) & 3 : (row >> 1) & 7; }
    // the fragment of matrix-instruction step k (0 / 1) of the stage, LDS row `row` of the operand's stage image
    __device__ static __forceinline__ v8i frag(const uint8_t* img, int row, int k, int h) {
        const uint8_t* p = img + row * ROW;
        const int f = swz(row);
        if constexpr (FP4) {
            const v4i x = *reinterpret_cast<const v4i*>(p + (((2 * k + h) ^ f) * 16));
            return (v8i){x[0], x[1], x[2], x[3], 0, 0, 0, 0};
        } else {
            const v4i x0 = *reinterpret_cast<const v4i*>(p + (((4 * k + h) ^ f) * 16));
            const v4i x1 = *reinterpret_cast<const v4i*>(p + (((4 * k + h + 2) ^ f) * 16));
            return (v8i){x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
        }
    }
};

// scale byte of row `row`, MX block kb: row-major [rows, K/32] or the packed [rows/128, K/128, 32, 4, 4] form
__device__ __forceinline__ int load_scale(const uint8_t* s, int row, int kb, int kblocks, bool packed) {
    if (!packed) return s[(int64_t)row * kblocks + kb];
    const int64_t chunk = (int64_t)(row >> 7) * (kblocks >> 2) + (kb >> 2);
    return s[chunk * 512 + (row & 31) * 16 + ((row >> 5) & 3) * 4 + (kb & 3)];
}

template <int FA, int FB>
constexpr int general_smem() { return 2 * (EdgeOp<FA>::BYTES + EdgeOp<FB>::BYTES); }

template <int FA, int FB, typename OutT>
__global__ __launch_bounds__(256, 2) void gemm_mx_general_kernel(GemmArgs g) {
    typedef EdgeOp<FA> OA;
    typedef EdgeOp<FB> OB;
    constexpr int STAGE = OA::BYTES + OB::BYTES;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int h = lane >> 5, r = lane & 31;
    const int rowb_a = OA::FP4 ? g.K / 2 : g.K;
    const int rowb_b = OB::FP4 ? g.K / 2 : g.K;
    const int kblocks = g.K / 32;
    const int tiles_n = (g.N + 127) / 128;
    const int tm0 = (blockIdx.x / tiles_n) * 128, tn0 = (blockIdx.x % tiles_n) * 128;   // the workgroup's tile
    const int m0 = tm0 + wm * 64, n0 = tn0 + wn * 64;                                   // the wave's
    const int bz = blockIdx.y;
    const int bb = bz / g.heads_a, ha = bz - bb * g.heads_a;
    const int64_t zb = (int64_t)bb * g.heads_b + ha / (g.heads_a / g.heads_b);
    const uint8_t* a = g.a + (int64_t)bz * g.M * rowb_a;
    const uint8_t* b = g.b + zb * g.N * rowb_b;
    const uint8_t* sa = g.sa + (int64_t)bz * g.M * kblocks;
    const uint8_t* sb = g.sb + zb * g.N * kblocks;
    const int steps = g.K / 64;                          // matrix-instruction steps
    const int nstages = (steps + 1) / 2;                 // the last stage is half a stage when `steps` is odd
    const bool words = (g.K % 128) == 0;                 // a row's four scale bytes of a stage are one aligned word

    // ---- staging: lane offsets of this wave's pieces (rows past the matrix clamp to its last row) ----
    uint32_t loa[OA::IPW], lob[OB::IPW];
    bool firsta[OA::IPW], firstb[OB::IPW];               // the piece lies in the stage's first half (first step)
#pragma unroll
    for (int c = 0; c < OA::IPW; ++c) {
        const int p = (wave * OA::IPW + c) * 64 + lane;
        const int row = p / OA::CPR, cb = (p % OA::CPR) ^ OA::swz(row);
        loa[c] = (uint32_t)min(tm0 + row, g.M - 1) * (uint32_t)rowb_a + cb * 16;
        firsta[c] = cb < OA::CPR / 2;
    }
#pragma unroll
    for (int c = 0; c < OB::IPW; ++c) {
        const int p = (wave * OB::IPW + c) * 64 + lane;
        const int row = p / OB::CPR, cb = (p % OB::CPR) ^ OB::swz(row);
        lob[c] = (uint32_t)min(tn0 + row, g.N - 1) * (uint32_t)rowb_b + cb * 16;
        firstb[c] = cb < OB::CPR / 2;
    }
    auto issue = [&](int s) __attribute__((always_inline)) {
        uint8_t* st = smem + (s & 1) * STAGE;
        const bool half = 2 * s + 1 >= steps;            // only the stage's first step exists
#pragma unroll
        for (int c = 0; c < OA::IPW; ++c)
            if (!half || firsta[c]) load_to_lds<16>(loa[c], a + (int64_t)s * OA::ROW, st + (wave * OA::IPW + c) * 1024);
#pragma unroll
        for (int c = 0; c < OB::IPW; ++c)
            if (!half || firstb[c]) load_to_lds<16>(lob[c], b + (int64_t)s * OB::ROW, st + OA::BYTES + (wave * OB::IPW + c) * 1024);
    };

    // ---- this lane's rows (for the scale bytes) and the scale words of a stage ----
    int ra[2], rb[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        ra[i] = min(m0 + i * 32 + r, g.M - 1);
        rb[i] = min(n0 + i * 32 + r, g.N - 1);
    }
    auto scale_word = [&](const uint8_t* sc, int row, int s) __attribute__((always_inline)) -> uint32_t {
        if (words) {
            const int64_t off = g.packed ? ((int64_t)(row >> 7) * (kblocks >> 2) + s) * 512 + (row & 31) * 16 + ((row >> 5) & 3) * 4
                                         : (int64_t)row * kblocks + 4 * s;
            return *reinterpret_cast<const uint32_t*>(sc + off);
        }
        uint32_t w = 0;                                  // K % 128 == 64 (row-major scales only): byte by byte
#pragma unroll
        for (int q = 0; q < 4; ++q)
            if (4 * s + q < kblocks) w |= (uint32_t)load_scale(sc, row, 4 * s + q, kblocks, false) << (8 * q);
        return w;
    };
    uint32_t wa[2], wb[2], na[2] = {0, 0}, nb[2] = {0, 0};
    auto fetch_scales = [&](int s, uint32_t (&xa)[2], uint32_t (&xb)[2]) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            xa[i] = scale_word(sa, ra[i], s);
            xb[i] = scale_word(sb, rb[i], s);
        }
    };

    v16f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    issue(0);
    fetch_scales(0, wa, wb);
    for (int s = 0; s < nstages; ++s) {
        // stage s has landed for every wave, and every wave is through with the buffer stage s + 1 goes to
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(0x0070);
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        if (s + 1 < nstages) {
            issue(s + 1);
            fetch_scales(s + 1, na, nb);
        }
        const uint8_t* ia = smem + (s & 1) * STAGE;
        const uint8_t* ib = ia + OA::BYTES;
        const int nk = min(2, steps - 2 * s);
        for (int k = 0; k < nk; ++k) {
            v8i fa[2], fb[2];
            int ca[2], cb[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                fa[i] = OA::frag(ia, wm * 64 + i * 32 + r, k, h);
                fb[i] = OB::frag(ib, wn * 64 + i * 32 + r, k, h);
                ca[i] = (int)(wa[i] >> (8 * (2 * k + h)));       // the matrix instruction takes the low byte
                cb[i] = (int)(wb[i] >> (8 * (2 * k + h)));
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[j], acc[i][j], FA, FB, 0, ca[i], 0, cb[j]);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) { wa[i] = na[i]; wb[i] = nb[i]; }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);                  // no direct-to-LDS load may outlive the workgroup

    // accumulator register e of lane (h, r) is C[8*(e/4) + 4*h + e%4][r] of its 32 x 32 block
    OutT* c = static_cast<OutT*>(g.c) + (int64_t)bz * g.M * g.ldc;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int col = n0 + j * 32 + r;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int row = m0 + i * 32 + 8 * (e >> 2) + 4 * h + (e & 3);
                if (row < g.M && col < g.N) c[(int64_t)row * g.ldc + col] = cvt_out<OutT>(acc[i][j][e]);
            }
        }
}

template <int FA, int FB, typename OutT>
struct GeneralLds {
    static inline const bool registered =
        mpsa_register_lds_kernel(reinterpret_cast<const void*>(gemm_mx_general_kernel<FA, FB, OutT>), general_smem<FA, FB>());
};

template <int FA, int FB, typename OutT>
void launch_general_kernel(const GemmArgs& g, dim3 grid, hipStream_t st) {
    if (!GeneralLds<FA, FB, OutT>::registered) return;
    constexpr int lds = general_smem<FA, FB>();
    hipLaunchKernelGGL((gemm_mx_general_kernel<FA, FB, OutT>), grid, dim3(256), lds, st, g);
}

template <int FA, int FB>
void launch_general_out(const GemmArgs& g, int c_dtype, dim3 grid, hipStream_t st) {
    if (c_dtype == MPSA_BF16)        launch_general_kernel<FA, FB, __bf16>(g, grid, st);
    else if (c_dtype == MPSA_F8E5M2) launch_general_kernel<FA, FB, OutE5M2>(g, grid, st);
    else if (c_dtype == MPSA_F16)    launch_general_kernel<FA, FB, _Float16>(g, grid, st);
    else                             launch_general_kernel<FA, FB, float>(g, grid, st);
}

template <int FA>
void launch_general_b(const GemmArgs& g, int fmt_b, int c_dtype, dim3 grid, hipStream_t st) {
    if (fmt_b == MPSA_FMT_E2M1)      launch_general_out<FA, MPSA_FMT_E2M1>(g, c_dtype, grid, st);
    else if (fmt_b == MPSA_FMT_E4M3) launch_general_out<FA, MPSA_FMT_E4M3>(g, c_dtype, grid, st);
    else                             launch_general_out<FA, MPSA_FMT_E5M2>(g, c_dtype, grid, st);
}

void launch_general(const GemmArgs& g, int fmt_a, int fmt_b, int c_dtype, dim3 grid, hipStream_t st) {
    if (fmt_a == MPSA_FMT_E2M1)      launch_general_b<MPSA_FMT_E2M1>(g, fmt_b, c_dtype, grid, st);
    else if (fmt_a == MPSA_FMT_E4M3) launch_general_b<MPSA_FMT_E4M3>(g, fmt_b, c_dtype, grid, st);
    else                             launch_general_b<MPSA_FMT_E5M2>(g, fmt_b, c_dtype, grid, st);
}

// MPSA_GEMM_GENERAL=1 in the environment sends every shape to the general kernel (cross-checking)
bool force_general() {
    static const bool on = [] {
        const char* v = getenv("MPSA_GEMM_GENERAL");
        return v && v[0] == '1';
    }();
    return on;
}

template <int FMT, int FMTB, typename OutT, bool WIDE, bool PK, bool PAIR>
struct GemmLds {
    static inline const bool registered =
        mpsa_register_lds_kernel(reinterpret_cast<const void*>(gemm_mx_kernel<FMT, FMTB, OutT, WIDE, PK, PAIR>), smem_bytes<WIDE>());
};

template <int FMT, int FMTB, typename OutT, bool WIDE, bool PK, bool PAIR>
void launch_kernel(const GemmArgs& g, dim3 grid, hipStream_t st) {
    if (!GemmLds<FMT, FMTB, OutT, WIDE, PK, PAIR>::registered) return;
    hipLaunchKernelGGL((gemm_mx_kernel<FMT, FMTB, OutT, WIDE, PK, PAIR>), grid, dim3(256), smem_bytes<WIDE>(), st, g);
}

template <int FMT, int FMTB, typename OutT, bool PAIR>
void launch_scales(const GemmArgs& g, dim3 grid, hipStream_t st) {
    if (g.packed)            launch_kernel<FMT, FMTB, OutT, false, true, PAIR>(g, grid, st);
    else if (g.K % 512 == 0) launch_kernel<FMT, FMTB, OutT, true, false, PAIR>(g, grid, st);
    else                     launch_kernel<FMT, FMTB, OutT, false, false, PAIR>(g, grid, st);
}

template <int FMT, int FMTB, typename OutT>
void launch_one(const GemmArgs& g, dim3 grid, hipStream_t st) {
    // whole cache lines per row (two stages at a time) need an even number of stages: always so with 8-bit codes
    // (K % 128 == 0), with 4-bit codes when K % 256 == 0
    if constexpr (FMT != MPSA_FMT_E2M1) {
        launch_scales<FMT, FMTB, OutT, true>(g, grid, st);
    } else {
        if (g.K % 256 == 0) launch_scales<FMT, FMTB, OutT, true>(g, grid, st);
        else                launch_scales<FMT, FMTB, OutT, false>(g, grid, st);
    }
}

template <int FMT, int FMTB>
void launch_fmt(const GemmArgs& g, int c_dtype, dim3 grid, hipStream_t st) {
    if (c_dtype == MPSA_BF16)      launch_one<FMT, FMTB, __bf16>(g, grid, st);
    else if (c_dtype == MPSA_F8E5M2) launch_one<FMT, FMTB, OutE5M2>(g, grid, st);
    else if (c_dtype == MPSA_F16)  launch_one<FMT, FMTB, _Float16>(g, grid, st);
    else                           launch_one<FMT, FMTB, float>(g, grid, st);
}

}  // namespace

static bool known_fmt(int f) { return f == MPSA_FMT_E2M1 || f == MPSA_FMT_E4M3 || f == MPSA_FMT_E5M2; }

static int gemm_entry(const uint8_t* a, const uint8_t* sa, int fmt_a, const uint8_t* b, const uint8_t* sb, int fmt_b, bool packed,
                      int64_t batch, int64_t heads_a, int64_t heads_b, int64_t M, int64_t N, int64_t K,
                      void* c, int c_dtype, int64_t ldc, mpsa_stream_t stream) {
    if (!a || !sa || !b || !sb || !c) return mpsa_fail(MPSA_EINVAL, "gemm: null pointer");
    if (!known_fmt(fmt_a) || !known_fmt(fmt_b)) return mpsa_fail(MPSA_EINVAL, "gemm: unknown format %d / %d", fmt_a, fmt_b);
    if (c_dtype != MPSA_BF16 && c_dtype != MPSA_F16 && c_dtype != MPSA_F32 && c_dtype != MPSA_F8E5M2) return mpsa_fail(MPSA_EINVAL, "gemm: unsupported output dtype %d", c_dtype);
    if (M <= 0 || N <= 0 || K <= 0 || ldc < N) return mpsa_fail(MPSA_EINVAL, "gemm: bad shape");
    if (batch <= 0 || heads_a <= 0 || heads_b <= 0 || heads_a % heads_b) return mpsa_fail(MPSA_EINVAL, "gemm: bad batch shape (batch=%lld heads_a=%lld heads_b=%lld)", (long long)batch, (long long)heads_a, (long long)heads_b);
    if (K % 64) return mpsa_fail(MPSA_EUNSUPPORTED, "gemm: K must be a multiple of 64 (got %lld)", (long long)K);
    if (packed && (M % 128 || N % 128 || K % 128)) return mpsa_fail(MPSA_EUNSUPPORTED, "gemm: packed scales need M, N and K in multiples of 128 (got %lld,%lld,%lld)", (long long)M, (long long)N, (long long)K);
    if (M > (1 << 30) || N > (1 << 30) || K > (1 << 24) || ((M + 127) / 128) * ((N + 127) / 128) > (int64_t(1) << 30) || batch * heads_a > 65535)
        return mpsa_fail(MPSA_EUNSUPPORTED, "gemm: shape too large");
    if (!mpsa_aligned16(a) || !mpsa_aligned16(b) || (reinterpret_cast<uintptr_t>(sa) & 3) || (reinterpret_cast<uintptr_t>(sb) & 3))
        return mpsa_fail(MPSA_EALIGN, "gemm: codes must be 16-byte and scales 4-byte aligned");
    if (packed && (!mpsa_aligned16(sa) || !mpsa_aligned16(sb))) return mpsa_fail(MPSA_EALIGN, "gemm: packed scales must be 16-byte aligned");
    GemmArgs g;
    g.a = a; g.sa = sa; g.b = b; g.sb = sb; g.c = c; g.ldc = ldc;
    g.M = (int)M; g.N = (int)N; g.K = (int)K;
    g.heads_a = (int)heads_a; g.heads_b = (int)heads_b;
    g.packed = packed ? 1 : 0;
    hipStream_t st = (hipStream_t)stream;
    const int rc = mpsa_ensure_init();
    if (rc != MPSA_OK) return rc;
    // whole 256 x 256 tiles of one element format, or of an 8-bit A against a 4-bit B (the reference's "mixed" type):
    // the LDS-staged kernel; everything else: the general one
    const bool mixed = fmt_a != MPSA_FMT_E2M1 && fmt_b == MPSA_FMT_E2M1;
    if ((fmt_a == fmt_b || mixed) && M % BM == 0 && N % BN == 0 && K % 128 == 0 && !force_general()) {
        dim3 grid((unsigned)((M / BM) * (N / BN)), (unsigned)(batch * heads_a));
        if (fmt_a == MPSA_FMT_E2M1)      launch_fmt<MPSA_FMT_E2M1, MPSA_FMT_E2M1>(g, c_dtype, grid, st);
        else if (fmt_a == MPSA_FMT_E4M3) mixed ? launch_fmt<MPSA_FMT_E4M3, MPSA_FMT_E2M1>(g, c_dtype, grid, st) : launch_fmt<MPSA_FMT_E4M3, MPSA_FMT_E4M3>(g, c_dtype, grid, st);
        else                             mixed ? launch_fmt<MPSA_FMT_E5M2, MPSA_FMT_E2M1>(g, c_dtype, grid, st) : launch_fmt<MPSA_FMT_E5M2, MPSA_FMT_E5M2>(g, c_dtype, grid, st);
    } else {
        dim3 grid((unsigned)(((M + 127) / 128) * ((N + 127) / 128)), (unsigned)(batch * heads_a));
        launch_general(g, fmt_a, fmt_b, c_dtype, grid, st);
    }
    MPSA_CHECK_LAUNCH("gemm");
    return MPSA_OK;
}

extern "C" int mpsa_gemm_mx_batched(const uint8_t* a, const uint8_t* sa, int fmt_a, const uint8_t* b, const uint8_t* sb, int fmt_b,
                                    int64_t batch, int64_t heads_a, int64_t heads_b, int64_t M, int64_t N, int64_t K,
                                    void* c, int c_dtype, int64_t ldc, mpsa_stream_t stream) {
    return gemm_entry(a, sa, fmt_a, b, sb, fmt_b, false, batch, heads_a, heads_b, M, N, K, c, c_dtype, ldc, stream);
}

extern "C" int mpsa_gemm_mx(const uint8_t* a, const uint8_t* sa, int fmt_a, const uint8_t* b, const uint8_t* sb, int fmt_b,
                            int64_t M, int64_t N, int64_t K, void* c, int c_dtype, int64_t ldc, mpsa_stream_t stream) {
    return gemm_entry(a, sa, fmt_a, b, sb, fmt_b, false, 1, 1, 1, M, N, K, c, c_dtype, ldc, stream);
}

extern "C" int mpsa_gemm_mx_packed(const uint8_t* a, const uint8_t* sa5, int fmt_a, const uint8_t* b, const uint8_t* sb5, int fmt_b,
                                   int64_t M, int64_t N, int64_t K, void* c, int c_dtype, int64_t ldc, mpsa_stream_t stream) {
    return gemm_entry(a, sa5, fmt_a, b, sb5, fmt_b, true, 1, 1, 1, M, N, K, c, c_dtype, ldc, stream);
}

extern "C" int mpsa_gemm_mx_batched_packed(const uint8_t* a, const uint8_t* sa5, int fmt_a, const uint8_t* b, const uint8_t* sb5, int fmt_b,
                                           int64_t batch, int64_t heads_a, int64_t heads_b, int64_t M, int64_t N, int64_t K,
                                           void* c, int c_dtype, int64_t ldc, mpsa_stream_t stream) {
    return gemm_entry(a, sa5, fmt_a, b, sb5, fmt_b, true, batch, heads_a, heads_b, M, N, K, c, c_dtype, ldc, stream);
}
