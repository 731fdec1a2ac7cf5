// Value-tile repack for the fused attention kernel (gfx950).
//
// The P.V product runs as O^T += V^T P^T on v_mfma_f32_32x32x16_{bf16,f16}: the V^T operand of one
// instruction is a 32(dim) x 16(key) block of which lane (h = lane/32, r = lane%32) supplies eight
// 16-bit values, dim 32*db + r, for the eight keys whose scores that same lane pair holds after the
// score MFMA.  This kernel writes V so that those eight values are one aligned 16-byte word and the
// 64 lanes of a wave read 1 KiB contiguously:
//
//   out[b][h][it][kb][c][db][lane][t] = v[b][h][key][32*db + r]
//   key = tile*it + 32*kb + 16*c + 8*(t/4) + 4*(lane/32) + t%4,  r = lane%32,  keys >= N read as zero.
//
// Replaces the reference wrapper's V normalisation (ours/mxfp_attn_kernel.py:27-31).  HBM-bound:
// 2 B/element in, 2 B/element out.
#include "mpsa_common.h"

namespace {

struct VTArgs {
    const unsigned short* v;
    int64_t sb, sh, sn;
    int n, nt;
    unsigned short* out;
};

template <int TILE, int D>
__global__ __launch_bounds__(256) void v_tiles_kernel(VTArgs a) {
    constexpr int NDB = D / 32;
    constexpr int KB = TILE / 32;
    const uint32_t per_head = (uint32_t)a.nt * (TILE * D / 8);
    const uint32_t o = blockIdx.x * 256u + threadIdx.x;
    if (o >= per_head) return;
    const uint32_t lane = o & 63u;
    uint32_t rest = o >> 6;
    const uint32_t db = rest % NDB; rest /= NDB;
    const uint32_t c = rest & 1u;   rest >>= 1;
    const uint32_t kb = rest % KB;
    const uint32_t it = rest / KB;
    const uint32_t h = lane >> 5, r = lane & 31u;
    const uint32_t key0 = TILE * it + 32u * kb + 16u * c + 4u * h;
    const unsigned short* src = a.v + (int64_t)blockIdx.z * a.sb + (int64_t)blockIdx.y * a.sh + (32u * db + r);
    v8us val;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const uint32_t key = key0 + 8u * (t >> 2) + (t & 3);
        val[t] = key < (uint32_t)a.n ? src[(int64_t)key * a.sn] : (unsigned short)0;
    }
    const int64_t head = (int64_t)blockIdx.z * gridDim.y + blockIdx.y;
    reinterpret_cast<v8us*>(a.out)[head * per_head + o] = val;
}

}  // namespace

extern "C" int mpsa_v_tiles(const void* v, int v_dtype, int64_t B, int64_t H, int64_t N, int64_t D,
                            const int64_t v_strides[4], int tile, void* v_tiles, mpsa_stream_t stream) {
    if (!v || !v_tiles || !v_strides) return mpsa_fail(MPSA_EINVAL, "v_tiles: null pointer");
    if (v_dtype != MPSA_BF16 && v_dtype != MPSA_F16) return mpsa_fail(MPSA_EINVAL, "v_tiles: dtype must be bf16 or f16");
    if (B < 0 || H < 0 || N <= 0) return mpsa_fail(MPSA_EINVAL, "v_tiles: bad shape");
    if (v_strides[3] != 1) return mpsa_fail(MPSA_EINVAL, "v_tiles: last dim must be contiguous");
    if (!mpsa_aligned16(v_tiles)) return mpsa_fail(MPSA_EALIGN, "v_tiles: output must be 16-byte aligned");
    if ((D != 64 && D != 128) || (tile != 64 && tile != 128))
        return mpsa_fail(MPSA_EUNSUPPORTED, "v_tiles: D=%lld tile=%d (D and tile must be 64 or 128)", (long long)D, tile);
    if (B == 0 || H == 0) return MPSA_OK;
    const int64_t nt = (N + tile - 1) / tile;
    const int64_t per_head = nt * (tile * D / 8);
    if (per_head >= (int64_t(1) << 31) || H > 65535 || B > 65535) return mpsa_fail(MPSA_EUNSUPPORTED, "v_tiles: tensor too large");
    VTArgs a;
    a.v = static_cast<const unsigned short*>(v);
    a.sb = v_strides[0]; a.sh = v_strides[1]; a.sn = v_strides[2];
    a.n = (int)N; a.nt = (int)nt;
    a.out = static_cast<unsigned short*>(v_tiles);
    dim3 grid((unsigned)((per_head + 255) / 256), (unsigned)H, (unsigned)B);
    hipStream_t st = (hipStream_t)stream;
    if (tile == 128 && D == 128)      hipLaunchKernelGGL((v_tiles_kernel<128, 128>), grid, dim3(256), 0, st, a);
    else if (tile == 128 && D == 64)  hipLaunchKernelGGL((v_tiles_kernel<128, 64>), grid, dim3(256), 0, st, a);
    else if (tile == 64 && D == 128)  hipLaunchKernelGGL((v_tiles_kernel<64, 128>), grid, dim3(256), 0, st, a);
    else                              hipLaunchKernelGGL((v_tiles_kernel<64, 64>), grid, dim3(256), 0, st, a);
    MPSA_CHECK_LAUNCH("v_tiles");
    return MPSA_OK;
}
