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
#include "v_tiles_kernel.h"

int mpsa_v_tiles_setup(const void* v, int v_dtype, int64_t B, int64_t H, int64_t N, int64_t D, const int64_t* v_strides,
                       int tile, void* v_tiles, VTArgs* out, unsigned* blocks) {
    *blocks = 0;
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
    VTArgs& a = *out;
    a.v = static_cast<const unsigned short*>(v);
    a.sb = v_strides[0]; a.sh = v_strides[1]; a.sn = v_strides[2];
    a.n = (int)N; a.nt = (int)nt;
    a.out = static_cast<unsigned short*>(v_tiles);
    *blocks = (unsigned)((per_head + 255) / 256);
    return MPSA_OK;
}

extern "C" int mpsa_v_tiles(const void* v, int v_dtype, int64_t B, int64_t H, int64_t N, int64_t D,
                            const int64_t v_strides[4], int tile, void* v_tiles, mpsa_stream_t stream) {
    VTArgs a;
    unsigned blocks = 0;
    const int rc = mpsa_v_tiles_setup(v, v_dtype, B, H, N, D, v_strides, tile, v_tiles, &a, &blocks);
    if (rc != MPSA_OK || blocks == 0) return rc;
    dim3 grid(blocks, (unsigned)H, (unsigned)B);
    hipStream_t st = (hipStream_t)stream;
    if (tile == 128 && D == 128)      hipLaunchKernelGGL((v_tiles_kernel<128, 128>), grid, dim3(256), 0, st, a);
    else if (tile == 128 && D == 64)  hipLaunchKernelGGL((v_tiles_kernel<128, 64>), grid, dim3(256), 0, st, a);
    else if (tile == 64 && D == 128)  hipLaunchKernelGGL((v_tiles_kernel<64, 128>), grid, dim3(256), 0, st, a);
    else                              hipLaunchKernelGGL((v_tiles_kernel<64, 64>), grid, dim3(256), 0, st, a);
    MPSA_CHECK_LAUNCH("v_tiles");
    return MPSA_OK;
}
