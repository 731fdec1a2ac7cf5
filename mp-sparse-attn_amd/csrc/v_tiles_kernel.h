// The value-tile repack's per-workgroup body, shared by v_tiles.hip and prepare.hip (layout: top of v_tiles.hip).
#pragma once
#include "mpsa_common.h"


struct VTArgs {
    const unsigned short* v;
    int64_t sb, sh, sn;
    int n, nt;
    unsigned short* out;
};

// host side, defined in v_tiles.hip: validates and fills the argument block; *blocks = workgroups per (batch, head)
int mpsa_v_tiles_setup(const void* v, int v_dtype, int64_t B, int64_t H, int64_t N, int64_t D, const int64_t* v_strides,
                       int tile, void* v_tiles, VTArgs* out, unsigned* blocks);

namespace {


// One workgroup's share: 256 consecutive 16-byte output words, starting at word 256*bx, of head hh of batch bb.
template <int TILE, int D>
__device__ __forceinline__ void v_tiles_block(const VTArgs& a, uint32_t bx, uint32_t hh, uint32_t bb, uint32_t nh) {
    constexpr int NDB = D / 32;
    constexpr int KB = TILE / 32;
    const uint32_t per_head = (uint32_t)a.nt * (TILE * D / 8);
    const uint32_t o = bx * 256u + threadIdx.x;
    if (o >= per_head) return;
    const uint32_t lane = o & 63u;
    uint32_t rest = o >> 6;
    const uint32_t db = rest % NDB; rest /= NDB;
    const uint32_t c = rest & 1u;   rest >>= 1;
    const uint32_t kb = rest % KB;
    const uint32_t it = rest / KB;
    const uint32_t h = lane >> 5, r = lane & 31u;
    const uint32_t key0 = TILE * it + 32u * kb + 16u * c + 4u * h;
    const unsigned short* src = a.v + (int64_t)bb * a.sb + (int64_t)hh * a.sh + (32u * db + r);
    v8us val;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
        const uint32_t key = key0 + 8u * (t >> 2) + (t & 3);
        val[t] = key < (uint32_t)a.n ? src[(int64_t)key * a.sn] : (unsigned short)0;
    }
    const int64_t head = (int64_t)bb * nh + hh;
    reinterpret_cast<v8us*>(a.out)[head * per_head + o] = val;
}

template <int TILE, int D>
__global__ __launch_bounds__(256) void v_tiles_kernel(VTArgs a) {
    v_tiles_block<TILE, D>(a, blockIdx.x, blockIdx.y, blockIdx.z, gridDim.y);
}

}  // namespace

