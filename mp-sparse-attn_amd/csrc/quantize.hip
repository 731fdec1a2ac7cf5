// MX quantizer for gfx950: bf16/f16 rows -> E2M1 / E4M3 / E5M2 codes + one E8M0 scale per 32 elements.
//
// Semantics follow the reference's quantizer (ours/quant_mxint8.py:276-351 for E2M1, :164-219 for the
// 8-bit format): x32 = f32(x) * pre; amax per 32 elements of the last dim; shared exponent
// floor(log2(amax)) - emax_elem; divide by that power of two; clamp; encode; scale byte
// clamp(shared_exp + 127, 0, 254).  The E2M1 encoder reproduces MXFP4Tensor._from_float
// (ours/mxfp.py:84-170) bit for bit, including its float32 1e-6 tie-break bias; codes leave the
// kernel already nibble-packed (ours/mxfp.py:196-205: even element in the low nibble).
//
// Smooth-K (ours/mxfp_attn.py:44-45, ours/mxfp_attn_kernel.py:33-34: k = k - k.mean(dim=-2, keepdim=True) in k's
// 16-bit dtype) is folded in: seq_mean_kernel + seq_mean_finish_kernel produce the per-(batch, head, channel) mean
// over the sequence, rounded to the input dtype, and the quantizer subtracts it - rounding the difference to the
// input dtype again, as the elementwise torch op would - before it does anything else.
//
// Work mapping: one lane owns 8 consecutive elements (one 128-bit load), four neighbouring lanes
// own one MX block, so the block maximum is two DPP quad exchanges.  The kernel is HBM-bound:
// 2 B/element in, 0.5 (+1) B/element of codes and 1/32 (x2) B/element of scales out.
#include "quantize_kernel.h"
#include <cstring>
#include <mutex>

namespace {

// ---- mean over the sequence, per (batch, head, channel) ----
constexpr int MEAN_ROWS = 256;     // rows per partial sum

struct MeanArgs {
    const void* x;
    int64_t sb, sh, sn;
    int n, d, nchunk;
    float* partial;            // [B,H,nchunk,D]
    void* mean;                // [B,H,D] of x's dtype
    float inv_n;
};

// One workgroup sums MEAN_ROWS rows of one head: a thread owns 8 channels of every (256*8/D)-th row; the row
// groups are then added in a fixed order through LDS, so the result does not depend on timing.
template <int XDT>
__global__ __launch_bounds__(256) void seq_mean_kernel(MeanArgs a) {
    __shared__ float part[256][9];
    const int cpr = a.d >> 3;                    // 8-channel groups per row (8 or 16)
    const int rthreads = 256 / cpr;
    const int cg = threadIdx.x % cpr, rt = threadIdx.x / cpr;
    const int chunk = blockIdx.x;
    const int row0 = chunk * MEAN_ROWS;
    const int row1 = min(row0 + MEAN_ROWS, a.n);
    const char* base = static_cast<const char*>(a.x) + 2 * ((int64_t)blockIdx.z * a.sb + (int64_t)blockIdx.y * a.sh + 8 * (int64_t)cg);
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int row = row0 + rt; row < row1; row += rthreads) {
        float x[8];
        load8<XDT>(base + 2 * (int64_t)row * a.sn, x);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] += x[i];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) part[threadIdx.x][i] = acc[i];
    __syncthreads();
    if (threadIdx.x < a.d) {
        const int c = threadIdx.x;               // channel
        float s = 0.0f;
        for (int t = 0; t < rthreads; ++t) s += part[t * cpr + (c >> 3)][c & 7];
        const int64_t head = (int64_t)blockIdx.z * gridDim.y + blockIdx.y;
        a.partial[(head * a.nchunk + chunk) * a.d + c] = s;
    }
}

// adds a head's partial sums in chunk order, multiplies by 1/N (float32) and rounds to the 16-bit dtype
template <int XDT>
__global__ __launch_bounds__(128) void seq_mean_finish_kernel(MeanArgs a) {
    const int c = threadIdx.x;
    if (c >= a.d) return;
    const int64_t head = blockIdx.x;
    float s = 0.0f;
    for (int k = 0; k < a.nchunk; ++k) s += a.partial[(head * a.nchunk + k) * a.d + c];
    const float m = s * a.inv_n;
    if constexpr (XDT == MPSA_BF16) {
        const uint32_t u = mpsa_f2u(m);
        static_cast<uint16_t*>(a.mean)[head * a.d + c] = (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
    } else {
        static_cast<_Float16*>(a.mean)[head * a.d + c] = (_Float16)m;
    }
}

// MPSA_FP8_ENCODE=sw or MPSA_FP4_ENCODE=sw in the environment selects the kernels that encode with explicit
// integer/float arithmetic only (no hardware conversion instructions), for cross-checking
bool use_sw_fp8() {
    static const bool sw = [] {
        const char* v = getenv("MPSA_FP8_ENCODE");
        const char* w = getenv("MPSA_FP4_ENCODE");
        return (v && v[0] == 's') || (w && w[0] == 's');
    }();
    return sw;
}

template <int XDT, bool DO4, bool DO8>
void launch(const QuantArgs& a, int fmt8, dim3 grid, hipStream_t st) {
    const bool sw = use_sw_fp8();
    if (!DO8 || fmt8 == MPSA_FMT_E4M3) {
        if (sw) hipLaunchKernelGGL((quantize_kernel<XDT, DO4, DO8, MPSA_FMT_E4M3, true>), grid, dim3(256), 0, st, a);
        else    hipLaunchKernelGGL((quantize_kernel<XDT, DO4, DO8, MPSA_FMT_E4M3, false>), grid, dim3(256), 0, st, a);
    } else {
        if (sw) hipLaunchKernelGGL((quantize_kernel<XDT, DO4, DO8, MPSA_FMT_E5M2, true>), grid, dim3(256), 0, st, a);
        else    hipLaunchKernelGGL((quantize_kernel<XDT, DO4, DO8, MPSA_FMT_E5M2, false>), grid, dim3(256), 0, st, a);
    }
}

int quantize_common(const void* x, int x_dtype, int64_t B, int64_t H, int64_t N, int64_t D, const int64_t* xs,
                    const void* sub, float pre, bool do4, int emax4, bool do8, int fmt8, int emax8,
                    uint8_t* c4, uint8_t* s4, uint8_t* c8, uint8_t* s8, int64_t out_rows, hipStream_t st) {
    QuantArgs a;
    unsigned blocks = 0;
    const int rc = mpsa_quantize_setup(x, x_dtype, B, H, N, D, xs, sub, pre, do4, emax4, do8, fmt8, emax8, c4, s4, c8, s8, out_rows, &a, &blocks);
    if (rc != MPSA_OK || blocks == 0) return rc;
    dim3 grid((blocks + 1) / 2, (unsigned)H, (unsigned)B);     // the kernel takes two blocks of chunks per workgroup
    if (x_dtype == MPSA_BF16) {
        if (do4 && do8) launch<MPSA_BF16, true, true>(a, fmt8, grid, st);
        else if (do4)   launch<MPSA_BF16, true, false>(a, fmt8, grid, st);
        else            launch<MPSA_BF16, false, true>(a, fmt8, grid, st);
    } else {
        if (do4 && do8) launch<MPSA_F16, true, true>(a, fmt8, grid, st);
        else if (do4)   launch<MPSA_F16, true, false>(a, fmt8, grid, st);
        else            launch<MPSA_F16, false, true>(a, fmt8, grid, st);
    }
    MPSA_CHECK_LAUNCH("quantize");
    return MPSA_OK;
}

}  // namespace

// Validates one quantizer job and fills its argument block; *blocks = workgroups per (batch, head), 0 for an empty job.
int mpsa_quantize_setup(const void* x, int x_dtype, int64_t B, int64_t H, int64_t N, int64_t D, const int64_t* xs,
                        const void* sub, float pre, bool do4, int emax4, bool do8, int fmt8, int emax8,
                        uint8_t* c4, uint8_t* s4, uint8_t* c8, uint8_t* s8, int64_t out_rows, QuantArgs* out, unsigned* blocks) {
    *blocks = 0;
    if (!xs) return mpsa_fail(MPSA_EINVAL, "quantize: null input");
    if (x_dtype != MPSA_BF16 && x_dtype != MPSA_F16) return mpsa_fail(MPSA_EINVAL, "quantize: x_dtype must be bf16 or f16");
    if (do8 && fmt8 != MPSA_FMT_E4M3 && fmt8 != MPSA_FMT_E5M2) return mpsa_fail(MPSA_EINVAL, "quantize: 8-bit format must be E4M3 or E5M2");
    if (B < 0 || H < 0 || N < 0 || D <= 0 || out_rows < N) return mpsa_fail(MPSA_EINVAL, "quantize: bad shape");
    if (D % 32) return mpsa_fail(MPSA_EINVAL, "quantize: D=%lld is not a multiple of 32", (long long)D);
    if (B == 0 || H == 0 || out_rows == 0) return MPSA_OK;                // nothing to write (pointers may be null)
    if (!x && N > 0) return mpsa_fail(MPSA_EINVAL, "quantize: null input");
    if ((do4 && (!c4 || !s4)) || (do8 && (!c8 || !s8))) return mpsa_fail(MPSA_EINVAL, "quantize: null output");
    if (xs[3] != 1) return mpsa_fail(MPSA_EINVAL, "quantize: last dim of x must be contiguous");
    if (!mpsa_aligned16(x) || (xs[0] % 8) || (xs[1] % 8) || (xs[2] % 8)) return mpsa_fail(MPSA_EALIGN, "quantize: x rows must be 16-byte aligned");
    if ((do4 && !mpsa_aligned16(c4)) || (do8 && !mpsa_aligned16(c8))) return mpsa_fail(MPSA_EALIGN, "quantize: outputs must be 16-byte aligned");
    if (sub && !mpsa_aligned16(sub)) return mpsa_fail(MPSA_EALIGN, "quantize: sub must be 16-byte aligned");
    const int64_t chunks = out_rows * (D / 8);
    if (chunks >= (int64_t(1) << 31) || H > 65535 || B > 65535) return mpsa_fail(MPSA_EUNSUPPORTED, "quantize: a head has too many elements, or too many heads");
    QuantArgs& a = *out;
    a.x = x; a.sub = sub; a.sb = xs[0]; a.sh = xs[1]; a.sn = xs[2];
    a.n = (int)N; a.d = (int)D; a.out_rows = (int)out_rows; a.pre = pre;
    {
        uint32_t pb;
        memcpy(&pb, &pre, 4);
        a.exact16 = ((pb & 0x007FFFFFu) == 0u && (pb & 0x7F800000u) != 0u && (pb & 0x7F800000u) != 0x7F800000u) ? 1 : 0;
    }
    a.emax4 = emax4; a.emax8 = emax8;
    a.codes4 = c4; a.scales4 = s4; a.codes8 = c8; a.scales8 = s8;
    *blocks = (unsigned)((chunks + 255) / 256);
    return MPSA_OK;
}

bool mpsa_quantize_sw_encoders() { return use_sw_fp8(); }

extern "C" int mpsa_quantize_mx(const void* x, int x_dtype, int64_t B, int64_t H, int64_t N, int64_t D,
                                const int64_t x_strides[4], const void* sub, float pre_scale, int fmt, int emax_elem,
                                uint8_t* codes, uint8_t* scales, int64_t out_rows, mpsa_stream_t stream) {
    if (fmt == MPSA_FMT_E2M1)
        return quantize_common(x, x_dtype, B, H, N, D, x_strides, sub, pre_scale, true, emax_elem, false, 0, 0,
                               codes, scales, nullptr, nullptr, out_rows, (hipStream_t)stream);
    if (fmt == MPSA_FMT_E4M3 || fmt == MPSA_FMT_E5M2)
        return quantize_common(x, x_dtype, B, H, N, D, x_strides, sub, pre_scale, false, 0, true, fmt, emax_elem,
                               nullptr, nullptr, codes, scales, out_rows, (hipStream_t)stream);
    return mpsa_fail(MPSA_EINVAL, "quantize: unknown format %d", fmt);
}

extern "C" int mpsa_quantize_mx_dual(const void* x, int x_dtype, int64_t B, int64_t H, int64_t N, int64_t D,
                                     const int64_t x_strides[4], const void* sub, float pre_scale, int emax4, int fmt8, int emax8,
                                     uint8_t* codes4, uint8_t* scales4, uint8_t* codes8, uint8_t* scales8,
                                     int64_t out_rows, mpsa_stream_t stream) {
    return quantize_common(x, x_dtype, B, H, N, D, x_strides, sub, pre_scale, true, emax4, true, fmt8, emax8,
                           codes4, scales4, codes8, scales8, out_rows, (hipStream_t)stream);
}

extern "C" int64_t mpsa_seq_mean_workspace(int64_t B, int64_t H, int64_t N, int64_t D) {
    if (B < 0 || H < 0 || N < 0 || D < 0) return 0;
    return B * H * ((N + MEAN_ROWS - 1) / MEAN_ROWS) * D * (int64_t)sizeof(float);
}

namespace {

int seq_mean_common(const void* x, int x_dtype, int64_t B, int64_t H, int64_t N, int64_t D,
                    const int64_t x_strides[4], float* workspace, void* mean, hipStream_t st) {
    if (!x || !x_strides || !workspace || !mean) return mpsa_fail(MPSA_EINVAL, "seq_mean: null pointer");
    if (x_dtype != MPSA_BF16 && x_dtype != MPSA_F16) return mpsa_fail(MPSA_EINVAL, "seq_mean: x_dtype must be bf16 or f16");
    if (B <= 0 || H <= 0 || N <= 0) return mpsa_fail(MPSA_EINVAL, "seq_mean: bad shape");
    if (D != 64 && D != 128) return mpsa_fail(MPSA_EUNSUPPORTED, "seq_mean: D must be 64 or 128 (got %lld)", (long long)D);
    if (x_strides[3] != 1) return mpsa_fail(MPSA_EINVAL, "seq_mean: last dim of x must be contiguous");
    if (!mpsa_aligned16(x) || (x_strides[0] % 8) || (x_strides[1] % 8) || (x_strides[2] % 8)) return mpsa_fail(MPSA_EALIGN, "seq_mean: x rows must be 16-byte aligned");
    if (H > 65535 || B > 65535 || N >= (int64_t(1) << 31)) return mpsa_fail(MPSA_EUNSUPPORTED, "seq_mean: shape too large");
    MeanArgs a;
    a.x = x; a.sb = x_strides[0]; a.sh = x_strides[1]; a.sn = x_strides[2];
    a.n = (int)N; a.d = (int)D; a.nchunk = (int)((N + MEAN_ROWS - 1) / MEAN_ROWS);
    a.partial = workspace; a.mean = mean; a.inv_n = 1.0f / (float)N;
    dim3 grid((unsigned)a.nchunk, (unsigned)H, (unsigned)B);
    if (x_dtype == MPSA_BF16) {
        hipLaunchKernelGGL(seq_mean_kernel<MPSA_BF16>, grid, dim3(256), 0, st, a);
        hipLaunchKernelGGL(seq_mean_finish_kernel<MPSA_BF16>, dim3((unsigned)(B * H)), dim3(128), 0, st, a);
    } else {
        hipLaunchKernelGGL(seq_mean_kernel<MPSA_F16>, grid, dim3(256), 0, st, a);
        hipLaunchKernelGGL(seq_mean_finish_kernel<MPSA_F16>, dim3((unsigned)(B * H)), dim3(128), 0, st, a);
    }
    MPSA_CHECK_LAUNCH("seq_mean");
    return MPSA_OK;
}

}  // namespace

extern "C" int mpsa_seq_mean(const void* x, int x_dtype, int64_t B, int64_t H, int64_t N, int64_t D,
                             const int64_t x_strides[4], float* workspace, void* mean, mpsa_stream_t stream) {
    return seq_mean_common(x, x_dtype, B, H, N, D, x_strides, workspace, mean, (hipStream_t)stream);
}

// ---- the same mean for callers that cannot allocate: the partial sums live in a device array of this library ----
// Every GPU the library runs on holds its own copy of the array (at its own address) until the process ends.  The
// name `scratch` is a host-side handle, not a device address: host code asks the runtime for the address once per
// device and passes that pointer on.
static __device__ __align__(256) float scratch[MPSA_SEQ_MEAN_STATIC_BYTES / sizeof(float)];

namespace {
std::mutex g_scratch_mutex;
float* g_scratch_ptr[MPSA_MAX_DEVICES] = {};

// device address of `scratch` on the current device (resolved on the first call per device)
int scratch_for_current_device(float** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return mpsa_fail(MPSA_ELAUNCH, "seq_mean_static: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= MPSA_MAX_DEVICES) return mpsa_fail(MPSA_EUNSUPPORTED, "seq_mean_static: device index %d beyond %d", dev, MPSA_MAX_DEVICES - 1);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        float* p = nullptr;
        e = hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return mpsa_fail(MPSA_ELAUNCH, "seq_mean_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return MPSA_OK;
}
}  // namespace

int mpsa_seq_mean_static_resolve() {
    float* p = nullptr;
    return scratch_for_current_device(&p);
}

extern "C" int mpsa_seq_mean_static(const void* x, int x_dtype, int64_t B, int64_t H, int64_t N, int64_t D,
                                    const int64_t x_strides[4], void* mean, mpsa_stream_t stream) {
    const int64_t need = mpsa_seq_mean_workspace(B, H, N, D);
    if (need > (int64_t)MPSA_SEQ_MEAN_STATIC_BYTES)
        return mpsa_fail(MPSA_EUNSUPPORTED, "seq_mean_static: B*H*ceil(N/256)*D*4 = %lld bytes of partial sums exceed the built-in %lld; use mpsa_seq_mean with a workspace",
                         (long long)need, (long long)MPSA_SEQ_MEAN_STATIC_BYTES);
    float* ws = nullptr;
    const int rc = scratch_for_current_device(&ws);
    if (rc != MPSA_OK) return rc;
    // nothing to clear: the first kernel writes every partial sum the second one reads
    return seq_mean_common(x, x_dtype, B, H, N, D, x_strides, ws, mean, (hipStream_t)stream);
}
