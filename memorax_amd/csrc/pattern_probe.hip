// Measurement only (part of libmemorax_amd_clk.so, never of the library): the memory side of the chunked
// kernels without their arithmetic.  One workgroup of four waves per (batch, head) sequence, two per compute
// unit, walks its sequence in chunks of C rows exactly as chunk_fwd_kernel / la_bwd_kernel / delta_bwd_kernel
// do -- 128-byte rows H * 128 bytes apart, 16 bytes per lane, the next chunk requested while the current one
// is written to LDS and read back -- reads NIN such arrays, writes NOUT, and moves a per-chunk block of
// residual bytes each way (state checkpoints, triangular factors).  Its time is what the access pattern costs
// on the device whatever the kernel computes: bench.py reports the kernels' times against it.
#include "common.h"
#include "hd.h"
#include "chunk_common.h"

namespace mrx {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr int PP_THREADS = 256, PP_MAXC = 64;
constexpr int PP_LDS = 75776;  // as much LDS as the chunk kernels take: two workgroups per compute unit

struct PatternArgs {
    const u32x4 *in[4];
    u32x4 *out[3];
    const u32x4 *res_in;  // (B*H, NC, res_in_segs) 16-byte segments read per chunk
    u32x4 *res_out;       // (B*H, NC, res_out_segs) written per chunk
    int res_in_segs, res_out_segs;
    int T, H, C;
    int reverse;  // walk the chunks from the last to the first (the backward kernels)
};

template <int NIN, int NOUT>
__global__ void __launch_bounds__(PP_THREADS, 2) pattern_kernel(PatternArgs a)
{
    extern __shared__ u32x4 lds[];
    const int tid = threadIdx.x, seg = tid % 8, r0 = tid / 8;
    constexpr int RPP = PP_THREADS / 8;  // 32 rows per pass of the threads
    const int bh = sequence_of_block(blockIdx.x, gridDim.x, a.H), b = bh / a.H, h = bh % a.H;  // as the kernels map them
    const int64_t rs = (int64_t)a.H * 8;  // row stride in 16-byte segments
    const int64_t base = ((int64_t)b * a.T * a.H + h) * 8 + seg;
    const int NC = a.T / a.C, passes = a.C / RPP;
    const int res_in_passes = (a.res_in_segs + PP_THREADS - 1) / PP_THREADS;
    const int res_out_passes = (a.res_out_segs + PP_THREADS - 1) / PP_THREADS;
    u32x4 r[NIN][PP_MAXC / RPP], rr[4];
    auto request = [&](int c) {
#pragma unroll
        for (int p = 0; p < PP_MAXC / RPP; ++p)
            if (p < passes) {
                const int64_t off = base + (int64_t)(c * a.C + r0 + p * RPP) * rs;
#pragma unroll
                for (int i = 0; i < NIN; ++i) r[i][p] = a.in[i][off];
            }
#pragma unroll
        for (int p = 0; p < 4; ++p)
            if (p < res_in_passes && tid + p * PP_THREADS < a.res_in_segs)
                rr[p] = __builtin_nontemporal_load(a.res_in + ((int64_t)bh * NC + c) * a.res_in_segs + tid + p * PP_THREADS);
    };
    request(a.reverse ? NC - 1 : 0);
    for (int i = 0; i < NC; ++i) {
        const int c = a.reverse ? NC - 1 - i : i;
        u32x4 x = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int p = 0; p < PP_MAXC / RPP; ++p)
            if (p < passes) {
                u32x4 y = r[0][p];
#pragma unroll
                for (int j = 1; j < NIN; ++j) y ^= r[j][p];
                lds[(r0 + p * RPP) * 9 + seg] = y;
            }
#pragma unroll
        for (int p = 0; p < 4; ++p)
            if (p < res_in_passes && tid + p * PP_THREADS < a.res_in_segs) x ^= rr[p];
        __syncthreads();
        if (i + 1 < NC) request(a.reverse ? c - 1 : c + 1);
#pragma unroll
        for (int p = 0; p < PP_MAXC / RPP; ++p)
            if (p < passes) {
                const int64_t off = base + (int64_t)(c * a.C + r0 + p * RPP) * rs;
                const u32x4 y = lds[(r0 + p * RPP) * 9 + ((seg + 1) & 7)] ^ x;
#pragma unroll
                for (int j = 0; j < NOUT; ++j) __builtin_nontemporal_store(y, a.out[j] + off);
            }
#pragma unroll
        for (int p = 0; p < 4; ++p)
            if (p < res_out_passes && tid + p * PP_THREADS < a.res_out_segs)
                a.res_out[((int64_t)bh * NC + c) * a.res_out_segs + tid + p * PP_THREADS] = x;
        __syncthreads();
    }
}

template <int NIN, int NOUT> struct PatternReg {
    static inline KernelRegistrar reg{reinterpret_cast<const void *>(pattern_kernel<NIN, NOUT>), PP_LDS};
};

template <int NIN, int NOUT> int launch_pattern(hipStream_t st, const PatternArgs &a, int64_t BH)
{
    (void)&PatternReg<NIN, NOUT>::reg;
    if (const int rc = prepare_device(); rc != MRX_OK) return rc;
    return launch_kernel(pattern_kernel<NIN, NOUT>, dim3((unsigned)BH), dim3(PP_THREADS), PP_LDS, st, a);
}

}  // namespace
}  // namespace mrx

// in: n_in <= 4 arrays of (B, T, H, 128 bytes) read; out: n_out <= 3 such arrays written; res_in / res_out: per
// (b, h, chunk) blocks of res_in_bytes / res_out_bytes (multiples of 16, at most 16 KB; may be null with 0 bytes).
// T a multiple of C, C 32 or 64.  Supported pairs (n_in, n_out): (3, 1), (4, 1), (4, 3).
extern "C" int mrx_pattern_probe(void *stream, const void *const *in, int n_in, void *const *out, int n_out, const void *res_in,
                                 int res_in_bytes, void *res_out, int res_out_bytes, int64_t B, int64_t T, int64_t H, int C,
                                 int reverse)
{
    using namespace mrx;
    if (!in || !out || B <= 0 || T <= 0 || H <= 0 || (C != 32 && C != 64) || T % C != 0) return MRX_ERR_INVALID_ARG;
    if (res_in_bytes < 0 || res_out_bytes < 0 || res_in_bytes % 16 || res_out_bytes % 16 || res_in_bytes > 16384 ||
        res_out_bytes > 16384 || (res_in_bytes && !res_in) || (res_out_bytes && !res_out))
        return MRX_ERR_INVALID_ARG;
    PatternArgs a{};
    for (int i = 0; i < n_in && i < 4; ++i) a.in[i] = static_cast<const u32x4 *>(in[i]);
    for (int i = 0; i < n_out && i < 3; ++i) a.out[i] = static_cast<u32x4 *>(out[i]);
    a.res_in = static_cast<const u32x4 *>(res_in);
    a.res_out = static_cast<u32x4 *>(res_out);
    a.res_in_segs = res_in_bytes / 16;
    a.res_out_segs = res_out_bytes / 16;
    a.T = (int)T;
    a.H = (int)H;
    a.C = C;
    a.reverse = reverse;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (n_in == 3 && n_out == 1) return launch_pattern<3, 1>(st, a, B * H);
    if (n_in == 4 && n_out == 1) return launch_pattern<4, 1>(st, a, B * H);
    if (n_in == 4 && n_out == 3) return launch_pattern<4, 3>(st, a, B * H);
    return MRX_ERR_UNSUPPORTED;
}
