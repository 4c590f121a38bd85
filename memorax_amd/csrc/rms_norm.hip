// Norms over the last axis, as the reference's blocks and read-outs apply them:
//   RMS norm    y = x * rsqrt(mean(x^2) + eps) * scale                 flax.linen.RMSNorm with its defaults: the
//               cells' read-outs (linear_attention.py:109-115), PreNorm blocks built with it
//   layer norm  y = (x - mean(x)) * rsqrt(var(x) + eps) * scale + bias  flax.linen.LayerNorm with its defaults: the
//               default norm of PreNorm / PostNorm (blocks/normalization.py:10-65)
//
// A row of a few hundred features is one wave's work: every lane holds four consecutive elements
// per 256 columns, a row statistic is six shuffle steps, and a row costs one trip to memory each
// way.  Around the sequence kernels the norms are passes over (B*T, features) arrays that the array
// library runs at a third of the memory rate (statistics in one kernel, parameter gradients in two more,
// casts in between); here the forward reads x once and writes y in the dtype its reader takes, and
// the backward reads x and dy once, writes dx, and leaves the parameters' gradients as per-workgroup
// partial sums that a second small kernel adds up in a fixed order.  CENTER selects the layer norm.
#include <math.h>

#include "common.h"

namespace mrx {
namespace {

constexpr int RN_WAVES = 4, RN_THREADS = 64 * RN_WAVES;
constexpr int RN_MAX_NV = 8;  // 256-column groups a lane can hold: rows of up to 2048 features

template <typename T> struct alignas(4 * sizeof(T)) Quad {
    T v[4];
};
struct F4 {
    float v[4];
};
constexpr F4 F4_ZERO{{0.f, 0.f, 0.f, 0.f}}, F4_ONE{{1.f, 1.f, 1.f, 1.f}};

template <typename T> __device__ __forceinline__ F4 load_quad(const T *p)
{
    const Quad<T> q = *reinterpret_cast<const Quad<T> *>(p);
    return F4{{(float)q.v[0], (float)q.v[1], (float)q.v[2], (float)q.v[3]}};
}
template <typename T> __device__ __forceinline__ void store_quad(T *p, const F4 &f)
{
    Quad<T> q;
#pragma unroll
    for (int e = 0; e < 4; ++e) q.v[e] = (T)f.v[e];
    *reinterpret_cast<Quad<T> *>(p) = q;
}

__device__ __forceinline__ float wave_sum(float x)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off);
    return x;
}

// The row held by a wave (columns past D hold zeros), centred in place if CENTER; returns rsqrt(mean of squares + eps).
template <int NV, bool CENTER> __device__ __forceinline__ float row_statistics(F4 (&xv)[NV], int lane, int D, float eps, float inv_D)
{
    if (CENTER) {
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) s += xv[i].v[e];
        const float mu = wave_sum(s) * inv_D;
#pragma unroll
        for (int i = 0; i < NV; ++i)
            if ((i * 64 + lane) * 4 < D) {
#pragma unroll
                for (int e = 0; e < 4; ++e) xv[i].v[e] -= mu;
            }
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) ss += xv[i].v[e] * xv[i].v[e];
    return rsqrtf(wave_sum(ss) * inv_D + eps);
}

// One wave per row, RPI rows in flight per wave; lane l holds columns (i * 64 + l) * 4 .. + 3 of its rows.
template <typename XT, typename YT, int NV, int RPI, bool CENTER>
__global__ void __launch_bounds__(RN_THREADS)
norm_fwd_kernel(const XT *__restrict__ x, const float *__restrict__ scale, const float *__restrict__ bias, YT *__restrict__ y,
                int64_t rows, int D, float eps, float inv_D)
{
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * RN_WAVES + (threadIdx.x >> 6), nwaves = (int64_t)gridDim.x * RN_WAVES;
    F4 sc[NV], bi[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int col = (i * 64 + lane) * 4;
        sc[i] = (scale && col < D) ? load_quad(scale + col) : F4_ONE;
        bi[i] = (CENTER && bias && col < D) ? load_quad(bias + col) : F4_ZERO;
    }
    for (int64_t r0 = wave * RPI; r0 < rows; r0 += nwaves * RPI) {
        F4 xv[RPI][NV];
#pragma unroll
        for (int j = 0; j < RPI; ++j)
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int col = (i * 64 + lane) * 4;
                xv[j][i] = (r0 + j < rows && col < D) ? load_quad(x + (r0 + j) * D + col) : F4_ZERO;
            }
#pragma unroll
        for (int j = 0; j < RPI; ++j) {
            const float rstd = row_statistics<NV, CENTER>(xv[j], lane, D, eps, inv_D);
            if (r0 + j < rows) {
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    const int col = (i * 64 + lane) * 4;
                    if (col < D) {
                        F4 o;
#pragma unroll
                        for (int e = 0; e < 4; ++e) o.v[e] = xv[j][i].v[e] * rstd * sc[i].v[e] + bi[i].v[e];
                        store_quad(y + (r0 + j) * D + col, o);
                    }
                }
            }
        }
    }
}

// With xc = x (RMS norm) or x - mean(x) (layer norm), r = rsqrt(mean(xc^2) + eps) and g = dy * scale:
//     dx = r g - xc r^3 mean(g xc)  [ - r mean(g), layer norm ] ,   dscale = sum over rows of dy xc r ,   dbias = sum of dy.
// The statistics are recomputed from x (it is read for dx anyway): nothing is kept from the forward.
// parts (gridDim.x, D) [then (gridDim.x, D) more for dbias]: this workgroup's share of the parameters' gradients
// (null: they are not wanted).  dx_add (nullable): a gradient that reaches x by another way -- the residual branch
// around a pre-norm block -- added here instead of by a pass of its own.
template <typename XT, typename GT, int NV, int RPI, bool CENTER>
__global__ void __launch_bounds__(RN_THREADS)
norm_bwd_kernel(const XT *__restrict__ x, const float *__restrict__ scale, const GT *__restrict__ dy, const XT *__restrict__ dx_add,
                XT *__restrict__ dx, float *__restrict__ parts, int64_t rows, int D, float eps, float inv_D)
{
    __shared__ float red[RN_WAVES][NV * 256];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int64_t wave = (int64_t)blockIdx.x * RN_WAVES + w, nwaves = (int64_t)gridDim.x * RN_WAVES;
    F4 sc[NV], ds[NV], db[CENTER ? NV : 1];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int col = (i * 64 + lane) * 4;
        sc[i] = (scale && col < D) ? load_quad(scale + col) : F4_ONE;
        ds[i] = F4_ZERO;
        if (CENTER) db[i] = F4_ZERO;
    }
    for (int64_t r0 = wave * RPI; r0 < rows; r0 += nwaves * RPI) {
        F4 xv[RPI][NV], gv[RPI][NV], av[RPI][NV];
#pragma unroll
        for (int j = 0; j < RPI; ++j)
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int col = (i * 64 + lane) * 4;
                const bool in = r0 + j < rows && col < D;
                xv[j][i] = in ? load_quad(x + (r0 + j) * D + col) : F4_ZERO;
                gv[j][i] = in ? load_quad(dy + (r0 + j) * D + col) : F4_ZERO;
                av[j][i] = (in && dx_add) ? load_quad(dx_add + (r0 + j) * D + col) : F4_ZERO;
            }
#pragma unroll
        for (int j = 0; j < RPI; ++j) {
            const float rstd = row_statistics<NV, CENTER>(xv[j], lane, D, eps, inv_D);
            float dot = 0.f, gsum = 0.f;
#pragma unroll
            for (int i = 0; i < NV; ++i)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float g = gv[j][i].v[e] * sc[i].v[e];
                    dot += g * xv[j][i].v[e];
                    if (CENTER) gsum += g;
                }
            const float c = wave_sum(dot) * inv_D * rstd * rstd * rstd;
            const float c1 = CENTER ? wave_sum(gsum) * inv_D * rstd : 0.f;
            if (r0 + j < rows) {   // rows past the end hold zeros: they add nothing to the sums either way
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    const int col = (i * 64 + lane) * 4;
                    if (col < D) {
                        F4 o;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            o.v[e] = av[j][i].v[e] + (gv[j][i].v[e] * sc[i].v[e] * rstd - xv[j][i].v[e] * c - c1);
                            ds[i].v[e] += gv[j][i].v[e] * xv[j][i].v[e] * rstd;
                            if (CENTER) db[i].v[e] += gv[j][i].v[e];
                        }
                        store_quad(dx + (r0 + j) * D + col, o);
                    }
                }
            }
        }
    }
    if (!parts) return;
#pragma unroll
    for (int pass = 0; pass < (CENTER ? 2 : 1); ++pass) {
        if (pass) __syncthreads();
#pragma unroll
        for (int i = 0; i < NV; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) red[w][(i * 64 + lane) * 4 + e] = pass ? db[CENTER ? i : 0].v[e] : ds[i].v[e];
        __syncthreads();
        float *out = parts + ((int64_t)pass * gridDim.x + blockIdx.x) * D;
        for (int col = threadIdx.x; col < D; col += RN_THREADS) {
            float s = 0.f;
#pragma unroll
            for (int j = 0; j < RN_WAVES; ++j) s += red[j][col];
            out[col] = s;
        }
    }
}

// out_y[col] = sum over the nparts rows of block y of parts, in a fixed order (y = 0: dscale, y = 1: dbias): 64 columns
// per workgroup, sixteen threads per column that each add every sixteenth row, four independent sums in flight per thread.
constexpr int RD_GROUPS = 16;
__global__ void __launch_bounds__(64 * RD_GROUPS) norm_param_grad_kernel(const float *__restrict__ parts, float *__restrict__ dscale,
                                                                      float *__restrict__ dbias, int nparts, int D)
{
    __shared__ float red[RD_GROUPS][64];
    const int c = threadIdx.x & 63, g = threadIdx.x >> 6, col = blockIdx.x * 64 + c;
    parts += (int64_t)blockIdx.y * nparts * D;
    float *out = blockIdx.y ? dbias : dscale;
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    if (col < D) {
        int p = g;
        for (; p + 3 * RD_GROUPS < nparts; p += 4 * RD_GROUPS)
#pragma unroll
            for (int u = 0; u < 4; ++u) s[u] += parts[(int64_t)(p + u * RD_GROUPS) * D + col];
        for (; p < nparts; p += RD_GROUPS) s[0] += parts[(int64_t)p * D + col];
    }
    red[g][c] = (s[0] + s[1]) + (s[2] + s[3]);
    __syncthreads();
    if (g == 0 && col < D) {
        float t = 0.f;
#pragma unroll
        for (int j = 0; j < RD_GROUPS; ++j) t += red[j][c];
        out[col] = t;
    }
}

bool known(int dtype) { return dtype == MRX_F32 || dtype == MRX_BF16; }
// rows are read and written four elements at a time
bool quad_aligned(const void *p, int dtype) { return aligned(p, dtype == MRX_F32 ? 16 : 8); }

// Workgroups of a launch: enough waves for RPI rows each, at most `cap` workgroups (the rest by striding).
unsigned grid_for(int64_t rows, int rpi, int cap)
{
    const int64_t waves = (rows + rpi - 1) / rpi, wgs = (waves + RN_WAVES - 1) / RN_WAVES;
    return (unsigned)(wgs < cap ? wgs : cap);
}

struct FwdCall {
    hipStream_t st;
    const void *x;
    const float *scale, *bias;
    void *y;
    int64_t rows;
    int D;
    float eps;
};

template <typename XT, typename YT, int NV, bool CENTER> int launch_fwd(const FwdCall &a)
{
    constexpr int RPI = NV <= 2 ? 4 : NV <= 4 ? 2 : 1;
    return launch_kernel(norm_fwd_kernel<XT, YT, NV, RPI, CENTER>, dim3(grid_for(a.rows, RPI, 4096)), dim3(RN_THREADS), 0, a.st,
                         static_cast<const XT *>(a.x), a.scale, a.bias, static_cast<YT *>(a.y), a.rows, a.D, a.eps, 1.f / (float)a.D);
}
template <typename XT, typename YT, bool CENTER> int fwd_by_width(const FwdCall &a)
{
    if (a.D <= 256) return launch_fwd<XT, YT, 1, CENTER>(a);
    if (a.D <= 512) return launch_fwd<XT, YT, 2, CENTER>(a);
    if (a.D <= 1024) return launch_fwd<XT, YT, 4, CENTER>(a);
    return launch_fwd<XT, YT, 8, CENTER>(a);
}
template <bool CENTER> int norm_fwd(const FwdCall &a, int x_dtype, int y_dtype)
{
    if (!a.x || !a.y || a.rows <= 0 || a.D <= 0) return MRX_ERR_INVALID_ARG;
    if (a.D % 4 != 0 || a.D > RN_MAX_NV * 256) return MRX_ERR_UNSUPPORTED;
    if (!known(x_dtype) || !known(y_dtype) || !(a.eps >= 0.f)) return MRX_ERR_INVALID_ARG;
    if (!quad_aligned(a.x, x_dtype) || !quad_aligned(a.y, y_dtype) || (a.scale && !aligned(a.scale, 16)) ||
        (a.bias && !aligned(a.bias, 16)))
        return MRX_ERR_INVALID_ARG;
    if (const int rc = prepare_device(); rc != MRX_OK) return rc;
    if (x_dtype == MRX_F32) return y_dtype == MRX_F32 ? fwd_by_width<float, float, CENTER>(a) : fwd_by_width<float, __bf16, CENTER>(a);
    return y_dtype == MRX_F32 ? fwd_by_width<__bf16, float, CENTER>(a) : fwd_by_width<__bf16, __bf16, CENTER>(a);
}

// Rows a wave of the backward kernel has in flight, by the 256-column groups a lane holds.
constexpr int bwd_rows_in_flight(int nv) { return nv <= 2 ? 2 : 1; }   // four at the narrowest width measured level

struct BwdCall {
    hipStream_t st;
    const void *x;
    const float *scale;
    const void *dy, *dx_add;
    void *dx;
    float *dscale, *dbias, *workspace;
    int64_t rows;
    int D;
    float eps;
    unsigned grid;
};

template <typename XT, typename GT, int NV, bool CENTER> int launch_bwd(const BwdCall &a)
{
    constexpr int RPI = bwd_rows_in_flight(NV);
    return launch_kernel(norm_bwd_kernel<XT, GT, NV, RPI, CENTER>, dim3(a.grid), dim3(RN_THREADS), 0, a.st, static_cast<const XT *>(a.x),
                         a.scale, static_cast<const GT *>(a.dy), static_cast<const XT *>(a.dx_add), static_cast<XT *>(a.dx),
                         (a.dscale || a.dbias) ? a.workspace : nullptr, a.rows, a.D, a.eps, 1.f / (float)a.D);
}
template <typename XT, typename GT, bool CENTER> int bwd_by_width(const BwdCall &a)
{
    if (a.D <= 256) return launch_bwd<XT, GT, 1, CENTER>(a);
    if (a.D <= 512) return launch_bwd<XT, GT, 2, CENTER>(a);
    if (a.D <= 1024) return launch_bwd<XT, GT, 4, CENTER>(a);
    return launch_bwd<XT, GT, 8, CENTER>(a);
}
template <bool CENTER> int norm_bwd(BwdCall a, int x_dtype, int dy_dtype)
{
    if (!a.x || !a.dx || !a.dy || a.rows <= 0 || a.D <= 0) return MRX_ERR_INVALID_ARG;
    if (a.D % 4 != 0 || a.D > RN_MAX_NV * 256) return MRX_ERR_UNSUPPORTED;
    if (!known(x_dtype) || !known(dy_dtype) || !(a.eps >= 0.f)) return MRX_ERR_INVALID_ARG;
    if (!quad_aligned(a.x, x_dtype) || !quad_aligned(a.dx, x_dtype) || !quad_aligned(a.dy, dy_dtype) ||
        (a.scale && !aligned(a.scale, 16)) || (a.dx_add && !quad_aligned(a.dx_add, x_dtype)))
        return MRX_ERR_INVALID_ARG;
    // the layer norm's parameters come as a pair, and so do their gradients
    if (CENTER && (a.dscale == nullptr) != (a.dbias == nullptr)) return MRX_ERR_INVALID_ARG;
    if ((a.dscale || a.dbias) && !a.workspace) return MRX_ERR_INVALID_ARG;
    if (const int rc = prepare_device(); rc != MRX_OK) return rc;
    a.grid = grid_for(a.rows, bwd_rows_in_flight((a.D + 255) / 256), MRX_RMS_NORM_PARTS);
    int rc;
    if (x_dtype == MRX_F32)
        rc = dy_dtype == MRX_F32 ? bwd_by_width<float, float, CENTER>(a) : bwd_by_width<float, __bf16, CENTER>(a);
    else
        rc = dy_dtype == MRX_F32 ? bwd_by_width<__bf16, float, CENTER>(a) : bwd_by_width<__bf16, __bf16, CENTER>(a);
    if (rc != MRX_OK || !a.dscale) return rc;
    return launch_kernel(norm_param_grad_kernel, dim3((unsigned)((a.D + 63) / 64), CENTER ? 2u : 1u), dim3(64 * RD_GROUPS), 0, a.st,
                         a.workspace, a.dscale, a.dbias, (int)a.grid, a.D);
}

}  // namespace
}  // namespace mrx

extern "C" int mrx_rms_norm_fwd(void *stream, const void *x, const float *scale, void *y, int64_t rows, int64_t D, int x_dtype,
                                int y_dtype, float eps)
{
    using namespace mrx;
    if (D > 0x7fffffff) return MRX_ERR_UNSUPPORTED;
    return norm_fwd<false>(FwdCall{static_cast<hipStream_t>(stream), x, scale, nullptr, y, rows, (int)D, eps}, x_dtype, y_dtype);
}

extern "C" int mrx_rms_norm_bwd(void *stream, const void *x, const float *scale, const void *dy, const void *dx_add, void *dx,
                                float *dscale, float *workspace, int64_t rows, int64_t D, int x_dtype, int dy_dtype, float eps)
{
    using namespace mrx;
    if (D > 0x7fffffff) return MRX_ERR_UNSUPPORTED;
    return norm_bwd<false>(BwdCall{static_cast<hipStream_t>(stream), x, scale, dy, dx_add, dx, dscale, nullptr, workspace, rows, (int)D,
                                   eps, 0u},
                           x_dtype, dy_dtype);
}

extern "C" int mrx_layer_norm_fwd(void *stream, const void *x, const float *scale, const float *bias, void *y, int64_t rows, int64_t D,
                                  int x_dtype, int y_dtype, float eps)
{
    using namespace mrx;
    if (D > 0x7fffffff) return MRX_ERR_UNSUPPORTED;
    return norm_fwd<true>(FwdCall{static_cast<hipStream_t>(stream), x, scale, bias, y, rows, (int)D, eps}, x_dtype, y_dtype);
}

extern "C" int mrx_layer_norm_bwd(void *stream, const void *x, const float *scale, const void *dy, const void *dx_add, void *dx,
                                  float *dscale, float *dbias, float *workspace, int64_t rows, int64_t D, int x_dtype, int dy_dtype,
                                  float eps)
{
    using namespace mrx;
    if (D > 0x7fffffff) return MRX_ERR_UNSUPPORTED;
    return norm_bwd<true>(BwdCall{static_cast<hipStream_t>(stream), x, scale, dy, dx_add, dx, dscale, dbias, workspace, rows, (int)D, eps,
                                  0u},
                          x_dtype, dy_dtype);
}
