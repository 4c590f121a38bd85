// RMS norm over the last axis: y = x * rsqrt(mean(x^2) + eps) * scale -- flax.linen.RMSNorm with its
// defaults, the norm of the cells' read-outs (linear_attention.py:109-115) and of the torso's PreNorm
// blocks (blocks/normalization.py:10-35 with RMSNorm as the norm).
//
// A row of a few hundred features is one wave's work: every lane holds four consecutive elements
// per 256 columns, the sum of squares is six shuffle steps, and a row costs one trip to memory each
// way.  Around the sequence kernels the norms are passes over (B*T, features) arrays that the array
// library runs at a third of the memory rate (statistics in one kernel, scale gradient in two more,
// casts in between); here the forward reads x once and writes y in the dtype its reader takes, and
// the backward reads x and dy once, writes dx, and leaves the scale's gradient as per-workgroup
// partial sums that a second small kernel adds up in a fixed order.
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

// One wave per row, RPI rows in flight per wave; lane l holds columns (i * 64 + l) * 4 .. + 3 of its rows.
template <typename XT, typename YT, int NV, int RPI>
__global__ void __launch_bounds__(RN_THREADS)
rms_norm_fwd_kernel(const XT *__restrict__ x, const float *__restrict__ scale, YT *__restrict__ y, int64_t rows, int D,
                    float eps, float inv_D)
{
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * RN_WAVES + (threadIdx.x >> 6), nwaves = (int64_t)gridDim.x * RN_WAVES;
    F4 sc[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int col = (i * 64 + lane) * 4;
        sc[i] = (scale && col < D) ? load_quad(scale + col) : F4{{1.f, 1.f, 1.f, 1.f}};
    }
    for (int64_t r0 = wave * RPI; r0 < rows; r0 += nwaves * RPI) {
        F4 xv[RPI][NV];
#pragma unroll
        for (int j = 0; j < RPI; ++j)
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int col = (i * 64 + lane) * 4;
                xv[j][i] = (r0 + j < rows && col < D) ? load_quad(x + (r0 + j) * D + col) : F4{{0.f, 0.f, 0.f, 0.f}};
            }
#pragma unroll
        for (int j = 0; j < RPI; ++j) {
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < NV; ++i)
#pragma unroll
                for (int e = 0; e < 4; ++e) ss += xv[j][i].v[e] * xv[j][i].v[e];
            const float rstd = rsqrtf(wave_sum(ss) * inv_D + eps);
            if (r0 + j < rows) {
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    const int col = (i * 64 + lane) * 4;
                    if (col < D) {
                        F4 o;
#pragma unroll
                        for (int e = 0; e < 4; ++e) o.v[e] = xv[j][i].v[e] * rstd * sc[i].v[e];
                        store_quad(y + (r0 + j) * D + col, o);
                    }
                }
            }
        }
    }
}

// With r = rsqrt(mean(x^2) + eps) and g = dy * scale:  dx = r g - x r^3 (g . x) / D,  dscale = sum over rows of
// dy x r.  The statistics are recomputed from x (it is read for dx anyway): nothing is kept from the forward.
// parts (gridDim.x, D): this workgroup's share of dscale (null: the scale's gradient is not wanted).
// dx_add (nullable): a gradient that reaches x by another way -- the residual branch around a pre-norm block --
// added here instead of by a pass of its own.
template <typename XT, typename GT, int NV, int RPI>
__global__ void __launch_bounds__(RN_THREADS)
rms_norm_bwd_kernel(const XT *__restrict__ x, const float *__restrict__ scale, const GT *__restrict__ dy,
                    const XT *__restrict__ dx_add, XT *__restrict__ dx, float *__restrict__ parts, int64_t rows, int D, float eps,
                    float inv_D)
{
    __shared__ float red[RN_WAVES][NV * 256];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    const int64_t wave = (int64_t)blockIdx.x * RN_WAVES + w, nwaves = (int64_t)gridDim.x * RN_WAVES;
    F4 sc[NV], ds[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int col = (i * 64 + lane) * 4;
        sc[i] = (scale && col < D) ? load_quad(scale + col) : F4{{1.f, 1.f, 1.f, 1.f}};
        ds[i] = F4{{0.f, 0.f, 0.f, 0.f}};
    }
    for (int64_t r0 = wave * RPI; r0 < rows; r0 += nwaves * RPI) {
        F4 xv[RPI][NV], gv[RPI][NV], av[RPI][NV];
#pragma unroll
        for (int j = 0; j < RPI; ++j)
#pragma unroll
            for (int i = 0; i < NV; ++i) {
                const int col = (i * 64 + lane) * 4;
                const bool in = r0 + j < rows && col < D;
                xv[j][i] = in ? load_quad(x + (r0 + j) * D + col) : F4{{0.f, 0.f, 0.f, 0.f}};
                gv[j][i] = in ? load_quad(dy + (r0 + j) * D + col) : F4{{0.f, 0.f, 0.f, 0.f}};
                av[j][i] = (in && dx_add) ? load_quad(dx_add + (r0 + j) * D + col) : F4{{0.f, 0.f, 0.f, 0.f}};
            }
#pragma unroll
        for (int j = 0; j < RPI; ++j) {
            float ss = 0.f, dot = 0.f;
#pragma unroll
            for (int i = 0; i < NV; ++i)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    ss += xv[j][i].v[e] * xv[j][i].v[e];
                    dot += gv[j][i].v[e] * sc[i].v[e] * xv[j][i].v[e];
                }
            const float rstd = rsqrtf(wave_sum(ss) * inv_D + eps);
            const float c = wave_sum(dot) * inv_D * rstd * rstd * rstd;
            if (r0 + j < rows) {   // rows past the end hold zeros: they add nothing to ds either way
#pragma unroll
                for (int i = 0; i < NV; ++i) {
                    const int col = (i * 64 + lane) * 4;
                    if (col < D) {
                        F4 o;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            o.v[e] = av[j][i].v[e] + (gv[j][i].v[e] * sc[i].v[e] * rstd - xv[j][i].v[e] * c);
                            ds[i].v[e] += gv[j][i].v[e] * xv[j][i].v[e] * rstd;
                        }
                        store_quad(dx + (r0 + j) * D + col, o);
                    }
                }
            }
        }
    }
    if (!parts) return;
#pragma unroll
    for (int i = 0; i < NV; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) red[w][(i * 64 + lane) * 4 + e] = ds[i].v[e];
    __syncthreads();
    for (int col = threadIdx.x; col < D; col += RN_THREADS) {
        float s = 0.f;
#pragma unroll
        for (int j = 0; j < RN_WAVES; ++j) s += red[j][col];
        parts[(int64_t)blockIdx.x * D + col] = s;
    }
}

// dscale[col] = sum over the nparts rows of parts, in a fixed order: 64 columns per workgroup, sixteen threads per
// column that each add every sixteenth row, four independent sums in flight per thread.
constexpr int RD_GROUPS = 16;
__global__ void __launch_bounds__(64 * RD_GROUPS) rms_norm_dscale_kernel(const float *__restrict__ parts, float *__restrict__ dscale,
                                                                      int nparts, int D)
{
    __shared__ float red[RD_GROUPS][64];
    const int c = threadIdx.x & 63, g = threadIdx.x >> 6, col = blockIdx.x * 64 + c;
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
        dscale[col] = t;
    }
}

int check_rows(const void *x, const void *out, int64_t rows, int64_t D)
{
    if (!x || !out || rows <= 0 || D <= 0) return MRX_ERR_INVALID_ARG;
    if (D % 4 != 0 || D > RN_MAX_NV * 256) return MRX_ERR_UNSUPPORTED;
    return MRX_OK;
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

template <typename XT, typename YT, int NV>
int launch_fwd(hipStream_t st, const void *x, const float *scale, void *y, int64_t rows, int D, float eps)
{
    constexpr int RPI = NV <= 2 ? 4 : NV <= 4 ? 2 : 1;
    return launch_kernel(rms_norm_fwd_kernel<XT, YT, NV, RPI>, dim3(grid_for(rows, RPI, 4096)), dim3(RN_THREADS), 0, st,
                         static_cast<const XT *>(x), scale, static_cast<YT *>(y), rows, D, eps, 1.f / (float)D);
}

template <typename XT, typename YT> int dispatch_fwd(hipStream_t st, const void *x, const float *scale, void *y, int64_t rows, int D, float eps)
{
    if (D <= 256) return launch_fwd<XT, YT, 1>(st, x, scale, y, rows, D, eps);
    if (D <= 512) return launch_fwd<XT, YT, 2>(st, x, scale, y, rows, D, eps);
    if (D <= 1024) return launch_fwd<XT, YT, 4>(st, x, scale, y, rows, D, eps);
    return launch_fwd<XT, YT, 8>(st, x, scale, y, rows, D, eps);
}

template <typename XT, typename GT, int NV>
int launch_bwd(hipStream_t st, const void *x, const float *scale, const void *dy, const void *dx_add, void *dx, float *parts,
               unsigned grid, int64_t rows, int D, float eps)
{
    constexpr int RPI = NV <= 2 ? 2 : 1;
    return launch_kernel(rms_norm_bwd_kernel<XT, GT, NV, RPI>, dim3(grid), dim3(RN_THREADS), 0, st, static_cast<const XT *>(x), scale,
                         static_cast<const GT *>(dy), static_cast<const XT *>(dx_add), static_cast<XT *>(dx), parts, rows, D, eps,
                         1.f / (float)D);
}

template <typename XT, typename GT>
int dispatch_bwd(hipStream_t st, const void *x, const float *scale, const void *dy, const void *dx_add, void *dx, float *parts,
                 unsigned grid, int64_t rows, int D, float eps)
{
    if (D <= 256) return launch_bwd<XT, GT, 1>(st, x, scale, dy, dx_add, dx, parts, grid, rows, D, eps);
    if (D <= 512) return launch_bwd<XT, GT, 2>(st, x, scale, dy, dx_add, dx, parts, grid, rows, D, eps);
    if (D <= 1024) return launch_bwd<XT, GT, 4>(st, x, scale, dy, dx_add, dx, parts, grid, rows, D, eps);
    return launch_bwd<XT, GT, 8>(st, x, scale, dy, dx_add, dx, parts, grid, rows, D, eps);
}

}  // namespace
}  // namespace mrx

extern "C" int mrx_rms_norm_fwd(void *stream, const void *x, const float *scale, void *y, int64_t rows, int64_t D, int x_dtype,
                                int y_dtype, float eps)
{
    using namespace mrx;
    if (const int rc = check_rows(x, y, rows, D); rc != MRX_OK) return rc;
    if (!known(x_dtype) || !known(y_dtype) || !(eps >= 0.f)) return MRX_ERR_INVALID_ARG;
    if (!quad_aligned(x, x_dtype) || !quad_aligned(y, y_dtype) || (scale && !aligned(scale, 16))) return MRX_ERR_INVALID_ARG;
    if (const int rc = prepare_device(); rc != MRX_OK) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int d = (int)D;
    if (x_dtype == MRX_F32)
        return y_dtype == MRX_F32 ? dispatch_fwd<float, float>(st, x, scale, y, rows, d, eps)
                                  : dispatch_fwd<float, __bf16>(st, x, scale, y, rows, d, eps);
    return y_dtype == MRX_F32 ? dispatch_fwd<__bf16, float>(st, x, scale, y, rows, d, eps)
                              : dispatch_fwd<__bf16, __bf16>(st, x, scale, y, rows, d, eps);
}

extern "C" int mrx_rms_norm_bwd(void *stream, const void *x, const float *scale, const void *dy, const void *dx_add, void *dx,
                                float *dscale, float *workspace, int64_t rows, int64_t D, int x_dtype, int dy_dtype, float eps)
{
    using namespace mrx;
    if (const int rc = check_rows(x, dx, rows, D); rc != MRX_OK) return rc;
    if (!dy || !known(x_dtype) || !known(dy_dtype) || !(eps >= 0.f)) return MRX_ERR_INVALID_ARG;
    if (!quad_aligned(x, x_dtype) || !quad_aligned(dx, x_dtype) || !quad_aligned(dy, dy_dtype) || (scale && !aligned(scale, 16)) ||
        (dx_add && !quad_aligned(dx_add, x_dtype)))
        return MRX_ERR_INVALID_ARG;
    if (dscale && !workspace) return MRX_ERR_INVALID_ARG;
    if (const int rc = prepare_device(); rc != MRX_OK) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int d = (int)D;
    const unsigned grid = grid_for(rows, d <= 512 ? 2 : 1, MRX_RMS_NORM_PARTS);
    float *parts = dscale ? workspace : nullptr;
    int rc;
    if (x_dtype == MRX_F32)
        rc = dy_dtype == MRX_F32 ? dispatch_bwd<float, float>(st, x, scale, dy, dx_add, dx, parts, grid, rows, d, eps)
                                 : dispatch_bwd<float, __bf16>(st, x, scale, dy, dx_add, dx, parts, grid, rows, d, eps);
    else
        rc = dy_dtype == MRX_F32 ? dispatch_bwd<__bf16, float>(st, x, scale, dy, dx_add, dx, parts, grid, rows, d, eps)
                                 : dispatch_bwd<__bf16, __bf16>(st, x, scale, dy, dx_add, dx, parts, grid, rows, d, eps);
    if (rc != MRX_OK || !dscale) return rc;
    return launch_kernel(rms_norm_dscale_kernel, dim3((unsigned)((d + 63) / 64)), dim3(64 * RD_GROUPS), 0, st, workspace, dscale,
                         (int)grid, d);
}
