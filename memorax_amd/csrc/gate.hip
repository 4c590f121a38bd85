// The gating product of the reference's GLU block (blocks/ffn.py:108-121: activation(gate) * value) with
// silu as the activation, as the torso's gated linear recurrence applies it to the scan's output:
//     y = h * silu(g) ,  silu(g) = g * sigmoid(g)
//     dh = dy * silu(g) ,  dg = dy * h * sigmoid(g) * (1 + g * (1 - sigmoid(g))).
// As array operations the pair is two passes forward and three backward over (B, T, F) arrays; here each
// direction reads its operands once.
#include <math.h>

#include <initializer_list>

#include "common.h"

namespace mrx {
namespace {

constexpr int GT_THREADS = 256;

template <typename T> struct GateVec;   // sixteen bytes of T
template <> struct GateVec<float> {
    static constexpr int N = 4;
};
template <> struct GateVec<__bf16> {
    static constexpr int N = 8;
};
template <typename T> struct alignas(16) Pack {
    T v[GateVec<T>::N];
};

__device__ __forceinline__ float sigmoidf(float x) { return 1.f / (1.f + __expf(-x)); }

template <typename T>
__global__ void __launch_bounds__(GT_THREADS) silu_gate_fwd_kernel(const T *__restrict__ h, const T *__restrict__ g, T *__restrict__ y,
                                                                int64_t n)
{
    constexpr int N = GateVec<T>::N;
    const int64_t stride = (int64_t)gridDim.x * GT_THREADS * N;
    for (int64_t i = ((int64_t)blockIdx.x * GT_THREADS + threadIdx.x) * N; i < n; i += stride) {
        if (i + N <= n) {
            const Pack<T> hv = *reinterpret_cast<const Pack<T> *>(h + i), gv = *reinterpret_cast<const Pack<T> *>(g + i);
            Pack<T> o;
#pragma unroll
            for (int e = 0; e < N; ++e) {
                const float x = (float)gv.v[e];
                o.v[e] = (T)((float)hv.v[e] * x * sigmoidf(x));
            }
            *reinterpret_cast<Pack<T> *>(y + i) = o;
        } else {
            for (int64_t j = i; j < n; ++j) {
                const float x = (float)g[j];
                y[j] = (T)((float)h[j] * x * sigmoidf(x));
            }
        }
    }
}

template <typename T>
__global__ void __launch_bounds__(GT_THREADS) silu_gate_bwd_kernel(const T *__restrict__ h, const T *__restrict__ g, const T *__restrict__ dy,
                                                                T *__restrict__ dh, T *__restrict__ dg, int64_t n)
{
    constexpr int N = GateVec<T>::N;
    const int64_t stride = (int64_t)gridDim.x * GT_THREADS * N;
    auto one = [](float hv, float x, float d, float &oh, float &og) {
        const float s = sigmoidf(x);
        oh = d * x * s;
        og = d * hv * s * (1.f + x * (1.f - s));
    };
    for (int64_t i = ((int64_t)blockIdx.x * GT_THREADS + threadIdx.x) * N; i < n; i += stride) {
        if (i + N <= n) {
            const Pack<T> hv = *reinterpret_cast<const Pack<T> *>(h + i), gv = *reinterpret_cast<const Pack<T> *>(g + i),
                          dv = *reinterpret_cast<const Pack<T> *>(dy + i);
            Pack<T> oh, og;
#pragma unroll
            for (int e = 0; e < N; ++e) {
                float a, b;
                one((float)hv.v[e], (float)gv.v[e], (float)dv.v[e], a, b);
                oh.v[e] = (T)a;
                og.v[e] = (T)b;
            }
            *reinterpret_cast<Pack<T> *>(dh + i) = oh;
            *reinterpret_cast<Pack<T> *>(dg + i) = og;
        } else {
            for (int64_t j = i; j < n; ++j) {
                float a, b;
                one((float)h[j], (float)g[j], (float)dy[j], a, b);
                dh[j] = (T)a;
                dg[j] = (T)b;
            }
        }
    }
}

unsigned gate_grid(int64_t n, int per_thread)
{
    const int64_t wgs = (n + (int64_t)GT_THREADS * per_thread - 1) / ((int64_t)GT_THREADS * per_thread);
    return (unsigned)(wgs < 8192 ? wgs : 8192);
}

bool gate_args_ok(std::initializer_list<const void *> ptrs, int64_t n, int dtype, int *rc)
{
    *rc = MRX_ERR_INVALID_ARG;
    if (n <= 0 || (dtype != MRX_F32 && dtype != MRX_BF16)) return false;
    for (const void *p : ptrs)
        if (!p || !aligned(p, 16)) return false;
    *rc = MRX_OK;
    return true;
}

}  // namespace
}  // namespace mrx

extern "C" int mrx_silu_gate_fwd(void *stream, const void *h, const void *g, void *y, int64_t n, int dtype)
{
    using namespace mrx;
    int rc;
    if (!gate_args_ok({h, g, y}, n, dtype, &rc)) return rc;
    if (const int st = prepare_device(); st != MRX_OK) return st;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == MRX_F32)
        return launch_kernel(silu_gate_fwd_kernel<float>, dim3(gate_grid(n, 4)), dim3(GT_THREADS), 0, s, static_cast<const float *>(h),
                             static_cast<const float *>(g), static_cast<float *>(y), n);
    return launch_kernel(silu_gate_fwd_kernel<__bf16>, dim3(gate_grid(n, 8)), dim3(GT_THREADS), 0, s, static_cast<const __bf16 *>(h),
                         static_cast<const __bf16 *>(g), static_cast<__bf16 *>(y), n);
}

extern "C" int mrx_silu_gate_bwd(void *stream, const void *h, const void *g, const void *dy, void *dh, void *dg, int64_t n, int dtype)
{
    using namespace mrx;
    int rc;
    if (!gate_args_ok({h, g, dy, dh, dg}, n, dtype, &rc)) return rc;
    if (const int st = prepare_device(); st != MRX_OK) return st;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype == MRX_F32)
        return launch_kernel(silu_gate_bwd_kernel<float>, dim3(gate_grid(n, 4)), dim3(GT_THREADS), 0, s, static_cast<const float *>(h),
                             static_cast<const float *>(g), static_cast<const float *>(dy), static_cast<float *>(dh),
                             static_cast<float *>(dg), n);
    return launch_kernel(silu_gate_bwd_kernel<__bf16>, dim3(gate_grid(n, 8)), dim3(GT_THREADS), 0, s, static_cast<const __bf16 *>(h),
                         static_cast<const __bf16 *>(g), static_cast<const __bf16 *>(dy), static_cast<__bf16 *>(dh),
                         static_cast<__bf16 *>(dg), n);
}
