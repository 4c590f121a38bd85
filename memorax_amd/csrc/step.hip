// Single-step (T = 1) state updates for acting/rollout loops: one time step of the linear
// attention and of the delta-rule recurrence per (b, h) sequence, fused with the read-out.
//
//   linear attention : S' = (done ? 0 : S) + v phi(k)^T ,  z' = (done ? 0 : z) + phi(k)
//                      o = S' phi(q)            [ / max(phi(q) . z', eps) when z is given ]
//   gated            : S' = (done ? 0 : exp(g) S) + v phi(k)^T ,  o = S' phi(q)   (g a log-decay per sequence)
//   delta rule       : S0 = done ? 0 : S ,  u = beta (v - S0 k) ,  S' = S0 + u k^T ,  o = S' q
//
// The state S:(B,H,d,d) fp32 ([dv][dk], d = 64 or 32) is read once and written once; everything else
// is a few hundred bytes per sequence, so the kernels are bound by HBM traffic of the state
// (32 KiB per (b,h) at d = 64).  One workgroup of 256 threads per (b,h): a row of the state is d / 4
// lanes of four consecutive dk each, the 256 threads cover 1024 / d rows at a time (d = 64: thread t
// owns dk = 4 (t & 15).. of rows dv = (t >> 4) + 16 p, p = 0..3), so that every load and store of S is a
// fully coalesced 16-byte access; row dot products reduce over the lanes of a row.
// Follows what Memoroid.__call__ computes for T = 1 (memoroid.py:93-109 with the cell algebra of
// linear_attention.py:62-117) and the delta-rule recurrence of the chunked kernels.
#include <type_traits>

#include "chunk_common.h"
#if MRX_HD == 64
#include "hd32_api.h"
#endif

namespace {
inline namespace MRX_HD_NS {

using namespace mrx;

constexpr int LPR = HD / 4;    // lanes per row of the state
constexpr int RPP = 256 / LPR;  // rows the workgroup covers at a time
constexpr int NP = HD / RPP;    // times it does so

__device__ __forceinline__ float reduce_row(float x)
{
    x += __shfl_xor(x, 1);
    x += __shfl_xor(x, 2);
    x += __shfl_xor(x, 4);
    if (LPR == 16) x += __shfl_xor(x, 8);
    return x;
}

template <typename T> __device__ __forceinline__ f32x4 load4(const T *p);
template <> __device__ __forceinline__ f32x4 load4<float>(const float *p) { return *reinterpret_cast<const f32x4 *>(p); }
template <> __device__ __forceinline__ f32x4 load4<__bf16>(const __bf16 *p)
{
    const bf16x4 x = *reinterpret_cast<const bf16x4 *>(p);
    return f32x4{(float)x[0], (float)x[1], (float)x[2], (float)x[3]};
}

__device__ __forceinline__ float dot4(const f32x4 &a, const f32x4 &b)
{
    return a[0] * b[0] + a[1] * b[1] + a[2] * b[2] + a[3] * b[3];
}

// NARROW: narrow heads -- q, k, z are dka wide, v, o dva, the state
// [dva][dka]; lanes and rows beyond take no part.
template <typename T, bool DELTA, bool FMAP, bool NARROW = false>
__global__ void __launch_bounds__(256)
step_kernel(const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v,
            const T *__restrict__ beta, const float *__restrict__ glog, const void *__restrict__ done, int done_f32,
            const float *S_in, const float *z_in, T *__restrict__ o, float *S_out, float *z_out, int H,
            float eps, int dka, int dva)  // S_in/S_out and z_in/z_out may alias (update in place)
{
    const int tid = threadIdx.x, c4 = tid % LPR, r0 = tid / LPR;
    const int64_t bh = blockIdx.x;
    const int b = (int)(bh / H);
    const bool reset = done_at(done, done_f32, b);
    const int dkw = NARROW ? dka : HD, dvw = NARROW ? dva : HD;
    const bool cin = !NARROW || 4 * c4 < dkw;  // this lane's four dk lie inside a row
    const T *qp = q + bh * dkw, *kp = k + bh * dkw, *vp = v + bh * dvw;

    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
    f32x4 k4 = cin ? load4<T>(kp + 4 * c4) : zero4, q4 = cin ? load4<T>(qp + 4 * c4) : zero4;
    if (FMAP && cin) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            k4[e] = elu1(k4[e]);
            q4[e] = elu1(q4[e]);
        }
    }
    const float *Sp = S_in ? S_in + bh * dvw * dkw : nullptr;
    const float decay = (!DELTA && glog) ? __expf(glog[bh]) : 1.f;  // gated linear attention: the carried state decays first
    f32x4 s[NP];
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const int row = r0 + RPP * p;
        // the carried state is loaded whether or not the flag says reset, and dropped by select below: a load
        // that waits for the flag would be a second trip to memory behind the first
        s[p] = (Sp && cin && (!NARROW || row < dvw)) ? *reinterpret_cast<const f32x4 *>(Sp + row * dkw + 4 * c4) : zero4;
    }
    float u[NP];
#pragma unroll
    for (int p = 0; p < NP; ++p) u[p] = (!NARROW || r0 + RPP * p < dvw) ? (float)vp[r0 + RPP * p] : 0.f;
#pragma unroll
    for (int p = 0; p < NP; ++p) s[p] = reset ? zero4 : s[p] * decay;
    if (DELTA) {
        const float bb = (float)beta[bh];
#pragma unroll
        for (int p = 0; p < NP; ++p) u[p] = bb * (u[p] - reduce_row(dot4(s[p], k4)));
    }
    float den = 1.f;
    if (!DELTA && z_out) {
        // every row's lanes recompute the normaliser of the sequence; row 0 stores it
        f32x4 z4 = (z_in && cin) ? *reinterpret_cast<const f32x4 *>(z_in + bh * dkw + 4 * c4) : zero4;
        if (reset) z4 = zero4;
        z4 += k4;
        // updated in place, z_out is z_in: every row's lanes must hold the carried z before row 0 overwrites it
        // (a row that read it afterwards would add k a second time and divide by the wrong normaliser)
        __syncthreads();
        if (r0 == 0 && cin) *reinterpret_cast<f32x4 *>(z_out + bh * dkw + 4 * c4) = z4;
        den = fmaxf(reduce_row(dot4(z4, q4)), eps);
    }
    float *So = S_out + bh * dvw * dkw;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const int row = r0 + RPP * p;
        s[p] += k4 * u[p];
        const bool rin = !NARROW || row < dvw;
        if (cin && rin) *reinterpret_cast<f32x4 *>(So + row * dkw + 4 * c4) = s[p];
        const float x = reduce_row(dot4(s[p], q4));
        if (c4 == 0 && rin) o[bh * dvw + row] = (T)(x / den);
    }
}

int check_step(const void *q, const void *k, const void *v, const void *done, const void *S_in,
               const void *o, const void *S_out, int64_t B, int64_t H, int64_t dk, int64_t dv, int dtype,
               int done_dtype, bool narrow = false)
{
    if (!q || !k || !v || !done || !o || !S_out) return MRX_ERR_INVALID_ARG;
    if (B <= 0 || H <= 0 || dk <= 0 || dv <= 0) return MRX_ERR_INVALID_ARG;
    if (dtype != MRX_F32 && dtype != MRX_BF16) return dtype == MRX_C64 ? MRX_ERR_UNSUPPORTED : MRX_ERR_INVALID_ARG;
    if (done_dtype != MRX_DONE_U8 && done_dtype != MRX_DONE_F32) return MRX_ERR_INVALID_ARG;
    // narrow: rows narrower than the build's head dim, in whole 16-byte segments
    const int64_t seg = dtype == MRX_BF16 ? 8 : 4;
    const bool narrow_ok = narrow && dk <= HD && dv <= HD && dk % seg == 0 && dv % seg == 0;
    if ((dk != HD || dv != HD) && !narrow_ok) return MRX_ERR_UNSUPPORTED;
    if (B * H >= (1ll << 31)) return MRX_ERR_INVALID_ARG;
    const void *ps[] = {q, k, v, S_in, o, S_out};
    for (const void *p : ps)
        if (!aligned(p, 16)) return MRX_ERR_INVALID_ARG;
    if (done_dtype == MRX_DONE_F32 && !aligned(done, 4)) return MRX_ERR_INVALID_ARG;
    return MRX_OK;
}

template <typename T, bool DELTA, bool FMAP>
int launch_step(hipStream_t st, const void *q, const void *k, const void *v, const void *beta, const void *done,
                int done_f32, const float *S_in, const float *z_in, void *o, float *S_out, float *z_out,
                int64_t B, int64_t H, float eps, int64_t dka = HD, int64_t dva = HD, const float *glog = nullptr)
{
    auto go = [&](auto narrow) {
        return launch_kernel((step_kernel<T, DELTA, FMAP, decltype(narrow)::value>), dim3((unsigned)(B * H)), dim3(256), 0, st,
                             (const T *)q, (const T *)k, (const T *)v, (const T *)beta, glog, done, done_f32, S_in, z_in,
                             (T *)o, S_out, z_out, (int)H, eps, (int)dka, (int)dva);
    };
    if (dka != HD || dva != HD) return go(std::true_type{});  // narrow heads
    return go(std::false_type{});
}

}  // namespace MRX_HD_NS
}  // namespace

MRX_EXPORT int MRX_API(mrx_linear_attn_step)(void *stream, const void *q, const void *k, const void *v, const void *done,
                                    const float *S_in, const float *z_in, void *o, float *S_out, float *z_out,
                                    int64_t B, int64_t H, int64_t dk, int64_t dv, int dtype, int done_dtype,
                                    int feature_map, float eps)
{
#if MRX_HD == 64
    if (dk <= 32 && dv <= 32) return mrx_linear_attn_step_hd32(stream, q, k, v, done, S_in, z_in, o, S_out, z_out, B, H, dk, dv, dtype, done_dtype, feature_map, eps);
#endif
    const int rc = check_step(q, k, v, done, S_in, o, S_out, B, H, dk, dv, dtype, done_dtype, true);
    if (rc != MRX_OK) return rc;
    if (feature_map != MRX_FMAP_NONE && feature_map != MRX_FMAP_ELU1) return MRX_ERR_INVALID_ARG;
    if ((z_in && !z_out) || !aligned(z_in, 16) || !aligned(z_out, 16)) return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const bool fm = feature_map == MRX_FMAP_ELU1;
    const int df = done_dtype == MRX_DONE_F32;
#define MRX_ARGS st, q, k, v, nullptr, done, df, S_in, z_in, o, S_out, z_out, B, H, eps, dk, dv
    if (dtype == MRX_BF16) return fm ? launch_step<__bf16, false, true>(MRX_ARGS) : launch_step<__bf16, false, false>(MRX_ARGS);
    return fm ? launch_step<float, false, true>(MRX_ARGS) : launch_step<float, false, false>(MRX_ARGS);
#undef MRX_ARGS
}

MRX_EXPORT int MRX_API(mrx_gated_linear_attn_step)(void *stream, const void *q, const void *k, const void *v,
                                          const float *g, const void *done, const float *S_in, void *o, float *S_out,
                                          int64_t B, int64_t H, int64_t dk, int64_t dv, int dtype, int done_dtype,
                                          int feature_map)
{
#if MRX_HD == 64
    if (dk <= 32 && dv <= 32) return mrx_gated_linear_attn_step_hd32(stream, q, k, v, g, done, S_in, o, S_out, B, H, dk, dv, dtype, done_dtype, feature_map);
#endif
    const int rc = check_step(q, k, v, done, S_in, o, S_out, B, H, dk, dv, dtype, done_dtype, true);
    if (rc != MRX_OK) return rc;
    if (!g || !aligned(g, 4)) return MRX_ERR_INVALID_ARG;
    if (feature_map != MRX_FMAP_NONE && feature_map != MRX_FMAP_ELU1) return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const bool fm = feature_map == MRX_FMAP_ELU1;
    const int df = done_dtype == MRX_DONE_F32;
#define MRX_ARGS st, q, k, v, nullptr, done, df, S_in, nullptr, o, S_out, nullptr, B, H, 0.f, dk, dv, g
    if (dtype == MRX_BF16) return fm ? launch_step<__bf16, false, true>(MRX_ARGS) : launch_step<__bf16, false, false>(MRX_ARGS);
    return fm ? launch_step<float, false, true>(MRX_ARGS) : launch_step<float, false, false>(MRX_ARGS);
#undef MRX_ARGS
}

MRX_EXPORT int MRX_API(mrx_delta_rule_step)(void *stream, const void *q, const void *k, const void *v, const void *beta,
                                   const void *done, const float *S_in, void *o, float *S_out, int64_t B,
                                   int64_t H, int64_t dk, int64_t dv, int dtype, int done_dtype)
{
#if MRX_HD == 64
    if (dk <= 32 && dv <= 32) return mrx_delta_rule_step_hd32(stream, q, k, v, beta, done, S_in, o, S_out, B, H, dk, dv, dtype, done_dtype);
#endif
    const int rc = check_step(q, k, v, done, S_in, o, S_out, B, H, dk, dv, dtype, done_dtype, true);
    if (rc != MRX_OK) return rc;
    if (!beta) return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const int df = done_dtype == MRX_DONE_F32;
    if (dtype == MRX_BF16)
        return launch_step<__bf16, true, false>(st, q, k, v, beta, done, df, S_in, nullptr, o, S_out, nullptr, B, H, 0.f, dk, dv);
    return launch_step<float, true, false>(st, q, k, v, beta, done, df, S_in, nullptr, o, S_out, nullptr, B, H, 0.f, dk, dv);
}
