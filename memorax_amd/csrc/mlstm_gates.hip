// The mLSTM cell's max-stabilised gates as one pass over time per (batch, head).
//
// The cell's elements (C, log_f, n, m) combine by the stabilised gated sum of mlstm.py:190-206 under the
// select-reset scan of memoroid.py:60-91.  Unrolled, the stabiliser is the recurrence
//     m_t = done_t ? log_i_t : max(m_{t-1} + log_f_t, log_i_t)
// and the state and the normaliser follow a gated linear recurrence whose log-decay and key weight are
//     g_t = done_t ? 0 : max(log_f_t + m_{t-1} - m_t, g_floor)          (<= 0)
//     w_t = exp(log_i_t - m_t)                                          (<= 1)
// -- what mrx_gated_linear_attn_* and mrx_linear_scan_* take.  (B,T,H) arrays are a sixty-fourth of the
// cell's (B,T,H,d) arrays; as array-library passes (a scan for the cumulative log f, a cumulative maximum per
// episode, a dozen element-wise steps, twice that in the backward) they cost more launches than bytes.
// One thread walks one (b, h): eight steps are loaded ahead of the chain that needs them.
#include <math.h>

#include "common.h"

namespace mrx {
namespace {

constexpr int MG_THREADS = 64, MG_STEPS = 8;
constexpr float MG_NO_CARRY = -1e9f;  // the cell's initial m (mlstm.py: initialize_carry)

__global__ void __launch_bounds__(MG_THREADS)
mlstm_gates_fwd_kernel(const float *__restrict__ log_i, const float *__restrict__ log_f, const void *__restrict__ done,
                       int done_f32, const float *__restrict__ m0, float *__restrict__ m, float *__restrict__ g,
                       float *__restrict__ w, int64_t BH, int T, int H, float g_floor)
{
    const int64_t idx = (int64_t)blockIdx.x * MG_THREADS + threadIdx.x;
    if (idx >= BH) return;
    const int64_t b = idx / H;
    const int h = (int)(idx % H);
    float mp = m0 ? m0[idx] : MG_NO_CARRY;
    for (int t0 = 0; t0 < T; t0 += MG_STEPS) {
        float li[MG_STEPS], lf[MG_STEPS];
        bool dn[MG_STEPS];
#pragma unroll
        for (int s = 0; s < MG_STEPS; ++s) {
            const bool in = t0 + s < T;
            const int64_t bt = b * T + (in ? t0 + s : T - 1);
            li[s] = log_i[bt * H + h];
            lf[s] = log_f[bt * H + h];
            dn[s] = done_at(done, done_f32, bt);
        }
#pragma unroll
        for (int s = 0; s < MG_STEPS; ++s) {
            if (t0 + s >= T) break;
            const float mt = dn[s] ? li[s] : fmaxf(mp + lf[s], li[s]);
            const int64_t o = (b * T + t0 + s) * H + h;
            m[o] = mt;
            g[o] = dn[s] ? 0.f : fmaxf(lf[s] + mp - mt, g_floor);
            w[o] = __expf(li[s] - mt);
            mp = mt;
        }
    }
}

// Gradients back through the recurrence, last step first.  M is the gradient that reaches m_t from everywhere:
// the caller's dm_t (the read-out's exp(-m), the carried m), g_t and w_t of its own step (-dg_t, -dw_t w_t)
// and what step t + 1 passes down (`below`: through g_{t+1}, which holds m_t, and through the maximum when
// the carried branch won it).  A reset cuts the chain; a clamped g passes nothing.
__global__ void __launch_bounds__(MG_THREADS)
mlstm_gates_bwd_kernel(const float *__restrict__ log_i, const float *__restrict__ log_f, const void *__restrict__ done,
                       int done_f32, const float *__restrict__ m0, const float *__restrict__ m,
                       const float *__restrict__ dm, const float *__restrict__ dg, const float *__restrict__ dw,
                       float *__restrict__ dlog_i, float *__restrict__ dlog_f, float *__restrict__ dm0, int64_t BH, int T, int H,
                       float g_floor)
{
    const int64_t idx = (int64_t)blockIdx.x * MG_THREADS + threadIdx.x;
    if (idx >= BH) return;
    const int64_t b = idx / H;
    const int h = (int)(idx % H);
    const float m_in = m0 ? m0[idx] : MG_NO_CARRY;
    float below = 0.f;
    for (int t1 = T; t1 > 0; t1 -= MG_STEPS) {  // steps t1 - 1 down to t1 - MG_STEPS
        float li[MG_STEPS], lf[MG_STEPS], mt[MG_STEPS + 1], gm[MG_STEPS], gg[MG_STEPS], gw[MG_STEPS];
        bool dn[MG_STEPS];
#pragma unroll
        for (int s = 0; s < MG_STEPS; ++s) {
            const int t = t1 - 1 - s;
            const int64_t bt = b * T + (t >= 0 ? t : 0), o = bt * H + h;
            li[s] = log_i[o];
            lf[s] = log_f[o];
            dn[s] = done_at(done, done_f32, bt);
            mt[s] = m[o];
            gm[s] = dm ? dm[o] : 0.f;
            gg[s] = dg ? dg[o] : 0.f;
            gw[s] = dw ? dw[o] : 0.f;
        }
        {
            const int t = t1 - 1 - MG_STEPS;  // the step before the block's first: its m enters the block's last
            mt[MG_STEPS] = t >= 0 ? m[(b * T + t) * H + h] : m_in;
        }
#pragma unroll
        for (int s = 0; s < MG_STEPS; ++s) {
            const int t = t1 - 1 - s;
            if (t < 0) break;
            const float mp = t == 0 ? m_in : mt[s + 1];
            const bool carried = !dn[s] && mp + lf[s] >= li[s];            // the branch of the maximum m_t took
            const bool open = !dn[s] && lf[s] + mp - mt[s] > g_floor;      // g_t neither reset nor clamped
            const float wt = __expf(li[s] - mt[s]);
            const float dgt = open ? gg[s] : 0.f;
            const float M = gm[s] + below - dgt - gw[s] * wt;
            const int64_t o = (b * T + t) * H + h;
            dlog_f[o] = dgt + (carried ? M : 0.f);
            dlog_i[o] = gw[s] * wt + (carried ? 0.f : M);
            below = dgt + (carried ? M : 0.f);
        }
    }
    if (dm0) dm0[idx] = below;
}

int check_gates(const void *log_i, const void *log_f, const void *done, int64_t B, int64_t T, int64_t H, int done_dtype)
{
    if (!log_i || !log_f || !done) return MRX_ERR_INVALID_ARG;
    if (B <= 0 || T <= 0 || H <= 0) return MRX_ERR_INVALID_ARG;
    if (done_dtype != MRX_DONE_U8 && done_dtype != MRX_DONE_F32) return MRX_ERR_INVALID_ARG;
    if (T > 0x7fffffff || H > 0x7fffffff) return MRX_ERR_UNSUPPORTED;
    return MRX_OK;
}

}  // namespace
}  // namespace mrx

extern "C" int mrx_mlstm_gates_fwd(void *stream, const float *log_i, const float *log_f, const void *done, const float *m0,
                                   float *m, float *g, float *w, int64_t B, int64_t T, int64_t H, int done_dtype,
                                   float g_floor)
{
    using namespace mrx;
    if (const int rc = check_gates(log_i, log_f, done, B, T, H, done_dtype); rc != MRX_OK) return rc;
    if (!m || !g || !w || !(g_floor <= 0.f)) return MRX_ERR_INVALID_ARG;
    if (const int rc = prepare_device(); rc != MRX_OK) return rc;
    const int64_t BH = B * H;
    return launch_kernel(mlstm_gates_fwd_kernel, dim3((unsigned)((BH + MG_THREADS - 1) / MG_THREADS)), dim3(MG_THREADS), 0,
                         static_cast<hipStream_t>(stream), log_i, log_f, done, done_dtype == MRX_DONE_F32 ? 1 : 0, m0, m, g, w,
                         BH, (int)T, (int)H, g_floor);
}

extern "C" int mrx_mlstm_gates_bwd(void *stream, const float *log_i, const float *log_f, const void *done, const float *m0,
                                   const float *m, const float *dm, const float *dg, const float *dw, float *dlog_i,
                                   float *dlog_f, float *dm0, int64_t B, int64_t T, int64_t H, int done_dtype, float g_floor)
{
    using namespace mrx;
    if (const int rc = check_gates(log_i, log_f, done, B, T, H, done_dtype); rc != MRX_OK) return rc;
    if (!m || !dlog_i || !dlog_f || !(g_floor <= 0.f)) return MRX_ERR_INVALID_ARG;
    if (const int rc = prepare_device(); rc != MRX_OK) return rc;
    const int64_t BH = B * H;
    return launch_kernel(mlstm_gates_bwd_kernel, dim3((unsigned)((BH + MG_THREADS - 1) / MG_THREADS)), dim3(MG_THREADS), 0,
                         static_cast<hipStream_t>(stream), log_i, log_f, done, done_dtype == MRX_DONE_F32 ? 1 : 0, m0, m, dm, dg,
                         dw, dlog_i, dlog_f, dm0, BH, (int)T, (int)H, g_floor);
}
