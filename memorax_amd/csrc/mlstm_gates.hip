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
// One wave walks one (b, h), sixty-four steps at a time: the lanes lie along time and scan their steps with
// shuffles -- m_t = max(m_{t-1} + A_t, B_t) composes as (A1, B1) then (A2, B2) = (A1 + A2, max(B1 + A2, B2)),
// a reset being an element whose A forgets the past -- so a block costs one trip to memory (the next block's
// loads are under way meanwhile) and six shuffle steps instead of sixty-four dependent steps.
#include <math.h>

#include "common.h"

namespace mrx {
namespace {

constexpr int MG_WAVES = 4, MG_THREADS = 64 * MG_WAVES;
constexpr float MG_NO_CARRY = -1e9f;  // the cell's initial m (mlstm.py: initialize_carry)
constexpr float MG_FORGET = -1e30f;   // "minus infinity" that stays finite under addition

struct GateIn {
    float li, lf;
    bool dn, in;
};

__global__ void __launch_bounds__(MG_THREADS)
mlstm_gates_fwd_kernel(const float *__restrict__ log_i, const float *__restrict__ log_f, const void *__restrict__ done,
                       int done_f32, const float *__restrict__ m0, float *__restrict__ m, float *__restrict__ g,
                       float *__restrict__ w, int64_t BH, int T, int H, float g_floor)
{
    const int lane = threadIdx.x & 63;
    const int64_t idx = (int64_t)blockIdx.x * MG_WAVES + (threadIdx.x >> 6);  // this wave's (b, h)
    if (idx >= BH) return;
    const int64_t b = idx / H;
    const int h = (int)(idx % H);
    auto fetch = [&](int t0) {
        GateIn x;
        const int t = t0 + lane;
        x.in = t < T;
        const int64_t bt = b * T + (x.in ? t : T - 1);
        x.li = log_i[bt * H + h];
        x.lf = log_f[bt * H + h];
        x.dn = done_at(done, done_f32, bt);
        return x;
    };
    float m_in = m0 ? m0[idx] : MG_NO_CARRY;
    GateIn nx = fetch(0);
    for (int t0 = 0; t0 < T; t0 += 64) {
        const GateIn x = nx;
        if (t0 + 64 < T) nx = fetch(t0 + 64);
        // steps past the end are the identity (0, forget): they pass the state through
        float A = !x.in ? 0.f : x.dn ? MG_FORGET : x.lf;
        float Bv = x.in ? x.li : MG_FORGET;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const float A1 = __shfl_up(A, off), B1 = __shfl_up(Bv, off);
            if (lane >= off) {
                Bv = fmaxf(B1 + A, Bv);
                A = fmaxf(A1 + A, MG_FORGET);  // several resets in a block: keep the sentinel in range
            }
        }
        const float mt = fmaxf(m_in + A, Bv);
        float mp = __shfl_up(mt, 1);
        if (lane == 0) mp = m_in;
        m_in = __shfl(mt, 63);
        if (x.in) {
            const int64_t o = (b * T + t0 + lane) * H + h;
            m[o] = mt;
            // where the carried branch wins, m_t - m_{t-1} and log f_t differ by rounding only: no decay above one
            g[o] = x.dn ? 0.f : fminf(fmaxf(x.lf + mp - mt, g_floor), 0.f);
            w[o] = __expf(x.li - mt);
        }
    }
}

// Gradients back through the recurrence.  M_t is the gradient that reaches m_t from everywhere: the caller's
// dm_t (the read-out's exp(-m), the carried m), g_t and w_t of its own step (-dg_t, -dw_t w_t) and what step
// t + 1 passes down -- through g_{t+1}, which holds m_t, and through the maximum when the carried branch won
// it.  With c_t = 1 where m_t took the carried branch (0 at a reset or where the input gate won) and
// x_t = dm_t - dg_t - dw_t w_t, what step t passes down is y_t = c_t y_{t+1} + (dg_t + c_t x_t): a linear
// recurrence running backwards in time, scanned over the lanes like the forward one.  A clamped g passes nothing.
struct GateBwdIn {
    float li, lf, mt, mp, gm, gg, gw;
    bool dn, in;
};

__global__ void __launch_bounds__(MG_THREADS)
mlstm_gates_bwd_kernel(const float *__restrict__ log_i, const float *__restrict__ log_f, const void *__restrict__ done,
                       int done_f32, const float *__restrict__ m0, const float *__restrict__ m,
                       const float *__restrict__ dm, const float *__restrict__ dg, const float *__restrict__ dw,
                       float *__restrict__ dlog_i, float *__restrict__ dlog_f, float *__restrict__ dm0, int64_t BH, int T, int H,
                       float g_floor)
{
    const int lane = threadIdx.x & 63;
    const int64_t idx = (int64_t)blockIdx.x * MG_WAVES + (threadIdx.x >> 6);
    if (idx >= BH) return;
    const int64_t b = idx / H;
    const int h = (int)(idx % H);
    const float m_first = m0 ? m0[idx] : MG_NO_CARRY;
    auto fetch = [&](int t0) {
        GateBwdIn x;
        const int t = t0 + lane;
        x.in = t < T;
        const int64_t bt = b * T + (x.in ? t : T - 1), o = bt * H + h;
        x.li = log_i[o];
        x.lf = log_f[o];
        x.dn = done_at(done, done_f32, bt);
        x.mt = m[o];
        x.mp = x.in && t > 0 ? m[o - H] : m_first;
        x.gm = dm ? dm[o] : 0.f;
        x.gg = dg ? dg[o] : 0.f;
        x.gw = dw ? dw[o] : 0.f;
        return x;
    };
    const int t_last = ((T - 1) / 64) * 64;
    float y_in = 0.f;  // what the block after this one passes down to this one's last step
    GateBwdIn nx = fetch(t_last);
    for (int t0 = t_last; t0 >= 0; t0 -= 64) {
        const GateBwdIn x = nx;
        if (t0 >= 64) nx = fetch(t0 - 64);
        const bool carried = x.in && !x.dn && x.mp + x.lf >= x.li;          // the branch of the maximum m_t took
        const bool open = x.in && !x.dn && x.lf + x.mp - x.mt > g_floor;     // g_t neither reset nor on the floor
        const float wt = __expf(x.li - x.mt);
        const float dgt = open ? x.gg : 0.f;
        const float xt = x.in ? x.gm - dgt - x.gw * wt : 0.f;
        // steps past the end are the identity (1, 0)
        float c = !x.in || carried ? 1.f : 0.f;
        float d = x.in ? dgt + (carried ? xt : 0.f) : 0.f;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const float c1 = __shfl_down(c, off), d1 = __shfl_down(d, off);
            if (lane + off < 64) {
                d = c * d1 + d;
                c = c * c1;
            }
        }
        const float y = c * y_in + d;        // what step t passes down to step t - 1
        float below = __shfl_down(y, 1);      // what reaches step t from step t + 1
        if (lane == 63) below = y_in;
        y_in = __shfl(y, 0);
        if (x.in) {
            const float M = xt + below;
            const int64_t o = (b * T + t0 + lane) * H + h;
            dlog_f[o] = dgt + (carried ? M : 0.f);
            dlog_i[o] = x.gw * wt + (carried ? 0.f : M);
        }
    }
    if (dm0 && lane == 0) dm0[idx] = y_in;
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
    return launch_kernel(mlstm_gates_fwd_kernel, dim3((unsigned)((BH + MG_WAVES - 1) / MG_WAVES)), dim3(MG_THREADS), 0,
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
    return launch_kernel(mlstm_gates_bwd_kernel, dim3((unsigned)((BH + MG_WAVES - 1) / MG_WAVES)), dim3(MG_THREADS), 0,
                         static_cast<hipStream_t>(stream), log_i, log_f, done, done_dtype == MRX_DONE_F32 ? 1 : 0, m0, m, dm, dg,
                         dw, dlog_i, dlog_f, dm0, BH, (int)T, (int)H, g_floor);
}
