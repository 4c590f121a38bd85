// The kernels declared in la_states.h.
#include "la_states.h"

#include "chunk_common.h"

namespace mrx {
inline namespace MRX_HD_NS {

namespace {

// One workgroup = one chunk of one sequence: slot <- sum over the kept rows r of y_r phi(x_r)^T,
// kept = the chunk's last episode (forward: what the chunk adds to the state that leaves it) or its
// first episode (backward: what it adds to the gradient of the state that enters it).
// NARROW: narrow heads -- x rows are dka wide in memory, y rows dva, a slot is [dva][dka]; the tiles keep the
// build's width with zeros beyond (after the feature map).
template <typename T, int C, bool FMAP, bool BWD, bool NARROW>
__global__ void __launch_bounds__(256)
la_chunk_state_kernel(const T *__restrict__ x, const T *__restrict__ y, const void *__restrict__ done, int done_f32,
                      float *__restrict__ slots, int Tlen, int H, int NC, int dka, int dva)
{
    constexpr int NW = 4, NTHR = 64 * NW, LDD = HD + pad_of<T>();
    using IO = TileIO<T, C, NTHR>;
    using TMS = TileMap<HD, HD, NW>;
    __shared__ __align__(16) T sX[C * LDD];
    __shared__ __align__(16) T sY[C * LDD];
    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    const int bh = blockIdx.x, c = blockIdx.y, b = bh / H, h = bh % H;
    const int t0 = c * C;
    const int dkw = NARROW ? dka : HD, dvw = NARROW ? dva : HD;
    const bool segx = !NARROW || (tid % IO::SEGS) * IO::KP < dkw, segy = !NARROW || (tid % IO::SEGS) * IO::KP < dvw;

    typename IO::Regs rx, ry;
    IO::zero(rx);
    IO::zero(ry);
    if (segx) IO::load(rx, x + ((int64_t)b * Tlen * H + h) * dkw, (int64_t)H * dkw, t0, Tlen, tid);
    if (segy) IO::load(ry, y + ((int64_t)b * Tlen * H + h) * dvw, (int64_t)H * dvw, t0, Tlen, tid);
    const bool dn = lane < C && t0 + lane < Tlen && done_at(done, done_f32, (int64_t)b * Tlen + t0 + lane);
    const unsigned long long dmask = __ballot(dn);
    const int nres = __popcll(dmask);
    if (segx) IO::template fmap<FMAP>(rx);  // columns beyond a narrow head's width stay zero
    if (nres != 0) {  // rows of other episodes leave by select: what they hold must not meet a zero in a product
        const int ep = BWD ? 0 : nres;
        auto keep = [&](int r) { return episode_of(dmask, r) == ep; };
        IO::mask_rows(rx, tid, keep);
        IO::mask_rows(ry, tid, keep);
    }
    // rows past the end of the sequence: y is zero there, and phi(0) = 1 in x is finite
    IO::to_lds(rx, sX, LDD, tid);
    IO::to_lds(ry, sY, LDD, tid);
    sync_lds();
    f32x4 acc[TMS::TPW];  // S^T: m = dk, n = dv
    zero_acc<TMS::TPW>(acc);
    gemm<T, HD, HD, C, KROW, KROW, NW>(acc, sX, LDD, sY, LDD, w, lane);
    float *slot = slots + ((int64_t)bh * NC + c) * (dvw * dkw);
#pragma unroll
    for (int j = 0; j < TMS::TPW; ++j) {
        const int dk0 = TMS::mt(w, j) * 16 + 4 * lg, dv = TMS::nt(w, j) * 16 + li;
        if (!NARROW || (dv < dvw && dk0 < dkw)) *reinterpret_cast<f32x4 *>(slot + dv * dkw + dk0) = acc[j];
    }
}

// grid (B * H, d * d / 1024): each thread carries four of the d x d state elements through the chunks.  Only the
// additions are sequential: the slots (and the reset flags) of the next group of eight chunks are
// requested before the current group is summed and written back, so that one trip to memory is exposed
// per sequence, not one per group.
// NARROW: narrow heads, the state's size is a run-time value.
template <bool NARROW>
__global__ void __launch_bounds__(256)
la_state_scan_kernel(float *__restrict__ slots, const float *__restrict__ init, float *__restrict__ fin,
                     const void *__restrict__ done, int done_f32, int Tlen, int H, int NC, int C, int backward, int Qn)
{
    const int Q = NARROW ? Qn : HD * HD / 4;  // f32x4 per state (d_v * d_k / 4)
    constexpr int G = 8;            // chunks per group
    const int tid = threadIdx.x, lane = tid & 63;
    const int bh = blockIdx.x, b = bh / H;
    const int idx = blockIdx.y * 256 + tid;
    const bool act = !NARROW || idx < Q;  // a narrow state has fewer elements than the workgroup has threads; the idle lanes
                                       // still bring their reset flags to the ballots
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    f32x4 S = init && act ? reinterpret_cast<const f32x4 *>(init)[(int64_t)bh * Q + idx] : zero;
    f32x4 *p = reinterpret_cast<f32x4 *>(slots) + (int64_t)bh * NC * Q + idx;
    auto chunk_of = [&](int s) { return backward ? NC - 1 - s : s; };
    f32x4 nt[G];
    uint32_t nd[G];  // raw reset flag of chunk row `lane`
    auto fetch = [&](int s0) {
#pragma unroll
        for (int u = 0; u < G; ++u) {
            const int s = s0 + u, c = chunk_of(s);
            nt[u] = zero;
            nd[u] = 0u;
            if (s < NC) {  // uniform over the workgroup
                if (act) nt[u] = p[(int64_t)c * Q];
                const int tt = c * C + lane;
                if (lane < C && tt < Tlen) nd[u] = done_raw(done, done_f32, (int64_t)b * Tlen + tt);
            }
        }
    };
    fetch(0);
    for (int s0 = 0; s0 < NC; s0 += G) {
        f32x4 t[G];
        bool cut[G];
#pragma unroll
        for (int u = 0; u < G; ++u) {
            t[u] = nt[u];
            cut[u] = __ballot(done_test(nd[u], done_f32)) != 0ull;
        }
        if (s0 + G < NC) fetch(s0 + G);
#pragma unroll
        for (int u = 0; u < G; ++u) {
            const int s = s0 + u;
            if (s < NC) {
                if (act) p[(int64_t)chunk_of(s) * Q] = S;
                S = cut[u] ? t[u] : S + t[u];
            }
        }
    }
    if (fin && act) reinterpret_cast<f32x4 *>(fin)[(int64_t)bh * Q + idx] = S;
}

template <typename T, int C>
int launch_states(hipStream_t st, const void *x, const void *y, const void *done, int done_f32, float *slots, int64_t B,
                  int64_t Tlen, int64_t H, bool fmap, bool backward, int64_t dk, int64_t dv)
{
    const int64_t NC = (Tlen + C - 1) / C;
    if (B * H > 0x7fffffffLL || NC > 65535) return MRX_ERR_INVALID_ARG;
    const dim3 grid((unsigned)(B * H), (unsigned)NC), block(256);
#define MRX_LAUNCH(FM, BW, RG)                                                                                         \
    launch_kernel((la_chunk_state_kernel<T, C, FM, BW, RG>), grid, block, 0, st, (const T *)x, (const T *)y, done,       \
                  done_f32, slots, (int)Tlen, (int)H, (int)NC, (int)dk, (int)dv)
    if (dk != HD || dv != HD) {  // narrow heads
        if (fmap) return backward ? MRX_LAUNCH(true, true, true) : MRX_LAUNCH(true, false, true);
        return backward ? MRX_LAUNCH(false, true, true) : MRX_LAUNCH(false, false, true);
    }
    if (fmap) return backward ? MRX_LAUNCH(true, true, false) : MRX_LAUNCH(true, false, false);
    return backward ? MRX_LAUNCH(false, true, false) : MRX_LAUNCH(false, false, false);
#undef MRX_LAUNCH
}

}  // namespace

int launch_la_chunk_states(hipStream_t st, const void *x, const void *y, const void *done, int done_f32, float *slots,
                           int64_t B, int64_t Tlen, int64_t H, int dtype, bool fmap, bool backward, int64_t dk, int64_t dv)
{
    if (dtype == MRX_BF16)
        return launch_states<__bf16, LA_BF16_CHUNK>(st, x, y, done, done_f32, slots, B, Tlen, H, fmap, backward, dk, dv);
    return launch_states<float, 32>(st, x, y, done, done_f32, slots, B, Tlen, H, fmap, backward, dk, dv);
}

int launch_la_state_scan(hipStream_t st, float *slots, const float *init, float *fin, const void *done, int done_f32,
                         int64_t B, int64_t Tlen, int64_t H, int C, bool backward, int64_t dk, int64_t dv)
{
    const int64_t NC = (Tlen + C - 1) / C;
    if (B * H > 0x7fffffffLL) return MRX_ERR_INVALID_ARG;
    const int Q = (int)(dk * dv / 4);
    const dim3 grid((unsigned)(B * H), (unsigned)((Q + 255) / 256));
    if (dk != HD || dv != HD)
        return launch_kernel(la_state_scan_kernel<true>, grid, dim3(256), 0, st, slots, init, fin, done, done_f32, (int)Tlen,
                             (int)H, (int)NC, C, backward ? 1 : 0, Q);
    return launch_kernel(la_state_scan_kernel<false>, grid, dim3(256), 0, st, slots, init, fin, done, done_f32, (int)Tlen,
                         (int)H, (int)NC, C, backward ? 1 : 0, Q);
}

}  // namespace MRX_HD_NS
}  // namespace mrx
