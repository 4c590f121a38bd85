// Backward of chunked causal linear attention and of the DeltaNet delta rule.
//
// Chunks are walked from the last to the first with dS (gradient of the state
// leaving the chunk) carried in MFMA accumulators; the state entering each chunk
// comes from the checkpoints the forward call wrote (S_chk), as does the delta rule's
// triangular factor Tm (Tm_chk); everything else of the forward (U', masked QK^T) is
// recomputed per chunk.  A chunk that
// contains resets is processed once per episode, last episode first, with the rows
// of the other episodes zeroed by select; dS only flows into the episode that
// leaves the chunk and only out of the episode that enters it.
//
// Linear attention per pass (rows i >= j; all rows of one episode):
//   Aqk = tril(Q K^T)                      dV  = Aqk^T dO + K dS^T
//   dAqk = tril(dO V^T)                    dQ  = dO S + dAqk K
//   dK  = dAqk^T Q + V dS                  dS <- dS + Q^T dO            (stored as dS^T)
// The delta rule's formulas stand at its kernel.
// Every tile lives in LDS once, in its natural orientation; products that contract over
// the row index read it through transpose loads (KROW operands).  Gradients leave through dead
// LDS tiles and are written to memory row-wise (tile_rows_to_global).
#include <type_traits>

#include "chunk_common.h"
#include "la_states.h"
#if MRX_HD == 64
#include "hd32_api.h"
#endif


namespace {
inline namespace MRX_HD_NS {

using namespace mrx;

template <typename T, int C> struct BwdDims {
    static constexpr int PAD = pad_of<T>();
    static constexpr int LDD = HD + PAD;  // leading dim of tiles with 64 columns
    static constexpr int LDC = C + PAD;   // leading dim of tiles with C columns
    static constexpr int szRD = C * LDD * sizeof(T);   // [C][64]
    static constexpr int szDD = HD * LDD * sizeof(T);  // [64][64]
    static constexpr int szCC = C * LDC * sizeof(T);   // [C][C]
};

// d(phi)/dx recovered from the staged phi(x): phi > 1 <=> x > 0 (derivative 1), else phi' = phi.
template <bool FMAP> __device__ __forceinline__ float fmap_grad(float phi) { return FMAP ? (phi > 1.f ? 1.f : phi) : 1.f; }

// =====================================================================================
// linear attention: 8 tiles, two workgroups per CU
// =====================================================================================
template <typename T, int C, bool GATED = false, bool NORM = false> struct LaBwdSmem : BwdDims<T, C> {
    using D = BwdDims<T, C>;
    static constexpr int oQ = 0, oK = oQ + D::szRD, oV = oK + D::szRD, oDO = oV + D::szRD,
                         oS = oDO + D::szRD, oDS = oS + D::szDD, oAqk = oDS + D::szDD,
                         oDAqk = oAqk + D::szCC,
                         oG = oDAqk + D::szCC,    // gated: G[C], [WM][C] row-dot partials, exp(G)[C]
                         oN = oG + (GATED ? (2 + TileMap<HD, C, 4>::WM) * C * 4 : 0),
                         // normalised read-out: dden fp32 [C], dden T-typed [C] (C * 4 bytes kept), z fp32 [64], dz fp32 [64]
                         total = oN + (NORM ? 2 * C * 4 + 2 * HD * 4 : 0);
};

// What the normalised read-out adds to the backward argument list.
struct NormBwdArgs {
    const void *o;        // (B,T,H,64) T-typed: the normalised outputs of the forward call
    const float *den;     // (B,T,H): the clamped denominators
    const float *z_chk;   // (B,H,NC,64): z entering each chunk
    const float *dz_last; // (B,H,64) or null
    float *dz0;           // (B,H,64) or null
    float eps;
    const float *d_ss;    // (B,H,T) or null: gradient of the forward call's sums of squares of the outputs
};

// GATED: S_t = r_t exp(g_t) S_{t-1} + v_t k_t^T.  With G the cumulative log-decay inside the chunk
// (per episode), a_i = exp(G_i), b_j = exp(G_last - G_j), c = exp(G_last), D_ij = exp(G_i - G_j):
//   Aqk, dAqk carry the factor D;  dV = Aqk^T dO + diag(b) K dS^T;  dQ = diag(a) dO S + dAqk K;
//   dK = dAqk^T Q + diag(b) V dS;  dS <- c dS + (diag(a) Q)^T dO.
// NORM (normalised read-out o_i = num_i / den_i, den_i = max(q_i . z_i, eps), z the running sum of
// the keys of the episode; a gradient d_ss of the forward call's row sums of squares ss_i = |o_i|^2
// first joins the output gradient, dout_i <- dout_i + 2 d_ss_i o_i): with dnum_i = dout_i / den_i taking the place of dO and
// dden_i = -(dout_i . o_i) / den_i (0 where the clamp is active),
//   dAqk_ij += dden_i (j <= i);  dQ_i += dden_i z_in;  dK_j += dz;  dz <- dz + sum_i dden_i Q_i,
// z_in the sum entering the chunk (first episode only), dz the gradient of the sum leaving it.
// The gradient of the log-decays follows from edot_i = q_i . dq_i - k_i . dk_i (taken on the
// feature-mapped q, k and their gradients): dg_t is the sum of edot over the rows i >= t of t's
// episode (plus <S_last, dS_last> when the episode reaches the end), 0 at a reset step.  The kernel
// walks the chunks and their episodes from the end anyway, so wave 0 carries that running sum in
// a register (a reverse cumulative sum over the chunk's rows by lane shuffles, cut at resets) and
// writes dg itself.
// PAR (plain linear attention): one workgroup per chunk (grid.y = chunk).  Slot c of S_chk holds, in
// fp32, the state entering chunk c and slot c of dS_last -- then a (B,H,NC,64,64) array -- the gradient
// of the state leaving it (la_states.h); the workgroup forms the chunk's dQ, dK, dV from them and neither
// walks the state nor accumulates its gradient.
// NARROW: narrow heads, as in the forward kernel: q, k and their gradients are dka wide in memory, v, dout, o and
// dv dva, states [dva][dka], z [dka]; tiles keep the build's width, zero beyond, and only the rows' own
// width is ever stored.
template <typename T, int C, bool FMAP, bool GATED, bool NORM, bool PAR = false, bool NARROW = false>
__global__ void __launch_bounds__(256, 2)
la_bwd_kernel(const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v,
              const float *__restrict__ glog, const void *__restrict__ done, int done_f32,
              const void *__restrict__ S_chk, const float *__restrict__ S_last, const T *__restrict__ dout,
              const float *__restrict__ dS_last, T *__restrict__ dq, T *__restrict__ dk, T *__restrict__ dv, float *__restrict__ dg,
              float *__restrict__ dS0, int Tlen, int H, NormBwdArgs na, int dka, int dva)
{
    static_assert(!(GATED && NORM), "the normalised read-out belongs to plain linear attention");
    static_assert(!PAR || (!GATED && !NORM), "one workgroup per chunk: plain linear attention only");
    constexpr int NW = 4, NTHR = 64 * NW;
    using L = LaBwdSmem<T, C, GATED, NORM>;
    using Frag = typename TT<T>::frag;
    using IO = TileIO<T, C, NTHR>;
    using IOS = TileIO<T, HD, NTHR>;
    using P4 = typename TT<T>::pack4;
    constexpr int LDD = L::LDD, LDC = L::LDC;
    extern __shared__ __align__(16) unsigned char smem[];
    T *sQ = reinterpret_cast<T *>(smem + L::oQ);
    T *sK = reinterpret_cast<T *>(smem + L::oK);
    T *sV = reinterpret_cast<T *>(smem + L::oV);
    T *sDO = reinterpret_cast<T *>(smem + L::oDO);
    T *sS = reinterpret_cast<T *>(smem + L::oS);
    T *sDS = reinterpret_cast<T *>(smem + L::oDS);
    T *sAqk = reinterpret_cast<T *>(smem + L::oAqk);
    T *sDAqk = reinterpret_cast<T *>(smem + L::oDAqk);
    float *sG = reinterpret_cast<float *>(smem + L::oG);
    float *sE = sG + C;  // [WM][C] partial row dots
    float *sEa = sE + TileMap<HD, C, 4>::WM * C;  // a_i = exp(G_i)
    float *sDd = reinterpret_cast<float *>(smem + L::oN);       // dden[C]
    T *sDdT = reinterpret_cast<T *>(smem + L::oN + C * 4);      // dden[C], T-typed (MFMA operand)
    float *sZf = reinterpret_cast<float *>(smem + L::oN + 2 * C * 4);  // z entering the chunk
    float *sDZ = sZf + HD;                                      // dz leaving the pass

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    const int bh = sequence_of_block(blockIdx.x, gridDim.x, H), b = bh / H, h = bh % H;
    const int dkw = NARROW ? dka : HD, dvw = NARROW ? dva : HD;  // row widths in memory
    const int64_t rs = (int64_t)H * dkw, rsv = (int64_t)H * dvw;  // row strides of q, k / v, dout, o
    const int64_t base = ((int64_t)b * Tlen * H + h) * dkw, basev = ((int64_t)b * Tlen * H + h) * dvw;
    const bool segk = !NARROW || (tid % (HD / TT<T>::KP)) * TT<T>::KP < dkw;  // this thread's 16-byte segment lies inside a q/k row
    const bool segv = !NARROW || (tid % (HD / TT<T>::KP)) * TT<T>::KP < dvw;  // ... inside a v row
    const int NC = (Tlen + C - 1) / C;
    const int c_hi = PAR ? (int)blockIdx.y : NC - 1, c_lo = PAR ? c_hi : 0;  // the chunks this workgroup walks, downwards
    const int64_t slot = PAR ? ((int64_t)bh * NC + c_hi) * dvw : (int64_t)bh * dvw;  // in state rows
    auto in_state = [&](int dvv, int dk0) { return !NARROW || (dvv < dvw && dk0 < dkw); };

    using TMS = TileMap<HD, HD, NW>;
    using TMA = TileMap<C, C, NW>;
    using TMR = TileMap<HD, C, NW>;
    f32x4 dSacc[TMS::TPW];  // dS^T: m = dk, n = dv
#pragma unroll
    for (int j = 0; j < TMS::TPW; ++j) {
        const int dk0 = TMS::mt(w, j) * 16 + 4 * lg, dvv = TMS::nt(w, j) * 16 + li;
        dSacc[j] = dS_last && in_state(dvv, dk0) ? *reinterpret_cast<const f32x4 *>(dS_last + (slot + dvv) * dkw + dk0)
                                                 : f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // normalised read-out: dz[dk], held like a column of dS^T; fp32 (VN): component 0 holds
    // dz[dk = 16 mt + li] and the sums run on the vector ALU (see the forward kernel's z)
    constexpr bool VN = sizeof(T) == 4;
    f32x4 dzacc[TMS::MBW];
#pragma unroll
    for (int mi = 0; mi < TMS::MBW; ++mi) {
        const int dkt = TMS::mt(w, mi * TMS::NBW) * 16;
        dzacc[mi] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (NORM && na.dz_last) {
            if (VN) { if (!NARROW || dkt + li < dkw) dzacc[mi][0] = na.dz_last[(int64_t)bh * dkw + dkt + li]; }
            else if (!NARROW || dkt + 4 * lg < dkw) dzacc[mi] = *reinterpret_cast<const f32x4 *>(na.dz_last + (int64_t)bh * dkw + dkt + 4 * lg);
        }
    }

    // The state leaving, then entering, the chunk at hand (S^T, in the layout of dS^T).  Without a decay
    // the update of a chunk can be undone, S_c = S_{c+1} - V_c^T K_c, so the state is walked back in
    // fp32 registers from the forward call's S_last and read from the forward call's (fp32) checkpoints
    // only where the walk cannot pass -- chunks with resets -- and at every walk_anchor()-th chunk, where it
    // starts afresh from the exact state: the chunks the forward call writes then.
    // Gated: every chunk has a checkpoint in the I/O type, staged row-wise.
    constexpr bool WALK = !GATED;
    constexpr int NSA = WALK ? TMS::TPW : 1;
    f32x4 Sacc[NSA];
    zero_acc<NSA>(Sacc);
    if (WALK) {
#pragma unroll
        for (int j = 0; j < NSA; ++j) {
            const int dk0 = TMS::mt(w, j) * 16 + 4 * lg, dvv = TMS::nt(w, j) * 16 + li;
            if (in_state(dvv, dk0))
                Sacc[j] = *reinterpret_cast<const f32x4 *>((PAR ? reinterpret_cast<const float *>(S_chk) : S_last) +
                                                           (slot + dvv) * dkw + dk0);
        }
    }

    // gated: the running sum behind dg, held by wave 0; it starts from <S_last, dS_last>
    float dg_carry = 0.f;
    if (GATED && dS_last && S_last) {
        float part = 0.f;
#pragma unroll
        for (int j = 0; j < TMS::TPW; ++j) {
            const int dk0 = TMS::mt(w, j) * 16 + 4 * lg, dvv = TMS::nt(w, j) * 16 + li;
            if (!in_state(dvv, dk0)) continue;
            const f32x4 sl = *reinterpret_cast<const f32x4 *>(S_last + ((int64_t)bh * dvw + dvv) * dkw + dk0);
            part += dSacc[j][0] * sl[0] + dSacc[j][1] * sl[1] + dSacc[j][2] * sl[2] + dSacc[j][3] * sl[3];
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) part += __shfl_xor(part, off);
        if (lane == 0) sE[w] = part;
        sync_lds();
        dg_carry = sE[0] + sE[1] + sE[2] + sE[3];
        sync_lds();  // sE is written again by the first pass
    }

    typename IO::Regs rq, rk, rv, rdo, ro;
    float rden[IO::PASSES], rdss[IO::PASSES];
#pragma unroll
    for (int p = 0; p < IO::PASSES; ++p) rdss[p] = 0.f;
    f32x4 rz = {0.f, 0.f, 0.f, 0.f};
    typename IOS::Regs rS;
    // raw bits, tested when the chunk is staged; the reset flags of the chunk after the next one too:
    // whether its checkpoint must be fetched is known when the next prefetch starts
    uint32_t rdone = 0u, rdone2 = 0u;
    // Does the chunk about to be prefetched take its entering state from S_chk?  Not known for the
    // first one (its reset flags are part of the same prefetch): if it does, the checkpoint is fetched
    // when the chunk is reached.
    bool need_S = false;
    float rg = 0.f;       // log-decay of chunk row `lane` (gated)
    // Running element offsets of this thread's loads, stepped back by one chunk per prefetch
    // (64-bit adds instead of per-chunk index multiplications).  The prefetch is issued in parts
    // spread over the phases so that the address unit works beside LDS and MFMA work:
    // part 0: q, k; 1: v, dout; 2: S and the per-row scalars.
    const int tlast = c_hi * C;
    int64_t roff[IO::PASSES];
    int64_t roffv[NARROW ? IO::PASSES : 1];  // v, dout, o where their rows are not as wide as those of q and k
#pragma unroll
    for (int p = 0; p < IO::PASSES; ++p) {
        roff[p] = base + (int64_t)(tlast + IO::row_of(tid, p)) * rs + (tid % IO::SEGS) * IO::KP;
        if (NARROW) roffv[p] = basev + (int64_t)(tlast + IO::row_of(tid, p)) * rsv + (tid % IO::SEGS) * IO::KP;
    }
    int64_t soff = ((int64_t)bh * NC + c_hi) * dvw * dkw +
                   (WALK ? li * dkw + 4 * lg : (tid / IOS::SEGS) * dkw + (tid % IOS::SEGS) * IOS::KP);
    int64_t doff = (int64_t)b * Tlen + tlast + lane;
    int64_t noff[IO::PASSES];  // den of the rows this thread stages
#pragma unroll
    for (int p = 0; p < IO::PASSES; ++p) noff[p] = (int64_t)bh * Tlen + tlast + IO::row_of(tid, p);  // den: (B,H,T)
    int64_t zoff = ((int64_t)bh * NC + c_hi) * dkw + 4 * (tid % (HD / 4));
    int tpre = tlast;
    auto prefetch_part = [&](int part) {
        typename IO::F z;
#pragma unroll
        for (int e = 0; e < IO::KP; ++e) z[e] = (T)0.f;
        if (part < 2) {
#pragma unroll
            for (int p = 0; p < IO::PASSES; ++p) {
                const bool in = (IO::FULL || IO::row_of(tid, p) < C) && tpre + IO::row_of(tid, p) < Tlen;
                if (part == 0) {
                    rq.v[p] = in && segk ? *reinterpret_cast<const typename IO::F *>(q + roff[p]) : z;
                    rk.v[p] = in && segk ? *reinterpret_cast<const typename IO::F *>(k + roff[p]) : z;
                } else {
                    const int64_t ov = NARROW ? roffv[p] : roff[p];
                    rv.v[p] = in && segv ? *reinterpret_cast<const typename IO::F *>(v + ov) : z;
                    rdo.v[p] = in && segv ? *reinterpret_cast<const typename IO::F *>(dout + ov) : z;
                    if (NORM) ro.v[p] = in && segv ? *reinterpret_cast<const typename IO::F *>((const T *)na.o + ov) : z;
                }
            }
        } else {
            if (!WALK) {
#pragma unroll
                for (int p = 0; p < IOS::PASSES; ++p)
                    if (IOS::FULL || IOS::row_of(tid, p) < HD) {  // a [32][32] tile has fewer segments than threads
                        if (!NARROW || (IOS::row_of(tid, p) < dvw && (tid % IOS::SEGS) * IOS::KP < dkw))
                            rS.v[p] = load_once<typename IOS::F>(reinterpret_cast<const T *>(S_chk) + soff + p * IOS::RPP * dkw);
                        else
                            rS.v[p] = z;
                    }
            } else if (need_S) {
                // straight into the state registers: the chunk at hand has formed its state (the first
                // phase), and the next chunk, taking a checkpoint, does not walk back from it
#pragma unroll
                for (int j = 0; j < NSA; ++j)
                    if (in_state(TMS::nt(w, j) * 16 + li, TMS::mt(w, j) * 16 + 4 * lg))
                        Sacc[j] = *reinterpret_cast<const f32x4 *>(reinterpret_cast<const float *>(S_chk) + soff +
                                                                   TMS::nt(w, j) * 16 * dkw + TMS::mt(w, j) * 16);
                    else
                        Sacc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
            rdone = 0u;
            rdone2 = 0u;
            rg = 0.f;
            if (lane < C && tpre + lane < Tlen) {
                rdone = done_raw(done, done_f32, doff);
                if (GATED) rg = glog[doff * H + h];
            }
            if (WALK && !PAR && lane < C && tpre >= C) rdone2 = done_raw(done, done_f32, doff - C);
            if (NORM) {
#pragma unroll
                for (int p = 0; p < IO::PASSES; ++p) {
                    const bool in = (IO::FULL || IO::row_of(tid, p) < C) && tpre + IO::row_of(tid, p) < Tlen;
                    rden[p] = in ? na.den[noff[p]] : 1.f;
                    if (na.d_ss) rdss[p] = in ? na.d_ss[noff[p]] : 0.f;
                    noff[p] -= C;
                }
                if (!NARROW || 4 * (tid % (HD / 4)) < dkw) rz = *reinterpret_cast<const f32x4 *>(na.z_chk + zoff);
                zoff -= dkw;
            }
#pragma unroll
            for (int p = 0; p < IO::PASSES; ++p) {
                roff[p] -= (int64_t)C * rs;
                if (NARROW) roffv[p] -= (int64_t)C * rsv;
            }
            soff -= dvw * dkw;
            doff -= C;
            tpre -= C;
        }
    };
#pragma unroll
    for (int part = 0; part < 3; ++part) prefetch_part(part);

    // Gradients leave through LDS as whole rows (a store from accumulators writes 16 pieces of 32 bytes
    // per instruction): at the end of a pass, once every product has read its operands, dV, dQ, dK are
    // written over V, Q, K; the next pass reads them back row-wise -- each thread exactly the 16 bytes it
    // is about to restage, so no barrier is needed in between -- after it has consumed its prefetched
    // registers (the wait for those then does not cover these stores).
    unsigned long long pend_dmask = 0ull;
    int pend_nres = 0, pend_pass = 0, pend_t0 = -1;
    auto flush_pending = [&]() {
        if (pend_t0 >= 0) {
            auto keep = [&](int r) { return pend_nres == 0 || episode_of(pend_dmask, r) == pend_pass; };
            const int64_t off = base + (int64_t)pend_t0 * rs;
            tile_rows_to_global<T, C, NTHR>(sV, LDD, dv + basev + (int64_t)pend_t0 * rsv, rsv, pend_t0, Tlen, tid, keep, dvw);
            tile_rows_to_global<T, C, NTHR>(sQ, LDD, dq + off, rs, pend_t0, Tlen, tid, keep, dkw);
            tile_rows_to_global<T, C, NTHR>(sK, LDD, dk + off, rs, pend_t0, Tlen, tid, keep, dkw);
        }
        pend_t0 = -1;
    };
    P4 hV[TMR::TPW], hQ[TMR::TPW], hK[TMR::TPW];  // the three gradients of a pass, rounded, until its operands are dead
    auto hold = [&](const f32x4 *acc, P4 *h, auto scale) {
#pragma unroll
        for (int j = 0; j < TMR::TPW; ++j) {
            const f32x4 sc = scale(TMR::nt(w, j) * 16 + li, TMR::mt(w, j) * 16 + 4 * lg);
            h[j] = TT<T>::pack(acc[j][0] * sc[0], acc[j][1] * sc[1], acc[j][2] * sc[2], acc[j][3] * sc[3]);
        }
    };
    auto park = [&](const P4 *h, T *dst) {
#pragma unroll
        for (int j = 0; j < TMR::TPW; ++j)
            *reinterpret_cast<P4 *>(dst + (TMR::nt(w, j) * 16 + li) * LDD + TMR::mt(w, j) * 16 + 4 * lg) = h[j];
    };

    for (int c = c_hi; c >= c_lo; --c) {
        const int t0 = c * C;
        const unsigned long long dmask = __ballot(done_test(rdone, done_f32) && lane < C);
        const int nres = __popcll(dmask);
        const bool ckpt = PAR || !WALK || nres != 0 || (c > 0 && c % walk_anchor<T>() == 0);  // the entering state comes from S_chk
        if (WALK && !PAR)  // for the chunk prefetched during this one
            need_S = __ballot(done_test(rdone2, done_f32) && lane < C) != 0ull || (c >= 2 && (c - 1) % walk_anchor<T>() == 0);
        for (int pass = nres; pass >= 0; --pass) {
            auto live = [&](int r) { return nres == 0 || episode_of(dmask, r) == pass; };
            // gated: cumulative log-decay of this pass's episode (as in the forward kernel)
            float G = 0.f, Glast = 0.f;
            if (GATED) {
                G = (lane < C && live(lane) && !((dmask >> lane) & 1ull)) ? rg : 0.f;
#pragma unroll
                for (int off = 1; off < C; off <<= 1) {
                    const float up = __shfl_up(G, off);
                    if (lane >= off) G += up;
                }
                Glast = __shfl(G, C - 1);
                if (w == 0 && lane < C) {
                    sG[lane] = G;
                    sEa[lane] = __expf(G);
                }
            }
            // ---- stage -------------------------------------------------------------
            {
                typename IO::Regs fq = rq, fk = rk, fv = rv, fdo = rdo;
                if (segk) {  // columns beyond a narrow head's width stay zero: phi(0) = 1 must not count
                    IO::template fmap<FMAP>(fq);
                    IO::template fmap<FMAP>(fk);
                }
                if (nres != 0) {
                    IO::mask_rows(fq, tid, live);
                    IO::mask_rows(fk, tid, live);
                    IO::mask_rows(fv, tid, live);
                    IO::mask_rows(fdo, tid, live);
                }
                if (NORM) {
                    // dden_i = -(dout_i . o_i) / den_i where the clamp is inactive; dO <- dout / den
                    float inv[IO::PASSES];
#pragma unroll
                    for (int p = 0; p < IO::PASSES; ++p) {
                        float dot = 0.f;
#pragma unroll
                        for (int e = 0; e < IO::KP; ++e) dot += (float)rdo.v[p][e] * (float)ro.v[p][e];
                        dot = seg_sum<IO::SEGS>(dot);
                        const int r = IO::row_of(tid, p);
                        const bool on = (IO::FULL || r < C) && live(r);
                        if (na.d_ss) {  // dout_i + 2 d_ss_i o_i takes the place of dout_i (live rows only, by select)
                            float oo = 0.f;
#pragma unroll
                            for (int e = 0; e < IO::KP; ++e) oo += (float)ro.v[p][e] * (float)ro.v[p][e];
                            oo = seg_sum<IO::SEGS>(oo);
                            const float two = 2.f * rdss[p];
                            dot += two * oo;
                            if (on) {
#pragma unroll
                                for (int e = 0; e < IO::KP; ++e) fdo.v[p][e] = (T)(((float)rdo.v[p][e] + two * (float)ro.v[p][e]) / rden[p]);
                            }
                        }
                        inv[p] = on ? 1.f / rden[p] : 1.f;
                        const float dd = (on && rden[p] > na.eps) ? -dot * inv[p] : 0.f;
                        if (tid % IO::SEGS == 0 && (IO::FULL || r < C)) {
                            sDd[r] = dd;
                            sDdT[r] = (T)dd;
                        }
                    }
                    if (!na.d_ss) IO::scale_rows(fdo, inv);
                    if (tid < HD / 4) *reinterpret_cast<f32x4 *>(sZf + 4 * tid) = rz;
                }
                flush_pending();  // reads what this thread is about to overwrite in sV, sQ, sK
                IO::to_lds(fq, sQ, LDD, tid);
                IO::to_lds(fk, sK, LDD, tid);
                IO::to_lds(fv, sV, LDD, tid);
                IO::to_lds(fdo, sDO, LDD, tid);
                if (!WALK) {
                    typename IOS::Regs fS = rS;
                    if (pass != 0) IOS::zero(fS);
                    IOS::to_lds(fS, sS, LDD, tid);  // S[dv][dk]
                }
            }
            if (pass != nres) zero_acc<TMS::TPW>(dSacc);  // an episode that ends inside the chunk
            store_acc<T, HD, HD, NW>(dSacc, sDS, LDD, w, lane);  // dS[dv][dk]
            if (NORM) {
                if (pass != nres) zero_acc<TMS::MBW>(dzacc);
                if (w < TMS::WM && (VN ? lg == 0 : li == 0)) {
#pragma unroll
                    for (int mi = 0; mi < TMS::MBW; ++mi) {
                        float *dst = sDZ + TMS::mt(w, mi * TMS::NBW) * 16;
                        if (VN) dst[li] = dzacc[mi][0];
                        else *reinterpret_cast<f32x4 *>(dst + 4 * lg) = dzacc[mi];
                    }
                }
            }
            sync_lds();
            const bool pre = pass == 0 && c > c_lo;
            if (pre) prefetch_part(0);

            // ---- Aqk[i][j] = q_i.k_j, dAqk[i][j] = do_i.v_j, both j <= i ------------------
            {
                f32x4 acc[TMA::TPW];
                zero_acc<TMA::TPW>(acc);
                // masked store; gated: times exp(G_i - G_j) (exponent <= 0 where kept)
                auto store_tril = [&](const f32x4 *a, T *dst, bool add_dden) {
#pragma unroll
                    for (int j = 0; j < TMA::TPW; ++j) {
                        const int m = TMA::mt(w, j) * 16 + 4 * lg, n = TMA::nt(w, j) * 16 + li;
                        float x[4];
                        const float dd = (NORM && add_dden) ? sDd[n] : 0.f;
                        if (GATED) {
                            const float gn = sG[n];
                            const f32x4 gm = *reinterpret_cast<const f32x4 *>(sG + m);
#pragma unroll
                            for (int e = 0; e < 4; ++e) x[e] = (m + e <= n) ? a[j][e] * __expf(gn - gm[e]) : 0.f;
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; ++e) x[e] = (m + e <= n) ? a[j][e] + dd : 0.f;
                        }
                        *reinterpret_cast<P4 *>(dst + n * LDC + m) = TT<T>::pack(x[0], x[1], x[2], x[3]);
                    }
                };
                gemm<T, C, C, HD, ROWK, ROWK, NW>(acc, sK, LDD, sQ, LDD, w, lane);  // D[m = j][n = i]
                store_tril(acc, sAqk, false);
                zero_acc<TMA::TPW>(acc);
                gemm<T, C, C, HD, ROWK, ROWK, NW>(acc, sV, LDD, sDO, LDD, w, lane);  // D[m = j][n = i]
                store_tril(acc, sDAqk, true);
            }
            // ---- the state entering the chunk, S^T[dk][dv] = S_leaving^T - sum_c K[c][dk] V[c][dv], or the
            //      forward call's checkpoint (first episode of a chunk with resets; the later ones start
            //      from zero); rounded into sS[dv][dk] -----------------------------------------------------
            if (WALK) {
                if (!ckpt) {
                    f32x4 acc[TMS::TPW];
                    zero_acc<TMS::TPW>(acc);
                    gemm<T, HD, HD, C, KROW, KROW, NW>(acc, sK, LDD, sV, LDD, w, lane);
#pragma unroll
                    for (int j = 0; j < NSA; ++j) Sacc[j] -= acc[j];
                    store_acc<T, HD, HD, NW>(Sacc, sS, LDD, w, lane);
                } else if (pass == 0) {
                    if (!PAR && c == NC - 1) {  // the one checkpoint no prefetch could know of (PAR: loaded at the start)
#pragma unroll
                        for (int j = 0; j < NSA; ++j)
                            if (in_state(TMS::nt(w, j) * 16 + li, TMS::mt(w, j) * 16 + 4 * lg))
                                Sacc[j] = *reinterpret_cast<const f32x4 *>(reinterpret_cast<const float *>(S_chk) +
                                                                           ((int64_t)bh * NC + c) * dvw * dkw + li * dkw + 4 * lg +
                                                                           TMS::nt(w, j) * 16 * dkw + TMS::mt(w, j) * 16);
                            else
                                Sacc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
                    }  // else the prefetch of the chunk before has left the checkpoint in Sacc
                    store_acc<T, HD, HD, NW>(Sacc, sS, LDD, w, lane);
                } else {
                    f32x4 zero[TMS::TPW];
                    zero_acc<TMS::TPW>(zero);
                    store_acc<T, HD, HD, NW>(zero, sS, LDD, w, lane);
                }
            }
            sync_lds();
            if (pre) prefetch_part(1);
            auto one = [](int, int) { return f32x4{1.f, 1.f, 1.f, 1.f}; };
            float ep[TMR::NBW];  // gated: per-lane partials of edot for rows nt * 16 + li
#pragma unroll
            for (int j = 0; j < TMR::NBW; ++j) ep[j] = 0.f;
            auto rowdot = [&](const f32x4 *acc, const T *X, float sign) {
#pragma unroll
                for (int j = 0; j < TMR::TPW; ++j) {
                    const int d0 = TMR::mt(w, j) * 16 + 4 * lg, r = TMR::nt(w, j) * 16 + li;
                    const P4 x = *reinterpret_cast<const P4 *>(X + r * LDD + d0);
                    ep[j % TMR::NBW] += sign * (acc[j][0] * (float)x[0] + acc[j][1] * (float)x[1] +
                                                acc[j][2] * (float)x[2] + acc[j][3] * (float)x[3]);
                }
            };
            // ---- dV^T[dv][j] = sum_i dO[i][dv] Aqk[i][j] + sum_dk dS[dv][dk] K[j][dk] -------
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                if (GATED) {  // the state term of row j carries b_j = exp(G_last - G_j)
                    gemm<T, HD, C, HD, ROWK, ROWK, NW>(acc, sDS, LDD, sK, LDD, w, lane);
#pragma unroll
                    for (int j = 0; j < TMR::TPW; ++j) acc[j] *= __expf(Glast - sG[TMR::nt(w, j) * 16 + li]);
                    gemm<T, HD, C, C, KROW, KROW, NW>(acc, sDO, LDD, sAqk, LDC, w, lane);
                } else {
                    gemm<T, HD, C, C, KROW, KROW, NW>(acc, sDO, LDD, sAqk, LDC, w, lane);
                    gemm<T, HD, C, HD, ROWK, ROWK, NW>(acc, sDS, LDD, sK, LDD, w, lane);
                }
                hold(acc, hV, one);
            }
            if (pre) prefetch_part(2);
            // ---- dQ^T[dk][i] = sum_dv S[dv][dk] dO[i][dv] + sum_j K[j][dk] dAqk[i][j] ---------
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                gemm<T, HD, C, HD, KROW, ROWK, NW>(acc, sS, LDD, sDO, LDD, w, lane);
                if (GATED) {  // the incoming state reaches row i decayed by a_i = exp(G_i)
#pragma unroll
                    for (int j = 0; j < TMR::TPW; ++j) acc[j] *= __expf(sG[TMR::nt(w, j) * 16 + li]);
                }
                gemm<T, HD, C, C, KROW, ROWK, NW>(acc, sK, LDD, sDAqk, LDC, w, lane);
                if (GATED) rowdot(acc, sQ, 1.f);
                if (NORM && pass == 0) {  // den_i = q_i . (z_in + ...): dQ_i += dden_i z_in
#pragma unroll
                    for (int j = 0; j < TMR::TPW; ++j) {
                        const f32x4 zz = *reinterpret_cast<const f32x4 *>(sZf + TMR::mt(w, j) * 16 + 4 * lg);
                        acc[j] += zz * sDd[TMR::nt(w, j) * 16 + li];
                    }
                }
                auto sc = [&](int r, int d0) {
                    const P4 x = *reinterpret_cast<const P4 *>(sQ + r * LDD + d0);
                    return f32x4{fmap_grad<FMAP>((float)x[0]), fmap_grad<FMAP>((float)x[1]),
                                 fmap_grad<FMAP>((float)x[2]), fmap_grad<FMAP>((float)x[3])};
                };
                hold(acc, hQ, sc);
            }
            // ---- dK^T[dk][j] = sum_i Q[i][dk] dAqk[i][j] + sum_dv dS[dv][dk] V[j][dv] -----------
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                if (GATED) {
                    gemm<T, HD, C, HD, KROW, ROWK, NW>(acc, sDS, LDD, sV, LDD, w, lane);
#pragma unroll
                    for (int j = 0; j < TMR::TPW; ++j) acc[j] *= __expf(Glast - sG[TMR::nt(w, j) * 16 + li]);
                    gemm<T, HD, C, C, KROW, KROW, NW>(acc, sQ, LDD, sDAqk, LDC, w, lane);
                    rowdot(acc, sK, -1.f);
                } else {
                    gemm<T, HD, C, C, KROW, KROW, NW>(acc, sQ, LDD, sDAqk, LDC, w, lane);
                    gemm<T, HD, C, HD, KROW, ROWK, NW>(acc, sDS, LDD, sV, LDD, w, lane);
                }
                if (NORM && pass == nres) {  // every key of the leaving episode is part of the z that leaves
#pragma unroll
                    for (int j = 0; j < TMR::TPW; ++j)
                        acc[j] += *reinterpret_cast<const f32x4 *>(sDZ + TMR::mt(w, j) * 16 + 4 * lg);
                }
                auto sc = [&](int r, int d0) {
                    const P4 x = *reinterpret_cast<const P4 *>(sK + r * LDD + d0);
                    return f32x4{fmap_grad<FMAP>((float)x[0]), fmap_grad<FMAP>((float)x[1]),
                                 fmap_grad<FMAP>((float)x[2]), fmap_grad<FMAP>((float)x[3])};
                };
                hold(acc, hK, sc);
            }
            // ---- dS^T[dk][dv] += sum_c Q[c][dk] dO[c][dv]  (gated: c dS + sum_c a_c Q[c] dO[c]) -----
            if (GATED) {
                const float cl = __expf(Glast);
#pragma unroll
                for (int j = 0; j < TMS::TPW; ++j) dSacc[j] *= cl;
#pragma unroll
                for (int j = 0; j < TMR::NBW; ++j) {
                    float x = ep[j];
                    x += __shfl_xor(x, 16);
                    x += __shfl_xor(x, 32);
                    if (lg == 0) sE[(w % TMR::WM) * C + TMR::nt(w, j) * 16 + li] = x;
                }
            }
            float dzpart[TMS::MBW];  // fp32: per-lane partial sums over the lane's k slots
#pragma unroll
            for (int mi = 0; mi < TMS::MBW; ++mi) dzpart[mi] = 0.f;
            auto dz_q = [&](int mi, int kb, Frag &xq) {
                if (NORM) {  // dz[dk] += sum_i Q[i][dk] dden_i
                    if (VN) {
                        const float *dd = sDd + kb * TT<T>::KB + TT<T>::KP * lg;
#pragma unroll
                        for (int e = 0; e < TT<T>::KP; ++e) dzpart[mi] += (float)xq[e] * dd[e];
                    } else {
                        dzacc[mi] = TT<T>::mma(xq, TT<T>::template load<ROWK>(sDdT, 0, 0, kb * TT<T>::KB, lane), dzacc[mi]);
                    }
                }
                if (GATED) {  // row c of Q enters the state update as a_c Q[c]: scale the fragment along k
                    const float *ea = sEa + kb * TT<T>::KB + TT<T>::KP * lg;
#pragma unroll
                    for (int e = 0; e < TT<T>::KP; ++e) xq[e] = (T)((float)xq[e] * ea[e]);
                }
            };
            if (!PAR) gemm<T, HD, HD, C, KROW, KROW, NW>(dSacc, sQ, LDD, sDO, LDD, w, lane, dz_q);
            if (NORM && VN) {
#pragma unroll
                for (int mi = 0; mi < TMS::MBW; ++mi) {
                    float x = dzpart[mi];
                    x += __shfl_xor(x, 16);
                    x += __shfl_xor(x, 32);
                    dzacc[mi][0] += x;
                }
            }
            sync_lds();  // every product has read its operands
            park(hV, sV);
            park(hQ, sQ);
            park(hK, sK);
            pend_dmask = dmask;
            pend_nres = nres;
            pend_pass = pass;
            pend_t0 = t0;
            sync_lds();
            if (GATED && w == 0) {
                const bool on = lane < C && live(lane);  // rows past the end of the sequence hold zeros
                float x = 0.f;
                if (on) {
#pragma unroll
                    for (int sl = 0; sl < TMR::WM; ++sl) x += sE[sl * C + lane];
                }
                // x_r <- sum over the rows i >= r of this pass's episode (its rows are consecutive)
#pragma unroll
                for (int off = 1; off < C; off <<= 1) {
                    const float up = __shfl_down(x, off);
                    if (lane + off < C) x += up;
                }
                if (pass == nres) x += dg_carry;  // the episode that reaches the end of the chunk goes on into the later steps
                if (on && t0 + lane < Tlen) dg[((int64_t)b * Tlen + t0 + lane) * H + h] = ((dmask >> lane) & 1ull) ? 0.f : x;
                if (pass == 0) dg_carry = (dmask & 1ull) ? 0.f : __shfl(x, 0);  // cut where the chunk opens with a reset
            }
        }
    }
    flush_pending();  // the last pass ended with a barrier
    if (dS0 && !PAR) {
#pragma unroll
        for (int j = 0; j < TMS::TPW; ++j) {
            const int dk0 = TMS::mt(w, j) * 16 + 4 * lg, dvv = TMS::nt(w, j) * 16 + li;
            if (in_state(dvv, dk0)) *reinterpret_cast<f32x4 *>(dS0 + ((int64_t)bh * dvw + dvv) * dkw + dk0) = dSacc[j];
        }
    }
    if (NORM && na.dz0 && w < TMS::WM && (VN ? lg == 0 : li == 0)) {
#pragma unroll
        for (int mi = 0; mi < TMS::MBW; ++mi) {
            const int dkt = TMS::mt(w, mi * TMS::NBW) * 16;
            float *dst = na.dz0 + (int64_t)bh * dkw + dkt;
            if (VN) { if (!NARROW || dkt + li < dkw) dst[li] = dzacc[mi][0]; }
            else if (!NARROW || dkt + 4 * lg < dkw) *reinterpret_cast<f32x4 *>(dst + 4 * lg) = dzacc[mi];
        }
    }
}

// =====================================================================================
// delta rule: fourteen LDS tiles (68 KB for bf16, 127 KB for fp32, C = 32), two of them reused
// once their first tenant is dead.  bf16: two workgroups per CU.
//
// Per pass, with S the state entering the chunk, Tm = (I + A)^-1 from the forward call:
//   V0 = V - K S^T,  V~ = diag(beta) V0,  U' = Tm V~            (W = T K and U = T V are never formed)
//   Aqk = tril(Q K^T),  dU' = Aqk^T dO + K dS^T,  dAqk = tril(dO U'^T)
//   Z = Tm^T dU',  dV = diag(beta) Z,  dbeta = rowdot(Z, V0) + rowdot(K, R)
//   dA = -tril(Z U'^T, -1),  R = dA K
//     (dTm = dU' V~^T and dA = -Tm^T dTm Tm^T = -(Tm^T dU')(Tm V~)^T; the part of dTm above the
//      diagonal, which is no parameter, only reaches the part of dA above the diagonal, so neither
//      dTm nor the two products with Tm^T are formed)
//   dQ = dO S + dAqk K
//   dK = dAqk^T Q + U' dS - (diag(beta) Z) S + diag(beta) R + dA^T (diag(beta) K)
//   dS <- dS + Q^T dO - K^T (diag(beta) Z)                       (stored as dS^T)
// =====================================================================================
template <typename T, int C, int NW> struct DeltaBwdSmem : BwdDims<T, C> {
    using D = BwdDims<T, C>;
    static_assert(D::szCC <= D::szRD && D::szCC <= D::szDD, "reused regions must hold a [C][C] tile");
    // nine [C][64] tiles, two [64][64], three [C][C]
    static constexpr int oK = 0, oV = oK + D::szRD, oQ = oV + D::szRD, oDO = oQ + D::szRD,
                         oBK = oDO + D::szRD, oVt = oBK + D::szRD, oU = oVt + D::szRD, oDU = oU + D::szRD,
                         oZb = oDU + D::szRD, oS = oZb + D::szRD, oDS = oS + D::szDD,
                         oAqk = oDS + D::szDD, oTm = oAqk + D::szCC, oDT = oTm + D::szCC,
                         oBeta = oDT + D::szCC, oDb = oBeta + C * 4;
    static constexpr int NSLOT = TileMap<HD, C, NW>::WM;  // dbeta partials per row: one per feature block
    // prologue variant: 1 / |k| per row, then [NSLOT][C] partials of k_n . dk_n
    static constexpr int oKinv = oDb + NSLOT * C * 4;
    static constexpr int oFlag = oKinv + (1 + NSLOT) * C * 4;  // merged episodes: one screen flag per wave
    static constexpr int total = oFlag + NW * 4;
};

// PRO: the cell's prologue is part of the call -- k_n = k / max(|k|, 1e-12), beta = sigmoid(b) are
// formed while staging (as in the forward kernel) and the gradients are taken back through them:
//   dk = (dk_n - k_n (k_n . dk_n)) / |k| ,   db = dbeta beta (1 - beta).
// NARROW: narrow heads, as in the linear-attention kernels -- q, k, dq, dk are dka wide in memory, v, dout, dv dva,
// the states [dva][dka]; tiles keep the build's width with zeros beyond, only the rows' own width is stored.
#ifdef MRX_PHASE_CLOCKS
// [0] cycles inside matrix products, [1] cycles alive, both summed over the waves of every workgroup of
// every delta_bwd_kernel launch since the last reset; [2] workgroups counted.
static __device__ unsigned long long g_phase_clocks[4];
#endif

// MERGE: a chunk that holds resets is done in ONE unit instead of one per episode, as in the forward kernel
// (chunk_fwd_kernel): masks keep the episodes apart where they could meet -- Aqk, dAqk and dA (pairs of one
// episode only), the three terms with the state entering the chunk (rows of the first episode), the two
// terms with the gradient of the state leaving it (rows of the last episode) and the update of that
// gradient (rows of the first episode) -- after a screen of the chunk's inputs that rules out any
// non-finite intermediate (chunk_common.h); a chunk that fails the screen takes the units per episode.
template <typename T, int C, int NW, bool PRO, bool NARROW = false, bool MERGE = false>
__global__ void __launch_bounds__(64 * NW, sizeof(T) == 2 ? 2 : 1)
delta_bwd_kernel(const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v,
                 const T *__restrict__ beta, const void *__restrict__ done, int done_f32,
                 const T *__restrict__ S_chk, const T *__restrict__ Tm_chk,
                 const T *__restrict__ dout, const float *__restrict__ dS_last, T *__restrict__ dq,
                 T *__restrict__ dk, T *__restrict__ dv, T *__restrict__ dbeta,
                 float *__restrict__ dS0, int Tlen, int H, int dka, int dva)
{
    constexpr int NTHR = 64 * NW;
    using L = DeltaBwdSmem<T, C, NW>;
    using IO = TileIO<T, C, NTHR>;
    using IOS = TileIO<T, HD, NTHR>;
    using IOT = TileIO<T, C, NTHR, C>;  // the [C][C] triangular factor
    using P4 = typename TT<T>::pack4;
    constexpr int LDD = L::LDD, LDC = L::LDC;
    extern __shared__ __align__(16) unsigned char smem[];
    auto at = [&](int off) { return reinterpret_cast<T *>(smem + off); };
    T *sK = at(L::oK), *sQ = at(L::oQ), *sDO = at(L::oDO), *sBK = at(L::oBK);
    T *sV = at(L::oV);                                    // V[c][dv] -> V0 = V - K S^T (in place)
    T *sVt = at(L::oVt), *sZ = at(L::oVt);                // V~ = beta V0 -> Z[c][dv]
    T *sU = at(L::oU), *sDU = at(L::oDU), *sZb = at(L::oZb);
    T *sS = at(L::oS);                                    // S[dv][dk]
    T *sDS = at(L::oDS);                                  // dS[dv][dk]
    T *sAqk = at(L::oAqk), *sDAqk = at(L::oAqk);          // Aqk^T[j][i] -> dAqk[i][j]
    T *sTm = at(L::oTm), *sDA = at(L::oDT);               // Tm[i][j], dA[i][j]
    float *sBeta = reinterpret_cast<float *>(smem + L::oBeta);
    float *sDb = reinterpret_cast<float *>(smem + L::oDb);  // [NSLOT][C] dbeta partials
    float *sKinv = reinterpret_cast<float *>(smem + L::oKinv);  // prologue: 1 / |k_row|
    float *sKd = sKinv + C;                                      // prologue: [NSLOT][C] partials of k_n . dk_n
    float *sFlag = reinterpret_cast<float *>(smem + L::oFlag);
    static_assert(!MERGE || !NARROW, "merged episodes: full-width heads");

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    const int bh = sequence_of_block(blockIdx.x, gridDim.x, H), b = bh / H, h = bh % H;
    const int dkw = NARROW ? dka : HD, dvw = NARROW ? dva : HD;  // row widths in memory
    const int64_t rs = (int64_t)H * dkw, rsv = (int64_t)H * dvw;  // row strides of q, k / v, dout
    const int64_t base = ((int64_t)b * Tlen * H + h) * dkw, basev = ((int64_t)b * Tlen * H + h) * dvw;
    const bool segk = !NARROW || (tid % (HD / TT<T>::KP)) * TT<T>::KP < dkw;  // this thread's 16-byte segment lies inside a q/k row
    const bool segv = !NARROW || (tid % (HD / TT<T>::KP)) * TT<T>::KP < dvw;  // ... inside a v row
    auto in_state = [&](int dvv, int dk0) { return !NARROW || (dvv < dvw && dk0 < dkw); };
    const int NC = (Tlen + C - 1) / C;

    using TMS = TileMap<HD, HD, NW>;
    using TMA = TileMap<C, C, NW>;
    using TMR = TileMap<HD, C, NW>;
    constexpr int NSLOT = L::NSLOT;
#ifdef MRX_PHASE_CLOCKS
    if (tid == 0) wg_product_clocks = 0ull;  // the first product comes after the staging barrier
    const long long kernel_clk0 = clock64();
#endif

    f32x4 dSacc[TMS::TPW];  // dS^T: m = dk, n = dv
#pragma unroll
    for (int j = 0; j < TMS::TPW; ++j) {
        const int dk0 = TMS::mt(w, j) * 16 + 4 * lg, dvv = TMS::nt(w, j) * 16 + li;
        dSacc[j] = dS_last && in_state(dvv, dk0) ? *reinterpret_cast<const f32x4 *>(dS_last + ((int64_t)bh * dvw + dvv) * dkw + dk0)
                                                 : f32x4{0.f, 0.f, 0.f, 0.f};
    }

    typename IO::Regs rq, rk, rv, rdo;
    typename IOS::Regs rS;
    typename IOT::Regs rTm;
    uint32_t rdone = 0u, rbeta = 0u;  // raw bits, converted when the chunk is staged
    uint32_t rbrow[IO::PASSES];       // beta of the rows this thread stages
    // Running element offsets of this thread's loads and stores, stepped back by one chunk per
    // iteration (64-bit adds instead of per-chunk index multiplications).
    const int tlast = (NC - 1) * C;
    int64_t roff[IO::PASSES], boff[IO::PASSES];
    int64_t roffv[NARROW ? IO::PASSES : 1];  // v, dout where their rows are not as wide as those of q and k
#pragma unroll
    for (int p = 0; p < IO::PASSES; ++p) {
        const int r = tlast + IO::row_of(tid, p);
        roff[p] = base + (int64_t)r * rs + (tid % IO::SEGS) * IO::KP;  // q/k/v/dout: row r, this thread's segment
        if (NARROW) roffv[p] = basev + (int64_t)r * rsv + (tid % IO::SEGS) * IO::KP;
        boff[p] = ((int64_t)b * Tlen + r) * H + h;                     // beta of row r
    }
    int64_t soff = ((int64_t)bh * NC + NC - 1) * dvw * dkw + (tid / IOS::SEGS) * dkw + (tid % IOS::SEGS) * IOS::KP;
    int64_t tmoff = ((int64_t)bh * NC + NC - 1) * C * C + (tid / IOT::SEGS) * C + (tid % IOT::SEGS) * IOT::KP;
    int64_t doff = (int64_t)b * Tlen + tlast + lane;  // done/beta of chunk row `lane`
    int tpre = tlast;                                 // first time step of the chunk about to be prefetched
    // The prefetch of the next chunk is issued in parts, two in each of the first three phases, so
    // that the address unit works through the loads beside the phases' LDS and MFMA work instead of
    // stalling every wave at one point, and all of them are under way before the first store of the
    // pass.  part 0: q, 1: k, 2: v, 3: dout, 4: S, 5: Tm and the per-row scalars.
    auto prefetch_part = [&](int part) {
        typename IO::F z;
#pragma unroll
        for (int e = 0; e < IO::KP; ++e) z[e] = (T)0.f;
        if (part < 4) {
            const T *src = part == 0 ? q : part == 1 ? k : part == 2 ? v : dout;
            typename IO::Regs &dst = part == 0 ? rq : part == 1 ? rk : part == 2 ? rv : rdo;
            const bool seg_in = part < 2 ? segk : segv;
#pragma unroll
            for (int p = 0; p < IO::PASSES; ++p)
                dst.v[p] = seg_in && (IO::FULL || IO::row_of(tid, p) < C) && tpre + IO::row_of(tid, p) < Tlen
                               ? *reinterpret_cast<const typename IO::F *>(src + (NARROW && part >= 2 ? roffv[p] : roff[p])) : z;
        } else if (part == 4) {
#pragma unroll
            for (int p = 0; p < IOS::PASSES; ++p)
                if (IOS::FULL || IOS::row_of(tid, p) < HD) {
                    if (!NARROW || (IOS::row_of(tid, p) < dvw && (tid % IOS::SEGS) * IOS::KP < dkw))
                        rS.v[p] = load_once<typename IOS::F>(S_chk + soff + p * IOS::RPP * dkw);
                    else
                        rS.v[p] = z;
                }
        } else {
#pragma unroll
            for (int p = 0; p < IOT::PASSES; ++p)
                if (IOT::FULL || IOT::row_of(tid, p) < C)  // a [C][C] tile may have fewer segments than threads
                    rTm.v[p] = load_once<typename IOT::F>(Tm_chk + tmoff + p * IOT::RPP * C);
#pragma unroll
            for (int p = 0; p < IO::PASSES; ++p) {
                rbrow[p] = (IO::FULL || IO::row_of(tid, p) < C) && tpre + IO::row_of(tid, p) < Tlen ? load_raw<T>(beta + boff[p]) : 0u;
                roff[p] -= (int64_t)C * rs;
                if (NARROW) roffv[p] -= (int64_t)C * rsv;
                boff[p] -= (int64_t)C * H;
            }
            rdone = 0u;
            rbeta = 0u;
            if (lane < C && tpre + lane < Tlen) {
                rdone = done_raw(done, done_f32, doff);
                if (w == 0) rbeta = load_raw<T>(beta + doff * H + h);
            }
            soff -= dvw * dkw;
            tmoff -= C * C;
            doff -= C;
            tpre -= C;
        }
    };
#pragma unroll
    for (int part = 0; part < 6; ++part) prefetch_part(part);
    int64_t dboff = ((int64_t)b * Tlen + tlast + tid) * H + h;

    // Gradients leave through LDS: an accumulator tile holds four features of sixteen rows per lane
    // group, so a store from accumulators writes 16 pieces of 32 bytes per instruction; written to a
    // dead LDS tile first (dV is there anyway) and read back row-wise, every instruction writes whole
    // 128-byte rows (measured: the three stores from accumulators cost a third of the kernel).
    // dK is complete only in a pass's last phase; it waits in sU -- not written again before the
    // next pass's second phase -- and goes to memory after the next pass has been staged, so that no
    // store is issued right before the wait for the prefetched loads.  dbeta waits in a register.
    unsigned long long pend_dmask = 0ull;
    int pend_nres = 0, pend_pass = 0, pend_t0 = -1;
    int64_t pend_dboff = 0;
    float pend_db = 0.f;
    bool pend_db_on = false;
    auto flush_pending = [&]() {  // call after a barrier that follows the writes to sU
        if (pend_t0 >= 0) {
            auto keep = [&](int r) { return pend_nres == 0 || episode_of(pend_dmask, r) == pend_pass; };
            tile_rows_to_global<T, C, NTHR>(sU, LDD, dk + base + (int64_t)pend_t0 * rs, rs, pend_t0, Tlen, tid, keep, dkw);
        }
        if (pend_db_on) dbeta[pend_dboff] = (T)pend_db;
        pend_t0 = -1;
        pend_db_on = false;
    };

    for (int c = NC - 1; c >= 0; --c, dboff -= (int64_t)C * H) {
        const int t0 = c * C;
        const unsigned long long dmask = __ballot(done_test(rdone, done_f32) && lane < C);
        const int nres = __popcll(dmask);
        bool mg = false;  // this chunk's episodes in one unit
        if constexpr (MERGE) {
            if (nres != 0) {
                bool ok = true;
                auto small = [](float x, float lim) { return fabsf(x) <= lim; };  // false for NaN
#pragma unroll
                for (int p = 0; p < IO::PASSES; ++p) {
#pragma unroll
                    for (int e = 0; e < IO::KP; ++e)
                        ok = ok && small((float)rq.v[p][e], MERGE_IN_MAX) && small((float)rk.v[p][e], MERGE_IN_MAX) &&
                             small((float)rv.v[p][e], MERGE_IN_MAX) && small((float)rdo.v[p][e], MERGE_IN_MAX);
                    ok = ok && small(raw_to_float<T>(rbrow[p]), MERGE_IN_MAX);
                }
#pragma unroll
                for (int p = 0; p < IOT::PASSES; ++p)
                    if (IOT::FULL || IOT::row_of(tid, p) < C) {
#pragma unroll
                        for (int e = 0; e < IOT::KP; ++e) ok = ok && small((float)rTm.v[p][e], MERGE_IN_MAX);
                    }
#pragma unroll
                for (int p = 0; p < IOS::PASSES; ++p)
                    if (IOS::FULL || IOS::row_of(tid, p) < HD) {
#pragma unroll
                        for (int e = 0; e < IOS::KP; ++e) ok = ok && small((float)rS.v[p][e], MERGE_STATE_MAX);
                    }
#pragma unroll
                for (int j = 0; j < TMS::TPW; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e) ok = ok && small(dSacc[j][e], MERGE_STATE_MAX);
                if (lane == 0) sFlag[w] = __ballot(!ok) != 0ull ? 1.f : 0.f;
                sync_lds();
                float bad = 0.f;
#pragma unroll
                for (int j = 0; j < NW; ++j) bad += sFlag[j];
                mg = bad == 0.f;
            }
        }
        const int r_first = mg ? (int)__builtin_ctzll(dmask) : C;        // rows below it: the episode that enters the chunk
        const int r_last = mg ? 63 - (int)__builtin_clzll(dmask) : 0;   // rows from it on: the episode that leaves it
        auto one_episode = [&](int lo, int hi) { return (dmask & ((2ull << hi) - (2ull << lo))) == 0ull; };  // no reset in rows lo + 1 .. hi
        // One unit of work: the rows of one episode of the chunk (`pass` counts the episodes), or -- merged
        // episodes, MG -- all rows of a chunk that holds resets at once (pass 0).  In the instance that can
        // merge, the masks are part of the straight-line code of every unit (all-pass values where there is
        // nothing to mask): a branch per mask would cut the phases into pieces the scheduler cannot overlap
        // (measured: 10 % on chunks without resets), two copies of the unit do not fit the registers.
        const bool MG = MERGE && mg;
        // ff / fl: 1 for the rows (nt * 16 + li of the wave's [C][64]-shaped tiles) of the first / last episode, else
        // 0; cw: the packed words of the wave's [C][C] tile j keep the bits of the elements that pair two rows of
        // one episode; fw: the words of an operand fragment read along the chunk rows (element e of the fragment of k block kb is
        // row kb KB + KP lg + e) keep the bits of the rows of the first episode; keep_dS: 0 where the gradient of
        // the state that leaves the chunk does not flow on past it
        constexpr int NKB = C / TT<T>::KB, WPF = TT<T>::KP * (int)sizeof(T) / 4;  // k blocks; 32-bit words per fragment
        float ff[TMR::NBW], fl[TMR::NBW], keep_dS = 1.f;
        constexpr int WPP = 4 * (int)sizeof(T) / 4;  // 32-bit words of four packed elements
        unsigned cw[TMA::TPW][WPP], fw[NKB][WPF];
#pragma unroll
        for (int j = 0; j < TMA::TPW; ++j)
#pragma unroll
            for (int i = 0; i < WPP; ++i) cw[j][i] = ~0u;
#pragma unroll
        for (int ni = 0; ni < TMR::NBW; ++ni) ff[ni] = fl[ni] = 1.f;
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
            for (int i = 0; i < WPF; ++i) fw[kb][i] = ~0u;
        if (MG) {  // once per chunk, outside the unit's phases
            keep_dS = 0.f;
#pragma unroll
            for (int ni = 0; ni < TMR::NBW; ++ni) {
                const int r = TMR::nt(w, ni) * 16 + li;
                ff[ni] = r < r_first ? 1.f : 0.f;
                fl[ni] = r >= r_last ? 1.f : 0.f;
            }
#pragma unroll
            for (int j = 0; j < TMA::TPW; ++j) {
                bool same[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int m = TMA::mt(w, j) * 16 + 4 * lg + e, n = TMA::nt(w, j) * 16 + li;
                    same[e] = one_episode(m < n ? m : n, m < n ? n : m);
                }
#pragma unroll
                for (int i = 0; i < WPP; ++i)
                    cw[j][i] = sizeof(T) == 2 ? (same[2 * i] ? 0x0000ffffu : 0u) | (same[2 * i + 1] ? 0xffff0000u : 0u)
                                              : (same[i % 4] ? ~0u : 0u);
            }
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                for (int i = 0; i < WPF; ++i) {
                    const int k0 = kb * TT<T>::KB + TT<T>::KP * lg;
                    if (sizeof(T) == 2)
                        fw[kb][i] = (k0 + 2 * i < r_first ? 0x0000ffffu : 0u) | (k0 + 2 * i + 1 < r_first ? 0xffff0000u : 0u);
                    else
                        fw[kb][i] = k0 + i < r_first ? ~0u : 0u;
                }
        }
        // masked store of a [C][C] product as dst[n][m]: tri(m, n) as in the other instance (a compile-time
        // pattern for most tiles), then the packed words ANDed with the chunk's episode mask
        auto store_cc = [&](const f32x4 *acc, T *dst, auto tri, float sign) {
#pragma unroll
            for (int j = 0; j < TMA::TPW; ++j) {
                const int m = TMA::mt(w, j) * 16 + 4 * lg, n = TMA::nt(w, j) * 16 + li;
                float x[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) x[e] = tri(m + e, n) ? sign * acc[j][e] : 0.f;
                typedef uint32_t words_t __attribute__((ext_vector_type(WPP)));
                words_t wv = __builtin_bit_cast(words_t, TT<T>::pack(x[0], x[1], x[2], x[3]));
#pragma unroll
                for (int i = 0; i < WPP; ++i) wv[i] &= cw[j][i];
                *reinterpret_cast<words_t *>(dst + n * LDC + m) = wv;
            }
        };
        for (int pass = MG ? 0 : nres; pass >= 0; --pass) {
            auto live = [&](int r) { return nres == 0 || MG || episode_of(dmask, r) == pass; };
            // ---- stage ---------------------------------------------------------------
            {
                typename IO::Regs fq = rq, fk = rk, fv = rv, fdo = rdo;
                if (nres != 0 && !MG) {
                    IO::mask_rows(fq, tid, live);
                    IO::mask_rows(fk, tid, live);
                    IO::mask_rows(fv, tid, live);
                    IO::mask_rows(fdo, tid, live);
                }
                if (PRO) {
                    float kinv[IO::PASSES];
#pragma unroll
                    for (int p = 0; p < IO::PASSES; ++p) {
                        float ss = 0.f;
#pragma unroll
                        for (int e = 0; e < IO::KP; ++e) ss += (float)fk.v[p][e] * (float)fk.v[p][e];
                        kinv[p] = inv_norm(seg_sum<IO::SEGS>(ss));
                        const int r = IO::row_of(tid, p);
                        if (tid % IO::SEGS == 0 && (IO::FULL || r < C)) sKinv[r] = kinv[p];
                    }
                    IO::scale_rows(fk, kinv);
                }
                IO::to_lds(fq, sQ, LDD, tid);
                IO::to_lds(fk, sK, LDD, tid);
                IO::to_lds(fv, sV, LDD, tid);
                IO::to_lds(fdo, sDO, LDD, tid);
                float bf[IO::PASSES];
#pragma unroll
                for (int p = 0; p < IO::PASSES; ++p)
                    bf[p] = !live(IO::row_of(tid, p)) ? 0.f  // by select: a NaN gate of another episode must not meet a zeroed row
                            : PRO ? sigmoidf(raw_to_float<T>(rbrow[p])) : raw_to_float<T>(rbrow[p]);
                IO::scale_rows(fk, bf);
                IO::to_lds(fk, sBK, LDD, tid);
                typename IOS::Regs fS = rS;
                if (pass != 0) IOS::zero(fS);
                IOS::to_lds(fS, sS, LDD, tid);
                // Tm[i][j] from the forward call (block diagonal by episode).  Rows of other episodes
                // are cleared by select: they only ever meet zeros, but a NaN key or gate of another
                // episode sits in them and must not meet those zeros.
                typename IOT::Regs fTm = rTm;
                if (nres != 0 && !MG) IOT::mask_rows(fTm, tid, live);
                IOT::to_lds(fTm, sTm, LDC, tid);
            }
            if (tid < C) sBeta[tid] = !live(tid) ? 0.f : PRO ? sigmoidf(raw_to_float<T>(rbeta)) : raw_to_float<T>(rbeta);
            if (pass != nres && !MG) zero_acc<TMS::TPW>(dSacc);
            store_acc<T, HD, HD, NW>(dSacc, sDS, LDD, w, lane);  // dS[dv][dk]
            sync_lds();
            flush_pending();
            const bool pre = pass == 0 && c > 0;
            if (pre) { prefetch_part(0); prefetch_part(1); }

            auto tril = [](int m, int n, float x) { return m <= n ? x : 0.f; };
            // ---- Aqk[i][j] = q_i . k_j, j <= i, stored transposed: D[m = i][n = j] -> sAqk[j][i], the
            //      orientation its one consumer (dU') contracts over without transpose reads -------------
            {
                f32x4 acc[TMA::TPW];
                zero_acc<TMA::TPW>(acc);
                gemm<T, C, C, HD, ROWK, ROWK, NW>(acc, sQ, LDD, sK, LDD, w, lane);
                if constexpr (MERGE)
                    store_cc(acc, sAqk, [](int m, int n) { return m >= n; }, 1.f);
                else
                    store_acc_f<T, C, C, NW>(acc, sAqk, LDC, w, lane, [](int m, int n, float x) { return m >= n ? x : 0.f; });
            }
            // ---- V0[c][dv] = V[c][dv] - sum_dk S[dv][dk] K[c][dk] (in place), V~ = beta_c V0 -> sVt ---
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                gemm<T, HD, C, HD, ROWK, ROWK, NW>(acc, sS, LDD, sK, LDD, w, lane);  // D[m = dv][n = c]
#pragma unroll
                for (int j = 0; j < TMR::TPW; ++j) {
                    const int d0 = TMR::mt(w, j) * 16 + 4 * lg, r = TMR::nt(w, j) * 16 + li;
                    const P4 x = *reinterpret_cast<const P4 *>(sV + r * LDD + d0);  // each lane rewrites what it read
                    const float bb = sBeta[r];
                    float y[4];
                    // merged episodes: the first one alone sees the entering state (a factor 0 on finite values)
                    const float sees_S = MERGE ? ff[j % TMR::NBW] : 1.f;
#pragma unroll
                    for (int e = 0; e < 4; ++e) y[e] = MERGE ? (float)x[e] - sees_S * acc[j][e] : (float)x[e] - acc[j][e];
                    const P4 v0 = TT<T>::pack(y[0], y[1], y[2], y[3]);
                    *reinterpret_cast<P4 *>(sV + r * LDD + d0) = v0;
                    // V~ from the rounded V0, so that dbeta = rowdot(Z, V0) matches what U' was built from
                    *reinterpret_cast<P4 *>(sVt + r * LDD + d0) =
                        TT<T>::pack(bb * (float)v0[0], bb * (float)v0[1], bb * (float)v0[2], bb * (float)v0[3]);
                }
            }
            sync_lds();
            if (pre) { prefetch_part(2); prefetch_part(3); }
            // ---- U'^T[dv][c] = sum_j V~[j][dv] Tm[c][j] -> sU[c][dv] ----------------------------------
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                gemm<T, HD, C, C, KROW, ROWK, NW>(acc, sVt, LDD, sTm, LDC, w, lane);
                store_acc<T, HD, C, NW>(acc, sU, LDD, w, lane);
            }
            // ---- dU'^T[dv][j] = sum_i dO[i][dv] Aqk[i][j] + sum_dk dS[dv][dk] K[j][dk] -> sDU[j][dv]
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                if constexpr (MERGE) {  // the term with dS first, so that it can be confined to the rows of the last episode
                    gemm<T, HD, C, HD, ROWK, ROWK, NW>(acc, sDS, LDD, sK, LDD, w, lane);
#pragma unroll
                    for (int j = 0; j < TMR::TPW; ++j) acc[j] *= fl[j % TMR::NBW];
                    gemm<T, HD, C, C, KROW, ROWK, NW>(acc, sDO, LDD, sAqk, LDC, w, lane);
                } else {
                    gemm<T, HD, C, C, KROW, ROWK, NW>(acc, sDO, LDD, sAqk, LDC, w, lane);
                    gemm<T, HD, C, HD, ROWK, ROWK, NW>(acc, sDS, LDD, sK, LDD, w, lane);
                }
                store_acc<T, HD, C, NW>(acc, sDU, LDD, w, lane);
            }
            sync_lds();  // sU, sDU visible; sAqk dead
            if (pre) { prefetch_part(4); prefetch_part(5); }
            float dbp[TMR::NBW];  // per-lane partials of dbeta for rows nt * 16 + li of the wave's tile columns
#pragma unroll
            for (int j = 0; j < TMR::NBW; ++j) dbp[j] = 0.f;
            auto rowdot = [&](const f32x4 *acc, const T *X) {
#pragma unroll
                for (int j = 0; j < TMR::TPW; ++j) {
                    const int d0 = TMR::mt(w, j) * 16 + 4 * lg, r = TMR::nt(w, j) * 16 + li;
                    const P4 x = *reinterpret_cast<const P4 *>(X + r * LDD + d0);
                    dbp[j % TMR::NBW] += acc[j][0] * (float)x[0] + acc[j][1] * (float)x[1] + acc[j][2] * (float)x[2] +
                                         acc[j][3] * (float)x[3];
                }
            };
            // ---- dAqk[i][j] = do_i . u'_j, j <= i -> sDAqk (over sAqk) ------------------------------
            {
                f32x4 acc[TMA::TPW];
                zero_acc<TMA::TPW>(acc);
                gemm<T, C, C, HD, ROWK, ROWK, NW>(acc, sU, LDD, sDO, LDD, w, lane);  // D[m = j][n = i]
                if constexpr (MERGE)
                    store_cc(acc, sDAqk, [](int m, int n) { return m <= n; }, 1.f);
                else
                    store_acc_f<T, C, C, NW>(acc, sDAqk, LDC, w, lane, tril);
            }
            // ---- Z^T[dv][j] = sum_i dU'[i][dv] Tm[i][j] : dV = beta_j Z -> global and sZb ; dbeta += Z_j . V0_j
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                gemm<T, HD, C, C, KROW, KROW, NW>(acc, sDU, LDD, sTm, LDC, w, lane);
                rowdot(acc, sV);
                store_acc<T, HD, C, NW>(acc, sZ, LDD, w, lane);  // V~ is dead: every wave has formed its U'
#pragma unroll
                for (int j = 0; j < TMR::TPW; ++j) acc[j] *= sBeta[TMR::nt(w, j) * 16 + li];
                store_acc<T, HD, C, NW>(acc, sZb, LDD, w, lane);  // = dV, written to memory from here after the barrier
            }
            sync_lds();  // sDAqk, sZ, sZb visible
            tile_rows_to_global<T, C, NTHR>(sZb, LDD, dv + basev + (int64_t)t0 * rsv, rsv, t0, Tlen, tid, live, dvw);
            // ---- dQ^T[dk][i] = sum_dv S[dv][dk] dO[i][dv] + sum_j K[j][dk] dAqk[i][j] -> global ----
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                gemm<T, HD, C, HD, KROW, ROWK, NW>(acc, sS, LDD, sDO, LDD, w, lane);
                if constexpr (MERGE) {
#pragma unroll
                    for (int j = 0; j < TMR::TPW; ++j) acc[j] *= ff[j % TMR::NBW];
                }
                gemm<T, HD, C, C, KROW, ROWK, NW>(acc, sK, LDD, sDAqk, LDC, w, lane);
                store_acc<T, HD, C, NW>(acc, sDU, LDD, w, lane);  // dU' is dead; to memory after the barrier
            }
            // ---- dK^T[dk][j] = sum_i Q[i][dk] dAqk[i][j] + sum_dv dS[dv][dk] U'[j][dv]
            //                    - sum_dv S[dv][dk] (beta Z)[j][dv]   (kept in registers) ---------------
            f32x4 dKacc[TMR::TPW];
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                zero_acc<TMR::TPW>(dKacc);
                gemm<T, HD, C, HD, KROW, ROWK, NW>(acc, sS, LDD, sZb, LDD, w, lane);
                if constexpr (MERGE) {  // the term with dS first: rows of the last episode; the term with S: rows of the first
                    gemm<T, HD, C, HD, KROW, ROWK, NW>(dKacc, sDS, LDD, sU, LDD, w, lane);
#pragma unroll
                    for (int j = 0; j < TMR::TPW; ++j) dKacc[j] *= fl[j % TMR::NBW];
                    gemm<T, HD, C, C, KROW, KROW, NW>(dKacc, sQ, LDD, sDAqk, LDC, w, lane);
#pragma unroll
                    for (int j = 0; j < TMR::TPW; ++j) dKacc[j] -= acc[j] * ff[j % TMR::NBW];
                } else {
                    gemm<T, HD, C, C, KROW, KROW, NW>(dKacc, sQ, LDD, sDAqk, LDC, w, lane);
                    gemm<T, HD, C, HD, KROW, ROWK, NW>(dKacc, sDS, LDD, sU, LDD, w, lane);
#pragma unroll
                    for (int j = 0; j < TMR::TPW; ++j) dKacc[j] -= acc[j];
                }
            }
            // ---- dS^T[dk][dv] += sum_c Q[c][dk] dO[c][dv] - sum_c K[c][dk] (beta Z)[c][dv] -----------
            {
                f32x4 acc[TMS::TPW];
                zero_acc<TMS::TPW>(acc);
                if constexpr (MERGE) {
                    // a merged chunk: what flows on to the chunk before is the first episode's own sum -- the
                    // incoming gradient is dropped and the operand fragments keep the first episode's rows
                    // (straight-line: all-pass values in every other chunk)
#pragma unroll
                    for (int j = 0; j < TMS::TPW; ++j) dSacc[j] *= keep_dS;
                    auto first_rows = [&](int, int kb, typename TT<T>::frag &x) {
                        typedef uint32_t words_t __attribute__((ext_vector_type(WPF)));
                        words_t wv = __builtin_bit_cast(words_t, x);
#pragma unroll
                        for (int i = 0; i < WPF; ++i) wv[i] &= fw[kb][i];
                        x = __builtin_bit_cast(typename TT<T>::frag, wv);
                    };
                    gemm<T, HD, HD, C, KROW, KROW, NW>(dSacc, sQ, LDD, sDO, LDD, w, lane, first_rows);
                    gemm<T, HD, HD, C, KROW, KROW, NW>(acc, sK, LDD, sZb, LDD, w, lane, first_rows);
                } else {
                    gemm<T, HD, HD, C, KROW, KROW, NW>(dSacc, sQ, LDD, sDO, LDD, w, lane);
                    gemm<T, HD, HD, C, KROW, KROW, NW>(acc, sK, LDD, sZb, LDD, w, lane);
                }
#pragma unroll
                for (int j = 0; j < TMS::TPW; ++j) dSacc[j] -= acc[j];
            }
            // ---- dA[i][j] = -z_i . u'_j, j < i : D[m = j][n = i] -> sDA[i][j] ---------------------------
            {
                f32x4 acc[TMA::TPW];
                zero_acc<TMA::TPW>(acc);
                gemm<T, C, C, HD, ROWK, ROWK, NW>(acc, sU, LDD, sZ, LDD, w, lane);
                if constexpr (MERGE)
                    store_cc(acc, sDA, [](int m, int n) { return m < n; }, -1.f);
                else
                    store_acc_f<T, C, C, NW>(acc, sDA, LDC, w, lane, [](int m, int n, float x) { return m < n ? -x : 0.f; });
            }
            sync_lds();  // sDA visible; sQ, sDO, sS, sDS, sDAqk, sZ, sZb dead
            tile_rows_to_global<T, C, NTHR>(sDU, LDD, dq + base + (int64_t)t0 * rs, rs, t0, Tlen, tid, live, dkw);
            // ---- R^T[dk][i] = sum_j K[j][dk] dA[i][j] : dbeta += K_i . R_i ; dK += beta_i R ;
            //      dK^T[dk][j] += sum_i beta_i K[i][dk] dA[i][j] -> global -------------------------------
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                gemm<T, HD, C, C, KROW, ROWK, NW>(acc, sK, LDD, sDA, LDC, w, lane);
                rowdot(acc, sK);
#pragma unroll
                for (int j = 0; j < TMR::TPW; ++j) dKacc[j] += acc[j] * sBeta[TMR::nt(w, j) * 16 + li];
                gemm<T, HD, C, C, KROW, KROW, NW>(dKacc, sBK, LDD, sDA, LDC, w, lane);
                if (!PRO) store_acc<T, HD, C, NW>(dKacc, sU, LDD, w, lane);
            }
            // prologue: dKacc holds the gradient of the normalised keys; its component along k_n is
            // removed once the row dots k_n . dk_n are summed over the feature blocks (after the barrier).
            // The k_n values and 1 / |k| are taken into registers now: sK is restaged right after.
            P4 kn[TMR::TPW];
            float kiv[TMR::NBW];
            if (PRO) {
                float sp[TMR::NBW];
#pragma unroll
                for (int j = 0; j < TMR::NBW; ++j) sp[j] = 0.f;
#pragma unroll
                for (int j = 0; j < TMR::TPW; ++j) {
                    const int d0 = TMR::mt(w, j) * 16 + 4 * lg, r = TMR::nt(w, j) * 16 + li;
                    kn[j] = *reinterpret_cast<const P4 *>(sK + r * LDD + d0);
                    sp[j % TMR::NBW] += dKacc[j][0] * (float)kn[j][0] + dKacc[j][1] * (float)kn[j][1] +
                                        dKacc[j][2] * (float)kn[j][2] + dKacc[j][3] * (float)kn[j][3];
                }
#pragma unroll
                for (int j = 0; j < TMR::NBW; ++j) {
                    float x = sp[j];
                    x += __shfl_xor(x, 16);
                    x += __shfl_xor(x, 32);
                    if (lg == 0) sKd[(w % TMR::WM) * C + TMR::nt(w, j) * 16 + li] = x;
                    kiv[j] = sKinv[TMR::nt(w, j) * 16 + li];
                }
            }
            // ---- dbeta: reduce the partials over lane groups, then over waves through LDS -----------
#pragma unroll
            for (int j = 0; j < TMR::NBW; ++j) {
                float x = dbp[j];
                x += __shfl_xor(x, 16);
                x += __shfl_xor(x, 32);
                if (lg == 0) sDb[(w % TMR::WM) * C + TMR::nt(w, j) * 16 + li] = x;
            }
            sync_lds();
            if (PRO) {
#pragma unroll
                for (int j = 0; j < TMR::TPW; ++j) {
                    const int r = TMR::nt(w, j) * 16 + li;
                    float sd = 0.f;
#pragma unroll
                    for (int sl = 0; sl < NSLOT; ++sl) sd += sKd[sl * C + r];
#pragma unroll
                    for (int e = 0; e < 4; ++e) dKacc[j][e] = (dKacc[j][e] - (float)kn[j][e] * sd) * kiv[j % TMR::NBW];
                }
                store_acc<T, HD, C, NW>(dKacc, sU, LDD, w, lane);
            }
            pend_dmask = dmask;
            pend_nres = MG ? 0 : nres;
            pend_pass = pass;
            pend_t0 = t0;
            if (tid < C && t0 + tid < Tlen && live(tid)) {
                float x = 0.f;
#pragma unroll
                for (int sl = 0; sl < NSLOT; ++sl) x += sDb[sl * C + tid];
                if (PRO) x *= sBeta[tid] * (1.f - sBeta[tid]);
                pend_db = x;
                pend_dboff = dboff;
                pend_db_on = true;
            }
            // no barrier: sDb, sKd are not written again before the next pass's last phase
        }
    }
    sync_lds();
    flush_pending();
#ifdef MRX_PHASE_CLOCKS
    if (tid == 0) {  // the waves of a workgroup move from barrier to barrier together: wave 0's lifetime stands for all
        atomicAdd(&g_phase_clocks[0], wg_product_clocks);
        atomicAdd(&g_phase_clocks[1], (unsigned long long)NW * (unsigned long long)(clock64() - kernel_clk0));
        atomicAdd(&g_phase_clocks[2], 1ull);
    }
#endif
    if (dS0) {
#pragma unroll
        for (int j = 0; j < TMS::TPW; ++j) {
            const int dk0 = TMS::mt(w, j) * 16 + 4 * lg, dvv = TMS::nt(w, j) * 16 + li;
            if (in_state(dvv, dk0)) *reinterpret_cast<f32x4 *>(dS0 + ((int64_t)bh * dvw + dvv) * dkw + dk0) = dSacc[j];
        }
    }
}

template <typename T, int C, bool FMAP, bool GATED, bool NORM, bool PAR, bool NARROW> struct LaBwdReg {
    static constexpr int smem = LaBwdSmem<T, C, GATED, NORM>::total;
    static inline KernelRegistrar reg{reinterpret_cast<const void *>(la_bwd_kernel<T, C, FMAP, GATED, NORM, PAR, NARROW>), smem};
};

template <typename T, int C, bool FMAP, bool GATED = false, bool NORM = false, bool PAR = false>
int launch_la(hipStream_t st, const void *q, const void *k, const void *v, const void *done,
              int done_f32, const void *S_chk, const void *S_last, const void *dout, const void *dS_last, void *dq,
              void *dk, void *dv, void *dS0, int64_t B, int64_t Tlen, int64_t H, const void *glog = nullptr,
              void *dg = nullptr, NormBwdArgs na = NormBwdArgs{}, int64_t dka = HD, int64_t dva = HD)
{
    if (const int rc = prepare_device(); rc != MRX_OK) return rc;
    const int64_t NC = (Tlen + C - 1) / C;
    if (PAR && NC > 65535) return MRX_ERR_INVALID_ARG;
    auto go = [&](auto narrow) {
        constexpr bool NARROW = decltype(narrow)::value;
        using Reg = LaBwdReg<T, C, FMAP, GATED, NORM, PAR, NARROW>;
        (void)&Reg::reg;  // the kernel is on the list mrx_init() walks
        return launch_kernel(la_bwd_kernel<T, C, FMAP, GATED, NORM, PAR, NARROW>,
                             dim3((unsigned)(B * H), PAR ? (unsigned)NC : 1u), dim3(256), Reg::smem, st, (const T *)q,
                             (const T *)k, (const T *)v, (const float *)glog, done, done_f32, S_chk,
                             (const float *)S_last, (const T *)dout, (const float *)dS_last, (T *)dq, (T *)dk, (T *)dv,
                             (float *)dg, (float *)dS0, (int)Tlen, (int)H, na, (int)dka, (int)dva);
    };
    if (dka != HD || dva != HD) return go(std::true_type{});  // narrow heads
    return go(std::false_type{});
}

int check_bwd(const void *q, const void *k, const void *v, const void *done, const void *S_chk,
              const void *dout, const void *dS_last, const void *dq, const void *dk_out,
              const void *dv_out, const void *dS0, int64_t B, int64_t T, int64_t H, int64_t dk,
              int64_t dv, int dtype, int done_dtype, bool narrow = false)
{
    if (!q || !k || !v || !done || !S_chk || !dout || !dq || !dk_out || !dv_out) return MRX_ERR_INVALID_ARG;
    if (B <= 0 || T <= 0 || H <= 0 || dk <= 0 || dv <= 0) return MRX_ERR_INVALID_ARG;
    if (dtype != MRX_F32 && dtype != MRX_BF16) return dtype == MRX_C64 ? MRX_ERR_UNSUPPORTED : MRX_ERR_INVALID_ARG;
    if (done_dtype != MRX_DONE_U8 && done_dtype != MRX_DONE_F32) return MRX_ERR_INVALID_ARG;
    // narrow: rows narrower than the build's head dim, in whole 16-byte segments
    const int64_t seg = dtype == MRX_BF16 ? 8 : 4;
    const bool narrow_ok = narrow && dk <= HD && dv <= HD && dk % seg == 0 && dv % seg == 0;
    if ((dk != HD || dv != HD) && !narrow_ok) return MRX_ERR_UNSUPPORTED;
    if (B * H >= (1ll << 31) || T >= (1ll << 30)) return MRX_ERR_INVALID_ARG;
    const void *ps[] = {q, k, v, S_chk, dout, dS_last, dq, dk_out, dv_out, dS0};
    for (const void *p : ps)
        if (!aligned(p, 16)) return MRX_ERR_INVALID_ARG;
    if (done_dtype == MRX_DONE_F32 && !aligned(done, 4)) return MRX_ERR_INVALID_ARG;
    return MRX_OK;
}

}  // namespace MRX_HD_NS
}  // namespace

MRX_EXPORT int MRX_API(mrx_linear_attn_bwd)(void *stream, const void *q, const void *k, const void *v,
                                   const void *done, const void *S_chk, const float *S_last, const void *dout,
                                   const void *dS_last, void *dq, void *dk_out, void *dv_out,
                                   void *dS0, int64_t B, int64_t T, int64_t H, int64_t dk, int64_t dv,
                                   int dtype, int done_dtype, int feature_map)
{
#if MRX_HD == 64
    if (dk <= 32 && dv <= 32) return mrx_linear_attn_bwd_hd32(stream, q, k, v, done, S_chk, S_last, dout, dS_last, dq, dk_out, dv_out, dS0, B, T, H, dk, dv, dtype, done_dtype, feature_map);
#endif
    const int rc = check_bwd(q, k, v, done, S_chk, dout, dS_last, dq, dk_out, dv_out, dS0, B, T, H, dk,
                             dv, dtype, done_dtype, true);
    if (rc != MRX_OK) return rc;
    if (!S_last || !aligned(S_last, 16)) return MRX_ERR_INVALID_ARG;
    if (feature_map != MRX_FMAP_NONE && feature_map != MRX_FMAP_ELU1) return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const bool fm = feature_map == MRX_FMAP_ELU1;
#define MRX_ARGS st, q, k, v, done, done_dtype, S_chk, S_last, dout, dS_last, dq, dk_out, dv_out, dS0, B, T, H, nullptr, nullptr, NormBwdArgs{}, dk, dv
    if (dtype == MRX_BF16) return fm ? launch_la<__bf16, LA_BF16_CHUNK, true>(MRX_ARGS) : launch_la<__bf16, LA_BF16_CHUNK, false>(MRX_ARGS);
    return fm ? launch_la<float, 32, true>(MRX_ARGS) : launch_la<float, 32, false>(MRX_ARGS);
#undef MRX_ARGS
}

MRX_EXPORT int MRX_API(mrx_linear_attn_bwd_chunk_parallel)(void *stream, const void *q, const void *k, const void *v,
                                                  const void *done, const float *S_chk, const void *dout,
                                                  const void *dS_last, void *dq, void *dk_out, void *dv_out,
                                                  void *dS0, float *workspace, int64_t B, int64_t T, int64_t H,
                                                  int64_t dk, int64_t dv, int dtype, int done_dtype, int feature_map)
{
#if MRX_HD == 64
    if (dk <= 32 && dv <= 32) return mrx_linear_attn_bwd_chunk_parallel_hd32(stream, q, k, v, done, S_chk, dout, dS_last, dq, dk_out, dv_out, dS0, workspace, B, T, H, dk, dv, dtype, done_dtype, feature_map);
#endif
    const int rc = check_bwd(q, k, v, done, S_chk, dout, dS_last, dq, dk_out, dv_out, dS0, B, T, H, dk,
                             dv, dtype, done_dtype, true);
    if (rc != MRX_OK) return rc;
    if (!workspace || !aligned(workspace, 16)) return MRX_ERR_INVALID_ARG;
    if (feature_map != MRX_FMAP_NONE && feature_map != MRX_FMAP_ELU1) return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const bool fm = feature_map == MRX_FMAP_ELU1;
    const int C = (int)mrx_chunk_size(dtype);
    if ((T + C - 1) / C > 65535) return MRX_ERR_INVALID_ARG;
    // per-chunk sums of do phi(q)^T -> gradients of the states leaving the chunks (and dS0) -> dQ, dK, dV
    int rc2 = launch_la_chunk_states(st, q, dout, done, done_dtype, workspace, B, T, H, dtype, fm, true, dk, dv);
    if (rc2 != MRX_OK) return rc2;
    rc2 = launch_la_state_scan(st, workspace, (const float *)dS_last, (float *)dS0, done, done_dtype, B, T, H, C, true, dk, dv);
    if (rc2 != MRX_OK) return rc2;
#define MRX_ARGS st, q, k, v, done, done_dtype, S_chk, nullptr, dout, workspace, dq, dk_out, dv_out, nullptr, B, T, H, nullptr, nullptr, NormBwdArgs{}, dk, dv
    if (dtype == MRX_BF16)
        return fm ? launch_la<__bf16, LA_BF16_CHUNK, true, false, false, true>(MRX_ARGS)
                  : launch_la<__bf16, LA_BF16_CHUNK, false, false, false, true>(MRX_ARGS);
    return fm ? launch_la<float, 32, true, false, false, true>(MRX_ARGS)
              : launch_la<float, 32, false, false, false, true>(MRX_ARGS);
#undef MRX_ARGS
}

MRX_EXPORT int MRX_API(mrx_linear_attn_norm_bwd)(void *stream, const void *q, const void *k, const void *v,
                                        const void *done, const void *S_chk, const float *S_last, const float *z_chk,
                                        const void *o, const float *den, const void *dout, const float *d_ss,
                                        const void *dS_last, const float *dz_last, void *dq, void *dk_out,
                                        void *dv_out, void *dS0, float *dz0, int64_t B, int64_t T, int64_t H,
                                        int64_t dk, int64_t dv, int dtype, int done_dtype, int feature_map,
                                        float eps)
{
#if MRX_HD == 64
    if (dk <= 32 && dv <= 32) return mrx_linear_attn_norm_bwd_hd32(stream, q, k, v, done, S_chk, S_last, z_chk, o, den, dout, d_ss, dS_last, dz_last, dq, dk_out, dv_out, dS0, dz0, B, T, H, dk, dv, dtype, done_dtype, feature_map, eps);
#endif
    const int rc = check_bwd(q, k, v, done, S_chk, dout, dS_last, dq, dk_out, dv_out, dS0, B, T, H, dk,
                             dv, dtype, done_dtype, true);
    if (rc != MRX_OK) return rc;
    if (!z_chk || !o || !den || !S_last || !aligned(S_last, 16)) return MRX_ERR_INVALID_ARG;
    if (!aligned(z_chk, 16) || !aligned(o, 16) || !aligned(den, 4) || !aligned(d_ss, 4) || !aligned(dz_last, 16) || !aligned(dz0, 16))
        return MRX_ERR_INVALID_ARG;
    if (feature_map != MRX_FMAP_NONE && feature_map != MRX_FMAP_ELU1) return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const bool fm = feature_map == MRX_FMAP_ELU1;
    const NormBwdArgs na{o, den, z_chk, dz_last, dz0, eps, d_ss};
#define MRX_ARGS st, q, k, v, done, done_dtype, S_chk, S_last, dout, dS_last, dq, dk_out, dv_out, dS0, B, T, H, nullptr, nullptr, na, dk, dv
    if (dtype == MRX_BF16)
        return fm ? launch_la<__bf16, LA_BF16_CHUNK, true, false, true>(MRX_ARGS)
                  : launch_la<__bf16, LA_BF16_CHUNK, false, false, true>(MRX_ARGS);
    return fm ? launch_la<float, 32, true, false, true>(MRX_ARGS) : launch_la<float, 32, false, false, true>(MRX_ARGS);
#undef MRX_ARGS
}

MRX_EXPORT int MRX_API(mrx_gated_linear_attn_bwd)(void *stream, const void *q, const void *k, const void *v,
                                         const void *g, const void *done, const void *S_chk, const float *S_last,
                                         const void *dout, const void *dS_last, void *dq, void *dk_out,
                                         void *dv_out, float *dg, void *dS0, int64_t B, int64_t T, int64_t H,
                                         int64_t dk, int64_t dv, int dtype, int done_dtype, int feature_map)
{
#if MRX_HD == 64
    if (dk <= 32 && dv <= 32) return mrx_gated_linear_attn_bwd_hd32(stream, q, k, v, g, done, S_chk, S_last, dout, dS_last, dq, dk_out, dv_out, dg, dS0, B, T, H, dk, dv, dtype, done_dtype, feature_map);
#endif
    const int rc = check_bwd(q, k, v, done, S_chk, dout, dS_last, dq, dk_out, dv_out, dS0, B, T, H, dk,
                             dv, dtype, done_dtype, true);
    if (rc != MRX_OK) return rc;
    if (!g || !dg || !aligned(g, 4) || !aligned(dg, 4) || !aligned(S_last, 16)) return MRX_ERR_INVALID_ARG;
    if (dS_last && !S_last) return MRX_ERR_INVALID_ARG;  // <S_last, dS_last> enters dg at the last step
    if (feature_map != MRX_FMAP_NONE && feature_map != MRX_FMAP_ELU1) return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const bool fm = feature_map == MRX_FMAP_ELU1;
#define MRX_ARGS st, q, k, v, done, done_dtype, S_chk, S_last, dout, dS_last, dq, dk_out, dv_out, dS0, B, T, H, g, dg, NormBwdArgs{}, dk, dv
    if (dtype == MRX_BF16)
        return fm ? launch_la<__bf16, LA_BF16_CHUNK, true, true>(MRX_ARGS) : launch_la<__bf16, LA_BF16_CHUNK, false, true>(MRX_ARGS);
    return fm ? launch_la<float, 32, true, true>(MRX_ARGS) : launch_la<float, 32, false, true>(MRX_ARGS);
#undef MRX_ARGS
}

namespace {
inline namespace MRX_HD_NS {

template <typename T, int C, bool PRO, bool NARROW, bool MERGE> struct DeltaBwdReg {
    static constexpr int NW = 4;
    static constexpr int smem = DeltaBwdSmem<T, C, NW>::total;
    static inline KernelRegistrar reg{reinterpret_cast<const void *>(delta_bwd_kernel<T, C, NW, PRO, NARROW, MERGE>), smem};
};

template <typename T, int C, bool PRO, bool MERGE = false>
int launch_delta_bwd(hipStream_t st, const void *q, const void *k, const void *v, const void *beta,
                     const void *done, int done_dtype, const void *S_chk, const void *Tm_chk, const void *dout,
                     const void *dS_last, void *dq, void *dk_out, void *dv_out, void *dbeta, void *dS0, int64_t B,
                     int64_t T_, int64_t H, int64_t dka, int64_t dva)
{
    if (const int rc = prepare_device(); rc != MRX_OK) return rc;
    auto go = [&](auto narrow) {
        constexpr bool MG = MERGE && !decltype(narrow)::value;  // narrow heads keep the units per episode
        using Reg = DeltaBwdReg<T, C, PRO, decltype(narrow)::value, MG>;
        (void)&Reg::reg;  // the kernel is on the list mrx_init() walks
        return launch_kernel(delta_bwd_kernel<T, C, Reg::NW, PRO, decltype(narrow)::value, MG>, dim3((unsigned)(B * H)),
                             dim3(64 * Reg::NW), Reg::smem, st, (const T *)q, (const T *)k, (const T *)v, (const T *)beta,
                             done, done_dtype, (const T *)S_chk, (const T *)Tm_chk, (const T *)dout,
                             (const float *)dS_last, (T *)dq, (T *)dk_out, (T *)dv_out, (T *)dbeta, (float *)dS0, (int)T_,
                             (int)H, (int)dka, (int)dva);
    };
    if (dka != HD || dva != HD) return go(std::true_type{});  // narrow heads
    return go(std::false_type{});
}

template <bool PRO>
int delta_bwd_entry(void *stream, const void *q, const void *k, const void *v, const void *beta, const void *done,
                    const void *S_chk, const void *Tm_chk, const void *dout, const void *dS_last, void *dq,
                    void *dk_out, void *dv_out, void *dbeta, void *dS0, int64_t B, int64_t T, int64_t H,
                    int64_t dk, int64_t dv, int dtype, int done_dtype, int reset_path)
{
    const int rc = check_bwd(q, k, v, done, S_chk, dout, dS_last, dq, dk_out, dv_out, dS0, B, T, H, dk,
                             dv, dtype, done_dtype, true);
    if (rc != MRX_OK) return rc;
    if (!beta || !dbeta || !Tm_chk || !aligned(Tm_chk, 16)) return MRX_ERR_INVALID_ARG;
    if (reset_path != MRX_RESETS_AUTO && reset_path != MRX_RESETS_PASSES && reset_path != MRX_RESETS_MERGED)
        return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
#if MRX_HD == 64
    // merged episodes: the build with 32-row chunks, whose bounds the screen was derived for
    if (reset_path == MRX_RESETS_MERGED && DELTA_BF16_CHUNK == 32) {
        if (dtype == MRX_BF16)
            return launch_delta_bwd<__bf16, 32, PRO, true>(st, q, k, v, beta, done, done_dtype, S_chk, Tm_chk, dout,
                                                           dS_last, dq, dk_out, dv_out, dbeta, dS0, B, T, H, dk, dv);
        return launch_delta_bwd<float, 32, PRO, true>(st, q, k, v, beta, done, done_dtype, S_chk, Tm_chk, dout, dS_last, dq,
                                                      dk_out, dv_out, dbeta, dS0, B, T, H, dk, dv);
    }
#endif
    if (dtype == MRX_BF16)
        return launch_delta_bwd<__bf16, DELTA_BF16_CHUNK, PRO>(st, q, k, v, beta, done, done_dtype, S_chk, Tm_chk, dout,
                                                               dS_last, dq, dk_out, dv_out, dbeta, dS0, B, T, H, dk, dv);
    return launch_delta_bwd<float, 32, PRO>(st, q, k, v, beta, done, done_dtype, S_chk, Tm_chk, dout, dS_last, dq,
                                            dk_out, dv_out, dbeta, dS0, B, T, H, dk, dv);
}

}  // namespace MRX_HD_NS
}  // namespace

MRX_EXPORT int MRX_API(mrx_delta_rule_bwd)(void *stream, const void *q, const void *k, const void *v,
                                  const void *beta, const void *done, const void *S_chk,
                                  const void *Tm_chk, const void *dout, const void *dS_last, void *dq,
                                  void *dk_out, void *dv_out, void *dbeta, void *dS0, int64_t B,
                                  int64_t T, int64_t H, int64_t dk, int64_t dv, int dtype,
                                  int done_dtype, int reset_path)
{
#if MRX_HD == 64
    if (dk <= 32 && dv <= 32) return mrx_delta_rule_bwd_hd32(stream, q, k, v, beta, done, S_chk, Tm_chk, dout, dS_last, dq, dk_out, dv_out, dbeta, dS0, B, T, H, dk, dv, dtype, done_dtype, reset_path);
#endif
    return delta_bwd_entry<false>(stream, q, k, v, beta, done, S_chk, Tm_chk, dout, dS_last, dq, dk_out, dv_out,
                                  dbeta, dS0, B, T, H, dk, dv, dtype, done_dtype, reset_path);
}

MRX_EXPORT int MRX_API(mrx_deltanet_bwd)(void *stream, const void *q, const void *k, const void *v,
                                const void *beta_raw, const void *done, const void *S_chk,
                                const void *Tm_chk, const void *dout, const void *dS_last, void *dq,
                                void *dk_out, void *dv_out, void *dbeta_raw, void *dS0, int64_t B,
                                int64_t T, int64_t H, int64_t dk, int64_t dv, int dtype,
                                int done_dtype, int reset_path)
{
#if MRX_HD == 64
    if (dk <= 32 && dv <= 32) return mrx_deltanet_bwd_hd32(stream, q, k, v, beta_raw, done, S_chk, Tm_chk, dout, dS_last, dq, dk_out, dv_out, dbeta_raw, dS0, B, T, H, dk, dv, dtype, done_dtype, reset_path);
#endif
    return delta_bwd_entry<true>(stream, q, k, v, beta_raw, done, S_chk, Tm_chk, dout, dS_last, dq, dk_out, dv_out,
                                 dbeta_raw, dS0, B, T, H, dk, dv, dtype, done_dtype, reset_path);
}

#if defined(MRX_PHASE_CLOCKS) && MRX_HD == 64
// Measurement build only: the clocks of delta_bwd_kernel (above), copied to out[0..2] after the device has
// finished what was enqueued; reset != 0 clears them afterwards.  Synchronises: not for use beside real work.
extern "C" int mrx_phase_clocks(unsigned long long *out, int reset)
{
    unsigned long long v[4] = {0ull, 0ull, 0ull, 0ull};
    if (hipDeviceSynchronize() != hipSuccess) return MRX_ERR_LAUNCH;
    if (hipMemcpyFromSymbol(v, HIP_SYMBOL(g_phase_clocks), sizeof(v)) != hipSuccess) return MRX_ERR_LAUNCH;
    if (out) for (int i = 0; i < 3; ++i) out[i] = v[i];
    if (reset) {
        const unsigned long long z[4] = {0ull, 0ull, 0ull, 0ull};
        if (hipMemcpyToSymbol(HIP_SYMBOL(g_phase_clocks), z, sizeof(z)) != hipSuccess) return MRX_ERR_LAUNCH;
    }
    return MRX_OK;
}
#endif
