// Backward of chunked causal linear attention and of the DeltaNet delta rule.
//
// Chunks are walked from the last to the first with dS (gradient of the state
// leaving the chunk) carried in MFMA accumulators; the state entering each chunk
// comes from the checkpoints the forward call wrote (S_chk), everything else of the
// forward (A, Tm, W, U', masked QK^T) is recomputed per chunk.  A chunk that
// contains resets is processed once per episode, last episode first, with the rows
// of the other episodes zeroed by select; dS only flows into the episode that
// leaves the chunk and only out of the episode that enters it.
//
// Per pass (rows i >= j; all rows of one episode):
//   Aqk = tril(Q K^T)                      dU' = Aqk^T dO + K dS^T
//   dAqk = tril(dO U'^T)                   dQ  = dO S + dAqk K
//   dK  = dAqk^T Q + U' dS                 dS <- dS + dO^T Q - dU'^T W
//   linear attention: U' = V, dV = dU', W = 0.
//   delta rule:  A = tril(diag(beta) K K^T, -1), Tm = (I+A)^-1, T = Tm diag(beta),
//     W = T K, U' = T V - W S^T, dW = -dU' S, Zu = Tm^T dU', Zw = Tm^T dW,
//     dV = diag(beta) Zu, dK += diag(beta) Zw, dbeta = rowdot(V, Zu) + rowdot(K, Zw),
//     dT = tril(dW K^T + dU' V^T), dA = -tril((Tm^T dT) T^T, -1),
//     R = dA K, dbeta += rowdot(K, R), dK += diag(beta) R + (diag(beta) dA)^T K.
#include "chunk_common.h"

namespace {

using namespace mrx;

template <typename T, int C> struct BwdDims {
    static constexpr int PAD = pad_of<T>();
    static constexpr int LDD = HD + PAD;  // leading dim of tiles with 64 columns
    static constexpr int LDC = C + PAD;   // leading dim of tiles with C columns
    static constexpr int szRD = C * LDD * sizeof(T);   // [C][64]
    static constexpr int szDR = HD * LDC * sizeof(T);  // [64][C]
    static constexpr int szDD = HD * LDD * sizeof(T);  // [64][64]
    static constexpr int szCC = C * LDC * sizeof(T);   // [C][C]
};

// d(phi)/dx recovered from the staged phi(x): phi > 1 <=> x > 0 (derivative 1), else phi' = phi.
template <bool FMAP> __device__ __forceinline__ float fmap_grad(float phi) { return FMAP ? (phi > 1.f ? 1.f : phi) : 1.f; }

// ---- shared pieces ----------------------------------------------------------------

// Stage dS (held as dS^T: m = dk, n = dv) into sdS[dv][dk] and sdSt[dk][dv].
template <typename T>
__device__ __forceinline__ void stage_dS(const f32x4 *dSacc, T *sdS, T *sdSt, int ld, int w, int lane)
{
    store_acc_t<T, HD, HD>(dSacc, sdS, ld, w, lane);
    store_acc_n<T, HD, HD>(dSacc, sdSt, ld, w, lane);
}

// Write an accumulator set holding X^T (m = feature, n = chunk row) to a (B,T,H,64)
// array: 4 consecutive features per lane.  scale(row) multiplies, keep(row) gates.
template <typename T, int C, typename ScaleF, typename KeepF>
__device__ __forceinline__ void store_rows_global(const f32x4 *acc, T *base, int64_t rs, int t0, int Tlen,
                                                  int w, int lane, ScaleF scale, KeepF keep)
{
    using TM = TileMap<HD, C>;
    using P4 = typename TT<T>::pack4;
    const int li = lane & 15, lg = lane >> 4;
#pragma unroll
    for (int j = 0; j < TM::TPW; ++j) {
        const int d0 = TM::mt(w) * 16 + 4 * lg, r = TM::nt(w, j) * 16 + li;
        if (t0 + r < Tlen && keep(r)) {
            const f32x4 s = scale(r, d0);
            *reinterpret_cast<P4 *>(base + (int64_t)(t0 + r) * rs + d0) =
                TT<T>::pack(acc[j][0] * s[0], acc[j][1] * s[1], acc[j][2] * s[2], acc[j][3] * s[3]);
        }
    }
}

// =====================================================================================
// linear attention
// =====================================================================================
template <typename T, int C> struct LaBwdSmem : BwdDims<T, C> {
    using D = BwdDims<T, C>;
    static constexpr int oQ = 0, oK = oQ + D::szRD, oV = oK + D::szRD, oDO = oV + D::szRD,
                         oQt = oDO + D::szRD, oKt = oQt + D::szDR, oDOt = oKt + D::szDR,
                         oSt = oDOt + D::szDR, oDS = oSt + D::szDD, oDSt = oDS + D::szDD,
                         oAqkT = oDSt + D::szDD, oDAqk = oAqkT + D::szCC, oDAqkT = oDAqk + D::szCC,
                         total = oDAqkT + D::szCC;
};

template <typename T, int C, bool FMAP>
__global__ void __launch_bounds__(NTHREADS)
la_bwd_kernel(const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v,
              const void *__restrict__ done, int done_f32, const T *__restrict__ S_chk,
              const T *__restrict__ dout, const float *__restrict__ dS_last, T *__restrict__ dq,
              T *__restrict__ dk, T *__restrict__ dv, float *__restrict__ dS0, int Tlen, int H)
{
    using L = LaBwdSmem<T, C>;
    using IO = TileIO<T, C>;
    using IOS = TileIO<T, HD>;
    using P4 = typename TT<T>::pack4;
    extern __shared__ __align__(16) unsigned char smem[];
    T *sQ = reinterpret_cast<T *>(smem + L::oQ);
    T *sK = reinterpret_cast<T *>(smem + L::oK);
    T *sV = reinterpret_cast<T *>(smem + L::oV);
    T *sDO = reinterpret_cast<T *>(smem + L::oDO);
    T *sQt = reinterpret_cast<T *>(smem + L::oQt);
    T *sKt = reinterpret_cast<T *>(smem + L::oKt);
    T *sDOt = reinterpret_cast<T *>(smem + L::oDOt);
    T *sSt = reinterpret_cast<T *>(smem + L::oSt);
    T *sDS = reinterpret_cast<T *>(smem + L::oDS);
    T *sDSt = reinterpret_cast<T *>(smem + L::oDSt);
    T *sAqkT = reinterpret_cast<T *>(smem + L::oAqkT);
    T *sDAqk = reinterpret_cast<T *>(smem + L::oDAqk);
    T *sDAqkT = reinterpret_cast<T *>(smem + L::oDAqkT);

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    const int bh = blockIdx.x, b = bh / H, h = bh % H;
    const int64_t rs = (int64_t)H * HD;
    const int64_t base = ((int64_t)b * Tlen * H + h) * HD;
    const int NC = (Tlen + C - 1) / C;

    using TMS = TileMap<HD, HD>;
    using TMA = TileMap<C, C>;
    using TMR = TileMap<HD, C>;
    f32x4 dSacc[TMS::TPW];  // dS^T: m = dk, n = dv
#pragma unroll
    for (int j = 0; j < TMS::TPW; ++j) {
        const int dk0 = TMS::mt(w) * 16 + 4 * lg, dvv = TMS::nt(w, j) * 16 + li;
        dSacc[j] = dS_last ? *reinterpret_cast<const f32x4 *>(dS_last + ((int64_t)bh * HD + dvv) * HD + dk0)
                           : f32x4{0.f, 0.f, 0.f, 0.f};
    }

    typename IO::Regs rq, rk, rv, rdo;
    typename IOS::Regs rS;
    uint32_t rdone = 0u;  // raw bits, tested when the chunk is staged
    auto prefetch = [&](int c) {
        const int t0 = c * C;
        IO::load(rq, q + base, rs, t0, Tlen, tid);
        IO::load(rk, k + base, rs, t0, Tlen, tid);
        IO::load(rv, v + base, rs, t0, Tlen, tid);
        IO::load(rdo, dout + base, rs, t0, Tlen, tid);
        IOS::load(rS, S_chk + ((int64_t)bh * NC + c) * HD * HD, HD, 0, HD, tid);
        rdone = 0u;
        if (lane < C && t0 + lane < Tlen) rdone = done_raw(done, done_f32, (int64_t)b * Tlen + t0 + lane);
    };
    prefetch(NC - 1);

    for (int c = NC - 1; c >= 0; --c) {
        const int t0 = c * C;
        const unsigned long long dmask = __ballot(done_test(rdone, done_f32) && lane < C);
        const int nres = __popcll(dmask);
        for (int pass = nres; pass >= 0; --pass) {
            auto live = [&](int r) { return nres == 0 || episode_of(dmask, r) == pass; };
            // ---- stage -------------------------------------------------------------
            {
                typename IO::Regs fq = rq, fk = rk, fv = rv, fdo = rdo;
                IO::template fmap<FMAP>(fq);
                IO::template fmap<FMAP>(fk);
                if (nres != 0) {
                    const int r0 = tid / IO::SEGS;
#pragma unroll
                    for (int p = 0; p < IO::PASSES; ++p) {
                        if (!live(r0 + p * IO::RPP)) {
#pragma unroll
                            for (int e = 0; e < IO::KP; ++e) {
                                fq.v[p][e] = (T)0.f; fk.v[p][e] = (T)0.f; fv.v[p][e] = (T)0.f; fdo.v[p][e] = (T)0.f;
                            }
                        }
                    }
                }
                IO::to_lds(fq, sQ, L::LDD, tid);
                IO::to_lds_t(fq, sQt, L::LDC, tid);
                IO::to_lds(fk, sK, L::LDD, tid);
                IO::to_lds_t(fk, sKt, L::LDC, tid);
                IO::to_lds(fv, sV, L::LDD, tid);
                IO::to_lds(fdo, sDO, L::LDD, tid);
                IO::to_lds_t(fdo, sDOt, L::LDC, tid);
                typename IOS::Regs fS = rS;
                if (pass != 0) {
#pragma unroll
                    for (int p = 0; p < IOS::PASSES; ++p)
#pragma unroll
                        for (int e = 0; e < IOS::KP; ++e) fS.v[p][e] = (T)0.f;
                }
                IOS::to_lds_t(fS, sSt, L::LDD, tid);  // S_chk is [dv][dk]; sSt[dk][dv]
            }
            if (pass != nres) zero_acc<TMS::TPW>(dSacc);  // an episode that ends inside the chunk
            stage_dS<T>(dSacc, sDS, sDSt, L::LDD, w, lane);
            sync_lds();
            if (pass == 0 && c > 0) prefetch(c - 1);

            // ---- Aqk^T[j][i] and dAqk[i][j] (+ transpose), causal -----------------------
            {
                f32x4 acc[TMA::TPW];
                zero_acc<TMA::TPW>(acc);
                gemm_nt<T, C, C, HD>(acc, sQ, L::LDD, sK, L::LDD, w, lane);  // D[m = i][n = j]
#pragma unroll
                for (int j = 0; j < TMA::TPW; ++j) {
                    const int m0 = TMA::mt(w) * 16 + 4 * lg, n = TMA::nt(w, j) * 16 + li;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (m0 + e < n) acc[j][e] = 0.f;
                }
                store_acc_t<T, C, C>(acc, sAqkT, L::LDC, w, lane);
                zero_acc<TMA::TPW>(acc);
                gemm_nt<T, C, C, HD>(acc, sV, L::LDD, sDO, L::LDD, w, lane);  // D[m = j][n = i]
#pragma unroll
                for (int j = 0; j < TMA::TPW; ++j) {
                    const int m0 = TMA::mt(w) * 16 + 4 * lg, n = TMA::nt(w, j) * 16 + li;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (m0 + e > n) acc[j][e] = 0.f;
                }
                store_acc_t<T, C, C>(acc, sDAqk, L::LDC, w, lane);
                store_acc_n<T, C, C>(acc, sDAqkT, L::LDC, w, lane);
            }
            sync_lds();
            auto one = [](int, int) { return f32x4{1.f, 1.f, 1.f, 1.f}; };
            // ---- dV^T[dv][j] = dO^T Aqk + dS K^T ---------------------------------------
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                gemm_nt<T, HD, C, C>(acc, sDOt, L::LDC, sAqkT, L::LDC, w, lane);
                gemm_nt<T, HD, C, HD>(acc, sDS, L::LDD, sK, L::LDD, w, lane);
                store_rows_global<T, C>(acc, dv + base, rs, t0, Tlen, w, lane, one, live);
            }
            // ---- dQ^T[dk][i] = S^T dO^T + K^T dAqk^T -----------------------------------
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                gemm_nt<T, HD, C, HD>(acc, sSt, L::LDD, sDO, L::LDD, w, lane);
                gemm_nt<T, HD, C, C>(acc, sKt, L::LDC, sDAqk, L::LDC, w, lane);
                auto sc = [&](int r, int d0) {
                    const P4 x = *reinterpret_cast<const P4 *>(sQ + r * L::LDD + d0);
                    return f32x4{fmap_grad<FMAP>((float)x[0]), fmap_grad<FMAP>((float)x[1]),
                                 fmap_grad<FMAP>((float)x[2]), fmap_grad<FMAP>((float)x[3])};
                };
                store_rows_global<T, C>(acc, dq + base, rs, t0, Tlen, w, lane, sc, live);
            }
            // ---- dK^T[dk][j] = Q^T dAqk + dS^T V^T --------------------------------------
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                gemm_nt<T, HD, C, C>(acc, sQt, L::LDC, sDAqkT, L::LDC, w, lane);
                gemm_nt<T, HD, C, HD>(acc, sDSt, L::LDD, sV, L::LDD, w, lane);
                auto sc = [&](int r, int d0) {
                    const P4 x = *reinterpret_cast<const P4 *>(sK + r * L::LDD + d0);
                    return f32x4{fmap_grad<FMAP>((float)x[0]), fmap_grad<FMAP>((float)x[1]),
                                 fmap_grad<FMAP>((float)x[2]), fmap_grad<FMAP>((float)x[3])};
                };
                store_rows_global<T, C>(acc, dk + base, rs, t0, Tlen, w, lane, sc, live);
            }
            // ---- dS^T[dk][dv] += Q^T dO ---------------------------------------------------
            gemm_nt<T, HD, HD, C>(dSacc, sQt, L::LDC, sDOt, L::LDC, w, lane);
            sync_lds();
        }
    }
    if (dS0) {
#pragma unroll
        for (int j = 0; j < TMS::TPW; ++j) {
            const int dk0 = TMS::mt(w) * 16 + 4 * lg, dvv = TMS::nt(w, j) * 16 + li;
            *reinterpret_cast<f32x4 *>(dS0 + ((int64_t)bh * HD + dvv) * HD + dk0) = dSacc[j];
        }
    }
}

// =====================================================================================
// delta rule (bf16, C = 64: seventeen 9 KiB regions, reused as operands die)
// =====================================================================================
template <typename T, int C> struct DeltaBwdSmem : BwdDims<T, C> {
    using D = BwdDims<T, C>;
    static constexpr int U = D::szDD;  // every tile type has this size for bf16 / C = 64
    static_assert(D::szRD == U && D::szDR == U && D::szCC == U, "regions assume equal tile sizes");
    static_assert(C * (C + 4) * 4 <= 2 * U, "fp32 A must fit two regions");
    static constexpr int NREG = 17;
    static constexpr int oBeta = NREG * U, oDb = oBeta + C * 4, total = oDb + NWAVES * C * 4;
};

template <typename T, int C>
__global__ void __launch_bounds__(NTHREADS)
delta_bwd_kernel(const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v,
                 const T *__restrict__ beta, const void *__restrict__ done, int done_f32,
                 const T *__restrict__ S_chk, const T *__restrict__ dout,
                 const float *__restrict__ dS_last, T *__restrict__ dq, T *__restrict__ dk,
                 T *__restrict__ dv, T *__restrict__ dbeta, float *__restrict__ dS0, int Tlen, int H)
{
    using L = DeltaBwdSmem<T, C>;
    using IO = TileIO<T, C>;
    using IOS = TileIO<T, HD>;
    using P4 = typename TT<T>::pack4;
    constexpr int LDD = L::LDD, LDC = L::LDC, LDA = C + 4;
    extern __shared__ __align__(16) unsigned char smem[];
    auto reg = [&](int r) { return reinterpret_cast<T *>(smem + r * L::U); };
    // region plan (-> marks reuse once the first tenant is dead)
    T *sK = reg(0), *sKt = reg(1), *sV = reg(2);
    T *sVt = reg(3), *sDU = reg(3);           // Vt -> dU'[c][dv]
    T *sQ = reg(4), *sDUt = reg(4);           // Q  -> dU'^T[dv][c]
    T *sQt = reg(5), *sDTt = reg(5);          // Qt -> dT^T[b][a]
    T *sDO = reg(6), *sDW = reg(6);           // dO -> dW[c][dk]
    T *sDOt = reg(7), *sDWt = reg(7);         // dOt -> dW^T[dk][c]
    T *sS = reg(8), *sU = reg(8);             // S[dv][dk] -> U'[c][dv]
    T *sSt = reg(9), *sY1 = reg(9);           // St[dk][dv] -> Y1[j][b]
    T *sDS = reg(10), *sDAqk = reg(10), *sDA = reg(10);  // dS[dv][dk] -> dAqk[i][j] -> dA[i][j]
    T *sDSt = reg(11), *sGt = reg(11);        // dSt[dk][dv] -> G^T[j][i]
    float *sA = reinterpret_cast<float *>(smem + 12 * L::U);  // regions 12,13 (fp32)
    T *sAqkT = reg(12);                       // after A is consumed
    T *sW = reg(13), *sDAqkT = reg(13);       // W[c][dk] -> dAqk^T[j][i]
    T *sT = reg(14), *sTmt = reg(15), *sWt = reg(16);
    float *sBeta = reinterpret_cast<float *>(smem + L::oBeta);
    float *sDb = reinterpret_cast<float *>(smem + L::oDb);

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    const int bh = blockIdx.x, b = bh / H, h = bh % H;
    const int64_t rs = (int64_t)H * HD;
    const int64_t base = ((int64_t)b * Tlen * H + h) * HD;
    const int NC = (Tlen + C - 1) / C;

    using TMS = TileMap<HD, HD>;
    using TMA = TileMap<C, C>;
    using TMR = TileMap<HD, C>;
    f32x4 dSacc[TMS::TPW];  // dS^T: m = dk, n = dv
#pragma unroll
    for (int j = 0; j < TMS::TPW; ++j) {
        const int dk0 = TMS::mt(w) * 16 + 4 * lg, dvv = TMS::nt(w, j) * 16 + li;
        dSacc[j] = dS_last ? *reinterpret_cast<const f32x4 *>(dS_last + ((int64_t)bh * HD + dvv) * HD + dk0)
                           : f32x4{0.f, 0.f, 0.f, 0.f};
    }

    typename IO::Regs rq, rk, rv, rdo;
    typename IOS::Regs rS;
    uint32_t rdone = 0u, rbeta = 0u;  // raw bits, converted when the chunk is staged
    auto prefetch = [&](int c) {
        const int t0 = c * C;
        IO::load(rq, q + base, rs, t0, Tlen, tid);
        IO::load(rk, k + base, rs, t0, Tlen, tid);
        IO::load(rv, v + base, rs, t0, Tlen, tid);
        IO::load(rdo, dout + base, rs, t0, Tlen, tid);
        IOS::load(rS, S_chk + ((int64_t)bh * NC + c) * HD * HD, HD, 0, HD, tid);
        rdone = 0u;
        rbeta = 0u;
        if (lane < C && t0 + lane < Tlen) {
            const int64_t bt = (int64_t)b * Tlen + t0 + lane;
            rdone = done_raw(done, done_f32, bt);
            if (w == 0) rbeta = load_raw<T>(beta + bt * H + h);
        }
    };
    prefetch(NC - 1);
    MRX_PHASE_INIT();

    for (int c = NC - 1; c >= 0; --c) {
        const int t0 = c * C;
        const unsigned long long dmask = __ballot(done_test(rdone, done_f32) && lane < C);
        const int nres = __popcll(dmask);
        for (int pass = nres; pass >= 0; --pass) {
            auto live = [&](int r) { return nres == 0 || episode_of(dmask, r) == pass; };
            // ---- stage ---------------------------------------------------------------
            {
                typename IO::Regs fq = rq, fk = rk, fv = rv, fdo = rdo;
                if (nres != 0) {
                    const int r0 = tid / IO::SEGS;
#pragma unroll
                    for (int p = 0; p < IO::PASSES; ++p) {
                        if (!live(r0 + p * IO::RPP)) {
#pragma unroll
                            for (int e = 0; e < IO::KP; ++e) {
                                fq.v[p][e] = (T)0.f; fk.v[p][e] = (T)0.f; fv.v[p][e] = (T)0.f; fdo.v[p][e] = (T)0.f;
                            }
                        }
                    }
                }
                IO::to_lds(fq, sQ, LDD, tid);
                IO::to_lds_t(fq, sQt, LDC, tid);
                IO::to_lds(fk, sK, LDD, tid);
                IO::to_lds_t(fk, sKt, LDC, tid);
                IO::to_lds(fv, sV, LDD, tid);
                IO::to_lds_t(fv, sVt, LDC, tid);
                IO::to_lds(fdo, sDO, LDD, tid);
                IO::to_lds_t(fdo, sDOt, LDC, tid);
                typename IOS::Regs fS = rS;
                if (pass != 0) {
#pragma unroll
                    for (int p = 0; p < IOS::PASSES; ++p)
#pragma unroll
                        for (int e = 0; e < IOS::KP; ++e) fS.v[p][e] = (T)0.f;
                }
                IOS::to_lds(fS, sS, LDD, tid);
                IOS::to_lds_t(fS, sSt, LDD, tid);
            }
            if (tid < C) sBeta[tid] = live(tid) ? raw_to_float<T>(rbeta) : 0.f;
            if (pass != nres) zero_acc<TMS::TPW>(dSacc);
            stage_dS<T>(dSacc, sDS, sDSt, LDD, w, lane);
            sync_lds();
            MRX_PHASE(11);
            if (pass == 0 && c > 0) prefetch(c - 1);

            // ---- A = beta_i (K K^T) strictly lower -> sA ---------------------------------
            {
                f32x4 acc[TMA::TPW];
                zero_acc<TMA::TPW>(acc);
                gemm_nt<T, C, C, HD>(acc, sK, LDD, sK, LDD, w, lane);
#pragma unroll
                for (int j = 0; j < TMA::TPW; ++j) {
                    const int m0 = TMA::mt(w) * 16 + 4 * lg, n = TMA::nt(w, j) * 16 + li;
                    const float bi = sBeta[n];
                    f32x4 r;
#pragma unroll
                    for (int e = 0; e < 4; ++e) r[e] = (m0 + e < n) ? bi * acc[j][e] : 0.f;
                    *reinterpret_cast<f32x4 *>(sA + n * LDA + m0) = r;
                }
            }
            sync_lds();
            MRX_PHASE(12);
            tri_inverse<C>(sA, LDA, w, lane);
            MRX_PHASE(13);
            // ---- sT[i][j] = Tm[i][j] beta_j ; sTmt[j][i] = Tm[i][j] ----------------------
            for (int idx = tid; idx < C * C / 4; idx += NTHREADS) {
                const int i = idx / (C / 4), j = (idx % (C / 4)) * 4;
                const f32x4 t = tri_inverse_get4(sA, LDA, i, j);
                *reinterpret_cast<P4 *>(sT + i * LDC + j) =
                    TT<T>::pack(t[0] * sBeta[j], t[1] * sBeta[j + 1], t[2] * sBeta[j + 2], t[3] * sBeta[j + 3]);
#pragma unroll
                for (int e = 0; e < 4; ++e) sTmt[(j + e) * LDC + i] = (T)t[e];
            }
            sync_lds();
            MRX_PHASE(14);
            // ---- Aqk^T[j][i] ; W^T[dk][c] = K^T T^T -> sW[c][dk], sWt[dk][c] ---------------
            {
                f32x4 acc[TMA::TPW];
                zero_acc<TMA::TPW>(acc);
                gemm_nt<T, C, C, HD>(acc, sQ, LDD, sK, LDD, w, lane);  // D[m = i][n = j]
#pragma unroll
                for (int j = 0; j < TMA::TPW; ++j) {
                    const int m0 = TMA::mt(w) * 16 + 4 * lg, n = TMA::nt(w, j) * 16 + li;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (m0 + e < n) acc[j][e] = 0.f;
                }
                store_acc_t<T, C, C>(acc, sAqkT, LDC, w, lane);
            }
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                gemm_nt<T, HD, C, C>(acc, sKt, LDC, sT, LDC, w, lane);  // D[m = dk][n = c]
                store_acc_t<T, HD, C>(acc, sW, LDD, w, lane);
                store_acc_n<T, HD, C>(acc, sWt, LDC, w, lane);
            }
            sync_lds();
            MRX_PHASE(15);
            // ---- U'^T[dv][c] = V^T T^T - S W^T -> sU[c][dv] (over sS) ------------------------
            {
                f32x4 acc[TMR::TPW], acc2[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                zero_acc<TMR::TPW>(acc2);
                gemm_nt<T, HD, C, C>(acc, sVt, LDC, sT, LDC, w, lane);
                gemm_nt<T, HD, C, HD>(acc2, sS, LDD, sW, LDD, w, lane);
#pragma unroll
                for (int j = 0; j < TMR::TPW; ++j) acc[j] -= acc2[j];
                sync_lds();  // every wave is done reading sS, sVt, sQ
                MRX_PHASE(16);
                store_acc_t<T, HD, C>(acc, sU, LDD, w, lane);
            }
            // ---- dU'^T[dv][j] = dO^T Aqk + dS K^T -> sDU[j][dv], sDUt[dv][j] -----------------
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                gemm_nt<T, HD, C, C>(acc, sDOt, LDC, sAqkT, LDC, w, lane);
                gemm_nt<T, HD, C, HD>(acc, sDS, LDD, sK, LDD, w, lane);
                store_acc_t<T, HD, C>(acc, sDU, LDD, w, lane);
                store_acc_n<T, HD, C>(acc, sDUt, LDC, w, lane);
            }
            sync_lds();  // sU, sDU, sDUt visible; sDS, sW dead
            MRX_PHASE(17);
            // ---- dAqk[i][j] = tril(dO U'^T) (+ transpose) ----------------------------------
            {
                f32x4 acc[TMA::TPW];
                zero_acc<TMA::TPW>(acc);
                gemm_nt<T, C, C, HD>(acc, sU, LDD, sDO, LDD, w, lane);  // D[m = j][n = i]
#pragma unroll
                for (int j = 0; j < TMA::TPW; ++j) {
                    const int m0 = TMA::mt(w) * 16 + 4 * lg, n = TMA::nt(w, j) * 16 + li;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (m0 + e > n) acc[j][e] = 0.f;
                }
                store_acc_t<T, C, C>(acc, sDAqk, LDC, w, lane);
                store_acc_n<T, C, C>(acc, sDAqkT, LDC, w, lane);
            }
            sync_lds();
            MRX_PHASE(18);
            auto one = [](int, int) { return f32x4{1.f, 1.f, 1.f, 1.f}; };
            // ---- dQ^T[dk][i] = S^T dO^T + K^T dAqk^T -> global -------------------------------
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                gemm_nt<T, HD, C, HD>(acc, sSt, LDD, sDO, LDD, w, lane);
                gemm_nt<T, HD, C, C>(acc, sKt, LDC, sDAqk, LDC, w, lane);
                store_rows_global<T, C>(acc, dq + base, rs, t0, Tlen, w, lane, one, live);
            }
            // ---- dK^T[dk][j] = Q^T dAqk + dS^T U'^T  (kept in registers) ----------------------
            f32x4 dKacc[TMR::TPW];
            zero_acc<TMR::TPW>(dKacc);
            gemm_nt<T, HD, C, C>(dKacc, sQt, LDC, sDAqkT, LDC, w, lane);
            gemm_nt<T, HD, C, HD>(dKacc, sDSt, LDD, sU, LDD, w, lane);
            // ---- dS^T[dk][dv] += Q^T dO - W^T dU' -----------------------------------------------
            {
                f32x4 acc[TMS::TPW];
                zero_acc<TMS::TPW>(acc);
                gemm_nt<T, HD, HD, C>(dSacc, sQt, LDC, sDOt, LDC, w, lane);
                gemm_nt<T, HD, HD, C>(acc, sWt, LDC, sDUt, LDC, w, lane);
#pragma unroll
                for (int j = 0; j < TMS::TPW; ++j) dSacc[j] -= acc[j];
            }
            sync_lds();  // sDO, sDOt, sQt, sDAqk*, sDSt dead
            MRX_PHASE(19);
            // ---- dW^T[dk][c] = -S^T dU'^T -> sDW[c][dk], sDWt[dk][c] ---------------------------
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                gemm_nt<T, HD, C, HD>(acc, sSt, LDD, sDU, LDD, w, lane);
#pragma unroll
                for (int j = 0; j < TMR::TPW; ++j) acc[j] = -acc[j];
                store_acc_t<T, HD, C>(acc, sDW, LDD, w, lane);
                store_acc_n<T, HD, C>(acc, sDWt, LDC, w, lane);
            }
            float dbp[TMR::TPW];  // per-lane partial of dbeta for row 16 j + li
#pragma unroll
            for (int j = 0; j < TMR::TPW; ++j) dbp[j] = 0.f;
            auto rowdot = [&](const f32x4 *acc, const T *X) {
#pragma unroll
                for (int j = 0; j < TMR::TPW; ++j) {
                    const int d0 = TMR::mt(w) * 16 + 4 * lg, r = TMR::nt(w, j) * 16 + li;
                    const P4 x = *reinterpret_cast<const P4 *>(X + r * LDD + d0);
                    dbp[j] += acc[j][0] * (float)x[0] + acc[j][1] * (float)x[1] + acc[j][2] * (float)x[2] +
                              acc[j][3] * (float)x[3];
                }
            };
            auto beta_of = [&](int r, int) { const float bb = sBeta[r]; return f32x4{bb, bb, bb, bb}; };
            // ---- Zu^T[dv][j] = dU'^T Tm -> dV = beta_j Zu ; dbeta += V_j . Zu_j -------------------
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                gemm_nt<T, HD, C, C>(acc, sDUt, LDC, sTmt, LDC, w, lane);
                rowdot(acc, sV);
                store_rows_global<T, C>(acc, dv + base, rs, t0, Tlen, w, lane, beta_of, live);
            }
            sync_lds();  // sDW, sDWt visible
            MRX_PHASE(20);
            // ---- Zw^T[dk][j] = dW^T Tm -> dK += beta_j Zw ; dbeta += K_j . Zw_j -------------------
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                gemm_nt<T, HD, C, C>(acc, sDWt, LDC, sTmt, LDC, w, lane);
                rowdot(acc, sK);
#pragma unroll
                for (int j = 0; j < TMR::TPW; ++j) {
                    const float bb = sBeta[TMR::nt(w, j) * 16 + li];
                    dKacc[j] += acc[j] * bb;
                }
            }
            // ---- dT^T: D[m = a][n = b] = dW K^T + dU' V^T, a >= b -> sDTt[b][a] --------------------
            {
                f32x4 acc[TMA::TPW];
                zero_acc<TMA::TPW>(acc);
                gemm_nt<T, C, C, HD>(acc, sDW, LDD, sK, LDD, w, lane);
                gemm_nt<T, C, C, HD>(acc, sDU, LDD, sV, LDD, w, lane);
#pragma unroll
                for (int j = 0; j < TMA::TPW; ++j) {
                    const int m0 = TMA::mt(w) * 16 + 4 * lg, n = TMA::nt(w, j) * 16 + li;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (m0 + e < n) acc[j][e] = 0.f;
                }
                store_acc_t<T, C, C>(acc, sDTt, LDC, w, lane);
            }
            sync_lds();
            MRX_PHASE(21);
            // ---- Y1: D[m = b][n = j] = dT^T Tm -> sY1[j][b] -----------------------------------------
            {
                f32x4 acc[TMA::TPW];
                zero_acc<TMA::TPW>(acc);
                gemm_nt<T, C, C, C>(acc, sDTt, LDC, sTmt, LDC, w, lane);
                store_acc_t<T, C, C>(acc, sY1, LDC, w, lane);
            }
            sync_lds();
            MRX_PHASE(22);
            // ---- dA: D[m = j][n = i] = -T Y1^T, j < i -> sDA[i][j] ; sGt[j][i] = beta_i dA[i][j] -----
            {
                f32x4 acc[TMA::TPW];
                zero_acc<TMA::TPW>(acc);
                gemm_nt<T, C, C, C>(acc, sT, LDC, sY1, LDC, w, lane);
#pragma unroll
                for (int j = 0; j < TMA::TPW; ++j) {
                    const int m0 = TMA::mt(w) * 16 + 4 * lg, n = TMA::nt(w, j) * 16 + li;
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[j][e] = (m0 + e < n) ? -acc[j][e] : 0.f;
                }
                store_acc_t<T, C, C>(acc, sDA, LDC, w, lane);
#pragma unroll
                for (int j = 0; j < TMA::TPW; ++j) acc[j] *= sBeta[TMA::nt(w, j) * 16 + li];
                store_acc_n<T, C, C>(acc, sGt, LDC, w, lane);
            }
            sync_lds();
            MRX_PHASE(23);
            // ---- R^T[dk][i] = K^T dA^T -> dK += beta_i R ; dbeta += K_i . R_i ; dK += K^T G ---------
            {
                f32x4 acc[TMR::TPW];
                zero_acc<TMR::TPW>(acc);
                gemm_nt<T, HD, C, C>(acc, sKt, LDC, sDA, LDC, w, lane);
                rowdot(acc, sK);
#pragma unroll
                for (int j = 0; j < TMR::TPW; ++j) {
                    const float bb = sBeta[TMR::nt(w, j) * 16 + li];
                    dKacc[j] += acc[j] * bb;
                }
                gemm_nt<T, HD, C, C>(dKacc, sKt, LDC, sGt, LDC, w, lane);
                store_rows_global<T, C>(dKacc, dk + base, rs, t0, Tlen, w, lane, one, live);
            }
            // ---- dbeta: reduce the partials over lane groups, then over waves through LDS ---------
#pragma unroll
            for (int j = 0; j < TMR::TPW; ++j) {
                float x = dbp[j];
                x += __shfl_xor(x, 16);
                x += __shfl_xor(x, 32);
                if (lg == 0) sDb[w * C + TMR::nt(w, j) * 16 + li] = x;
            }
            sync_lds();
            MRX_PHASE(24);
            if (tid < C && t0 + tid < Tlen && live(tid)) {
                float x = 0.f;
#pragma unroll
                for (int ww = 0; ww < NWAVES; ++ww) x += sDb[ww * C + tid];
                dbeta[((int64_t)b * Tlen + t0 + tid) * H + h] = (T)x;
            }
            sync_lds();
            MRX_PHASE(25);
        }
    }
    if (dS0) {
#pragma unroll
        for (int j = 0; j < TMS::TPW; ++j) {
            const int dk0 = TMS::mt(w) * 16 + 4 * lg, dvv = TMS::nt(w, j) * 16 + li;
            *reinterpret_cast<f32x4 *>(dS0 + ((int64_t)bh * HD + dvv) * HD + dk0) = dSacc[j];
        }
    }
}

template <typename K> int set_smem(K kern, int smem, bool &flag)
{
    if (!flag) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                hipFuncAttributeMaxDynamicSharedMemorySize, smem) != hipSuccess)
            return MRX_ERR_LAUNCH;
        flag = true;
    }
    return MRX_OK;
}

template <typename T, int C, bool FMAP>
int launch_la(hipStream_t st, const void *q, const void *k, const void *v, const void *done,
              int done_f32, const void *S_chk, const void *dout, const void *dS_last, void *dq,
              void *dk, void *dv, void *dS0, int64_t B, int64_t Tlen, int64_t H)
{
    auto kern = la_bwd_kernel<T, C, FMAP>;
    constexpr int smem = LaBwdSmem<T, C>::total;
    static bool attr_set = false;
    if (set_smem(kern, smem, attr_set) != MRX_OK) return MRX_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)(B * H)), dim3(NTHREADS), smem, st, (const T *)q,
                       (const T *)k, (const T *)v, done, done_f32, (const T *)S_chk,
                       (const T *)dout, (const float *)dS_last, (T *)dq, (T *)dk, (T *)dv,
                       (float *)dS0, (int)Tlen, (int)H);
    return launch_status();
}

int check_bwd(const void *q, const void *k, const void *v, const void *done, const void *S_chk,
              const void *dout, const void *dS_last, const void *dq, const void *dk_out,
              const void *dv_out, const void *dS0, int64_t B, int64_t T, int64_t H, int64_t dk,
              int64_t dv, int dtype, int done_dtype)
{
    if (!q || !k || !v || !done || !S_chk || !dout || !dq || !dk_out || !dv_out) return MRX_ERR_INVALID_ARG;
    if (B <= 0 || T <= 0 || H <= 0 || dk <= 0 || dv <= 0) return MRX_ERR_INVALID_ARG;
    if (dtype != MRX_F32 && dtype != MRX_BF16) return dtype == MRX_C64 ? MRX_ERR_UNSUPPORTED : MRX_ERR_INVALID_ARG;
    if (done_dtype != MRX_DONE_U8 && done_dtype != MRX_DONE_F32) return MRX_ERR_INVALID_ARG;
    if (dk != HD || dv != HD) return MRX_ERR_UNSUPPORTED;
    if (B * H >= (1ll << 31) || T >= (1ll << 30)) return MRX_ERR_INVALID_ARG;
    const void *ps[] = {q, k, v, S_chk, dout, dS_last, dq, dk_out, dv_out, dS0};
    for (const void *p : ps)
        if (!aligned(p, 16)) return MRX_ERR_INVALID_ARG;
    if (done_dtype == MRX_DONE_F32 && !aligned(done, 4)) return MRX_ERR_INVALID_ARG;
    return MRX_OK;
}

}  // namespace

extern "C" int mrx_linear_attn_bwd(void *stream, const void *q, const void *k, const void *v,
                                   const void *done, const void *S_chk, const void *dout,
                                   const void *dS_last, void *dq, void *dk_out, void *dv_out,
                                   void *dS0, int64_t B, int64_t T, int64_t H, int64_t dk, int64_t dv,
                                   int dtype, int done_dtype, int feature_map)
{
    const int rc = check_bwd(q, k, v, done, S_chk, dout, dS_last, dq, dk_out, dv_out, dS0, B, T, H, dk,
                             dv, dtype, done_dtype);
    if (rc != MRX_OK) return rc;
    if (feature_map != MRX_FMAP_NONE && feature_map != MRX_FMAP_ELU1) return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const bool fm = feature_map == MRX_FMAP_ELU1;
#define MRX_ARGS st, q, k, v, done, done_dtype, S_chk, dout, dS_last, dq, dk_out, dv_out, dS0, B, T, H
    if (dtype == MRX_BF16) return fm ? launch_la<__bf16, 64, true>(MRX_ARGS) : launch_la<__bf16, 64, false>(MRX_ARGS);
    return fm ? launch_la<float, 32, true>(MRX_ARGS) : launch_la<float, 32, false>(MRX_ARGS);
#undef MRX_ARGS
}

extern "C" int mrx_delta_rule_bwd(void *stream, const void *q, const void *k, const void *v,
                                  const void *beta, const void *done, const void *S_chk,
                                  const void *dout, const void *dS_last, void *dq, void *dk_out,
                                  void *dv_out, void *dbeta, void *dS0, int64_t B, int64_t T, int64_t H,
                                  int64_t dk, int64_t dv, int dtype, int done_dtype)
{
    const int rc = check_bwd(q, k, v, done, S_chk, dout, dS_last, dq, dk_out, dv_out, dS0, B, T, H, dk,
                             dv, dtype, done_dtype);
    if (rc != MRX_OK) return rc;
    if (!beta || !dbeta) return MRX_ERR_INVALID_ARG;
    if (dtype != MRX_BF16) return MRX_ERR_UNSUPPORTED;  // fp32 delta-rule backward: not built yet
    hipStream_t st = (hipStream_t)stream;
    auto kern = delta_bwd_kernel<__bf16, 64>;
    constexpr int smem = DeltaBwdSmem<__bf16, 64>::total;
    static bool attr_set = false;
    if (set_smem(kern, smem, attr_set) != MRX_OK) return MRX_ERR_LAUNCH;
    hipLaunchKernelGGL(kern, dim3((unsigned)(B * H)), dim3(NTHREADS), smem, st, (const __bf16 *)q,
                       (const __bf16 *)k, (const __bf16 *)v, (const __bf16 *)beta, done, done_dtype,
                       (const __bf16 *)S_chk, (const __bf16 *)dout, (const float *)dS_last,
                       (__bf16 *)dq, (__bf16 *)dk_out, (__bf16 *)dv_out, (__bf16 *)dbeta, (float *)dS0,
                       (int)T, (int)H);
    return launch_status();
}
