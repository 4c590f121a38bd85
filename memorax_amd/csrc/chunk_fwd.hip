// Forward of chunked causal linear attention and of the DeltaNet delta rule (WY/UT form).
//
// Per chunk (rows i, j of the chunk; S = state entering the chunk, d_v x d_k, fp32):
//   linear attention:  U' = V
//   delta rule:        A  = tril(diag(beta) (K K^T . M), -1),  Tm = (I + A)^-1,  T = Tm diag(beta)
//                      W  = T K,  U' = T V - diag(m) W S^T
//   both:              O  = diag(m) Q S^T + (tril(Q K^T) . M) U'
//                      S <- l S + (diag(e) U')^T K
// M, m, e, l are the episode masks of the chunk; they are realised by processing a
// chunk that contains resets once per episode with the other episodes' rows zeroed
// by select, so inside a pass only the causal mask remains.  The state is
// kept transposed (S^T, d_k x d_v) in MFMA accumulators for the whole sequence and
// re-staged to LDS as a T-typed d_v x d_k tile once per chunk.
#include "chunk_common.h"

namespace {

using namespace mrx;

template <typename T, int C, bool DELTA> struct FwdSmem {
    static constexpr int PAD = pad_of<T>();
    static constexpr int LDD = HD + PAD;  // tiles with 64 columns
    static constexpr int LDC = C + PAD;   // tiles with C columns
    static constexpr int LDA = C + 4;     // fp32 C x C
    static constexpr int szQ = C * LDD * sizeof(T);    // sQ, later sW   [C][64]
    static constexpr int szK = szQ;                    // sK            [C][64]
    static constexpr int szKt = HD * LDC * sizeof(T);  // sKt           [64][C]
    static constexpr int szVt = szKt;                  // sVt, later sUt [64][C]
    static constexpr int szS = HD * LDD * sizeof(T);   // sS            [64][64]
    static constexpr int szT = DELTA ? C * LDC * sizeof(T) : 0;  // sT   [C][C]
    static constexpr int szAq = C * LDC * sizeof(T);   // sAqk          [C][C]
    static constexpr int szA = DELTA ? C * LDA * 4 : 0;  // sA fp32 [C][C], overlaid by sAqk afterwards
    static constexpr int szAA = szA > szAq ? szA : szAq;
    static constexpr int oQ = 0, oK = oQ + szQ, oKt = oK + szK, oVt = oKt + szKt, oS = oVt + szVt,
                         oT = oS + szS, oA = oT + szT, oBeta = oA + szAA, total = oBeta + C * 4;
};

template <typename T, int C, bool DELTA, bool FMAP>
__global__ void __launch_bounds__(NTHREADS, 2)  // 2 waves per SIMD: two workgroups share a CU
chunk_fwd_kernel(const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v,
                 const T *__restrict__ beta, const void *__restrict__ done, int done_f32,
                 const float *__restrict__ S0, T *__restrict__ o, float *__restrict__ S_last,
                 T *__restrict__ S_chk, int Tlen, int H)
{
    using L = FwdSmem<T, C, DELTA>;
    using IO = TileIO<T, C>;
    using P4 = typename TT<T>::pack4;
    extern __shared__ __align__(16) unsigned char smem[];
    T *sQ = reinterpret_cast<T *>(smem + L::oQ);
    T *sW = sQ;
    T *sK = reinterpret_cast<T *>(smem + L::oK);
    T *sKt = reinterpret_cast<T *>(smem + L::oKt);
    T *sVt = reinterpret_cast<T *>(smem + L::oVt);
    T *sUt = sVt;
    T *sS = reinterpret_cast<T *>(smem + L::oS);
    T *sT = reinterpret_cast<T *>(smem + L::oT);
    float *sA = reinterpret_cast<float *>(smem + L::oA);
    T *sAqk = reinterpret_cast<T *>(smem + L::oA);
    float *sBeta = reinterpret_cast<float *>(smem + L::oBeta);

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    const int bh = blockIdx.x, b = bh / H, h = bh % H;
    const int64_t rs = (int64_t)H * HD;  // row stride of q/k/v/o
    const T *qb = q + ((int64_t)b * Tlen * H + h) * HD;
    const T *kb = k + ((int64_t)b * Tlen * H + h) * HD;
    const T *vb = v + ((int64_t)b * Tlen * H + h) * HD;
    T *ob = o + ((int64_t)b * Tlen * H + h) * HD;
    const int NC = (Tlen + C - 1) / C;

    // state S^T (m = d_k, n = d_v) in accumulators
    using TMS = TileMap<HD, HD>;
    f32x4 Sacc[TMS::TPW];
#pragma unroll
    for (int j = 0; j < TMS::TPW; ++j) {
        const int dk0 = TMS::mt(w) * 16 + 4 * lg, dv = TMS::nt(w, j) * 16 + li;
        Sacc[j] = S0 ? *reinterpret_cast<const f32x4 *>(S0 + ((int64_t)bh * HD + dv) * HD + dk0)
                     : f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // register prefetch of the next chunk
    typename IO::Regs rq, rk, rv;
    uint32_t rbeta = 0u, rdone = 0u;  // raw bits, converted when the chunk is staged
    auto prefetch = [&](int c) {
        const int t0 = c * C;
        IO::load(rq, qb, rs, t0, Tlen, tid);
        IO::load(rk, kb, rs, t0, Tlen, tid);
        IO::load(rv, vb, rs, t0, Tlen, tid);
        rdone = 0u;
        rbeta = 0u;
        if (lane < C && t0 + lane < Tlen) {
            const int64_t bt = (int64_t)b * Tlen + t0 + lane;
            rdone = done_raw(done, done_f32, bt);
            if (DELTA && w == 0) rbeta = load_raw<T>(beta + bt * H + h);
        }
    };
    MRX_WG_BEGIN();
    prefetch(0);
    MRX_PHASE_INIT();

    for (int c = 0; c < NC; ++c) {
        const int t0 = c * C;
        // Episode structure of the chunk, known to every wave from its own ballot.
        // A chunk that contains resets is processed once per episode ("pass") with
        // the rows of all other episodes replaced by zeros *by select*, so that a
        // non-finite value never meets a masked-out zero inside a matrix product.
        const unsigned long long dmask = __ballot(done_test(rdone, done_f32) && lane < C);
        const int nres = __popcll(dmask);
        for (int pass = 0; pass <= nres; ++pass) {
        // ---- P0: stage the chunk -------------------------------------------------
        {
            typename IO::Regs fq = rq, fk = rk, fv = rv;
            IO::template fmap<FMAP>(fq);
            IO::template fmap<FMAP>(fk);
            if (nres != 0) {
                const int r0 = tid / IO::SEGS;
#pragma unroll
                for (int p = 0; p < IO::PASSES; ++p) {
                    const int r = r0 + p * IO::RPP;
                    if (episode_of(dmask, r) != pass) {
#pragma unroll
                        for (int e = 0; e < IO::KP; ++e) {
                            fq.v[p][e] = (T)0.f; fk.v[p][e] = (T)0.f; fv.v[p][e] = (T)0.f;
                        }
                    }
                }
            }
            IO::to_lds(fq, sQ, L::LDD, tid);
            IO::to_lds(fk, sK, L::LDD, tid);
            IO::to_lds_t(fk, sKt, L::LDC, tid);
            IO::to_lds_t(fv, sVt, L::LDC, tid);
        }
        if (tid < C) {
            const int sg = episode_of(dmask, tid);
            if (DELTA) sBeta[tid] = (nres == 0 || sg == pass) ? raw_to_float<T>(rbeta) : 0.f;
        }
        if (pass != 0) zero_acc<TMS::TPW>(Sacc);  // an episode that starts in the chunk starts from 0
        store_acc_t<T, HD, HD>(Sacc, sS, L::LDD, w, lane);  // sS[dv][dk]
        if (S_chk && pass == 0) {
            T *dst = S_chk + ((int64_t)bh * NC + c) * HD * HD;
#pragma unroll
            for (int j = 0; j < TMS::TPW; ++j) {
                const int dk0 = TMS::mt(w) * 16 + 4 * lg, dv = TMS::nt(w, j) * 16 + li;
                *reinterpret_cast<P4 *>(dst + dv * HD + dk0) =
                    TT<T>::pack(Sacc[j][0], Sacc[j][1], Sacc[j][2], Sacc[j][3]);
            }
        }
        sync_lds();
        MRX_PHASE(1);
        if (pass == nres && c + 1 < NC) prefetch(c + 1);

        // ---- P1: O^T = m . S Q^T (m over columns), A = beta_i (K K^T) strictly lower ----
        using TMO = TileMap<HD, C>;  // O^T: m = dv, n = c
        f32x4 Oacc[TMO::TPW];
        zero_acc<TMO::TPW>(Oacc);
        gemm_nt<T, HD, C, HD>(Oacc, sS, L::LDD, sQ, L::LDD, w, lane);
        using TMA = TileMap<C, C>;
        if (DELTA) {
            f32x4 acc[TMA::TPW];
            zero_acc<TMA::TPW>(acc);
            gemm_nt<T, C, C, HD>(acc, sK, L::LDD, sK, L::LDD, w, lane);
            // lane holds KK[i = n][j = m..m+3]; write sA[i][j] = beta_i KK [j < i, same episode]
#pragma unroll
            for (int j = 0; j < TMA::TPW; ++j) {
                const int m0 = TMA::mt(w) * 16 + 4 * lg, n = TMA::nt(w, j) * 16 + li;
                const float bi = sBeta[n];
                f32x4 r;
#pragma unroll
                for (int e = 0; e < 4; ++e) r[e] = (m0 + e < n) ? bi * acc[j][e] : 0.f;
                *reinterpret_cast<f32x4 *>(sA + n * L::LDA + m0) = r;
            }
        }
        sync_lds();
        MRX_PHASE(2);

        if (DELTA) {
            // ---- P2/P3: Tm = (I + A)^-1 ; sT[i][j] = Tm[i][j] beta_j -----------------
            tri_inverse<C>(sA, L::LDA, w, lane);
            MRX_PHASE(3);
            for (int idx = tid; idx < C * C / 4; idx += NTHREADS) {
                const int i = idx / (C / 4), j = (idx % (C / 4)) * 4;
                const f32x4 t = tri_inverse_get4(sA, L::LDA, i, j);
                *reinterpret_cast<P4 *>(sT + i * L::LDC + j) =
                    TT<T>::pack(t[0] * sBeta[j], t[1] * sBeta[j + 1], t[2] * sBeta[j + 2], t[3] * sBeta[j + 3]);
            }
            sync_lds();
        MRX_PHASE(4);
        }

        // ---- P4: Aqk[i][j] = (q_i . k_j) [j <= i, same episode] ; U = T V ------------
        {
            f32x4 acc[TMA::TPW];
            zero_acc<TMA::TPW>(acc);
            gemm_nt<T, C, C, HD>(acc, sK, L::LDD, sQ, L::LDD, w, lane);  // D[m = j][n = i]
#pragma unroll
            for (int j = 0; j < TMA::TPW; ++j) {
                const int m0 = TMA::mt(w) * 16 + 4 * lg, n = TMA::nt(w, j) * 16 + li;
                float r[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) r[e] = (m0 + e <= n) ? acc[j][e] : 0.f;
                *reinterpret_cast<P4 *>(sAqk + n * L::LDC + m0) = TT<T>::pack(r[0], r[1], r[2], r[3]);
            }
        }
        if (DELTA) {
            using TMU = TileMap<C, HD>;  // U: m = c, n = dv
            f32x4 Uacc[TMU::TPW];
            zero_acc<TMU::TPW>(Uacc);
            gemm_nt<T, C, HD, C>(Uacc, sT, L::LDC, sVt, L::LDC, w, lane);
            sync_lds();  // sQ and sVt are dead, sAqk visible
        MRX_PHASE(5);
            // ---- P5: W^T = K^T T^T -> sW[c][dk] ---------------------------------------
            {
                using TMW = TileMap<HD, C>;  // m = dk, n = c
                f32x4 acc[TMW::TPW];
                zero_acc<TMW::TPW>(acc);
                gemm_nt<T, HD, C, C>(acc, sKt, L::LDC, sT, L::LDC, w, lane);
                store_acc_t<T, HD, C>(acc, sW, L::LDD, w, lane);
            }
            sync_lds();
        MRX_PHASE(6);
            // ---- P6: U' = U - m . W S^T -> sUt[dv][c] -----------------------------------
            {
                f32x4 acc[TMU::TPW];
                zero_acc<TMU::TPW>(acc);
                gemm_nt<T, C, HD, HD>(acc, sW, L::LDD, sS, L::LDD, w, lane);
#pragma unroll
                for (int j = 0; j < TMU::TPW; ++j) Uacc[j] -= acc[j];
                store_acc_t<T, C, HD>(Uacc, sUt, L::LDC, w, lane);
            }
        }
        sync_lds();
        MRX_PHASE(7);

        // ---- P7: O^T += U'^T Aqk^T ; store O ----------------------------------------
        gemm_nt<T, HD, C, C>(Oacc, sUt, L::LDC, sAqk, L::LDC, w, lane);
#pragma unroll
        for (int j = 0; j < TMO::TPW; ++j) {
            const int dv0 = TMO::mt(w) * 16 + 4 * lg, cc = TMO::nt(w, j) * 16 + li;
            if (t0 + cc < Tlen && (nres == 0 || episode_of(dmask, cc) == pass))
                *reinterpret_cast<P4 *>(ob + (int64_t)(t0 + cc) * rs + dv0) =
                    TT<T>::pack(Oacc[j][0], Oacc[j][1], Oacc[j][2], Oacc[j][3]);
        }
        // ---- P8: S^T <- S^T + K^T U'  (only the episode that leaves the chunk) ---------
        if (pass == nres) gemm_nt<T, HD, HD, C>(Sacc, sKt, L::LDC, sUt, L::LDC, w, lane);
        sync_lds();
        MRX_PHASE(8);
        }  // pass
    }

    MRX_WG_END();
    if (S_last) {
#pragma unroll
        for (int j = 0; j < TMS::TPW; ++j) {
            const int dk0 = TMS::mt(w) * 16 + 4 * lg, dv = TMS::nt(w, j) * 16 + li;
            *reinterpret_cast<f32x4 *>(S_last + ((int64_t)bh * HD + dv) * HD + dk0) = Sacc[j];
        }
    }
}

template <typename T, int C, bool DELTA, bool FMAP>
int launch(hipStream_t st, const void *q, const void *k, const void *v, const void *beta,
           const void *done, int done_f32, const void *S0, void *o, void *S_last, void *S_chk,
           int64_t B, int64_t Tlen, int64_t H)
{
    auto kern = chunk_fwd_kernel<T, C, DELTA, FMAP>;
    constexpr int smem = FwdSmem<T, C, DELTA>::total;
    static bool attr_set = false;  // idempotent; a race only repeats the call
    if (!attr_set) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                hipFuncAttributeMaxDynamicSharedMemorySize, smem) != hipSuccess)
            return MRX_ERR_LAUNCH;
        attr_set = true;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)(B * H)), dim3(NTHREADS), smem, st, (const T *)q,
                       (const T *)k, (const T *)v, (const T *)beta, done, done_f32,
                       (const float *)S0, (T *)o, (float *)S_last, (T *)S_chk, (int)Tlen, (int)H);
    return launch_status();
}

int check_common(const void *q, const void *k, const void *v, const void *done, const void *o,
                 const void *S0, const void *S_last, const void *S_chk, int64_t B, int64_t T,
                 int64_t H, int64_t dk, int64_t dv, int dtype, int done_dtype)
{
    if (!q || !k || !v || !done || !o) return MRX_ERR_INVALID_ARG;
    if (B <= 0 || T <= 0 || H <= 0 || dk <= 0 || dv <= 0) return MRX_ERR_INVALID_ARG;
    if (dtype != MRX_F32 && dtype != MRX_BF16) return dtype == MRX_C64 ? MRX_ERR_UNSUPPORTED : MRX_ERR_INVALID_ARG;
    if (done_dtype != MRX_DONE_U8 && done_dtype != MRX_DONE_F32) return MRX_ERR_INVALID_ARG;
    if (dk != HD || dv != HD) return MRX_ERR_UNSUPPORTED;
    if (B * H >= (1ll << 31) || T >= (1ll << 30)) return MRX_ERR_INVALID_ARG;
    if (!aligned(q, 16) || !aligned(k, 16) || !aligned(v, 16) || !aligned(o, 16) || !aligned(S0, 16) ||
        !aligned(S_last, 16) || !aligned(S_chk, 16))
        return MRX_ERR_INVALID_ARG;
    if (done_dtype == MRX_DONE_F32 && !aligned(done, 4)) return MRX_ERR_INVALID_ARG;
    return MRX_OK;
}

}  // namespace

extern "C" int64_t mrx_chunk_size(int dtype) { return dtype == MRX_BF16 ? 64 : (dtype == MRX_F32 ? 32 : 0); }

extern "C" int mrx_linear_attn_fwd(void *stream, const void *q, const void *k, const void *v,
                                   const void *done, const void *S0, void *o, void *S_last,
                                   void *S_chk, int64_t B, int64_t T, int64_t H, int64_t dk,
                                   int64_t dv, int dtype, int done_dtype, int feature_map)
{
    const int rc = check_common(q, k, v, done, o, S0, S_last, S_chk, B, T, H, dk, dv, dtype, done_dtype);
    if (rc != MRX_OK) return rc;
    if (feature_map != MRX_FMAP_NONE && feature_map != MRX_FMAP_ELU1) return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const bool fm = feature_map == MRX_FMAP_ELU1;
    if (dtype == MRX_BF16)
        return fm ? launch<__bf16, 64, false, true>(st, q, k, v, nullptr, done, done_dtype, S0, o, S_last, S_chk, B, T, H)
                  : launch<__bf16, 64, false, false>(st, q, k, v, nullptr, done, done_dtype, S0, o, S_last, S_chk, B, T, H);
    return fm ? launch<float, 32, false, true>(st, q, k, v, nullptr, done, done_dtype, S0, o, S_last, S_chk, B, T, H)
              : launch<float, 32, false, false>(st, q, k, v, nullptr, done, done_dtype, S0, o, S_last, S_chk, B, T, H);
}

extern "C" int mrx_delta_rule_fwd(void *stream, const void *q, const void *k, const void *v,
                                  const void *beta, const void *done, const void *S0, void *o,
                                  void *S_last, void *S_chk, int64_t B, int64_t T, int64_t H,
                                  int64_t dk, int64_t dv, int dtype, int done_dtype)
{
    const int rc = check_common(q, k, v, done, o, S0, S_last, S_chk, B, T, H, dk, dv, dtype, done_dtype);
    if (rc != MRX_OK) return rc;
    if (!beta) return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == MRX_BF16)
        return launch<__bf16, 64, true, false>(st, q, k, v, beta, done, done_dtype, S0, o, S_last, S_chk, B, T, H);
    return launch<float, 32, true, false>(st, q, k, v, beta, done, done_dtype, S0, o, S_last, S_chk, B, T, H);
}
