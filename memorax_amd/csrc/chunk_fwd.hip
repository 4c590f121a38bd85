// Forward of chunked causal linear attention and of the DeltaNet delta rule (WY/UT form).
//
// Per chunk (rows i >= j of the chunk; S = state entering the chunk, d_v x d_k, fp32):
//   linear attention:  U' = V
//   delta rule:        A  = tril(diag(beta) K K^T, -1),  Tm = (I + A)^-1,  T = Tm diag(beta)
//                      W  = T K,  U' = T V - W S^T
//   both:              O  = Q S^T + tril(Q K^T) U' ,   S <- S + U'^T K
//   normalised read-out (linear attention only): z <- z + sum_j K_j,
//                      den_i = max(Q_i . z + sum_{j<=i} (Q K^T)_ij, eps),  O_i <- O_i / den_i
// Episode resets: a chunk that contains resets is processed once per episode ("pass")
// with the rows of all other episodes replaced by zeros *by select*; the episode that
// enters the chunk sees S, later episodes start from 0, and only the episode that
// leaves the chunk updates S.  Inside a pass only the causal mask remains, and a
// non-finite value can never meet a masked-out zero inside a matrix product.
// The state is kept transposed (S^T, d_k x d_v) in MFMA accumulators for the whole
// sequence and re-staged to LDS as a T-typed d_v x d_k tile once per chunk.
#include <type_traits>

#include "chunk_common.h"
#include "delta_tm.h"
#include "la_states.h"
#if MRX_HD == 64
#include "hd32_api.h"
#endif

namespace {
inline namespace MRX_HD_NS {

using namespace mrx;

constexpr int NW = 4;             // waves per workgroup
constexpr int NTHR = 64 * NW;

template <typename T, int C, bool DELTA, bool GATED = false, bool NORM = false> struct FwdSmem {
    static constexpr int PAD = pad_of<T>();
    static constexpr int LDD = HD + PAD;  // tiles with 64 columns
    static constexpr int LDC = C + PAD;   // tiles with C columns
    static constexpr int LDA = C + 4;     // fp32 C x C
    static constexpr int szRD = C * LDD * sizeof(T);   // [C][64]
    static constexpr int szDD = HD * LDD * sizeof(T);  // [64][64]
    static constexpr int szCC = C * LDC * sizeof(T);   // [C][C]
    static constexpr int szA = DELTA ? C * LDA * 4 : 0;
    // region A: fp32 A during the inverse; afterwards Aqk (offset 0) and W (offset szCC)
    static constexpr int szAW = DELTA ? szCC + szRD : szCC;
    static constexpr int szRA = szA > szAW ? szA : szAW;
    static constexpr int oQ = 0;                          // Q [C][dk], later U' [C][dv]
    static constexpr int oK = oQ + szRD;                  // K [C][dk]
    static constexpr int oV = oK + szRD;                  // V [C][dv]  (delta rule: beta_j V_j)
    static constexpr int oBK = oV + szRD;                 // beta_j K_j [C][dk] (delta rule)
    static constexpr int oS = oBK + (DELTA ? szRD : 0);   // S [dv][dk]
    static constexpr int oTm = oS + szDD;                 // Tm [C][C]  (delta rule only)
    static constexpr int oA = oTm + (DELTA ? szCC : 0);
    static constexpr int oBeta = oA + szRA;
    static constexpr int oG = oBeta + C * 4;              // gated: cumulative log-decay G of the chunk rows, then exp(G_last - G)
    static constexpr int oZ = oG + 2 * C * 4;             // z entering the pass, T-typed row of 64 (normalised read-out)
    // normalised read-out: per-row partial sums of squares of the outputs, one slot per feature block of waves
    static constexpr int oSS = oZ + (NORM ? HD * (int)sizeof(T) : 0);
    static constexpr int oO = oSS + (NORM ? TileMap<HD, C, 4>::WM * C * 4 : 0);  // O [C][dv] on its way to memory
    static constexpr int total = oO + szRD;
};

// What the normalised read-out adds to the argument list.
struct NormArgs {
    const float *z0;  // (B,H,64) or null
    float *den;       // (B,T,H): the clamped denominators (residual of the backward call)
    float *z_last;    // (B,H,64) or null
    float *z_chk;     // (B,H,NC,64) or null: z entering each chunk
    float eps;
    float *ss;        // (B,H,T) or null: sum over the value features of the squared (rounded) outputs of each step
};

// PRO (delta rule): the cell's prologue runs on the staged rows -- keys are L2-normalised
// (k / max(|k|, 1e-12), in fp32, then rounded to T) and beta = sigmoid(raw beta).
// TMIN (delta rule): the triangular factors have been computed by delta_tm_kernel and are read from
// Tm_chk like any other input; the kernel then has neither the K K^T product nor the inverse and
// a chunk costs four barriers.  Without it (no Tm_chk buffer given) the inverse runs in here.
// PAR (plain linear attention): one workgroup per chunk (grid.y = chunk) instead of one per sequence.
// S_chk then is an input: slot c holds, in fp32, the state entering chunk c (la_states.h); the
// workgroup forms the chunk's outputs from it and neither updates nor writes any state.
// NARROW (every variant): narrow heads.  Keys and queries are dka wide in memory, values
// and outputs dva (both at most the head dim of the build, whole 16-byte segments), and so are the
// states (B,H,dva,dka) and z (B,H,dka).  Tiles in LDS and registers keep the build's width: what lies
// beyond the rows' width is loaded as zero (after the feature map, phi(0) = 1 must not count) and never
// stored.
// MERGE (delta rule with TMIN): a chunk that holds resets is done in ONE unit instead of one per episode.  The
// episodes are kept apart by masks on the three places where they could meet -- Q K^T (pairs of one episode
// only), the terms with the state entering the chunk (rows of the first episode only) and the state update
// (rows of the last episode only) -- and the triangular factor arrives block diagonal by episode.  A masked
// zero then multiplies values of other episodes inside the products, which is exact as long as those
// values are finite, so the chunk is screened first: every input of the chunk at most MERGE_IN_MAX in
// magnitude and the state at most MERGE_STATE_MAX (bounds under which no intermediate of the chunk can
// leave the float32 range, so a non-finite value cannot arise either), else the chunk takes the units
// per episode, whose zeros are put in by select.  Results equal those of the units per episode.
template <typename T, int C, bool DELTA, bool FMAP, bool GATED, bool NORM, bool PRO = false, bool TMIN = false,
          bool PAR = false, bool NARROW = false, bool MERGE = false>
__global__ void __launch_bounds__(NTHR, 2)  // 2 waves per SIMD: two workgroups share a CU
chunk_fwd_kernel(const T *__restrict__ q, const T *__restrict__ k, const T *__restrict__ v,
                 const T *__restrict__ beta, const float *__restrict__ glog,
                 const void *__restrict__ done, int done_f32,
                 const float *__restrict__ S0, T *__restrict__ o, float *__restrict__ S_last,
                 void *__restrict__ S_chk, T *__restrict__ Tm_chk, int Tlen, int H, NormArgs na, int dka, int dva)
{
    static_assert(!(DELTA && GATED), "the gated variant is linear attention with a decay");
    static_assert(!NORM || (!DELTA && !GATED), "the normalised read-out belongs to plain linear attention");
    static_assert(!PRO || DELTA, "the prologue belongs to the delta rule");
    static_assert(!TMIN || (DELTA && C == 32), "precomputed factors belong to the delta rule's 32-row chunks");
    static_assert(!PAR || (!DELTA && !GATED && !NORM), "one workgroup per chunk: plain linear attention only");
    static_assert(!MERGE || (TMIN && !NARROW), "merged episodes: the delta rule on precomputed factors, full-width heads");
    using IOT = TileIO<T, C, NTHR, C>;  // the [C][C] triangular factor
    using L = FwdSmem<T, C, DELTA, GATED, NORM>;
    using Frag = typename TT<T>::frag;
    using IO = TileIO<T, C, NTHR>;
    using P4 = typename TT<T>::pack4;
    constexpr int LDD = L::LDD, LDC = L::LDC, LDA = L::LDA;
    extern __shared__ __align__(16) unsigned char smem[];
    T *sQ = reinterpret_cast<T *>(smem + L::oQ);
    T *sK = reinterpret_cast<T *>(smem + L::oK);
    T *sV = reinterpret_cast<T *>(smem + L::oV);    // delta rule: holds beta_j V_j
    T *sBK = reinterpret_cast<T *>(smem + L::oBK);
    T *sS = reinterpret_cast<T *>(smem + L::oS);
    T *sTm = reinterpret_cast<T *>(smem + L::oTm);
    float *sA = reinterpret_cast<float *>(smem + L::oA);
    T *sAqk = reinterpret_cast<T *>(smem + L::oA);
    T *sW = reinterpret_cast<T *>(smem + L::oA + L::szCC);
    T *sU = sV;                                      // U' [C][dv] (delta rule: over beta V once U is taken)
    float *sBeta = reinterpret_cast<float *>(smem + L::oBeta);
    float *sG = reinterpret_cast<float *>(smem + L::oG);
    float *sEb = sG + C;                             // gated: b_j = exp(G_last - G_j)
    T *sZ = reinterpret_cast<T *>(smem + L::oZ);
    float *sSS = reinterpret_cast<float *>(smem + L::oSS);
    T *sO = reinterpret_cast<T *>(smem + L::oO);

    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    const int bh = sequence_of_block(blockIdx.x, gridDim.x, H), b = bh / H, h = bh % H;
    const int dkw = NARROW ? dka : HD, dvw = NARROW ? dva : HD;  // row widths in memory
    const int64_t rs = (int64_t)H * dkw;   // row stride of q/k
    const int64_t rsv = (int64_t)H * dvw;  // ... of v/o
    const int64_t base = ((int64_t)b * Tlen * H + h) * dkw, basev = ((int64_t)b * Tlen * H + h) * dvw;
    const bool segk = !NARROW || (tid % (HD / TT<T>::KP)) * TT<T>::KP < dkw;  // this thread's 16-byte segment lies inside a q/k row
    const bool segv = !NARROW || (tid % (HD / TT<T>::KP)) * TT<T>::KP < dvw;  // ... inside a v row
    const int NC = (Tlen + C - 1) / C;
    const int c_first = PAR ? (int)blockIdx.y : 0, c_end = PAR ? c_first + 1 : NC;  // the chunks this workgroup walks

    using TMS = TileMap<HD, HD, NW>;  // S^T : m = dk, n = dv
    using TMO = TileMap<HD, C, NW>;   // X^T : m = feature, n = chunk row
    using TMA = TileMap<C, C, NW>;
    using TMK = TileMap<C, C, NW, 1>;  // K K^T: a row of tiles per wave, so that every wave owns one diagonal tile
    f32x4 Sacc[TMS::TPW];
#pragma unroll
    for (int j = 0; j < TMS::TPW; ++j) {
        const int dk0 = TMS::mt(w, j) * 16 + 4 * lg, dv = TMS::nt(w, j) * 16 + li;
        const bool in = !NARROW || (dv < dvw && dk0 < dkw);
        Sacc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (PAR) {
            if (in) Sacc[j] = *reinterpret_cast<const f32x4 *>(reinterpret_cast<const float *>(S_chk) +
                                                              (((int64_t)bh * NC + c_first) * dvw + dv) * dkw + dk0);
        } else if (S0 && in) {
            Sacc[j] = *reinterpret_cast<const f32x4 *>(S0 + ((int64_t)bh * dvw + dv) * dkw + dk0);
        }
    }

    // normalised read-out: z[dk] of the running episode.  bf16: held like a column of S^T (every
    // lane of a 16-lane group carries the same four dk = 4 lg + v of each of the wave's m-tiles) and
    // maintained with MFMAs on a tile of ones.  fp32 (VN): a 16x16x4 MFMA per four terms of a row
    // sum is a bad trade, so the sums run on the vector ALU over the same fragments and component 0
    // holds z[dk = 16 mt + li] (every lane group the same).
    constexpr bool VN = sizeof(T) == 4;
    f32x4 zacc[TMS::MBW];
#pragma unroll
    for (int mi = 0; mi < TMS::MBW; ++mi) {
        const int dkt = TMS::mt(w, mi * TMS::NBW) * 16;
        zacc[mi] = f32x4{0.f, 0.f, 0.f, 0.f};
        if (NORM && na.z0) {
            if (VN) { if (!NARROW || dkt + li < dkw) zacc[mi][0] = na.z0[(int64_t)bh * dkw + dkt + li]; }
            else if (!NARROW || dkt + 4 * lg < dkw) zacc[mi] = *reinterpret_cast<const f32x4 *>(na.z0 + (int64_t)bh * dkw + dkt + 4 * lg);
        }
    }
    const Frag ones = TT<T>::ones();
    int64_t den_off = (int64_t)bh * Tlen + c_first * C + li;  // den[b][h][t0 + li]: contiguous in time per sequence

    // register prefetch of the next chunk (raw bits only: no arithmetic on in-flight loads)
    typename IO::Regs rq, rk, rv;
    uint32_t rbeta = 0u, rdone = 0u;
    float rg = 0.f;  // log-decay of chunk row `lane` (gated)
    uint32_t rbrow[IO::PASSES];  // beta of the rows this thread stages
    // Element offsets of what this thread loads for the chunk about to be prefetched; they advance
    // by one chunk per call (64-bit adds instead of per-chunk index multiplications).
    int64_t roff[IO::PASSES], boff[IO::PASSES];
    int64_t roffv[NARROW ? IO::PASSES : 1];  // v, where its rows are not as wide as those of q and k
#pragma unroll
    for (int p = 0; p < IO::PASSES; ++p) {
        const int r = IO::row_of(tid, p);
        roff[p] = base + (int64_t)(c_first * C + r) * rs + (tid % IO::SEGS) * IO::KP;  // q/k/v: row r, this thread's 16-byte segment
        if (NARROW) roffv[p] = basev + (int64_t)(c_first * C + r) * rsv + (tid % IO::SEGS) * IO::KP;
        boff[p] = ((int64_t)b * Tlen + c_first * C + r) * H + h;                       // beta of row r
    }
    int64_t doff = (int64_t)b * Tlen + c_first * C + lane;  // done of chunk row `lane`
    int tpre = c_first * C;                                 // first time step of the chunk about to be prefetched
    typename IOT::Regs rTm;                   // TMIN: the factor of the chunk about to be staged
    int64_t tmoff = (int64_t)bh * ((Tlen + C - 1) / C) * C * C + (tid / IOT::SEGS) * C + (tid % IOT::SEGS) * IOT::KP;
    // The prefetch is issued in parts spread over the first phases, so that the address unit works
    // through the loads beside LDS and MFMA work.  part 0: q, 1: k, 2: v, 3: per-row scalars.
    auto prefetch_part = [&](int part) {
        typename IO::F z;
#pragma unroll
        for (int e = 0; e < IO::KP; ++e) z[e] = (T)0.f;
        if (part < 3) {
            const T *src = part == 0 ? q : part == 1 ? k : v;
            typename IO::Regs &dst = part == 0 ? rq : part == 1 ? rk : rv;
            const bool seg_in = part == 2 ? segv : segk;
#pragma unroll
            for (int p = 0; p < IO::PASSES; ++p)
                dst.v[p] = seg_in && (IO::FULL || IO::row_of(tid, p) < C) && tpre + IO::row_of(tid, p) < Tlen
                               ? *reinterpret_cast<const typename IO::F *>(src + (NARROW && part == 2 ? roffv[p] : roff[p])) : z;
        } else {
#pragma unroll
            for (int p = 0; p < IO::PASSES; ++p) {
                if (DELTA) rbrow[p] = (IO::FULL || IO::row_of(tid, p) < C) && tpre + IO::row_of(tid, p) < Tlen ? load_raw<T>(beta + boff[p]) : 0u;
                roff[p] += (int64_t)C * rs;
                if (NARROW) roffv[p] += (int64_t)C * rsv;
                boff[p] += (int64_t)C * H;
            }
            if (TMIN) {
#pragma unroll
                for (int p = 0; p < IOT::PASSES; ++p)
                    if (IOT::FULL || IOT::row_of(tid, p) < C)  // a [C][C] tile may have fewer segments than threads
                        rTm.v[p] = *reinterpret_cast<const typename IOT::F *>(Tm_chk + tmoff + p * IOT::RPP * C);
                tmoff += C * C;
            }
            rdone = 0u;
            rbeta = 0u;
            rg = 0.f;
            if (lane < C && tpre + lane < Tlen) {
                rdone = done_raw(done, done_f32, doff);
                if (DELTA && !TMIN && w == 0) rbeta = load_raw<T>(beta + doff * H + h);
                if (GATED) rg = glog[doff * H + h];
            }
            doff += C;
            tpre += C;
        }
    };
#pragma unroll
    for (int part = 0; part < 4; ++part) prefetch_part(part);
    if (DELTA && !TMIN) {
        // blocks above the block diagonal of Tm are never written again
        for (int idx = tid; idx < C * LDC * (int)sizeof(T) / 4; idx += NTHR) reinterpret_cast<uint32_t *>(sTm)[idx] = 0u;
    }

    static_assert(C * C / 4 % NTHR == 0, "Tm tile copy assumes whole passes");
    // running element offsets of this thread's stores, advanced by one chunk per iteration
    unsigned long long pend_dmask = 0ull;  // the unit whose output waits in sO
    int pend_nres = 0, pend_pass = 0, pend_t0 = -1;
    auto flush_o = [&]() {  // call after a barrier that follows the writes to sO
        if (pend_t0 >= 0) {
            auto keep = [&](int r) { return pend_nres == 0 || episode_of(pend_dmask, r) == pend_pass; };
            tile_rows_to_global<T, C, NTHR>(sO, LDD, o + basev + (int64_t)pend_t0 * rsv, rsv, pend_t0, Tlen, tid, keep, dvw);
        }
        pend_t0 = -1;
    };
    int64_t schk_off = (int64_t)bh * NC * dvw * dkw;                                 // S_chk[c]
    int64_t tmchk_off = (int64_t)bh * NC * C * C + (int64_t)tid * 4;                                  // row-major C x C
    for (int c = c_first; c < c_end; ++c, schk_off += dvw * dkw, tmchk_off += C * C, den_off += C) {
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
                             small((float)rv.v[p][e], MERGE_IN_MAX);
                    ok = ok && small(raw_to_float<T>(rbrow[p]), MERGE_IN_MAX);
                }
#pragma unroll
                for (int p = 0; p < IOT::PASSES; ++p)
                    if (IOT::FULL || IOT::row_of(tid, p) < C) {
#pragma unroll
                        for (int e = 0; e < IOT::KP; ++e) ok = ok && small((float)rTm.v[p][e], MERGE_IN_MAX);
                    }
#pragma unroll
                for (int j = 0; j < TMS::TPW; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e) ok = ok && small(Sacc[j][e], MERGE_STATE_MAX);
                // sBeta is free in this variant (the factors arrive ready): one flag per wave
                if (lane == 0) sBeta[w] = __ballot(!ok) != 0ull ? 1.f : 0.f;
                sync_lds();
                mg = sBeta[0] + sBeta[1] + sBeta[2] + sBeta[3] == 0.f;
            }
        }
        const int npass = mg ? 0 : nres;
        const int r_first = mg ? (int)__builtin_ctzll(dmask) : C;        // rows below it: the episode that enters the chunk
        const int r_last = mg ? 63 - (int)__builtin_clzll(dmask) : 0;   // rows from it on: the episode that leaves it
        for (int pass = 0; pass <= npass; ++pass) {
            auto live = [&](int r) { return nres == 0 || mg || episode_of(dmask, r) == pass; };
            // gated: G_i = sum of the log-decays of this pass's episode up to row i (the decay of an
            // episode's first step multiplies a zero state and is left out); every wave scans its copy
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
                    sEb[lane] = __expf(Glast - G);
                }
            }
            // ---- stage the chunk ---------------------------------------------------
            {
                typename IO::Regs fq = rq, fk = rk, fv = rv;
                if (segk) {  // columns beyond a narrow head's width stay zero: phi(0) = 1 must not count
                    IO::template fmap<FMAP>(fq);
                    IO::template fmap<FMAP>(fk);
                }
                if (nres != 0 && !mg) {
                    IO::mask_rows(fq, tid, live);
                    IO::mask_rows(fk, tid, live);
                    IO::mask_rows(fv, tid, live);
                }
                if (PRO) {
                    float kinv[IO::PASSES];
#pragma unroll
                    for (int p = 0; p < IO::PASSES; ++p) {
                        float ss = 0.f;
#pragma unroll
                        for (int e = 0; e < IO::KP; ++e) ss += (float)fk.v[p][e] * (float)fk.v[p][e];
                        kinv[p] = inv_norm(seg_sum<IO::SEGS>(ss));
                    }
                    IO::scale_rows(fk, kinv);
                }
                // rows past the end of the sequence: phi(0) = 1 must not count towards z
                if (NORM && FMAP && t0 + C > Tlen) IO::mask_rows(fk, tid, [&](int r) { return t0 + r < Tlen; });
                IO::to_lds(fq, sQ, LDD, tid);
                IO::to_lds(fk, sK, LDD, tid);
                if (DELTA) {
                    float bf[IO::PASSES];
#pragma unroll
                    for (int p = 0; p < IO::PASSES; ++p)
                        bf[p] = !live(IO::row_of(tid, p)) ? 0.f  // by select: a NaN gate of another episode must not meet a zeroed row
                            : PRO ? sigmoidf(raw_to_float<T>(rbrow[p])) : raw_to_float<T>(rbrow[p]);
                    IO::scale_rows(fk, bf);
                    IO::scale_rows(fv, bf);
                    IO::to_lds(fk, sBK, LDD, tid);
                }
                IO::to_lds(fv, sV, LDD, tid);
            }
            if (DELTA && !TMIN && tid < C)
                sBeta[tid] = !live(tid) ? 0.f : PRO ? sigmoidf(raw_to_float<T>(rbeta)) : raw_to_float<T>(rbeta);
            if (TMIN) {
                // rows of other episodes are cleared by select: they only ever meet zeros, but a NaN key
                // or gate of another episode sits in them
                typename IOT::Regs fTm = rTm;
                if (nres != 0 && !mg) IOT::mask_rows(fTm, tid, live);
                IOT::to_lds(fTm, sTm, LDC, tid);
            }
            if (pass != 0) zero_acc<TMS::TPW>(Sacc);  // an episode that starts in the chunk starts from 0
            store_acc<T, HD, HD, NW>(Sacc, sS, LDD, w, lane);  // sS[dv][dk]
            if (NORM) {
                if (pass != 0) zero_acc<TMS::MBW>(zacc);
                if (w < TMS::WM && (VN ? lg == 0 : li == 0)) {
#pragma unroll
                    for (int mi = 0; mi < TMS::MBW; ++mi) {
                        const int dkt = TMS::mt(w, mi * TMS::NBW) * 16;
                        float *zc = (na.z_chk && pass == 0) ? na.z_chk + ((int64_t)bh * NC + c) * dkw + dkt : nullptr;
                        if (VN) {
                            sZ[dkt + li] = (T)zacc[mi][0];
                            if (zc && (!NARROW || dkt + li < dkw)) zc[li] = zacc[mi][0];
                        } else {
                            *reinterpret_cast<P4 *>(sZ + dkt + 4 * lg) = TT<T>::pack(zacc[mi][0], zacc[mi][1], zacc[mi][2], zacc[mi][3]);
                            if (zc && (!NARROW || dkt + 4 * lg < dkw)) *reinterpret_cast<f32x4 *>(zc + 4 * lg) = zacc[mi];
                        }
                    }
                }
            }
            sync_lds();
            // Outputs leave through LDS as whole rows (an accumulator tile would write 16 pieces of
            // 32 bytes per instruction): the output of the previous unit, parked in sO at its end, and
            // the state checkpoint from the copy of S that has just been staged.
            flush_o();
            // Plain and normalised linear attention: the backward call walks the state back from chunk to
            // chunk in fp32, starting from S_last (S_c = S_{c+1} - V_c^T K_c undoes a chunk's update), so a
            // checkpoint is written only where that walk cannot pass: for a chunk with resets, whose entering
            // state the state that leaves it does not determine.  Those are written in fp32 from the
            // accumulators (rare; the walk carries their rounding to the chunks before), as is every
            // walk_anchor()-th chunk, where the walk starts afresh from the exact state.  The decayed update
            // of the gated variant is not undone (it would divide by the decay), and for the delta rule the
            // walk needs U' as a residual and an extra product, which measured slower than reading the
            // states: there every chunk is written, in the I/O type, from the copy of S just staged.
            constexpr bool DENSE_CHK = GATED || DELTA;
            if (!PAR && S_chk && pass == 0 && (DENSE_CHK || nres != 0 || (c > 0 && c % walk_anchor<T>() == 0))) {
                if (DENSE_CHK) {
                    using IOS = TileIO<T, HD, NTHR>;
#pragma unroll
                    for (int p = 0; p < IOS::PASSES; ++p) {
                        const int r = IOS::row_of(tid, p), seg = tid % IOS::SEGS;
                        if ((IOS::FULL || r < HD) && (!NARROW || (r < dvw && seg * IOS::KP < dkw)))  // a [32][32] tile has fewer segments than threads
                            *reinterpret_cast<typename IOS::F *>(reinterpret_cast<T *>(S_chk) + schk_off + r * dkw + seg * IOS::KP) =
                                *reinterpret_cast<const typename IOS::F *>(sS + r * LDD + seg * IOS::KP);
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < TMS::TPW; ++j) {
                        const int dk0 = TMS::mt(w, j) * 16 + 4 * lg, dv = TMS::nt(w, j) * 16 + li;
                        if (!NARROW || (dv < dvw && dk0 < dkw))
                            *reinterpret_cast<f32x4 *>(reinterpret_cast<float *>(S_chk) + schk_off + dv * dkw + dk0) = Sacc[j];
                    }
                }
            }
            const bool pre = pass == npass && c + 1 < c_end;
            if (pre) { prefetch_part(0); prefetch_part(1); }
            if (TMIN && pre) { prefetch_part(2); prefetch_part(3); }
            // ---- A[i][j] = beta_i (k_i . k_j), j < i ----------------------------------
            if (DELTA && !TMIN) {
                f32x4 acc[TMK::TPW];
                zero_acc<TMK::TPW>(acc);
                gemm<T, C, C, HD, ROWK, ROWK, NW, 1>(acc, sK, LDD, sK, LDD, w, lane);  // D[m = j][n = i]
                // sA[i][j] = beta_i (k_i . k_j) for j < i, else 0 (beta read once per tile, then selects)
#pragma unroll
                for (int j = 0; j < TMK::TPW; ++j) {
                    const int m = TMK::mt(w, j) * 16 + 4 * lg, n = TMK::nt(w, j) * 16 + li;
                    const float bn = sBeta[n];
                    f32x4 a;
#pragma unroll
                    for (int e = 0; e < 4; ++e) a[e] = (m + e < n) ? bn * acc[j][e] : 0.f;
                    *reinterpret_cast<f32x4 *>(sA + n * LDA + m) = a;
                }
                // the wave that holds the diagonal tile (b, b) inverts that block from registers
                int diag = -1;
                f32x4 kk = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < TMK::TPW; ++j)
                    if (TMK::nt(w, j) == TMK::mt(w, j)) { diag = TMK::mt(w, j); kk = acc[j]; }
                f32x4 Xcc = {0.f, 0.f, 0.f, 0.f};
                if (diag >= 0) Xcc = tri_diag_block<T>(kk, sBeta, diag, sA, LDA, sTm, LDC, lane);
                sync_lds();
                if (pre) { prefetch_part(2); prefetch_part(3); }
                if (diag >= 0) tri_block_column<C, T>(sA, LDA, sTm, LDC, diag, Xcc, lane);
                sync_lds();
            }
            // ---- Aqk[i][j] = (q_i . k_j), j <= i ; delta rule: W = Tm (beta K), U = Tm (beta V) ----
            {
                f32x4 acc[TMA::TPW];
                zero_acc<TMA::TPW>(acc);
                gemm<T, C, C, HD, ROWK, ROWK, NW>(acc, sK, LDD, sQ, LDD, w, lane);  // D[m = j][n = i]
                if (GATED) {
                    // Aqk[i][j] = exp(G_i - G_j) (q_i . k_j), j <= i (exponent <= 0 for log-decays <= 0)
#pragma unroll
                    for (int j = 0; j < TMA::TPW; ++j) {
                        const int m = TMA::mt(w, j) * 16 + 4 * lg, n = TMA::nt(w, j) * 16 + li;
                        const float gn = sG[n];
                        const f32x4 gm = *reinterpret_cast<const f32x4 *>(sG + m);
                        float x[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) x[e] = (m + e <= n) ? acc[j][e] * __expf(gn - gm[e]) : 0.f;
                        *reinterpret_cast<P4 *>(sAqk + n * LDC + m) = TT<T>::pack(x[0], x[1], x[2], x[3]);
                    }
                } else if (MERGE && mg) {
                    // pairs (i = n, j = m <= n) of one episode only: no reset in rows m + 1 .. n
                    store_acc_f<T, C, C, NW>(acc, sAqk, LDC, w, lane, [&](int m, int n, float x) {
                        return m <= n && (dmask & ((2ull << n) - (2ull << m))) == 0ull ? x : 0.f;
                    });
                } else {
                    store_acc_f<T, C, C, NW>(acc, sAqk, LDC, w, lane,
                                             [](int m, int n, float x) { return m <= n ? x : 0.f; });
                }
            }
            if (DELTA) {
                f32x4 Uacc[TMO::TPW];
                zero_acc<TMO::TPW>(Uacc);
                gemm<T, HD, C, C, KROW, ROWK, NW>(Uacc, sV, LDD, sTm, LDC, w, lane);  // U^T[dv][c]
                {
                    f32x4 acc[TMO::TPW];
                    zero_acc<TMO::TPW>(acc);
                    gemm<T, HD, C, C, KROW, ROWK, NW>(acc, sBK, LDD, sTm, LDC, w, lane);  // W^T[dk][c]
                    store_acc<T, HD, C, NW>(acc, sW, LDD, w, lane);
                }
                if (Tm_chk && !TMIN) {
                    // residual for the backward call: the rows of this pass's episode (rows past
                    // the end of the sequence count as the last episode: identity rows)
#pragma unroll
                    for (int it = 0; it < C * C / 4 / NTHR; ++it) {
                        const int idx = tid + it * NTHR, i = idx / (C / 4), j = (idx % (C / 4)) * 4;
                        if (live(i))
                            *reinterpret_cast<P4 *>(Tm_chk + tmchk_off + it * NTHR * 4) =
                                *reinterpret_cast<const P4 *>(sTm + i * LDC + j);
                    }
                }
                sync_lds();  // sW, sAqk visible; every wave is done with beta V
                // U'^T[dv][c] = U^T - S W^T -> sU[c][dv] (over beta V)
                {
                    f32x4 acc[TMO::TPW];
                    zero_acc<TMO::TPW>(acc);
                    gemm<T, HD, C, HD, ROWK, ROWK, NW>(acc, sS, LDD, sW, LDD, w, lane);
#pragma unroll
                    for (int j = 0; j < TMO::TPW; ++j) {
                        // merged episodes: only the rows of the episode that entered the chunk see its state
                        if (!(MERGE && mg) || TMO::nt(w, j) * 16 + li < r_first) Uacc[j] -= acc[j];
                    }
                    store_acc<T, HD, C, NW>(Uacc, sU, LDD, w, lane);
                }
            }
            sync_lds();
            // ---- O^T[dv][i] = sum_dk S[dv][dk] Q[i][dk] + sum_j U'[j][dv] Aqk[i][j] ; store O -------
            if (!DELTA && pre) { prefetch_part(2); prefetch_part(3); }
            f32x4 Oacc[TMO::TPW];
            zero_acc<TMO::TPW>(Oacc);
            // normalised read-out: den_i = Q_i . z + sum_j Aqk[i][j], taken from the Q and Aqk
            // fragments the two products load anyway (z as a tile of equal rows, a tile of ones)
            f32x4 dacc[TMO::NBW];
            zero_acc<TMO::NBW>(dacc);
            auto den_q = [&](int ni, int kb, const Frag &yq) {
                if (!NORM) return;
                const Frag zf = TT<T>::template load<ROWK>(sZ, 0, 0, kb * TT<T>::KB, lane);  // z[k], the lane's k slots
                if (VN) {
#pragma unroll
                    for (int e = 0; e < TT<T>::KP; ++e) dacc[ni][0] += (float)zf[e] * (float)yq[e];
                } else {
                    dacc[ni] = TT<T>::mma(zf, yq, dacc[ni]);
                }
            };
            auto den_a = [&](int ni, int, const Frag &ya) {
                if (!NORM) return;
                if (VN) {
#pragma unroll
                    for (int e = 0; e < TT<T>::KP; ++e) dacc[ni][0] += (float)ya[e];
                } else {
                    dacc[ni] = TT<T>::mma(ones, ya, dacc[ni]);
                }
            };
            gemm<T, HD, C, HD, ROWK, ROWK, NW>(Oacc, sS, LDD, sQ, LDD, w, lane, NoHook(), den_q);
            if (MERGE && mg) {
#pragma unroll
                for (int j = 0; j < TMO::TPW; ++j)
                    if (TMO::nt(w, j) * 16 + li >= r_first) Oacc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
            if (GATED) {  // the incoming state reaches row i decayed by exp(G_i)
#pragma unroll
                for (int j = 0; j < TMO::TPW; ++j) Oacc[j] *= __expf(sG[TMO::nt(w, j) * 16 + li]);
            }
            gemm<T, HD, C, C, KROW, ROWK, NW>(Oacc, sU, LDD, sAqk, LDC, w, lane, NoHook(), den_a);
            if (NORM) {
                if (VN) {  // the lane groups hold partial sums over their k slots
#pragma unroll
                    for (int ni = 0; ni < TMO::NBW; ++ni) {
                        float x = dacc[ni][0];
                        x += __shfl_xor(x, 16);
                        x += __shfl_xor(x, 32);
                        dacc[ni][0] = x;
                    }
                }
#pragma unroll
                for (int j = 0; j < TMO::TPW; ++j) {
                    const int cc = TMO::nt(w, j) * 16 + li;
                    const float den = fmaxf(dacc[j % TMO::NBW][0], na.eps);
                    Oacc[j] *= 1.f / den;
                    if (t0 + cc < Tlen && live(cc) && TMO::mt(w, j) == 0 && lg == 0)
                        na.den[den_off + TMO::nt(w, j) * 16] = den;
                }
            }
            store_acc<T, HD, C, NW>(Oacc, sO, LDD, w, lane);  // to memory once the next unit has been staged
            if (NORM && na.ss) {
                // sum of squares of each output row as it is stored (rounded to T), for an RMS norm over the
                // heads that follows the read-out (linear_attention.py:114): the wave's feature tiles, the four
                // lane groups, then one slot per feature block of waves; summed after the unit's last barrier
                float sq[TMO::NBW];
#pragma unroll
                for (int ni = 0; ni < TMO::NBW; ++ni) sq[ni] = 0.f;
#pragma unroll
                for (int j = 0; j < TMO::TPW; ++j) {
                    const P4 r4 = TT<T>::pack(Oacc[j][0], Oacc[j][1], Oacc[j][2], Oacc[j][3]);
#pragma unroll
                    for (int e = 0; e < 4; ++e) sq[j % TMO::NBW] += (float)r4[e] * (float)r4[e];
                }
#pragma unroll
                for (int ni = 0; ni < TMO::NBW; ++ni) {
                    float x = sq[ni];
                    x += __shfl_xor(x, 16);
                    x += __shfl_xor(x, 32);
                    if (lg == 0) sSS[(w % TMO::WM) * C + TMO::nt(w, ni) * 16 + li] = x;
                }
            }
            pend_dmask = dmask;
            pend_nres = mg ? 0 : nres;
            pend_pass = pass;
            pend_t0 = t0;
            // ---- S^T[dk][dv] += sum_c K[c][dk] U'[c][dv]  (only the episode that leaves the chunk)
            if (pass == npass && !PAR) {
                if (MERGE && mg) zero_acc<TMS::TPW>(Sacc);  // a chunk with resets: the state that leaves is the last episode's own
                if (GATED) {  // S <- exp(G_last) S + sum_c exp(G_last - G_c) K[c] U'[c]
                    const float cl = __expf(Glast);
#pragma unroll
                    for (int j = 0; j < TMS::TPW; ++j) Sacc[j] *= cl;
                }
                float zpart[TMS::MBW];  // fp32: per-lane partial column sums of K over the lane's k slots
#pragma unroll
                for (int mi = 0; mi < TMS::MBW; ++mi) zpart[mi] = 0.f;
                auto z_k = [&](int mi, int kb, Frag &xk) {
                    if (NORM) {  // z[dk] += sum_c K[c][dk]
                        if (VN) {
#pragma unroll
                            for (int e = 0; e < TT<T>::KP; ++e) zpart[mi] += (float)xk[e];
                        } else {
                            zacc[mi] = TT<T>::mma(xk, ones, zacc[mi]);
                        }
                    }
                    if (GATED) {  // row c of K enters the state update as b_c K[c]: scale the fragment along k
                        const float *eb = sEb + kb * TT<T>::KB + TT<T>::KP * lg;
#pragma unroll
                        for (int e = 0; e < TT<T>::KP; ++e) xk[e] = (T)((float)xk[e] * eb[e]);
                    }
                    if (MERGE && mg) {  // rows of the last episode only (element e of the fragment is chunk row k0 + e)
                        const int k0 = kb * TT<T>::KB + TT<T>::KP * lg;
#pragma unroll
                        for (int e = 0; e < TT<T>::KP; ++e)
                            if (k0 + e < r_last) xk[e] = (T)0.f;
                    }
                };
                gemm<T, HD, HD, C, KROW, KROW, NW>(Sacc, sK, LDD, sU, LDD, w, lane, z_k);
                if (NORM && VN) {
#pragma unroll
                    for (int mi = 0; mi < TMS::MBW; ++mi) {
                        float x = zpart[mi];
                        x += __shfl_xor(x, 16);
                        x += __shfl_xor(x, 32);
                        zacc[mi][0] += x;
                    }
                }
            }
            sync_lds();
            if (NORM && na.ss && tid < C && t0 + tid < Tlen && live(tid)) {
                float x = 0.f;
#pragma unroll
                for (int sl = 0; sl < TMO::WM; ++sl) x += sSS[sl * C + tid];
                na.ss[(int64_t)bh * Tlen + t0 + tid] = x;  // the slots are next written after the next unit's barriers
            }
        }
    }
    flush_o();  // the last unit ended with a barrier

    if (S_last && !PAR) {
#pragma unroll
        for (int j = 0; j < TMS::TPW; ++j) {
            const int dk0 = TMS::mt(w, j) * 16 + 4 * lg, dv = TMS::nt(w, j) * 16 + li;
            if (!NARROW || (dv < dvw && dk0 < dkw))
                *reinterpret_cast<f32x4 *>(S_last + ((int64_t)bh * dvw + dv) * dkw + dk0) = Sacc[j];
        }
    }
    if (NORM && na.z_last && w < TMS::WM && (VN ? lg == 0 : li == 0)) {
#pragma unroll
        for (int mi = 0; mi < TMS::MBW; ++mi) {
            const int dkt = TMS::mt(w, mi * TMS::NBW) * 16;
            float *zl = na.z_last + (int64_t)bh * dkw + dkt;
            if (VN) { if (!NARROW || dkt + li < dkw) zl[li] = zacc[mi][0]; }
            else if (!NARROW || dkt + 4 * lg < dkw) *reinterpret_cast<f32x4 *>(zl + 4 * lg) = zacc[mi];
        }
    }
}

template <typename T, int C, bool DELTA, bool FMAP, bool GATED, bool NORM, bool PRO, bool TMIN, bool PAR, bool NARROW, bool MERGE> struct FwdReg {
    static constexpr int smem = FwdSmem<T, C, DELTA, GATED, NORM>::total;
    static inline KernelRegistrar reg{
        reinterpret_cast<const void *>(chunk_fwd_kernel<T, C, DELTA, FMAP, GATED, NORM, PRO, TMIN, PAR, NARROW, MERGE>), smem};
};

// dka, dva: widths of the q/k and v/o rows in memory; less than the build's head dim (narrow heads)
// selects the kernel instance that pads on the fly.
template <typename T, int C, bool DELTA, bool FMAP, bool GATED = false, bool NORM = false, bool PRO = false,
          bool TMIN = false, bool PAR = false, bool MERGE = false>
int launch(hipStream_t st, const void *q, const void *k, const void *v, const void *beta,
           const void *done, int done_f32, const void *S0, void *o, void *S_last, void *S_chk,
           void *Tm_chk, int64_t B, int64_t Tlen, int64_t H, const void *glog = nullptr, NormArgs na = NormArgs{},
           int64_t dka = HD, int64_t dva = HD)
{
    if (const int rc = prepare_device(); rc != MRX_OK) return rc;
    const int64_t NC = (Tlen + C - 1) / C;
    if (PAR && NC > 65535) return MRX_ERR_INVALID_ARG;
    auto go = [&](auto narrow) {
        constexpr bool NARROW = decltype(narrow)::value;
        constexpr bool MG = MERGE && !NARROW;  // narrow heads keep the units per episode
        using Reg = FwdReg<T, C, DELTA, FMAP, GATED, NORM, PRO, TMIN, PAR, NARROW, MG>;
        (void)&Reg::reg;  // the kernel is on the list mrx_init() walks
        return launch_kernel(chunk_fwd_kernel<T, C, DELTA, FMAP, GATED, NORM, PRO, TMIN, PAR, NARROW, MG>,
                             dim3((unsigned)(B * H), PAR ? (unsigned)NC : 1u), dim3(NTHR), Reg::smem, st, (const T *)q,
                             (const T *)k, (const T *)v, (const T *)beta, (const float *)glog, done, done_f32,
                             (const float *)S0, (T *)o, (float *)S_last, S_chk, (T *)Tm_chk, (int)Tlen, (int)H, na,
                             (int)dka, (int)dva);
    };
    if (dka != HD || dva != HD) return go(std::true_type{});
    return go(std::false_type{});
}

// narrow: the entry point also serves heads narrower than the build's (rows of whole 16-byte segments,
// padded inside the kernels)
int check_common(const void *q, const void *k, const void *v, const void *done, const void *o,
                 const void *S0, const void *S_last, const void *S_chk, int64_t B, int64_t T,
                 int64_t H, int64_t dk, int64_t dv, int dtype, int done_dtype, bool narrow = false)
{
    if (!q || !k || !v || !done || !o) return MRX_ERR_INVALID_ARG;
    if (B <= 0 || T <= 0 || H <= 0 || dk <= 0 || dv <= 0) return MRX_ERR_INVALID_ARG;
    if (dtype != MRX_F32 && dtype != MRX_BF16) return dtype == MRX_C64 ? MRX_ERR_UNSUPPORTED : MRX_ERR_INVALID_ARG;
    if (done_dtype != MRX_DONE_U8 && done_dtype != MRX_DONE_F32) return MRX_ERR_INVALID_ARG;
    const int64_t seg = dtype == MRX_BF16 ? 8 : 4;  // elements per 16 bytes
    const bool narrow_ok = narrow && dk <= HD && dv <= HD && dk % seg == 0 && dv % seg == 0;
    if ((dk != HD || dv != HD) && !narrow_ok) return MRX_ERR_UNSUPPORTED;
    if (B * H >= (1ll << 31) || T >= (1ll << 30)) return MRX_ERR_INVALID_ARG;
    if (!aligned(q, 16) || !aligned(k, 16) || !aligned(v, 16) || !aligned(o, 16) || !aligned(S0, 16) ||
        !aligned(S_last, 16) || !aligned(S_chk, 16))
        return MRX_ERR_INVALID_ARG;
    if (done_dtype == MRX_DONE_F32 && !aligned(done, 4)) return MRX_ERR_INVALID_ARG;
    return MRX_OK;
}

// Two ways to the triangular factors.  With a buffer for them and at most two workgroups per compute
// unit, the chunk-parallel kernel fills the buffer and the sequential kernel reads it: the
// sequential kernel loses half of its per-chunk dependency chain, which is what bounds it while
// the device is not full.  With more sequences than that the device is bound by memory traffic,
// other workgroups hide the inverse, and the second pass over the keys plus the round trip of the
// factors (a fifth more traffic) would only cost: the sequential kernel inverts in place then, as it
// does when there is no buffer.  factor_path (mrx_factor_path) overrides the rule: the reset rate,
// which the host cannot see, moves the break-even point (a chunk with resets repeats the in-kernel
// inverse per episode, the chunk-parallel kernel does that off the sequential path).
template <bool PRO>
int delta_fwd_dispatch(hipStream_t st, const void *q, const void *k, const void *v, const void *beta, const void *done,
                       int done_dtype, const void *S0, void *o, void *S_last, void *S_chk, void *Tm_chk, int64_t B,
                       int64_t T, int64_t H, int dtype, int factor_path, int64_t dk = HD, int64_t dv = HD,
                       int reset_path = MRX_RESETS_AUTO)
{
    // delta_tm_kernel is written for 32-row chunks: a build with 64-row bf16 chunks (the measurement
    // variant, MRX_DELTA_BF16_CHUNK=64) always inverts inside the sequential kernel
    constexpr bool TM_KERNEL = DELTA_BF16_CHUNK == 32;
    int cus = 0;
    if (const int rc = prepare_device(&cus); rc != MRX_OK) return rc;
    // fp32: the in-kernel inverse is the longer part of a chunk's chain at any occupancy (measured on
    // full devices, 1024 to 8192 sequences: 8 % faster with the chunk-parallel kernel), so the rule by
    // occupancy is the bf16 kernels' only
    const bool parallel = Tm_chk && factor_path != MRX_FACTORS_INLINE && T <= DELTA_TM_MAX_T &&
                          (factor_path == MRX_FACTORS_PARALLEL || dtype == MRX_F32 || B * H <= 2 * (int64_t)cus);
    // merged episodes run on precomputed factors (which arrive block diagonal by episode, and screened like any
    // other input): where the factor path is the chunk-parallel kernel; with the inverse inside the sequential
    // kernel the units per episode stay (on a full device, where that path is the rule, a chunk with resets
    // costs the forward a few per cent, less than the factor kernel would)
    const bool merged = MRX_HD == 64 && TM_KERNEL && reset_path == MRX_RESETS_MERGED && parallel;
    (void)merged;  // the head-dim-32 build has no merged instances
    if (!TM_KERNEL && factor_path == MRX_FACTORS_PARALLEL) return MRX_ERR_UNSUPPORTED;
    if constexpr (TM_KERNEL) if (parallel) {
        const int rc = launch_delta_tm(st, k, beta, done, done_dtype, Tm_chk, B, T, H, dtype, PRO, dk);
        if (rc != MRX_OK) return rc;
#define MRX_ARGS st, q, k, v, beta, done, done_dtype, S0, o, S_last, S_chk, Tm_chk, B, T, H, nullptr, NormArgs{}, dk, dv
#if MRX_HD == 64
        if (merged)
            return dtype == MRX_BF16 ? launch<__bf16, 32, true, false, false, false, PRO, true, false, true>(MRX_ARGS)
                                     : launch<float, 32, true, false, false, false, PRO, true, false, true>(MRX_ARGS);
#endif
        if (dtype == MRX_BF16) return launch<__bf16, 32, true, false, false, false, PRO, true>(MRX_ARGS);
        return launch<float, 32, true, false, false, false, PRO, true>(MRX_ARGS);
#undef MRX_ARGS
    }
    if (dtype == MRX_BF16)
        return launch<__bf16, DELTA_BF16_CHUNK, true, false, false, false, PRO, false>(st, q, k, v, beta, done, done_dtype, S0, o,
                                                                                      S_last, S_chk, Tm_chk, B, T, H, nullptr,
                                                                                      NormArgs{}, dk, dv);
    return launch<float, 32, true, false, false, false, PRO, false>(st, q, k, v, beta, done, done_dtype, S0, o, S_last,
                                                                    S_chk, Tm_chk, B, T, H, nullptr, NormArgs{}, dk, dv);
}

bool factor_path_ok(int f) { return f == MRX_FACTORS_AUTO || f == MRX_FACTORS_PARALLEL || f == MRX_FACTORS_INLINE; }
bool reset_path_ok(int r) { return r == MRX_RESETS_AUTO || r == MRX_RESETS_PASSES || r == MRX_RESETS_MERGED; }

#if MRX_HD == 64
// ---- static scratch of the entry point that allocates nothing --------------------------------------
// Room for the triangular factors of MRX_NOALLOC_SCRATCH_BYTES / (32 * 32 * sizeof(element)) chunks.
// Every device the library runs on holds its own copy at its own address; host code only ever uses
// the address resolve_scratch() obtained for the current device, never the array's name.
// The build with 64-step delta-rule chunks has no chunk-parallel factor kernel, hence no use for the
// array (its mrx_delta_rule_fwd_noalloc answers MRX_ERR_UNSUPPORTED) and does not hold it.
constexpr bool HAS_SCRATCH = DELTA_BF16_CHUNK == 32;
static __device__ __align__(256) unsigned char scratch[HAS_SCRATCH ? MRX_NOALLOC_SCRATCH_BYTES : 256];
void *g_scratch_ptr[64] = {nullptr};

#endif
}  // namespace MRX_HD_NS
}  // namespace

#if MRX_HD == 64
int mrx::resolve_scratch(int dev)
{
    if (dev < 0 || dev >= 64) return MRX_ERR_UNSUPPORTED;
    if (!HAS_SCRATCH) return MRX_OK;
    void *p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) {
        (void)hipGetLastError();  // reported through the return value; not left for the host framework's next call
        return MRX_ERR_LAUNCH;
    }
    g_scratch_ptr[dev] = p;
    return MRX_OK;
}

extern "C" int64_t mrx_chunk_size(int dtype) { return dtype == MRX_BF16 ? LA_BF16_CHUNK : (dtype == MRX_F32 ? 32 : 0); }

extern "C" int64_t mrx_delta_chunk_size(int dtype) { return dtype == MRX_BF16 ? DELTA_BF16_CHUNK : (dtype == MRX_F32 ? 32 : 0); }

#endif

MRX_EXPORT int MRX_API(mrx_linear_attn_fwd)(void *stream, const void *q, const void *k, const void *v,
                                   const void *done, const void *S0, void *o, void *S_last,
                                   void *S_chk, int64_t B, int64_t T, int64_t H, int64_t dk,
                                   int64_t dv, int dtype, int done_dtype, int feature_map)
{
#if MRX_HD == 64
    if (dk <= 32 && dv <= 32) return mrx_linear_attn_fwd_hd32(stream, q, k, v, done, S0, o, S_last, S_chk, B, T, H, dk, dv, dtype, done_dtype, feature_map);
#endif
    const int rc = check_common(q, k, v, done, o, S0, S_last, S_chk, B, T, H, dk, dv, dtype, done_dtype, true);
    if (rc != MRX_OK) return rc;
    if (feature_map != MRX_FMAP_NONE && feature_map != MRX_FMAP_ELU1) return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const bool fm = feature_map == MRX_FMAP_ELU1;
    if (dtype == MRX_BF16)
        return fm ? launch<__bf16, LA_BF16_CHUNK, false, true>(st, q, k, v, nullptr, done, done_dtype, S0, o, S_last, S_chk, nullptr, B, T, H, nullptr, NormArgs{}, dk, dv)
                  : launch<__bf16, LA_BF16_CHUNK, false, false>(st, q, k, v, nullptr, done, done_dtype, S0, o, S_last, S_chk, nullptr, B, T, H, nullptr, NormArgs{}, dk, dv);
    return fm ? launch<float, 32, false, true>(st, q, k, v, nullptr, done, done_dtype, S0, o, S_last, S_chk, nullptr, B, T, H, nullptr, NormArgs{}, dk, dv)
              : launch<float, 32, false, false>(st, q, k, v, nullptr, done, done_dtype, S0, o, S_last, S_chk, nullptr, B, T, H, nullptr, NormArgs{}, dk, dv);
}

MRX_EXPORT int MRX_API(mrx_linear_attn_fwd_chunk_parallel)(void *stream, const void *q, const void *k, const void *v,
                                                  const void *done, const void *S0, void *o, void *S_last,
                                                  float *S_chk, int64_t B, int64_t T, int64_t H, int64_t dk,
                                                  int64_t dv, int dtype, int done_dtype, int feature_map)
{
#if MRX_HD == 64
    if (dk <= 32 && dv <= 32) return mrx_linear_attn_fwd_chunk_parallel_hd32(stream, q, k, v, done, S0, o, S_last, S_chk, B, T, H, dk, dv, dtype, done_dtype, feature_map);
#endif
    const int rc = check_common(q, k, v, done, o, S0, S_last, S_chk, B, T, H, dk, dv, dtype, done_dtype, true);
    if (rc != MRX_OK) return rc;
    if (!S_chk) return MRX_ERR_INVALID_ARG;  // the per-chunk states live there
    if (feature_map != MRX_FMAP_NONE && feature_map != MRX_FMAP_ELU1) return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const bool fm = feature_map == MRX_FMAP_ELU1;
    const int C = (int)mrx_chunk_size(dtype);
    if ((T + C - 1) / C > 65535) return MRX_ERR_INVALID_ARG;
    // per-chunk sums of v phi(k)^T -> states entering the chunks (and S_last) -> outputs, chunk by chunk
    int rc2 = launch_la_chunk_states(st, k, v, done, done_dtype, S_chk, B, T, H, dtype, fm, false, dk, dv);
    if (rc2 != MRX_OK) return rc2;
    rc2 = launch_la_state_scan(st, S_chk, (const float *)S0, (float *)S_last, done, done_dtype, B, T, H, C, false, dk, dv);
    if (rc2 != MRX_OK) return rc2;
#define MRX_ARGS st, q, k, v, nullptr, done, done_dtype, nullptr, o, nullptr, S_chk, nullptr, B, T, H, nullptr, NormArgs{}, dk, dv
    if (dtype == MRX_BF16)
        return fm ? launch<__bf16, LA_BF16_CHUNK, false, true, false, false, false, false, true>(MRX_ARGS)
                  : launch<__bf16, LA_BF16_CHUNK, false, false, false, false, false, false, true>(MRX_ARGS);
    return fm ? launch<float, 32, false, true, false, false, false, false, true>(MRX_ARGS)
              : launch<float, 32, false, false, false, false, false, false, true>(MRX_ARGS);
#undef MRX_ARGS
}

#if MRX_HD == 64
extern "C" int mrx_linear_attn_chunk_parallel_pays(int64_t B, int64_t T, int64_t H, int dtype)
{
    const int64_t C = mrx_chunk_size(dtype);
    int cus = 0;
    if (C == 0 || B <= 0 || T <= 0 || H <= 0 || prepare_device(&cus) != MRX_OK) return 0;
    const int64_t NC = (T + C - 1) / C;
    // Measured on MI355X (forward + backward, fp32 and bf16, 8 to 192 sequences of 128 to 2048 steps): with
    // at most one sequence per two compute units and eight or more chunks each the pair is 1.1x (128
    // sequences) to 6x (8 sequences x 2048 steps) faster than one workgroup per sequence; with more
    // sequences the per-chunk state traffic (a 16 KB slot written, summed and read per chunk) costs more
    // than the idle compute units, and with fewer chunks the two extra launches do.
    return 2 * B * H <= (int64_t)cus && NC >= 8 && NC <= 65535;
}
#endif

MRX_EXPORT int MRX_API(mrx_delta_rule_fwd)(void *stream, const void *q, const void *k, const void *v,
                                  const void *beta, const void *done, const void *S0, void *o,
                                  void *S_last, void *S_chk, void *Tm_chk, int64_t B, int64_t T,
                                  int64_t H, int64_t dk, int64_t dv, int dtype, int done_dtype, int factor_path,
                                  int reset_path)
{
#if MRX_HD == 64
    if (dk <= 32 && dv <= 32) return mrx_delta_rule_fwd_hd32(stream, q, k, v, beta, done, S0, o, S_last, S_chk, Tm_chk, B, T, H, dk, dv, dtype, done_dtype, factor_path, reset_path);
#endif
    const int rc = check_common(q, k, v, done, o, S0, S_last, S_chk, B, T, H, dk, dv, dtype, done_dtype, true);
    if (rc != MRX_OK) return rc;
    if (!beta || !aligned(Tm_chk, 16) || !factor_path_ok(factor_path) || !reset_path_ok(reset_path)) return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    return delta_fwd_dispatch<false>(st, q, k, v, beta, done, done_dtype, S0, o, S_last, S_chk, Tm_chk, B, T, H, dtype,
                                     factor_path, dk, dv, reset_path);
}

#if MRX_HD == 64
extern "C" int mrx_delta_rule_fwd_noalloc(void *stream, const void *q, const void *k, const void *v,
                                          const void *beta, const void *done, const void *S0, void *o,
                                          void *S_last, int64_t B, int64_t T, int64_t H, int64_t dk,
                                          int64_t dv, int dtype, int done_dtype)
{
    const int rc = check_common(q, k, v, done, o, S0, S_last, nullptr, B, T, H, dk, dv, dtype, done_dtype);
    if (rc != MRX_OK) return rc;
    if (!beta) return MRX_ERR_INVALID_ARG;
    if (!HAS_SCRATCH) return MRX_ERR_UNSUPPORTED;
    const int64_t NC = (T + 31) / 32, esize = dtype == MRX_BF16 ? 2 : 4;
    if (T > DELTA_TM_MAX_T || B * H * NC > (int64_t)MRX_NOALLOC_SCRATCH_BYTES / (32 * 32 * esize)) return MRX_ERR_SCRATCH;
    int dev = -1;
    if (const int rc2 = prepare_device(nullptr, &dev); rc2 != MRX_OK) return rc2;
    void *factors = g_scratch_ptr[dev];  // this device's copy of the array, resolved at set-up
    if (!factors) return MRX_ERR_LAUNCH;
    hipStream_t st = (hipStream_t)stream;
    return delta_fwd_dispatch<false>(st, q, k, v, beta, done, done_dtype, S0, o, S_last, nullptr, factors, B, T, H, dtype,
                                     MRX_FACTORS_PARALLEL);
}
#endif

MRX_EXPORT int MRX_API(mrx_gated_linear_attn_fwd)(void *stream, const void *q, const void *k, const void *v,
                                         const void *g, const void *done, const void *S0, void *o,
                                         void *S_last, void *S_chk, int64_t B, int64_t T, int64_t H,
                                         int64_t dk, int64_t dv, int dtype, int done_dtype, int feature_map)
{
#if MRX_HD == 64
    if (dk <= 32 && dv <= 32) return mrx_gated_linear_attn_fwd_hd32(stream, q, k, v, g, done, S0, o, S_last, S_chk, B, T, H, dk, dv, dtype, done_dtype, feature_map);
#endif
    const int rc = check_common(q, k, v, done, o, S0, S_last, S_chk, B, T, H, dk, dv, dtype, done_dtype, true);
    if (rc != MRX_OK) return rc;
    if (!g || !aligned(g, 4)) return MRX_ERR_INVALID_ARG;
    if (feature_map != MRX_FMAP_NONE && feature_map != MRX_FMAP_ELU1) return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const bool fm = feature_map == MRX_FMAP_ELU1;
#define MRX_ARGS st, q, k, v, nullptr, done, done_dtype, S0, o, S_last, S_chk, nullptr, B, T, H, g, NormArgs{}, dk, dv
    if (dtype == MRX_BF16)
        return fm ? launch<__bf16, LA_BF16_CHUNK, false, true, true>(MRX_ARGS) : launch<__bf16, LA_BF16_CHUNK, false, false, true>(MRX_ARGS);
    return fm ? launch<float, 32, false, true, true>(MRX_ARGS) : launch<float, 32, false, false, true>(MRX_ARGS);
#undef MRX_ARGS
}

MRX_EXPORT int MRX_API(mrx_linear_attn_norm_fwd)(void *stream, const void *q, const void *k, const void *v,
                                        const void *done, const void *S0, const float *z0, void *o,
                                        float *den, float *ss, void *S_last, float *z_last, void *S_chk, float *z_chk,
                                        int64_t B, int64_t T, int64_t H, int64_t dk, int64_t dv, int dtype,
                                        int done_dtype, int feature_map, float eps)
{
#if MRX_HD == 64
    if (dk <= 32 && dv <= 32) return mrx_linear_attn_norm_fwd_hd32(stream, q, k, v, done, S0, z0, o, den, ss, S_last, z_last, S_chk, z_chk, B, T, H, dk, dv, dtype, done_dtype, feature_map, eps);
#endif
    const int rc = check_common(q, k, v, done, o, S0, S_last, S_chk, B, T, H, dk, dv, dtype, done_dtype, true);
    if (rc != MRX_OK) return rc;
    if (!den || !aligned(den, 4) || !aligned(ss, 4) || !aligned(z0, 16) || !aligned(z_last, 16) || !aligned(z_chk, 16))
        return MRX_ERR_INVALID_ARG;
    if (feature_map != MRX_FMAP_NONE && feature_map != MRX_FMAP_ELU1) return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const bool fm = feature_map == MRX_FMAP_ELU1;
    const NormArgs na{z0, den, z_last, z_chk, eps, ss};
#define MRX_ARGS st, q, k, v, nullptr, done, done_dtype, S0, o, S_last, S_chk, nullptr, B, T, H, nullptr, na, dk, dv
    if (dtype == MRX_BF16)
        return fm ? launch<__bf16, LA_BF16_CHUNK, false, true, false, true>(MRX_ARGS)
                  : launch<__bf16, LA_BF16_CHUNK, false, false, false, true>(MRX_ARGS);
    return fm ? launch<float, 32, false, true, false, true>(MRX_ARGS) : launch<float, 32, false, false, false, true>(MRX_ARGS);
#undef MRX_ARGS
}

MRX_EXPORT int MRX_API(mrx_deltanet_fwd)(void *stream, const void *q, const void *k, const void *v,
                                const void *beta_raw, const void *done, const void *S0, void *o,
                                void *S_last, void *S_chk, void *Tm_chk, int64_t B, int64_t T,
                                int64_t H, int64_t dk, int64_t dv, int dtype, int done_dtype, int factor_path,
                                int reset_path)
{
#if MRX_HD == 64
    if (dk <= 32 && dv <= 32) return mrx_deltanet_fwd_hd32(stream, q, k, v, beta_raw, done, S0, o, S_last, S_chk, Tm_chk, B, T, H, dk, dv, dtype, done_dtype, factor_path, reset_path);
#endif
    const int rc = check_common(q, k, v, done, o, S0, S_last, S_chk, B, T, H, dk, dv, dtype, done_dtype, true);
    if (rc != MRX_OK) return rc;
    if (!beta_raw || !aligned(Tm_chk, 16) || !factor_path_ok(factor_path) || !reset_path_ok(reset_path)) return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    return delta_fwd_dispatch<true>(st, q, k, v, beta_raw, done, done_dtype, S0, o, S_last, S_chk, Tm_chk, B, T, H, dtype,
                                    factor_path, dk, dv, reset_path);
}
