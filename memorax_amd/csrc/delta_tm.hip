// The kernel declared in delta_tm.h.  Its own translation unit: it is built with the compiler
// option that keeps MFMA results in ordinary vector registers (-mllvm -amdgpu-mfma-vgpr-form),
// because every product here is consumed by the vector ALU at once and a result in accumulation
// registers costs four extra moves.
#include "delta_tm.h"

#include <type_traits>

#include "chunk_common.h"

namespace mrx {
inline namespace MRX_HD_NS {

// NARROW: the key rows are dka wide in memory, less than the build's head dim; the fragments' further
// columns are zeros.
template <typename T, bool PRO, bool NARROW = false>
__global__ void __launch_bounds__(256)
delta_tm_kernel(const T *__restrict__ k, const T *__restrict__ beta, const void *__restrict__ done, int done_f32,
                T *__restrict__ Tm_chk, int Tlen, int H, int NC, int dka)
{
    constexpr int C = 32;
    using Frag = typename TT<T>::frag;
    using P4 = typename TT<T>::pack4;
    using Op = Op16<T>;
    constexpr int KB = TT<T>::KB, KP = TT<T>::KP, NKB = HD / KB;
    const int lane = threadIdx.x & 63, li = lane & 15, lg = lane >> 4;
    // grid: x = sequence (b, h), y = group of four chunks; 32-bit arithmetic on wave-uniform values
    const int c = (int)blockIdx.y * 4 + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));  // this wave's chunk
    if (c >= NC) return;
    const unsigned bh = blockIdx.x, b = bh / (unsigned)H, h = bh - b * (unsigned)H;
    const int t0 = c * C;

    // ---- K rows 16 rb + li as operand fragments: lane (li, lg) holds columns KB kb + KP lg .. ----
    Frag f[2][NKB];
    Frag zf;
#pragma unroll
    for (int e = 0; e < KP; ++e) zf[e] = (T)0.f;
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
        const int t = t0 + 16 * rb + li;
        const T *row = k + (((int64_t)b * Tlen + t) * H + h) * (NARROW ? dka : HD) + KP * lg;
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb)
            f[rb][kb] = (t < Tlen && (!NARROW || kb * KB + KP * lg < dka)) ? *reinterpret_cast<const Frag *>(row + kb * KB) : zf;
    }
    // gates and reset flags of the 32 rows, one per lane
    float bl = 0.f;
    bool dl = false;
    if (lane < C && t0 + lane < Tlen) {
        const int64_t r = (int64_t)b * Tlen + t0 + lane;
        bl = (float)beta[r * H + h];
        if (PRO) bl = sigmoidf(bl);
        dl = done_at(done, done_f32, r);
    }
    const unsigned long long dmask = __ballot(dl);
    const int nres = __popcll(dmask);
    if (PRO) {
        // |k_row|^2 with the summation tree of the staging code (16-byte segments in order, pairs,
        // pairs of pairs, halves), so that the normalised keys round to the same values
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
            float tq[NKB];
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb) {
                float ss = 0.f;
#pragma unroll
                for (int e = 0; e < KP; ++e) ss += (float)f[rb][kb][e] * (float)f[rb][kb][e];
                ss += __shfl_xor(ss, 16);
                ss += __shfl_xor(ss, 32);
                tq[kb] = ss;
            }
            float tot = tq[0];  // pairs, then pairs of pairs: the staging code's order
            if (NKB >= 2) tot += tq[NKB >= 2 ? 1 : 0];
            if (NKB == 4) tot += tq[NKB == 4 ? 2 : 0] + tq[NKB == 4 ? 3 : 0];
            const float inv = inv_norm(tot);
#pragma unroll
            for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
                for (int e = 0; e < KP; ++e) f[rb][kb][e] = (T)((float)f[rb][kb][e] * inv);
        }
    }
    // ---- K K^T: kk[rb][v] = k_{16 rb + 4 lg + v} . k_{16 rb + li}; kk10[v] = k_{16 + 4 lg + v} . k_{li} ------
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    f32x4 kk[2] = {zero, zero}, kk10 = zero;
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb) {
        kk[0] = TT<T>::mma(f[0][kb], f[0][kb], kk[0]);
        kk[1] = TT<T>::mma(f[1][kb], f[1][kb], kk[1]);
        kk10 = TT<T>::mma(f[1][kb], f[0][kb], kk10);
    }
    // the gates the tiles need, fetched from their lanes once (every lane takes part: not under a select)
    float beta_i[2], beta_r[2][4];
#pragma unroll
    for (int bb = 0; bb < 2; ++bb) {
        beta_i[bb] = __shfl(bl, 16 * bb + li);
#pragma unroll
        for (int e = 0; e < 4; ++e) beta_r[bb][e] = __shfl(bl, 16 * bb + 4 * lg + e);
    }
    T *out = Tm_chk + ((int64_t)bh * NC + c) * (C * C);
    // One episode of the chunk.  RES false: the chunk has no reset, every row is live and the code
    // carries no masks (the common case gets a copy of its own: this kernel is bound by the vector ALU).
    auto episode = [&](auto res_tag, const int pass) {
        constexpr bool RES = decltype(res_tag)::value;
        auto live = [&](int r) { return !RES || episode_of(dmask, r) == pass; };
        // N = -A_bb (strictly lower) and R = I + N, each with its transpose, in accumulator layout.
        // mm(P, Q) = P^T Q, so a product and its transpose come from the same two operands swapped.
        f32x4 M[2], Mt[2], R[2], Rt[2];
#pragma unroll
        for (int bb = 0; bb < 2; ++bb) {
            const bool live_i = live(16 * bb + li);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int r = 4 * lg + e;
                const bool on = live_i && live(16 * bb + r);
                M[bb][e] = (on && li < r) ? -beta_r[bb][e] * kk[bb][e] : 0.f;   // N[r][i]
                Mt[bb][e] = (on && r < li) ? -beta_i[bb] * kk[bb][e] : 0.f;     // N^T[r][i] = N[i][r]
                R[bb][e] = M[bb][e] + (r == li ? 1.f : 0.f);
                Rt[bb][e] = Mt[bb][e] + (r == li ? 1.f : 0.f);
            }
        }
        // (I - N)^-1 = (I + N)(I + N^2)(I + N^4)(I + N^8), the two blocks interleaved
        Op oM[2] = {Op::of(M[0]), Op::of(M[1])}, oMt[2] = {Op::of(Mt[0]), Op::of(Mt[1])};
        Op oR0 = Op::of(R[0]);  // only the last value is used
#pragma unroll
        for (int lvl = 0; lvl < 3; ++lvl) {
#pragma unroll
            for (int bb = 0; bb < 2; ++bb) {
                const f32x4 M2 = Op::mm(oMt[bb], oM[bb], zero);                   // N^2
                const Op oRt = Op::of(Rt[bb]);
                const Op oM2 = Op::of(M2);
                if (bb == 0) R[0] = Op::mm(oRt, oM2, R[0]);                        // R + R N^2 (block 1: not needed)
                Rt[bb] = Op::mm(oM2, oRt, Rt[bb]);                                // R^T + (N^2)^T R^T
                if (lvl < 2) {
                    const f32x4 M2t = Op::mm(oM[bb], oMt[bb], zero);              // (N^2)^T
                    oMt[bb] = Op::of(M2t);
                }
                oM[bb] = oM2;
            }
        }
        oR0 = Op::of(R[0]);
        // X_10^T = -X_00^T (A_10^T X_11^T); A_10^T as the left operand is A_10 in accumulator layout
        f32x4 a10;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            a10[e] = (live(16 + 4 * lg + e) && live(li)) ? beta_r[1][e] * kk10[e] : 0.f;  // A_10[4 lg + e][li]
        const f32x4 pt = Op::mm(Op::of(a10), Op::of(Rt[1]), zero);
        const f32x4 x10t = Op::mm(oR0, Op::of(pt), zero);  // X_10[li][4 lg + v], sign pending
        // rows of this pass's episode (rows past the end count as the last episode: identity rows)
        if (live(li)) {
            *reinterpret_cast<P4 *>(out + li * C + 4 * lg) = TT<T>::pack(Rt[0][0], Rt[0][1], Rt[0][2], Rt[0][3]);
            *reinterpret_cast<P4 *>(out + li * C + 16 + 4 * lg) = TT<T>::pack(0.f, 0.f, 0.f, 0.f);
        }
        if (live(16 + li)) {
            *reinterpret_cast<P4 *>(out + (16 + li) * C + 4 * lg) = TT<T>::pack(-x10t[0], -x10t[1], -x10t[2], -x10t[3]);
            *reinterpret_cast<P4 *>(out + (16 + li) * C + 16 + 4 * lg) = TT<T>::pack(Rt[1][0], Rt[1][1], Rt[1][2], Rt[1][3]);
        }
    };
    if (nres == 0) {
        episode(std::false_type{}, 0);
    } else {
        for (int pass = 0; pass <= nres; ++pass) episode(std::true_type{}, pass);
    }
}

namespace {
template <typename T, bool PRO>
int launch_tm(hipStream_t st, const void *k, const void *beta, const void *done, int done_f32, void *Tm_chk, int64_t B,
              int64_t Tlen, int64_t H, int64_t dk)
{
    const int64_t NC = (Tlen + 31) / 32, groups = (NC + 3) / 4;
    if (B * H > 0x7fffffffLL || groups > 65535) return MRX_ERR_INVALID_ARG;
    const dim3 grid((unsigned)(B * H), (unsigned)groups);
    if (dk != HD)
        return launch_kernel((delta_tm_kernel<T, PRO, true>), grid, dim3(256), 0, st, (const T *)k, (const T *)beta, done,
                             done_f32, (T *)Tm_chk, (int)Tlen, (int)H, (int)NC, (int)dk);
    return launch_kernel((delta_tm_kernel<T, PRO, false>), grid, dim3(256), 0, st, (const T *)k, (const T *)beta, done,
                         done_f32, (T *)Tm_chk, (int)Tlen, (int)H, (int)NC, (int)dk);
}
}  // namespace

int launch_delta_tm(hipStream_t st, const void *k, const void *beta, const void *done, int done_f32, void *Tm_chk,
                    int64_t B, int64_t Tlen, int64_t H, int dtype, bool prologue, int64_t dk)
{
    if (dtype == MRX_BF16)
        return prologue ? launch_tm<__bf16, true>(st, k, beta, done, done_f32, Tm_chk, B, Tlen, H, dk)
                        : launch_tm<__bf16, false>(st, k, beta, done, done_f32, Tm_chk, B, Tlen, H, dk);
    return prologue ? launch_tm<float, true>(st, k, beta, done, done_f32, Tm_chk, B, Tlen, H, dk)
                    : launch_tm<float, false>(st, k, beta, done, done_f32, Tm_chk, B, Tlen, H, dk);
}

}  // namespace MRX_HD_NS
}  // namespace mrx
