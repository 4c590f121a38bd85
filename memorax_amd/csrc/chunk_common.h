// Building blocks of the chunked linear-attention / delta-rule kernels (gfx950).
//
// One workgroup = 4 waves = one (batch, head) sequence, head dim 64, walking the
// time axis in chunks of C rows.  All matrix products are "NT" products
//     D[m][n] = sum_k X[m][k] * Y[n][k]
// of two LDS tiles that are both contiguous along k, executed with 16x16 MFMA
// tiles (bf16: v_mfma_f32_16x16x32_bf16, fp32: v_mfma_f32_16x16x4_f32) and fp32
// accumulation.  A wave lane (i = lane % 16, g = lane / 16) holds, for a 16x16
// accumulator tile, the four elements D[4g + v][i], v = 0..3; so four
// consecutive m-indices sit in one lane and a tile can be stored k-contiguously
// as the [n][m] (transposed) matrix with one 8/16-byte LDS write per lane.
// Every product below is oriented so that its result lands k-contiguous for
// the next product that consumes it.
#pragma once
#include "common.h"

namespace mrx {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also drains the
// vector-memory counter, which would make every barrier wait for the next chunk's
// global prefetch; the compiler still inserts the vmcnt wait where a prefetched
// register is first consumed.
__device__ __forceinline__ void sync_lds()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

constexpr int NWAVES = 4;
constexpr int NTHREADS = 64 * NWAVES;
constexpr int HD = 64;  // head dim (d_k = d_v)

template <typename T> struct TT;
template <> struct TT<__bf16> {
    static constexpr int KP = 8;   // elements per 16-byte fragment
    static constexpr int KB = 32;  // k extent of one fragment pair
    using frag = bf16x8;
    using pack4 = bf16x4;
    static __device__ __forceinline__ f32x4 mma(frag a, frag b, f32x4 c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ pack4 pack(float a, float b, float c, float d)
    {
        pack4 r;
        r[0] = (__bf16)a; r[1] = (__bf16)b; r[2] = (__bf16)c; r[3] = (__bf16)d;
        return r;
    }
};
template <> struct TT<float> {
    static constexpr int KP = 4;
    static constexpr int KB = 16;
    using frag = f32x4;
    using pack4 = f32x4;
    static __device__ __forceinline__ f32x4 mma(frag a, frag b, f32x4 c)
    {
        // lane group g supplies k = 4g + s to the s-th instruction (same map for both operands)
#pragma unroll
        for (int s = 0; s < 4; ++s) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[s], b[s], c, 0, 0, 0);
        return c;
    }
    static __device__ __forceinline__ pack4 pack(float a, float b, float c, float d)
    {
        pack4 r = {a, b, c, d};
        return r;
    }
};

// 16-byte LDS row padding (in elements) keeps 16-lane fragment reads conflict free.
template <typename T> constexpr int pad_of() { return 16 / (int)sizeof(T); }

// Which 16x16 tiles of an M x N result a wave owns: slot j -> (mt, nt).
template <int M, int N> struct TileMap {
    static constexpr int MT = M / 16, NT = N / 16;
    static constexpr int TPW = MT * NT / NWAVES;
    static_assert(MT == 2 || MT == 4, "M must be 32 or 64");
    static_assert(MT * NT % NWAVES == 0, "tiles must divide over the waves");
    static __device__ __forceinline__ int mt(int w) { return MT == 4 ? w : (w & 1); }
    static __device__ __forceinline__ int nt(int w, int j) { return MT == 4 ? j : (w >> 1) * TPW + j; }
};

// acc[j] += X[mt-th 16 rows][:] . Y[nt_j-th 16 rows][:]^T over K columns.
template <typename T, int M, int N, int K>
__device__ __forceinline__ void gemm_nt(f32x4 *acc, const T *X, int ldx, const T *Y, int ldy,
                                        int w, int lane)
{
    using TM = TileMap<M, N>;
    using F = typename TT<T>::frag;
    constexpr int KP = TT<T>::KP, KB = TT<T>::KB;
    static_assert(K % KB == 0, "K must be a multiple of the fragment k extent");
    const int i = lane & 15, g = lane >> 4;
    const T *xp = X + (TM::mt(w) * 16 + i) * ldx + g * KP;
#pragma unroll
    for (int kb = 0; kb < K / KB; ++kb) {
        const F a = *reinterpret_cast<const F *>(xp + kb * KB);
#pragma unroll
        for (int j = 0; j < TM::TPW; ++j) {
            const F b = *reinterpret_cast<const F *>(Y + (TM::nt(w, j) * 16 + i) * ldy + kb * KB + g * KP);
            acc[j] = TT<T>::mma(a, b, acc[j]);
        }
    }
}

template <int N> __device__ __forceinline__ void zero_acc(f32x4 *acc)
{
#pragma unroll
    for (int j = 0; j < N; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
}

// Store an accumulator tile set as the k-contiguous matrix dst[n][m] (type T).
template <typename T, int M, int N>
__device__ __forceinline__ void store_acc_t(const f32x4 *acc, T *dst, int ld, int w, int lane)
{
    using TM = TileMap<M, N>;
    using P = typename TT<T>::pack4;
    const int i = lane & 15, g = lane >> 4;
#pragma unroll
    for (int j = 0; j < TM::TPW; ++j) {
        const int m = TM::mt(w) * 16 + 4 * g, n = TM::nt(w, j) * 16 + i;
        *reinterpret_cast<P *>(dst + n * ld + m) = TT<T>::pack(acc[j][0], acc[j][1], acc[j][2], acc[j][3]);
    }
}

// Store an accumulator tile set as dst[m][n] (element-wise writes; use when the
// consumer needs the other orientation too).
template <typename T, int M, int N>
__device__ __forceinline__ void store_acc_n(const f32x4 *acc, T *dst, int ld, int w, int lane)
{
    using TM = TileMap<M, N>;
    const int i = lane & 15, g = lane >> 4;
#pragma unroll
    for (int j = 0; j < TM::TPW; ++j) {
        const int m = TM::mt(w) * 16 + 4 * g, n = TM::nt(w, j) * 16 + i;
#pragma unroll
        for (int v = 0; v < 4; ++v) dst[(m + v) * ld + n] = (T)acc[j][v];
    }
}

// Raw bits of one T-typed scalar (converted to float only when consumed).
template <typename T> __device__ __forceinline__ uint32_t load_raw(const T *p);
template <> __device__ __forceinline__ uint32_t load_raw<__bf16>(const __bf16 *p)
{
    return (uint32_t) *reinterpret_cast<const uint16_t *>(p);
}
template <> __device__ __forceinline__ uint32_t load_raw<float>(const float *p)
{
    return *reinterpret_cast<const uint32_t *>(p);
}
template <typename T> __device__ __forceinline__ float raw_to_float(uint32_t raw);
template <> __device__ __forceinline__ float raw_to_float<__bf16>(uint32_t raw) { return __uint_as_float(raw << 16); }
template <> __device__ __forceinline__ float raw_to_float<float>(uint32_t raw) { return __uint_as_float(raw); }

__device__ __forceinline__ float elu1(float x) { return x > 0.f ? x + 1.f : __expf(x); }
__device__ __forceinline__ float delu1(float x) { return x > 0.f ? 1.f : __expf(x); }

// ---- global <-> register <-> LDS movement of one [C][64] input tile ----------
// A tile is C rows of 64 T = C * SEGS 16-byte segments; thread tid owns segment
// (tid % SEGS) of rows (tid / SEGS) + p * RPP, p = 0..PASSES-1.
template <typename T, int C> struct TileIO {
    static constexpr int KP = TT<T>::KP;
    static constexpr int SEGS = HD / KP;
    static constexpr int RPP = NTHREADS / SEGS;
    static constexpr int PASSES = C / RPP;
    static_assert(PASSES >= 1 && C % RPP == 0, "chunk rows must be a multiple of rows per pass");
    using F = typename TT<T>::frag;
    struct Regs {
        F v[PASSES];
    };

    // rows t0.. of a (B,T,H,64) array whose (b,h) base pointer is `base`; rows >= Tlen read as 0
    static __device__ __forceinline__ void load(Regs &r, const T *base, int64_t row_stride, int t0,
                                                int Tlen, int tid)
    {
        const int seg = tid % SEGS, r0 = tid / SEGS;
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            const int t = t0 + r0 + p * RPP;
            F z;
#pragma unroll
            for (int e = 0; e < KP; ++e) z[e] = (T)0.f;
            r.v[p] = t < Tlen ? *reinterpret_cast<const F *>(base + (int64_t)t * row_stride + seg * KP) : z;
        }
    }

    template <bool FMAP> static __device__ __forceinline__ void fmap(Regs &r)
    {
        if (FMAP) {
#pragma unroll
            for (int p = 0; p < PASSES; ++p)
#pragma unroll
                for (int e = 0; e < KP; ++e) r.v[p][e] = (T)elu1((float)r.v[p][e]);
        }
    }

    // dst[row][col], row-major with leading dim ld
    static __device__ __forceinline__ void to_lds(const Regs &r, T *dst, int ld, int tid)
    {
        const int seg = tid % SEGS, r0 = tid / SEGS;
#pragma unroll
        for (int p = 0; p < PASSES; ++p)
            *reinterpret_cast<F *>(dst + (r0 + p * RPP) * ld + seg * KP) = r.v[p];
    }

    // dst[col][row]
    static __device__ __forceinline__ void to_lds_t(const Regs &r, T *dst, int ld, int tid)
    {
        const int seg = tid % SEGS, r0 = tid / SEGS;
#pragma unroll
        for (int p = 0; p < PASSES; ++p)
#pragma unroll
            for (int e = 0; e < KP; ++e) dst[(seg * KP + e) * ld + r0 + p * RPP] = r.v[p][e];
    }
};

// ---- per-chunk reset bookkeeping ------------------------------------------------
// dmask has bit r set when row r of the chunk starts a new episode.  episode_of(r)
// counts the resets at rows <= r; rows interact iff they have the same count.
__device__ __forceinline__ int episode_of(unsigned long long dmask, int r)
{
    return __popcll(dmask & ((2ull << r) - 1ull));
}

// ---- inverse of a unit lower-triangular matrix, in place, fp32 -------------------
// sA holds A (strictly lower part used), C x C with leading dim ld; on return the
// inverse X of (I + A) is stored as: diagonal 16x16 blocks in place; block (b, c),
// b > c, in the unused upper position (c, b) (same orientation).  Needs all 4 waves
// (contains workgroup barriers).
template <int C> __device__ __forceinline__ void tri_inverse(float *sA, int ld, int w, int lane)
{
    constexpr int NB = C / 16;
    const int i = lane & 15, g = lane >> 4;
    if (w < NB) {
        // Diagonal block w by repeated squaring, entirely in registers.  With N = -A
        // (nilpotent, N^16 = 0): (I + A)^-1 = (I + N)(I + N^2)(I + N^4)(I + N^8).
        // A 16x16 product P = X Y on the fp32 MFMA takes X^T and Y both in accumulator
        // layout (lane (i,g) holds Z[4g+v][i]), so each matrix is carried together with
        // its transpose and no operand goes through LDS.
        float *blk = sA + (16 * w) * ld + 16 * w;
        auto mm = [](const f32x4 &xt, const f32x4 &y, f32x4 c) {
#pragma unroll
            for (int s = 0; s < 4; ++s) c = __builtin_amdgcn_mfma_f32_16x16x4f32(xt[s], y[s], c, 0, 0, 0);
            return c;
        };
        const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
        f32x4 M, Mt, R, Rt;
        Mt = *reinterpret_cast<const f32x4 *>(blk + i * ld + 4 * g);  // A[i][4g+v] = (A^T)[4g+v][i]
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int r = 4 * g + v;
            M[v] = (i < r) ? -blk[r * ld + i] : 0.f;   // N[r][i], strictly lower
            Mt[v] = (r < i) ? -Mt[v] : 0.f;            // N^T[r][i] = N[i][r], strictly upper
            R[v] = M[v] + (r == i ? 1.f : 0.f);
            Rt[v] = Mt[v] + (r == i ? 1.f : 0.f);
        }
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            const f32x4 M2 = mm(Mt, M, zero);    // N^2  : X = M,  Y = M
            const f32x4 M2t = mm(M, Mt, zero);   // (N^2)^T = M^T M^T : X = M^T, Y = M^T
            const f32x4 R2 = mm(Rt, M2, R);      // R + R M2
            const f32x4 R2t = mm(M2, Rt, Rt);    // R^T + M2^T R^T
            M = M2; Mt = M2t; R = R2; Rt = R2t;
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) blk[(4 * g + v) * ld + i] = R[v];
    }
    sync_lds();
#pragma unroll
    for (int d = 1; d < NB; ++d) {
        if (w < NB - d) {
            const int b = w + d, c = w;  // block (b, c)
            f32x4 tmp = {0.f, 0.f, 0.f, 0.f};
            for (int k = c; k < b; ++k) {
                // tmp += A_bk . X_kc ; X_kc lives at rows 16c.., cols 16k.. (diagonal when k == c)
                const f32x4 a4 = *reinterpret_cast<const f32x4 *>(sA + (16 * b + i) * ld + 16 * k + 4 * g);
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const float bop = sA[(16 * c + 4 * g + s) * ld + 16 * k + i];
                    tmp = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[s], bop, tmp, 0, 0, 0);
                }
            }
            // X_bc = -X_bb . tmp ; the accumulator layout of tmp is already the B-operand layout
            f32x4 res = {0.f, 0.f, 0.f, 0.f};
            const f32x4 a4 = *reinterpret_cast<const f32x4 *>(sA + (16 * b + i) * ld + 16 * b + 4 * g);
#pragma unroll
            for (int s = 0; s < 4; ++s) res = __builtin_amdgcn_mfma_f32_16x16x4f32(a4[s], tmp[s], res, 0, 0, 0);
#pragma unroll
            for (int v = 0; v < 4; ++v) sA[(16 * c + 4 * g + v) * ld + 16 * b + i] = -res[v];
        }
        sync_lds();
    }
}

// Element (i, j..j+3) of the inverse stored by tri_inverse (j multiple of 4).
__device__ __forceinline__ f32x4 tri_inverse_get4(const float *sA, int ld, int i, int j)
{
    const int bi = i >> 4, bj = j >> 4;
    if (bi == bj) return *reinterpret_cast<const f32x4 *>(sA + i * ld + j);
    if (bi > bj) return *reinterpret_cast<const f32x4 *>(sA + (16 * bj + (i & 15)) * ld + 16 * bi + (j & 15));
    return f32x4{0.f, 0.f, 0.f, 0.f};
}

}  // namespace mrx
