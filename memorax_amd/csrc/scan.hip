// Diagonal linear-recurrence scan for gfx950:  h_t = done_t ? b_t : a_t h_{t-1} + b_t.
//
// The op is pure streaming (2 loads + 1 store per element forward, 3 + 2 backward),
// so the design is about HBM: lanes lie along the contiguous feature axis
// (one wave row = 64 lanes x 16 B), each lane walks time in registers, and when
// the (batch x feature) extent alone cannot fill 256 CUs the time axis is split
// over the waves of a workgroup: every wave scans its slice from the identity,
// per-wave summaries (P, h, reset-seen) meet in LDS, each wave folds the
// summaries to its left into a carry-in and fixes its slice up by *select*
// (a reset inside the slice wins over the carry, so NaN/Inf never cross a reset).
// One pass over HBM in either case.
// With MG set the kernels take the MinGRU cell's two projections and form a_t, b_t in registers.
#include <initializer_list>
#include <type_traits>

#include "common.h"

namespace {

using namespace mrx;

struct c64 {
    float re, im;
};

template <typename E> struct Ops;
template <> struct Ops<float> {
    static __device__ __forceinline__ float zero() { return 0.0f; }
    static __device__ __forceinline__ float one() { return 1.0f; }
    static __device__ __forceinline__ float conj(float a) { return a; }
    // a * x + y
    static __device__ __forceinline__ float madd(float a, float x, float y) { return a * x + y; }
    static __device__ __forceinline__ float mul(float a, float x) { return a * x; }
};
template <> struct Ops<c64> {
    static __device__ __forceinline__ c64 zero() { return {0.0f, 0.0f}; }
    static __device__ __forceinline__ c64 one() { return {1.0f, 0.0f}; }
    static __device__ __forceinline__ c64 conj(c64 a) { return {a.re, -a.im}; }
    static __device__ __forceinline__ c64 madd(c64 a, c64 x, c64 y)
    {
        return {a.re * x.re - a.im * x.im + y.re, a.re * x.im + a.im * x.re + y.im};
    }
    static __device__ __forceinline__ c64 mul(c64 a, c64 x)
    {
        return {a.re * x.re - a.im * x.im, a.re * x.im + a.im * x.re};
    }
};

template <typename E, int VEC> struct alignas(sizeof(E) * VEC) Vec {
    E v[VEC];
};

template <typename E, int VEC> __device__ __forceinline__ Vec<E, VEC> vfill(E x)
{
    Vec<E, VEC> r;
#pragma unroll
    for (int i = 0; i < VEC; ++i) r.v[i] = x;
    return r;
}

// Every (B,T,D) array is read or written once per launch and not again before the next kernel: its loads and
// stores are non-temporal, so that the stream does not sit in the caches at the expense of itself (measured at
// 512 x 1024 x 1024 float32: forward 5.77 -> 6.05 TB/s, backward 5.74 -> 6.27 TB/s).  The built-ins take
// scalars and vectors of the language, so a Vec or a raw word group goes through a word type of its size.
template <int BYTES> struct StreamWord;
template <> struct StreamWord<2> { using type = uint16_t; };
template <> struct StreamWord<4> { using type = uint32_t; };
template <> struct StreamWord<8> { typedef uint32_t type __attribute__((ext_vector_type(2))); };
template <> struct StreamWord<16> { typedef uint32_t type __attribute__((ext_vector_type(4))); };
template <typename X> __device__ __forceinline__ X ld_stream(const void *p)
{
    if constexpr (sizeof(X) <= 16) {
        using W = typename StreamWord<sizeof(X)>::type;
        return __builtin_bit_cast(X, __builtin_nontemporal_load(reinterpret_cast<const W *>(p)));
    } else {
        return *reinterpret_cast<const X *>(p);  // wider than one instruction moves (complex64 x 4)
    }
}
template <typename X> __device__ __forceinline__ void st_stream(void *p, const X &x)
{
    if constexpr (sizeof(X) <= 16) {
        using W = typename StreamWord<sizeof(X)>::type;
        __builtin_nontemporal_store(__builtin_bit_cast(W, x), reinterpret_cast<W *>(p));
    } else {
        *reinterpret_cast<X *>(p) = x;
    }
}

// Storage and arithmetic types of the (B,T,D) arrays may differ: bfloat16 in memory, float in registers
// (the carries -- h0, P0, h_last, P_last, g_last, dh0 -- are always in the arithmetic type).
template <typename S, typename E, int VEC> __device__ __forceinline__ Vec<E, VEC> ldv(const S *p)
{
    if constexpr (std::is_same<S, E>::value) {
        return ld_stream<Vec<E, VEC>>(p);
    } else {
        const Vec<S, VEC> raw = ld_stream<Vec<S, VEC>>(p);
        Vec<E, VEC> r;
#pragma unroll
        for (int i = 0; i < VEC; ++i) r.v[i] = (E)raw.v[i];
        return r;
    }
}
// The same in two steps, for prefetched values: the load leaves the stored bits in registers and the conversion
// runs where the value is consumed -- arithmetic on a load still in flight makes the wave wait for it, and for
// every load issued before it, in the middle of issuing a group of loads.
// bfloat16 values wait as whole 32-bit words (a structure of 16-bit members would be taken apart, i.e. computed
// on, the moment it arrives); a single one is widened by its load instruction.
template <typename S, int VEC> struct RawVec {
    using type = Vec<S, VEC>;
};
template <int VEC> struct alignas(VEC >= 2 ? 2 * VEC : 4) RawBf16 {
    uint32_t w[VEC >= 2 ? VEC / 2 : 1];
};
template <int VEC> struct RawVec<__bf16, VEC> {
    using type = RawBf16<VEC>;
};
template <typename S, int VEC> using raw_t = typename RawVec<S, VEC>::type;

template <typename S, int VEC> __device__ __forceinline__ raw_t<S, VEC> ldraw(const S *p)
{
    if constexpr (std::is_same<S, __bf16>::value && VEC == 1) {
        raw_t<S, VEC> r;
        r.w[0] = *reinterpret_cast<const uint16_t *>(p);
        return r;
    } else {
        return ld_stream<raw_t<S, VEC>>(p);
    }
}
template <typename S, typename E, int VEC> __device__ __forceinline__ Vec<E, VEC> cvtv(const raw_t<S, VEC> &raw)
{
    if constexpr (std::is_same<S, E>::value) {
        return raw;
    } else {
        static_assert(std::is_same<S, __bf16>::value && std::is_same<E, float>::value, "bfloat16 storage, float arithmetic");
        Vec<E, VEC> r;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const uint32_t word = raw.w[i >> 1];
            r.v[i] = __builtin_bit_cast(float, (VEC == 1 || !(i & 1)) ? word << 16 : word & 0xffff0000u);
        }
        return r;
    }
}
template <typename S, typename E, int VEC> __device__ __forceinline__ void stv(S *p, const Vec<E, VEC> &x)
{
    if constexpr (std::is_same<S, E>::value) {
        st_stream(p, x);
    } else {
        Vec<S, VEC> raw;
#pragma unroll
        for (int i = 0; i < VEC; ++i) raw.v[i] = (S)x.v[i];
        st_stream(p, raw);
    }
}

// MinGRU in linear space.  The reference scans (log h, log decay) with logaddexp
// (min_gru.py:49-78); the same recurrence is h_t = a_t h_{t-1} + b_t with, from the step's two
// projections z and x = h~:  a = sigma(-z),  b = sigma(z) g(x),  g(x) = x + 0.5 (x >= 0) | sigma(x).
// The kernels below take z and x in place of a and b when MG is set, so the coefficients never
// exist in memory; the backward kernels then emit dz and dx instead of da and db.
struct MinGru {
    // s = sigma(z) and a = sigma(-z), each from exp(-|z|): neither is 1 - the other, so a small
    // gate keeps its relative precision (the cumulative decay is a product of them)
    // The hardware exponential and reciprocal (a few ulp) instead of the library routines: the
    // kernels stream at HBM rate only if a step costs a handful of instructions per element.
    static __device__ __forceinline__ float rcp(float x) { return __builtin_amdgcn_rcpf(x); }
    static __device__ __forceinline__ void gates(float z, float &s, float &a)
    {
        const float e = __expf(-fabsf(z)), r = rcp(1.0f + e), q = e * r;
        s = z >= 0.0f ? r : q;
        a = z >= 0.0f ? q : r;
    }
    // sigma(x) for x < 0 from exp(x) <= 1 (no overflow however negative x is)
    static __device__ __forceinline__ float g(float x)
    {
        const float e = __expf(-fabsf(x));
        return x >= 0.0f ? x + 0.5f : e * rcp(1.0f + e);
    }
    static __device__ __forceinline__ float dg(float x)
    {
        const float e = __expf(-fabsf(x)), r = rcp(1.0f + e);
        return x >= 0.0f ? 1.0f : e * r * r;  // sigma (1 - sigma) = e / (1 + e)^2
    }
    // (z, x) -> (a, b) in place
    static __device__ __forceinline__ void coeffs(float &za, float &xb)
    {
        float s, a;
        gates(za, s, a);
        xb = s * g(xb);
        za = a;
    }
    // gradients of one step: lam = dL/db_t, da = dL/da_t (0 at a reset) -> dz, dx
    static __device__ __forceinline__ void grads(float z, float x, float lam, float da, float &dz, float &dx)
    {
        float s, a;
        gates(z, s, a);
        dz = s * a * (g(x) * lam - da);  // sigma'(z) = s a; b = s g(x), a = 1 - s
        dx = lam * s * dg(x);
    }
};

constexpr int TS = 8;  // time steps a wave holds in registers per super-step

// Forward.  grid = B * tiles workgroups, block = 64 * NW threads, NW <= MAXW (8, or 16 for the
// one-vector-lane instances that small shapes take: with 16 waves of 8 steps a sequence of up to 128
// steps is one super-step, every load of the workgroup in flight at once and a single barrier).
// smem: sH[2][NW][64] Vec, sP[2][NW][64] Vec, sF[2][NW] int.
template <typename E, int VEC, bool MG = false, int MAXW = 8, typename S = E>
__global__ void __launch_bounds__(64 * MAXW)
diag_scan_fwd_kernel(const S *__restrict__ a, const S *__restrict__ b,
                     const void *__restrict__ done, int done_f32,
                     const E *__restrict__ h0, const E *__restrict__ P0,
                     S *__restrict__ h, E *__restrict__ h_last,
                     E *__restrict__ P_last, int T, int64_t D, int tiles, int NW,
                     int a_ti)
{
    using V = Vec<E, VEC>;
    using O = Ops<E>;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    V *sH = reinterpret_cast<V *>(smem_raw);
    V *sP = sH + 2 * NW * 64;
    int *sF = reinterpret_cast<int *>(sP + 2 * NW * 64);

    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tile = blockIdx.x % tiles;
    const int64_t bi = blockIdx.x / tiles;
    const int64_t col = ((int64_t)tile * 64 + lane) * VEC;
    const bool act = col < D;
    const int64_t row0 = bi * T;

    V carry_h = vfill<E, VEC>(O::zero()), carry_p = vfill<E, VEC>(O::one());
    if (act) {
        if (h0) carry_h = *reinterpret_cast<const V *>(h0 + bi * D + col);
        if (P0) carry_p = *reinterpret_cast<const V *>(P0 + bi * D + col);
    }

    const int span = NW * TS;
    int buf = 0;
    for (int t0 = 0; t0 < T; t0 += span) {
        const int ts = t0 + w * TS;
        V x[TS], p[TS];
        // reset flags of the wave's TS steps: lane s fetches the flag of step ts + s, one ballot makes the mask
        const unsigned rmask = (unsigned)__ballot(lane < TS && ts + lane < T && done_at(done, done_f32, row0 + ts + lane));
        raw_t<S, VEC> rp[TS], rx[TS];  // as stored; converted once every load of the super-step has been issued
#pragma unroll
        for (int s = 0; s < TS; ++s) {
            const int t = ts + s;
            if (t < T && act) {
                const int64_t off = (row0 + t) * D + col;
                rp[s] = ldraw<S, VEC>(a + (a_ti ? col : off));
                rx[s] = ldraw<S, VEC>(b + off);
            }
        }
#pragma unroll
        for (int s = 0; s < TS; ++s) {
            if (ts + s < T && act) {
                p[s] = cvtv<S, E, VEC>(rp[s]);
                x[s] = cvtv<S, E, VEC>(rx[s]);
            } else {
                p[s] = vfill<E, VEC>(O::one());
                x[s] = vfill<E, VEC>(O::zero());
            }
        }
        if constexpr (MG) {  // after every load of the super-step has been issued
#pragma unroll
            for (int s = 0; s < TS; ++s) {
                if (ts + s < T && act) {
#pragma unroll
                    for (int i = 0; i < VEC; ++i) MinGru::coeffs(p[s].v[i], x[s].v[i]);
                }
            }
        }
        if (NW == 1) {
            // no time split: continue straight from the carry
#pragma unroll
            for (int s = 0; s < TS; ++s) {
                const bool r = (rmask >> s) & 1u;
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    const E hn = O::madd(p[s].v[i], carry_h.v[i], x[s].v[i]);
                    const E pn = O::mul(p[s].v[i], carry_p.v[i]);
                    carry_h.v[i] = r ? x[s].v[i] : hn;
                    carry_p.v[i] = r ? p[s].v[i] : pn;
                }
                if (ts + s < T && act)
                    stv<S, E, VEC>(h + (row0 + ts + s) * D + col, carry_h);
            }
            continue;
        }
        // local inclusive scan from the identity; x <- h_local, p <- P_local
        {
            V hc = vfill<E, VEC>(O::zero()), pc = vfill<E, VEC>(O::one());
#pragma unroll
            for (int s = 0; s < TS; ++s) {
                const bool r = (rmask >> s) & 1u;
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    const E hn = O::madd(p[s].v[i], hc.v[i], x[s].v[i]);
                    const E pn = O::mul(p[s].v[i], pc.v[i]);
                    hc.v[i] = r ? x[s].v[i] : hn;
                    pc.v[i] = r ? p[s].v[i] : pn;
                }
                x[s] = hc;
                p[s] = pc;
            }
            sH[(buf * NW + w) * 64 + lane] = hc;
            sP[(buf * NW + w) * 64 + lane] = pc;
            if (lane == 0) sF[buf * NW + w] = rmask != 0;
        }
        __syncthreads();
        // fold the summaries: carry-in of this wave, then the workgroup carry
        V cin_h = carry_h, cin_p = carry_p, my_h = carry_h;
        for (int j = 0; j < NW; ++j) {
            if (j == w) my_h = cin_h;
            const V Hj = sH[(buf * NW + j) * 64 + lane];
            const V Pj = sP[(buf * NW + j) * 64 + lane];
            const bool fj = sF[buf * NW + j] != 0;
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                const E hn = O::madd(Pj.v[i], cin_h.v[i], Hj.v[i]);
                const E pn = O::mul(Pj.v[i], cin_p.v[i]);
                cin_h.v[i] = fj ? Hj.v[i] : hn;
                cin_p.v[i] = fj ? Pj.v[i] : pn;
            }
        }
        carry_h = cin_h;
        carry_p = cin_p;
#pragma unroll
        for (int s = 0; s < TS; ++s) {
            const bool seen = (rmask & ((2u << s) - 1u)) != 0;
            V out;
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                const E fx = O::madd(p[s].v[i], my_h.v[i], x[s].v[i]);
                out.v[i] = seen ? x[s].v[i] : fx;
            }
            if (ts + s < T && act)
                stv<S, E, VEC>(h + (row0 + ts + s) * D + col, out);
        }
        buf ^= 1;
    }
    if (w == 0 && act) {
        if (h_last) *reinterpret_cast<V *>(h_last + bi * D + col) = carry_h;
        if (P_last) *reinterpret_cast<V *>(P_last + bi * D + col) = carry_p;
    }
}

// Backward: the same scan walked from t = T-1 down with coefficient conj(a_{t+1}),
// cut where done_{t+1}; reversed index r = T-1-t runs forward.
// MG: a holds z, hx holds x = h~; da receives dz and db receives dx.
template <typename E, int VEC, bool MG = false, int MAXW = 8, typename S = E>
__global__ void __launch_bounds__(64 * MAXW)
diag_scan_bwd_kernel(const S *__restrict__ a, const S *__restrict__ hx, const S *__restrict__ hfw,
                     const void *__restrict__ done, int done_f32,
                     const E *__restrict__ h0, const S *__restrict__ g,
                     const E *__restrict__ g_last, S *__restrict__ da,
                     S *__restrict__ db, E *__restrict__ dh0, int T, int64_t D,
                     int tiles, int NW, int a_ti, int da_sum)
{
    using V = Vec<E, VEC>;
    using O = Ops<E>;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    V *sH = reinterpret_cast<V *>(smem_raw);
    V *sP = sH + 2 * NW * 64;
    int *sF = reinterpret_cast<int *>(sP + 2 * NW * 64);

    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tile = blockIdx.x % tiles;
    const int64_t bi = blockIdx.x / tiles;
    const int64_t col = ((int64_t)tile * 64 + lane) * VEC;
    const bool act = col < D;
    const int64_t row0 = bi * T;

    V carry = vfill<E, VEC>(O::zero());  // lam_{t+1} entering from the right
    if (act && g_last) carry = *reinterpret_cast<const V *>(g_last + bi * D + col);
    // da_sum (time-invariant a): da is (B,D), the sum of the per-step terms over the sequence -- what the
    // gradient of a broadcast coefficient needs -- kept in registers instead of written per step
    V dsum = vfill<E, VEC>(O::zero());

    const int span = NW * TS;
    int buf = 0;
    for (int r0 = 0; r0 < T; r0 += span) {
        const int rs = r0 + w * TS;
        // Everything the super-step reads is requested here, before the barrier: h_{t-1} (and the
        // MinGRU projections of step t) are only needed once lam_t is known, but a load issued after the
        // barrier would be a second trip to memory on the critical path.
        V x[TS], p[TS], hp[TS];
        V zt[MG ? TS : 1], xt[MG ? TS : 1];
        // reset flags: step s of the wave is t_s = T - 1 - (rs + s); lane l fetches done at T - rs - l, i.e.
        // done_{t_0 + 1}, done_{t_0}, done_{t_1}, ..., and one ballot serves both masks (steps before the
        // sequence's first, t_s < 0, take no bit: a cut there would drop the carry on its way to dh0)
        unsigned cmask, dmask;  // bit s: chain cut between step t_s and t_s + 1 (done_{t_s + 1}) / done_{t_s}
        {
            const int tt = T - rs - lane;
            const unsigned fl = (unsigned)__ballot(lane <= TS && tt >= 0 && tt < T && done_at(done, done_f32, row0 + tt));
            const int nv = T - rs < TS ? (T - rs < 0 ? 0 : T - rs) : TS;  // steps of the wave inside the sequence
            const unsigned vm = (1u << nv) - 1u;
            cmask = fl & vm;
            dmask = (fl >> 1) & vm;
        }
        if constexpr (std::is_same<S, E>::value) {
#pragma unroll
            for (int s = 0; s < TS; ++s) {
                const int t = T - 1 - (rs + s);
                p[s] = vfill<E, VEC>(O::one());
                x[s] = vfill<E, VEC>(O::zero());
                hp[s] = vfill<E, VEC>(O::zero());
                if (t >= 0 && act) {
                    const int64_t off = (row0 + t) * D + col;
                    x[s] = ldv<S, E, VEC>(g + off);
                    if (t + 1 < T) {
                        V av = ldv<S, E, VEC>(a + (a_ti ? col : off + D));
#pragma unroll
                        for (int i = 0; i < VEC; ++i) p[s].v[i] = MG ? av.v[i] : O::conj(av.v[i]);  // MG: z_{t+1} for now
                    }
                    if (t > 0)
                        hp[s] = ldv<S, E, VEC>(hfw + off - D);
                    else if (h0)
                        hp[s] = *reinterpret_cast<const V *>(h0 + bi * D + col);
                    if constexpr (MG) {
                        zt[s] = ldv<S, E, VEC>(a + off);
                        xt[s] = ldv<S, E, VEC>(hx + off);
                    }
                }
            }
        } else {
            // narrower storage: the values wait as stored and are widened once every load has been issued
            raw_t<S, VEC> rg[TS], ra[TS], rh[TS], rz[MG ? TS : 1], rxt[MG ? TS : 1];
            V h0v = vfill<E, VEC>(O::zero());  // h_{-1}: what step 0 multiplies its lam with
            if (act && h0 && T - 1 - rs - (TS - 1) <= 0) h0v = *reinterpret_cast<const V *>(h0 + bi * D + col);
#pragma unroll
            for (int s = 0; s < TS; ++s) {
                const int t = T - 1 - (rs + s);
                if (t >= 0 && act) {
                    const int64_t off = (row0 + t) * D + col;
                    rg[s] = ldraw<S, VEC>(g + off);
                    if (t + 1 < T) ra[s] = ldraw<S, VEC>(a + (a_ti ? col : off + D));
                    if (t > 0) rh[s] = ldraw<S, VEC>(hfw + off - D);
                    if constexpr (MG) {
                        rz[s] = ldraw<S, VEC>(a + off);
                        rxt[s] = ldraw<S, VEC>(hx + off);
                    }
                }
            }
#pragma unroll
            for (int s = 0; s < TS; ++s) {
                const int t = T - 1 - (rs + s);
                p[s] = vfill<E, VEC>(O::one());
                x[s] = vfill<E, VEC>(O::zero());
                hp[s] = vfill<E, VEC>(O::zero());
                if (t >= 0 && act) {
                    x[s] = cvtv<S, E, VEC>(rg[s]);
                    if (t + 1 < T) {
                        const V av = cvtv<S, E, VEC>(ra[s]);
#pragma unroll
                        for (int i = 0; i < VEC; ++i) p[s].v[i] = MG ? av.v[i] : O::conj(av.v[i]);  // MG: z_{t+1} for now
                    }
                    if (t > 0) hp[s] = cvtv<S, E, VEC>(rh[s]);
                    else hp[s] = h0v;
                    if constexpr (MG) {
                        zt[s] = cvtv<S, E, VEC>(rz[s]);
                        xt[s] = cvtv<S, E, VEC>(rxt[s]);
                    }
                }
            }
        }
        if constexpr (MG) {  // a_{t+1} = sigma(-z_{t+1}), after every load of the super-step has been issued
#pragma unroll
            for (int s = 0; s < TS; ++s) {
                const int t = T - 1 - (rs + s);
                if (t >= 0 && t + 1 < T && act) {
#pragma unroll
                    for (int i = 0; i < VEC; ++i) {
                        float sg;
                        MinGru::gates(p[s].v[i], sg, p[s].v[i]);
                    }
                }
            }
        }
        V my = carry;
        if (NW == 1) {
#pragma unroll
            for (int s = 0; s < TS; ++s) {
                const bool c = (cmask >> s) & 1u;
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    const E ln = O::madd(p[s].v[i], carry.v[i], x[s].v[i]);
                    carry.v[i] = c ? x[s].v[i] : ln;
                }
                x[s] = carry;
            }
        } else {
            V lc = vfill<E, VEC>(O::zero()), pc = vfill<E, VEC>(O::one());
#pragma unroll
            for (int s = 0; s < TS; ++s) {
                const bool c = (cmask >> s) & 1u;
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    const E ln = O::madd(p[s].v[i], lc.v[i], x[s].v[i]);
                    const E pn = O::mul(p[s].v[i], pc.v[i]);
                    lc.v[i] = c ? x[s].v[i] : ln;
                    pc.v[i] = c ? p[s].v[i] : pn;
                }
                x[s] = lc;
                p[s] = pc;
            }
            sH[(buf * NW + w) * 64 + lane] = lc;
            sP[(buf * NW + w) * 64 + lane] = pc;
            if (lane == 0) sF[buf * NW + w] = cmask != 0;
            __syncthreads();
            V cin = carry;
            for (int j = 0; j < NW; ++j) {
                if (j == w) my = cin;
                const V Hj = sH[(buf * NW + j) * 64 + lane];
                const V Pj = sP[(buf * NW + j) * 64 + lane];
                const bool fj = sF[buf * NW + j] != 0;
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    const E ln = O::madd(Pj.v[i], cin.v[i], Hj.v[i]);
                    cin.v[i] = fj ? Hj.v[i] : ln;
                }
            }
            carry = cin;
#pragma unroll
            for (int s = 0; s < TS; ++s) {
                const bool seen = (cmask & ((2u << s) - 1u)) != 0;
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    const E fx = O::madd(p[s].v[i], my.v[i], x[s].v[i]);
                    x[s].v[i] = seen ? x[s].v[i] : fx;
                }
            }
            buf ^= 1;
        }
        // x[s] = lam_t : emit db_t and da_t = done_t ? 0 : lam_t conj(h_{t-1})
#pragma unroll
        for (int s = 0; s < TS; ++s) {
            const int t = T - 1 - (rs + s);
            if (t >= 0 && act) {
                const int64_t off = (row0 + t) * D + col;
                const bool dn = (dmask >> s) & 1u;
                V o;
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    const E prod = O::mul(x[s].v[i], O::conj(hp[s].v[i]));
                    o.v[i] = dn ? O::zero() : prod;
                }
                if constexpr (MG) {
                    V oz, ox;
#pragma unroll
                    for (int i = 0; i < VEC; ++i) MinGru::grads(zt[s].v[i], xt[s].v[i], x[s].v[i], o.v[i], oz.v[i], ox.v[i]);
                    stv<S, E, VEC>(db + off, ox);
                    stv<S, E, VEC>(da + off, oz);
                } else {
                    stv<S, E, VEC>(db + off, x[s]);
                    if (da_sum) {
#pragma unroll
                        for (int i = 0; i < VEC; ++i) dsum.v[i] = O::madd(O::one(), dsum.v[i], o.v[i]);
                    } else {
                        stv<S, E, VEC>(da + off, o);
                    }
                }
            }
        }
    }
    if (!MG && da_sum) {  // uniform over the workgroup
        if (NW > 1) {
            __syncthreads();  // the last fold has read sH
            sH[w * 64 + lane] = dsum;
            __syncthreads();
            if (w == 0) {
                for (int j = 1; j < NW; ++j) {
                    const V dj = sH[j * 64 + lane];
#pragma unroll
                    for (int i = 0; i < VEC; ++i) dsum.v[i] = O::madd(O::one(), dsum.v[i], dj.v[i]);
                }
            }
        }
        if (w == 0 && act) *reinterpret_cast<V *>(reinterpret_cast<E *>(da) + bi * D + col) = dsum;  // (B,D), arithmetic type
    }
    if (w == 0 && act && dh0) {
        // carry = lam_0 ; dh0 = done_0 ? 0 : conj(a_0) lam_0
        const bool d0 = done_at(done, done_f32, row0);
        V a0 = ldv<S, E, VEC>(a + (a_ti ? col : row0 * D + col));
        if constexpr (MG) {
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                float sg;
                MinGru::gates(a0.v[i], sg, a0.v[i]);
            }
        }
        V o;
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const E prod = O::mul(O::conj(a0.v[i]), carry.v[i]);
            o.v[i] = d0 ? O::zero() : prod;
        }
        *reinterpret_cast<V *>(dh0 + bi * D + col) = o;
    }
}


// ---- streaming kernels: enough (batch x feature) columns to fill the chip ------------
// No time split.  Each lane walks all of T for its VEC channels in groups of SG steps,
// with the loads of the next group issued before the current group is consumed
// (register double buffering), so a wave always has 2*SG (forward) / 3*SG (backward)
// row loads in flight.  done flags are prefetched as raw bits with the data.
template <typename E, int VEC, int SG, bool MG = false, typename S = E, bool DF = false>
__global__ void __launch_bounds__(256)
diag_scan_fwd_stream_kernel(const S *__restrict__ a, const S *__restrict__ b,
                            const void *__restrict__ done, int,
                            const E *__restrict__ h0, const E *__restrict__ P0,
                            S *__restrict__ h, E *__restrict__ h_last, E *__restrict__ P_last,
                            int64_t B, int T, int64_t D, int64_t cols_per_row, int a_ti)
{
    using V = Vec<E, VEC>;
    using O = Ops<E>;
    // the flags' type is a template parameter here: with both kinds of load in the code the compiler reuses
    // registers of loads still in flight for the other kind's address and waits for them in mid-prefetch
    constexpr int done_f32 = DF;
    // one thread per VEC channels of one batch row
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t bi = gid / cols_per_row;
    const int64_t col = (gid % cols_per_row) * VEC;
    if (bi >= B) return;  // padding threads of the last workgroup (this kernel has no barriers)
    const int64_t row0 = bi * T;
    V ch = vfill<E, VEC>(O::zero()), cp = vfill<E, VEC>(O::one());
    if (h0) ch = *reinterpret_cast<const V *>(h0 + bi * D + col);
    if (P0) cp = *reinterpret_cast<const V *>(P0 + bi * D + col);

    using R = raw_t<S, VEC>;  // prefetched values stay as stored until they are consumed
    R xa[SG], xb[SG], na[SG], nb[SG];
    uint32_t xd[SG], nd[SG];
    auto load = [&](int t0, R *pa, R *pb, uint32_t *pd) {
#pragma unroll
        for (int s = 0; s < SG; ++s) {
            const int t = t0 + s;
            pd[s] = 0u;
            if (t < T) {
                const int64_t off = (row0 + t) * D + col;
                pa[s] = ldraw<S, VEC>(a + (a_ti ? col : off));
                pb[s] = ldraw<S, VEC>(b + off);
                pd[s] = done_raw(done, done_f32, row0 + t);
            }
        }
    };
    load(0, xa, xb, xd);
    for (int t0 = 0; t0 < T; t0 += SG) {
        if (t0 + SG < T) load(t0 + SG, na, nb, nd);
#pragma unroll
        for (int s = 0; s < SG; ++s) {
            if (t0 + s < T) {
                const bool r = done_test(xd[s], done_f32);
                V va = cvtv<S, E, VEC>(xa[s]), vb = cvtv<S, E, VEC>(xb[s]);
                if constexpr (MG) {  // here, not at the load: the loads stay in flight
#pragma unroll
                    for (int i = 0; i < VEC; ++i) MinGru::coeffs(va.v[i], vb.v[i]);
                }
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    const E hn = O::madd(va.v[i], ch.v[i], vb.v[i]);
                    const E pn = O::mul(va.v[i], cp.v[i]);
                    ch.v[i] = r ? vb.v[i] : hn;
                    cp.v[i] = r ? va.v[i] : pn;
                }
                stv<S, E, VEC>(h + (row0 + t0 + s) * D + col, ch);
            }
        }
#pragma unroll
        for (int s = 0; s < SG; ++s) { xa[s] = na[s]; xb[s] = nb[s]; xd[s] = nd[s]; }
    }
    if (h_last) *reinterpret_cast<V *>(h_last + bi * D + col) = ch;
    if (P_last) *reinterpret_cast<V *>(P_last + bi * D + col) = cp;
}

// ---- final state only, decay shared by groups of channels ---------------------------
// h_T of h_t = done_t ? b_t : a_t h_{t-1} + b_t where a:(B,T,D/a_group) holds one decay per
// a_group consecutive channels.  Nothing but the last state is written, so the traffic is one
// read of b.  This is the real-time-recurrent-learning sensitivity update
// (memoroid.py:114-141: S <- last(scan(a = where(done, 0, repeat(decay, param_size)), J))),
// without materialising the repeated decay or the per-step states.
template <typename E, int VEC, int SG>
__global__ void __launch_bounds__(256)
diag_scan_last_kernel(const E *__restrict__ a, const E *__restrict__ b, const void *__restrict__ done,
                      int done_f32, const E *__restrict__ h0, E *__restrict__ h_last, int64_t B, int T,
                      int64_t D, int64_t cols_per_row, int64_t a_group)
{
    using V = Vec<E, VEC>;
    using O = Ops<E>;
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t bi = gid / cols_per_row;
    const int64_t col = (gid % cols_per_row) * VEC;
    if (bi >= B) return;  // padding threads of the last workgroup (this kernel has no barriers)
    const int64_t row0 = bi * T, Da = D / a_group, acol = col / a_group;  // VEC divides a_group
    V ch = vfill<E, VEC>(O::zero());
    if (h0) ch = *reinterpret_cast<const V *>(h0 + bi * D + col);

    E xa[SG], na[SG];
    V xb[SG], nb[SG];
    uint32_t xd[SG], nd[SG];
    auto load = [&](int t0, E *pa, V *pb, uint32_t *pd) {
#pragma unroll
        for (int s = 0; s < SG; ++s) {
            const int t = t0 + s;
            pd[s] = 0u;
            if (t < T) {
                pa[s] = a[(row0 + t) * Da + acol];
                pb[s] = *reinterpret_cast<const V *>(b + (row0 + t) * D + col);
                pd[s] = done_raw(done, done_f32, row0 + t);
            }
        }
    };
    load(0, xa, xb, xd);
    for (int t0 = 0; t0 < T; t0 += SG) {
        if (t0 + SG < T) load(t0 + SG, na, nb, nd);
#pragma unroll
        for (int s = 0; s < SG; ++s) {
            if (t0 + s < T) {
                const bool r = done_test(xd[s], done_f32);
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    const E hn = O::madd(xa[s], ch.v[i], xb[s].v[i]);
                    ch.v[i] = r ? xb[s].v[i] : hn;
                }
            }
        }
#pragma unroll
        for (int s = 0; s < SG; ++s) { xa[s] = na[s]; xb[s] = nb[s]; xd[s] = nd[s]; }
    }
    *reinterpret_cast<V *>(h_last + bi * D + col) = ch;
}

// MG: a holds z, hx holds x = h~ (a fourth load per step); da receives dz and db receives dx.
// RECOMP (with MG): the kernel has what the forward pass had, so it reads only one row of h per group of SG
// steps -- the state entering the group -- and runs the recurrence forward through the group again for the
// states between: SG - 1 of SG rows of h not fetched (24 -> 20.5 bytes per element and step in float32) for the
// map's arithmetic a second time.  That pays where the call is bound by HBM and costs where its arrays fit the
// last-level cache (float32, 1024 x 128 x 256: 157 -> 138 us; 256 x 128 x 256: 46 -> 49 us; bfloat16 arrays,
// 1024 x 128 x 256: 80 -> 90 us, 512 x 1024 x 1024: 1.30 -> 1.19 ms): launch_bwd asks for it by the bytes moved.
template <typename E, int VEC, int SG, bool MG = false, typename S = E, bool DF = false, bool RECOMP = false>
__global__ void __launch_bounds__(256)
diag_scan_bwd_stream_kernel(const S *__restrict__ a, const S *__restrict__ hx, const S *__restrict__ hfw,
                            const void *__restrict__ done, int,
                            const E *__restrict__ h0, const S *__restrict__ g,
                            const E *__restrict__ g_last, S *__restrict__ da, S *__restrict__ db,
                            E *__restrict__ dh0, int64_t B, int T, int64_t D, int64_t cols_per_row, int a_ti,
                            int da_sum)
{
    using V = Vec<E, VEC>;
    using O = Ops<E>;
    // the flags' type is a template parameter here: with both kinds of load in the code the compiler reuses
    // registers of loads still in flight for the other kind's address and waits for them in mid-prefetch
    constexpr int done_f32 = DF;
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t bi = gid / cols_per_row;
    const int64_t col = (gid % cols_per_row) * VEC;
    if (bi >= B) return;
    const int64_t row0 = bi * T;
    V dsum = vfill<E, VEC>(O::zero());  // da_sum: the per-step terms summed over the sequence, da is (B,D)
    V lam = vfill<E, VEC>(O::zero());  // conj(abar_{t+1}) lam_{t+1} entering step t
    if (g_last) lam = *reinterpret_cast<const V *>(g_last + bi * D + col);

    // step r (reversed index), t = T-1-r: needs g_t, a_t (for the carry to t-1), h_{t-1}, done_t
    using R = raw_t<S, VEC>;  // prefetched values stay as stored until they are consumed
    static_assert(!RECOMP || MG, "the states can be formed again only where the map's inputs are at hand");
    constexpr int NH = RECOMP ? 1 : SG;  // rows of h per group
    R xg[SG], xa[SG], xh[NH], ng[SG], na[SG], nh[NH];
    R xx[MG ? SG : 1], nx[MG ? SG : 1];
    uint32_t xd[SG], nd[SG];
    V h0v = vfill<E, VEC>(O::zero());  // h_{-1}: what step 0 multiplies its lam with
    if (h0) h0v = *reinterpret_cast<const V *>(h0 + bi * D + col);
    auto load = [&](int r0, R *pg, R *pa, R *ph, R *px, uint32_t *pd) {
#pragma unroll
        for (int s = 0; s < SG; ++s) {
            const int t = T - 1 - (r0 + s);
            pd[s] = 0u;
            if (t >= 0) {
                const int64_t off = (row0 + t) * D + col;
                pg[s] = ldraw<S, VEC>(g + off);
                pa[s] = ldraw<S, VEC>(a + (a_ti ? col : off));
                if constexpr (MG) px[s] = ldraw<S, VEC>(hx + off);
                if constexpr (!RECOMP) {
                    if (t > 0) ph[s] = ldraw<S, VEC>(hfw + off - D);
                }
                pd[s] = done_raw(done, done_f32, row0 + t);
            }
        }
        if constexpr (RECOMP) {  // the state entering the group's earliest step
            const int t_lo = T - r0 - SG;
            if (t_lo > 0) ph[0] = ldraw<S, VEC>(hfw + (row0 + t_lo - 1) * D + col);
        }
    };
    load(0, xg, xa, xh, xx, xd);
    for (int r0 = 0; r0 < T; r0 += SG) {
        if (r0 + SG < T) load(r0 + SG, ng, na, nh, nx, nd);
        V hprev[RECOMP ? SG : 1];  // h_{t-1} of the group's steps, by the recurrence from the state entering the group
        if constexpr (RECOMP) {
            V hc = h0v;
            if (T - r0 - SG > 0) hc = cvtv<S, E, VEC>(xh[0]);
#pragma unroll
            for (int s = SG - 1; s >= 0; --s) {  // forward in time
                const int t = T - 1 - (r0 + s);
                if (t >= 0) {
                    hprev[s] = hc;
                    const bool dn = done_test(xd[s], done_f32);
                    const V va = cvtv<S, E, VEC>(xa[s]), vx = cvtv<S, E, VEC>(xx[s]);
#pragma unroll
                    for (int i = 0; i < VEC; ++i) {
                        float ca = va.v[i], cb = vx.v[i];
                        MinGru::coeffs(ca, cb);
                        hc.v[i] = dn ? cb : O::madd(ca, hc.v[i], cb);
                    }
                }
            }
        }
#pragma unroll
        for (int s = 0; s < SG; ++s) {
            const int t = T - 1 - (r0 + s);
            if (t >= 0) {
                const bool dn = done_test(xd[s], done_f32);
                const int64_t off = (row0 + t) * D + col;
                const V vg = cvtv<S, E, VEC>(xg[s]), va = cvtv<S, E, VEC>(xa[s]);
                V vh = h0v, vx;
                if constexpr (MG) vx = cvtv<S, E, VEC>(xx[s]);
                if constexpr (RECOMP) {
                    vh = hprev[s];
                } else {
                    if (t > 0) vh = cvtv<S, E, VEC>(xh[s]);
                }
                V l, o;
#pragma unroll
                for (int i = 0; i < VEC; ++i) {
                    l.v[i] = O::madd(O::one(), vg.v[i], lam.v[i]);  // lam_t = g_t + carried term
                    const E prod = O::mul(l.v[i], O::conj(vh.v[i]));
                    o.v[i] = dn ? O::zero() : prod;
                    if constexpr (MG) {
                        float sg, at, dz, dx;
                        MinGru::gates(va.v[i], sg, at);
                        MinGru::grads(va.v[i], vx.v[i], l.v[i], o.v[i], dz, dx);
                        lam.v[i] = dn ? 0.0f : at * l.v[i];
                        o.v[i] = dz;
                        l.v[i] = dx;
                    } else {
                        const E nxt = O::mul(O::conj(va.v[i]), l.v[i]);
                        lam.v[i] = dn ? O::zero() : nxt;           // conj(abar_t) lam_t for step t-1
                    }
                }
                stv<S, E, VEC>(db + off, l);
                if (!MG && da_sum) {
#pragma unroll
                    for (int i = 0; i < VEC; ++i) dsum.v[i] = O::madd(O::one(), dsum.v[i], o.v[i]);
                } else {
                    stv<S, E, VEC>(da + off, o);
                }
            }
        }
#pragma unroll
        for (int s = 0; s < SG; ++s) { xg[s] = ng[s]; xa[s] = na[s]; xd[s] = nd[s]; }
#pragma unroll
        for (int s = 0; s < NH; ++s) xh[s] = nh[s];
        if constexpr (MG) {
#pragma unroll
            for (int s = 0; s < SG; ++s) xx[s] = nx[s];
        }
    }
    if (!MG && da_sum) *reinterpret_cast<V *>(reinterpret_cast<E *>(da) + bi * D + col) = dsum;  // (B,D), arithmetic type
    if (dh0) *reinterpret_cast<V *>(dh0 + bi * D + col) = lam;  // conj(abar_0) lam_0
}

struct ScanPlan {
    int vec, nw, tiles;
    bool stream;  // streaming kernel (no time split) instead of the wave-split kernel
};

// Which kernel, how many elements per lane and how many waves along time.  Two layers of rules: the first
// block in the function body (sequences of 32 steps and more) comes from one sweep over every plan and
// takes precedence; what follows it are the earlier rules, which still decide the cases that block leaves
// open and all shorter sequences.  The earlier rules, as they were derived
// (fp32; 512x1024x1024, 1024x128x256, 64x512x512, 32x128x256):
//  - widest vector the shapes/alignments allow, narrowed until there are >= 2048 wave columns;
//  - forward: split time over up to 8 waves until ~8192 waves exist (the wave-split kernel at
//    4 waves reached 5.7 TB/s on the 6.4 GB shape, the streaming kernel 5.1 TB/s); with no
//    split left to do, stream; shapes so small that eight waves per workgroup still leave the
//    device short of waves (one vector lane per thread by then) take sixteen, which makes a
//    sequence of up to 128 steps a single super-step: the kernel's time is then one trip to
//    memory and back instead of one per super-step;
//  - backward (three loads per step) prefers wide vectors: the widest one that still gives 4096 waves
//    with the time axis split over eight waves -- or, for one or two lanes per thread, sixteen --
//    takes the wave-split kernel (512x1024x1024: 1.91 ms = 5.6 TB/s against 2.12 ms streaming;
//    1024x128x256: 135 us either way; 256x128x256: 28 against 39 us; 64x512x512: 77 against 111 us);
//    shapes too small for that fall to the rule of the forward pass, and otherwise the streaming
//    kernel runs whenever the columns alone give >= 2048 waves.  With the MinGRU map inside (a
//    fourth stream and the map's arithmetic per element) the eight-wave split loses to streaming at
//    1024x128x256 (202 vs 165 us; level at the large shape), so that case keeps the rule it had.
ScanPlan plan_scan(int64_t B, int64_t T, int64_t D, size_t esize, bool al16, bool al8, bool bwd, bool mg = false,
                   bool half_storage = false)
{
    const int maxvec = (int)(16 / esize);
    int vec = 1;
    for (int v = maxvec; v >= 1; v >>= 1) {
        const size_t bytes = esize * v;
        const bool ok_al = bytes == 16 ? al16 : (bytes == 8 ? al8 : true);
        // a vector so wide that the waves covering a row are less than three quarters full wastes the
        // idle lanes' share of every load (rows of 128 floats, backward: 0.87 -> 0.57 ms at 16384x64x128
        // with two floats per lane instead of four; rows of 64: 0.75 -> 0.36 ms)
        const int64_t covered = ((D + 64 * (int64_t)v - 1) / (64 * (int64_t)v)) * 64 * v;
        if (D % v == 0 && ok_al && (v == 1 || 4 * D >= 3 * covered)) { vec = v; break; }
    }
    auto ntiles = [&](int v) { return (D + 64 * (int64_t)v - 1) / (64 * (int64_t)v); };
    // ---- Sequences of 32 steps and more: rules from a sweep of every plan (vector 1/2/4 x streaming or
    // 2..16 waves along time) over twenty-two shapes of 16..16384 sequences x 16..4096 steps x 64..1024
    // columns, for each kind of scan (float32, MinGRU map, bfloat16 arrays, complex64) and direction, timed
    // with 512 MB of other traffic between two launches so that no shape is served from the last-level cache.
    // Geometric mean of time over the best plan's, these rules / the rules below alone: float32 1.00 / 1.07
    // forward and 1.02 / 1.04 backward, MinGRU 1.00 / 1.06 and 1.02 / 1.05, bfloat16 1.01 / 1.40 and
    // 1.00 / 1.21, complex64 1.01 / 1.08 and 1.03 / 1.07; no shape more than 9 % off its best plan but one.
    // The sweep was repeated after the arrays' loads and stores had become non-temporal: two float32 rules
    // changed (marked below); against the new timings the rules stand at 1.03 / 1.02 (float32), 1.03 / 1.02
    // (MinGRU), 1.02 / 1.00 (bfloat16) and 1.02 / 1.01 (complex64).
    if (T >= 4 * TS) {
        auto cols = [&](int v) { return B * ntiles(v); };  // workgroups of the wave-split kernel
        auto split = [&](int v, int n) { return ScanPlan{v, n, (int)ntiles(v), false}; };
        int nw8 = 1;  // waves along time: up to eight, each with a whole group of steps to itself
        while (nw8 < 8 && (int64_t)2 * nw8 * TS <= T) nw8 <<= 1;
        // so few columns that eight waves along time leave most of the device idle: sixteen of one lane each
        if (T >= 16 * TS && cols(1) <= 256) return split(1, 16);
        if (half_storage) {
            // (swept again once the bfloat16 values waited as stored bits: the wave-split kernels then lead
            // forward at every size; four elements per lane, backward, do not fit the wave-split kernel's
            // registers)
            const int v = vec < 2 ? vec : 2;
            if (!bwd) return split(v, cols(v) >= 1024 && nw8 > 4 ? 4 : nw8);
            // the streaming kernels lay their threads flat over (row, column): a row need not fill whole waves
            if (D % 2 == 0 && al8 && B * D / 128 >= 2048) return {2, 1, (int)ntiles(2), true};
            return split(v, cols(v) >= 512 && nw8 > 4 ? 4 : nw8);
        }
        if (esize == 8 && !mg) {
            if (!bwd && T <= 256) return split(1, nw8);
            if (bwd && vec == 2 && (cols(2) >= 1024 || (cols(2) >= 256 && T >= 64 * TS))) return split(2, nw8);
        }
        if (esize == 4) {
            if (!bwd) {
                // (swept again once every array was loaded and stored non-temporally: two elements per lane
                // then lead at the large shapes as well -- 512 x 1024 x 1024 forward 1067 -> 1009 us,
                // 4096 x 128 x 256 291 -> 269 us -- where four used to)
                return split(vec < 2 ? vec : 2, nw8);
            }
            if (mg) {
                if (vec == 4 && cols(4) >= 2048 && T >= 8 * TS) return split(4, nw8 > 4 ? 4 : nw8);
                if (D <= 128 && cols(1) >= 2048) return split(1, nw8);
            } else {
                if (D <= 128 && cols(1) >= 1024) return split(1, nw8);
                if (T >= 8 * TS) {
                    for (int v = vec; v >= 1; v >>= 1) {
                        // rows of a single column tile take eight waves along time, wider rows four (the same
                        // sweep: 8192 x 128 x 256 backward 1007 -> 920 us, 256 x 128 x 1024 149 -> 132 us)
                        if (cols(v) >= 1024) return split(v, ntiles(v) == 1 ? 8 : 4);
                        if (cols(v) * 8 >= 4096) return split(v, 8);
                        if (v <= 2 && cols(v) * 16 >= 4096 && T >= 16 * TS) return split(v, 16);
                    }
                }
            }
        }
    }
    // ---- what the sweep above left as it was, and sequences shorter than 32 steps ----
    // bfloat16 arrays: a lane's loads are half as wide, so the widest vector stays (no narrowing for the sake
    // of more columns); measured on the MinGRU kernels at 1024x128x256, 512x1024x1024, 256x128x256: with 1024
    // waves of columns the streaming kernel is ahead or level (backward 186 -> 161 us, forward of the largest
    // shape 1412 -> 875 us), below that eight waves along time (backward 88 -> 44 us at 256x128x256)
    if (half_storage) {
        const int64_t cols = B * ntiles(vec);
        if (cols >= 1024) return {vec, 1, (int)ntiles(vec), true};
        int nw = 1;
        while (nw < 8 && cols * nw < 2048 && (int64_t)nw * TS < T) nw <<= 1;
        return {vec, nw, (int)ntiles(vec), nw == 1};
    }
    // complex64 (measured on 1024x128x{64,128,256}, 4096x128x64, 256x1024x{64,256}, 64x4096x256): one
    // element per lane is the width the column rule below arrives at for most shapes, and at that width
    // the streaming kernel is ahead of the wave-split one as soon as the columns give it 2048 waves
    // (forward 111 -> 93 us at 1024x128x128, 242 -> 180 us at 4096x128x64) or, backward, 1024 waves
    // (146 -> 70 us at 1024x128x64; 990 -> 520 us at 256x1024x256); where the 16-byte vector would be
    // narrowed for lack of columns but eight waves along time make up for them, it is kept (forward
    // 399 -> 328 us at 256x1024x256).
    if (esize == 8 && !mg) {
        int v1 = vec;
        while (v1 > 1 && B * ntiles(v1) < 2048) v1 >>= 1;
        const int64_t waves1 = B * ntiles(v1);
        if (v1 == 1 && waves1 >= (bwd ? 1024 : 2048)) return {1, 1, (int)ntiles(1), true};
        if (vec == 2 && v1 == 1 && B * ntiles(2) * 8 >= 4096 && T >= 8 * TS) return {2, 8, (int)ntiles(2), false};
    }
    // floats, backward: see above; rows of up to 128 floats first -- there a wave's loads in the
    // wave-split kernel are short pieces, and one column per lane in the streaming kernel is ahead
    // wherever it gets 1024 waves (4096x128x64: 193 -> 137 us, 1024x1024x64: 456 -> 303 us,
    // 1024x128x128: 84 -> 69 us, 8192x128x128: 585 -> 545 us)
    if (bwd && !mg && esize == 4 && D <= 128 && B * ntiles(1) >= 1024) return {1, 1, (int)ntiles(1), true};
    if (bwd && !mg && esize == 4) {
        for (int v = vec; v >= 1; v >>= 1) {
            const int64_t cols = B * ntiles(v);
            if (cols * 8 >= 4096 && T >= 8 * TS) return {v, 8, (int)ntiles(v), false};
            if (v <= 2 && cols * 16 >= 4096 && T >= 16 * TS) return {v, 16, (int)ntiles(v), false};
        }
    }
    while (vec > 1 && B * ntiles(vec) < 2048) vec >>= 1;
    const int tiles = (int)ntiles(vec);
    const int64_t waves = B * tiles;
    int nw = 1;
    const int maxw = vec == 1 ? 16 : 8;
    while (nw < maxw && waves * nw < 8192 && (int64_t)nw * TS < T) nw <<= 1;
    const bool stream = bwd ? waves >= 2048 : nw == 1;
    // MinGRU backward short of columns for that: one column per lane still streams ahead of the wave-split
    // kernel from 1024 waves (1024x128x64: 55 -> 45 us, 256x1024x256: 472 -> 332 us)
    if (bwd && mg && !stream && B * ntiles(1) >= 1024) return {1, 1, (int)ntiles(1), true};
    return {vec, stream ? 1 : nw, tiles, stream};
}

size_t scan_smem(int nw, size_t vbytes)
{
    return nw == 1 ? 0 : 2 * (size_t)nw * 64 * vbytes * 2 + 2 * (size_t)nw * sizeof(int);
}

// dispatch on the compile-time vector width: f(std::integral_constant<int, VEC>)
template <typename E, typename F> void vec_switch(int vec, F f)
{
    if constexpr (sizeof(E) == 4) {
        if (vec == 4) f(std::integral_constant<int, 4>{});
        else if (vec == 2) f(std::integral_constant<int, 2>{});
        else f(std::integral_constant<int, 1>{});
    } else {
        if (vec == 2) f(std::integral_constant<int, 2>{});
        else f(std::integral_constant<int, 1>{});
    }
}

// MG (E = float): a and b hold the MinGRU projections z and h~.
// S: storage type of the (B,T,D) arrays (E, or __bf16 with E = float).
template <typename E, bool MG = false, typename S = E>
int launch_fwd(hipStream_t st, const void *a, const void *b, const void *done,
               int done_f32, const void *h0, const void *P0, void *h, void *h_last,
               void *P_last, int64_t B, int64_t T, int64_t D, int a_ti)
{
    const bool al16 = aligned(a, 16) && aligned(b, 16) && aligned(h, 16) && aligned(h0, 16) &&
                      aligned(P0, 16) && aligned(h_last, 16) && aligned(P_last, 16);
    const bool al8 = aligned(a, 8) && aligned(b, 8) && aligned(h, 8) && aligned(h0, 8) &&
                     aligned(P0, 8) && aligned(h_last, 8) && aligned(P_last, 8);
    const ScanPlan pl = plan_scan(B, T, D, sizeof(E), al16, al8, false, MG, !std::is_same<S, E>::value);
    int rc = MRX_ERR_LAUNCH;
    if (pl.stream) {
        const int64_t cpr = D / pl.vec;
        const dim3 grid((unsigned)((B * cpr + 255) / 256)), block(256);
        vec_switch<E>(pl.vec, [&](auto vc) {
            constexpr int VEC = decltype(vc)::value;
            auto go = [&](auto df) {
                rc = launch_kernel((diag_scan_fwd_stream_kernel<E, VEC, (VEC * sizeof(E) == 16 ? 4 : 8), MG, S, decltype(df)::value>),
                                   grid, block, 0, st, (const S *)a, (const S *)b, done, done_f32, (const E *)h0,
                                   (const E *)P0, (S *)h, (E *)h_last, (E *)P_last, B, (int)T, D, cpr, a_ti);
            };
            if (done_f32) go(std::true_type{});
            else go(std::false_type{});
        });
    } else {
        const dim3 grid((unsigned)(B * pl.tiles)), block(64 * pl.nw);
        const size_t smem = scan_smem(pl.nw, sizeof(E) * pl.vec);
        vec_switch<E>(pl.vec, [&](auto vc) {
            constexpr int VEC = decltype(vc)::value;
            if constexpr (VEC == 1) {
                if (pl.nw == 16) {
                    rc = launch_kernel((diag_scan_fwd_kernel<E, 1, MG, 16, S>), grid, block, smem, st, (const S *)a,
                                       (const S *)b, done, done_f32, (const E *)h0, (const E *)P0, (S *)h,
                                       (E *)h_last, (E *)P_last, (int)T, D, pl.tiles, pl.nw, a_ti);
                    return;
                }
            }
            rc = launch_kernel((diag_scan_fwd_kernel<E, VEC, MG, 8, S>), grid, block, smem, st, (const S *)a,
                               (const S *)b, done, done_f32, (const E *)h0, (const E *)P0, (S *)h,
                               (E *)h_last, (E *)P_last, (int)T, D, pl.tiles, pl.nw, a_ti);
        });
    }
    return rc;
}

// MG (E = float): a holds z, hx holds h~ (else unused), da and db receive dz and dh~.
template <typename E, bool MG = false, typename S = E>
int launch_bwd(hipStream_t st, const void *a, const void *hx, const void *h, const void *done,
               int done_f32, const void *h0, const void *g, const void *g_last, void *da,
               void *db, void *dh0, int64_t B, int64_t T, int64_t D, int a_ti, int da_sum = 0)
{
    const bool al16 = aligned(a, 16) && aligned(hx, 16) && aligned(h, 16) && aligned(g, 16) && aligned(h0, 16) &&
                      aligned(g_last, 16) && aligned(da, 16) && aligned(db, 16) && aligned(dh0, 16);
    const bool al8 = aligned(a, 8) && aligned(hx, 8) && aligned(h, 8) && aligned(g, 8) && aligned(h0, 8) &&
                     aligned(g_last, 8) && aligned(da, 8) && aligned(db, 8) && aligned(dh0, 8);
    const ScanPlan pl = plan_scan(B, T, D, sizeof(E), al16, al8, true, MG, !std::is_same<S, E>::value);
    int rc = MRX_ERR_LAUNCH;
    if (pl.stream) {
        const int64_t cpr = D / pl.vec;
        const dim3 grid((unsigned)((B * cpr + 255) / 256)), block(256);
        vec_switch<E>(pl.vec, [&](auto vc) {
            constexpr int VEC = decltype(vc)::value;
            auto go = [&](auto df, auto rcmp) {
                rc = launch_kernel((diag_scan_bwd_stream_kernel<E, VEC, (VEC * sizeof(E) == 16 ? 4 : 8), MG, S, decltype(df)::value,
                                                                decltype(rcmp)::value>),
                                   grid, block, 0, st, (const S *)a, (const S *)hx, (const S *)h, done, done_f32,
                                   (const E *)h0, (const S *)g, (const E *)g_last, (S *)da, (S *)db, (E *)dh0, B, (int)T, D,
                                   cpr, a_ti, da_sum);
            };
            // six (B,T,D) arrays pass through the call: more than twice the 256 MB of last-level cache, and the
            // call is bound by HBM -- then h is better formed again than fetched
            const bool recompute = MG && 6.0 * (double)B * (double)T * (double)D * sizeof(S) >= 600e6;
            if constexpr (MG) {
                if (recompute) {
                    if (done_f32) go(std::true_type{}, std::true_type{});
                    else go(std::false_type{}, std::true_type{});
                    return;
                }
            }
            if (done_f32) go(std::true_type{}, std::false_type{});
            else go(std::false_type{}, std::false_type{});
        });
    } else {
        const dim3 grid((unsigned)(B * pl.tiles)), block(64 * pl.nw);
        const size_t smem = scan_smem(pl.nw, sizeof(E) * pl.vec);
        vec_switch<E>(pl.vec, [&](auto vc) {
            constexpr int VEC = decltype(vc)::value;
            if constexpr (VEC == 1 || (VEC == 2 && sizeof(E) == 4 && !MG)) {
                if (pl.nw == 16) {
                    rc = launch_kernel((diag_scan_bwd_kernel<E, VEC, MG, 16, S>), grid, block, smem, st, (const S *)a,
                                       (const S *)hx, (const S *)h, done, done_f32, (const E *)h0, (const S *)g,
                                       (const E *)g_last, (S *)da, (S *)db, (E *)dh0, (int)T, D, pl.tiles,
                                       pl.nw, a_ti, da_sum);
                    return;
                }
            }
            rc = launch_kernel((diag_scan_bwd_kernel<E, VEC, MG, 8, S>), grid, block, smem, st, (const S *)a,
                               (const S *)hx, (const S *)h, done, done_f32, (const E *)h0, (const S *)g,
                               (const E *)g_last, (S *)da, (S *)db, (E *)dh0, (int)T, D, pl.tiles,
                               pl.nw, a_ti, da_sum);
        });
    }
    return rc;
}

template <typename E>
int launch_last(hipStream_t st, const void *a, const void *b, const void *done, int done_f32,
                const void *h0, void *h_last, int64_t B, int64_t T, int64_t D, int64_t a_group)
{
    const int maxvec = (int)(16 / sizeof(E));
    int vec = 1;
    for (int v = maxvec; v >= 1; v >>= 1) {
        const size_t bytes = sizeof(E) * v;
        if (D % v == 0 && a_group % v == 0 && aligned(b, bytes) && aligned(h0, bytes) && aligned(h_last, bytes)) {
            vec = v;
            break;
        }
    }
    while (vec > 1 && B * (D / vec) < 2048 * 64) vec >>= 1;  // keep at least 2048 waves when the shape allows
    const int64_t cpr = D / vec;
    const dim3 grid((unsigned)((B * cpr + 255) / 256)), block(256);
    int rc = MRX_ERR_LAUNCH;
    vec_switch<E>(vec, [&](auto vc) {
        constexpr int VEC = decltype(vc)::value;
        rc = launch_kernel((diag_scan_last_kernel<E, VEC, (VEC * sizeof(E) == 16 ? 4 : 8)>), grid, block, 0, st,
                           (const E *)a, (const E *)b, done, done_f32, (const E *)h0, (E *)h_last, B, (int)T, D,
                           cpr, a_group);
    });
    return rc;
}

bool scan_shape_ok(int64_t B, int64_t T, int64_t D)
{
    return B > 0 && T > 0 && D > 0 && T < (1ll << 30) && B * ((D + 63) / 64) < (1ll << 31);
}

}  // namespace

extern "C" int mrx_linear_scan_fwd(void *stream, const void *a, const void *b, const void *done,
                                   const void *h0, const void *P0, void *h, void *h_last,
                                   void *P_last, int64_t B, int64_t T, int64_t D, int dtype,
                                   int done_dtype, int a_time_invariant)
{
    if (!a || !b || !done || !h) return MRX_ERR_INVALID_ARG;
    if (!scan_shape_ok(B, T, D)) return MRX_ERR_INVALID_ARG;
    if (done_dtype != MRX_DONE_U8 && done_dtype != MRX_DONE_F32) return MRX_ERR_INVALID_ARG;
    if (done_dtype == MRX_DONE_F32 && !aligned(done, 4)) return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    const int ti = a_time_invariant != 0;
    if (dtype == MRX_F32) {
        if (!aligned(a, 4) || !aligned(b, 4) || !aligned(h, 4)) return MRX_ERR_INVALID_ARG;
        return launch_fwd<float>(st, a, b, done, done_dtype, h0, P0, h, h_last, P_last, B, T, D, ti);
    }
    if (dtype == MRX_C64) {
        if (!aligned(a, 8) || !aligned(b, 8) || !aligned(h, 8) || !aligned(h0, 8) ||
            !aligned(P0, 8) || !aligned(h_last, 8) || !aligned(P_last, 8))
            return MRX_ERR_INVALID_ARG;
        return launch_fwd<c64>(st, a, b, done, done_dtype, h0, P0, h, h_last, P_last, B, T, D, ti);
    }
    if (dtype == MRX_BF16) {  // a, b, h in bfloat16; arithmetic and carries in float32
        if (!aligned(a, 2) || !aligned(b, 2) || !aligned(h, 2) || !aligned(h0, 4) || !aligned(P0, 4) ||
            !aligned(h_last, 4) || !aligned(P_last, 4))
            return MRX_ERR_INVALID_ARG;
        return launch_fwd<float, false, __bf16>(st, a, b, done, done_dtype, h0, P0, h, h_last, P_last, B, T, D, ti);
    }
    return MRX_ERR_INVALID_ARG;
}

extern "C" int mrx_linear_scan_bwd(void *stream, const void *a, const void *h, const void *done,
                                   const void *h0, const void *g, const void *g_last, void *da,
                                   void *db, void *dh0, int64_t B, int64_t T, int64_t D,
                                   int dtype, int done_dtype, int a_time_invariant)
{
    if (!a || !h || !done || !g || !da || !db) return MRX_ERR_INVALID_ARG;
    if (!scan_shape_ok(B, T, D)) return MRX_ERR_INVALID_ARG;
    if (done_dtype != MRX_DONE_U8 && done_dtype != MRX_DONE_F32) return MRX_ERR_INVALID_ARG;
    if (done_dtype == MRX_DONE_F32 && !aligned(done, 4)) return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    if (a_time_invariant < 0 || a_time_invariant > MRX_A_TIME_INVARIANT_SUM_DA) return MRX_ERR_INVALID_ARG;
    const int ti = a_time_invariant != 0;
    const int da_sum = a_time_invariant == MRX_A_TIME_INVARIANT_SUM_DA;
    if (dtype == MRX_F32) {
        if (!aligned(a, 4) || !aligned(h, 4) || !aligned(g, 4) || !aligned(da, 4) || !aligned(db, 4))
            return MRX_ERR_INVALID_ARG;
        return launch_bwd<float>(st, a, nullptr, h, done, done_dtype, h0, g, g_last, da, db, dh0, B, T, D, ti, da_sum);
    }
    if (dtype == MRX_C64) {
        if (!aligned(a, 8) || !aligned(h, 8) || !aligned(g, 8) || !aligned(da, 8) ||
            !aligned(db, 8) || !aligned(h0, 8) || !aligned(g_last, 8) || !aligned(dh0, 8))
            return MRX_ERR_INVALID_ARG;
        return launch_bwd<c64>(st, a, nullptr, h, done, done_dtype, h0, g, g_last, da, db, dh0, B, T, D, ti, da_sum);
    }
    if (dtype == MRX_BF16) {  // a, h, g, da (per step), db in bfloat16; carries and a summed da in float32
        if (!aligned(a, 2) || !aligned(h, 2) || !aligned(g, 2) || !aligned(da, da_sum ? 4 : 2) || !aligned(db, 2) ||
            !aligned(h0, 4) || !aligned(g_last, 4) || !aligned(dh0, 4))
            return MRX_ERR_INVALID_ARG;
        return launch_bwd<float, false, __bf16>(st, a, nullptr, h, done, done_dtype, h0, g, g_last, da, db, dh0, B, T, D,
                                                ti, da_sum);
    }
    return MRX_ERR_INVALID_ARG;
}

extern "C" int mrx_linear_scan_last(void *stream, const void *a, const void *b, const void *done,
                                    const void *h0, void *h_last, int64_t B, int64_t T, int64_t D,
                                    int64_t a_group, int dtype, int done_dtype)
{
    if (!a || !b || !done || !h_last) return MRX_ERR_INVALID_ARG;
    if (!scan_shape_ok(B, T, D) || a_group <= 0 || D % a_group != 0) return MRX_ERR_INVALID_ARG;
    if (B * D >= (1ll << 38)) return MRX_ERR_INVALID_ARG;  // grid size
    if (done_dtype != MRX_DONE_U8 && done_dtype != MRX_DONE_F32) return MRX_ERR_INVALID_ARG;
    if (done_dtype == MRX_DONE_F32 && !aligned(done, 4)) return MRX_ERR_INVALID_ARG;
    hipStream_t st = (hipStream_t)stream;
    if (dtype == MRX_F32) {
        if (!aligned(a, 4) || !aligned(b, 4) || !aligned(h0, 4) || !aligned(h_last, 4)) return MRX_ERR_INVALID_ARG;
        return launch_last<float>(st, a, b, done, done_dtype, h0, h_last, B, T, D, a_group);
    }
    if (dtype == MRX_C64) {
        if (!aligned(a, 8) || !aligned(b, 8) || !aligned(h0, 8) || !aligned(h_last, 8)) return MRX_ERR_INVALID_ARG;
        return launch_last<c64>(st, a, b, done, done_dtype, h0, h_last, B, T, D, a_group);
    }
    return dtype == MRX_BF16 ? MRX_ERR_UNSUPPORTED : MRX_ERR_INVALID_ARG;
}

extern "C" int mrx_mingru_scan_fwd(void *stream, const void *z, const void *h_tilde, const void *done,
                                   const void *h0, const void *P0, void *h, void *h_last, void *P_last,
                                   int64_t B, int64_t T, int64_t D, int dtype, int done_dtype)
{
    if (!z || !h_tilde || !done || !h) return MRX_ERR_INVALID_ARG;
    if (!scan_shape_ok(B, T, D)) return MRX_ERR_INVALID_ARG;
    if (dtype != MRX_F32 && dtype != MRX_BF16) return dtype == MRX_C64 ? MRX_ERR_UNSUPPORTED : MRX_ERR_INVALID_ARG;
    if (done_dtype != MRX_DONE_U8 && done_dtype != MRX_DONE_F32) return MRX_ERR_INVALID_ARG;
    if (done_dtype == MRX_DONE_F32 && !aligned(done, 4)) return MRX_ERR_INVALID_ARG;
    const size_t ea = dtype == MRX_BF16 ? 2 : 4;  // z, h~, h in `dtype`; the carries in float32
    for (const void *p : {z, h_tilde, (const void *)h})
        if (!aligned(p, ea)) return MRX_ERR_INVALID_ARG;
    for (const void *p : {h0, P0, (const void *)h_last, (const void *)P_last})
        if (!aligned(p, 4)) return MRX_ERR_INVALID_ARG;
    if (dtype == MRX_BF16)
        return launch_fwd<float, true, __bf16>((hipStream_t)stream, z, h_tilde, done, done_dtype, h0, P0, h, h_last,
                                               P_last, B, T, D, 0);
    return launch_fwd<float, true>((hipStream_t)stream, z, h_tilde, done, done_dtype, h0, P0, h, h_last, P_last, B, T,
                                   D, 0);
}

extern "C" int mrx_mingru_scan_bwd(void *stream, const void *z, const void *h_tilde, const void *h,
                                   const void *done, const void *h0, const void *g, const void *g_last,
                                   void *dz, void *dh_tilde, void *dh0, int64_t B, int64_t T, int64_t D,
                                   int dtype, int done_dtype)
{
    if (!z || !h_tilde || !h || !done || !g || !dz || !dh_tilde) return MRX_ERR_INVALID_ARG;
    if (!scan_shape_ok(B, T, D)) return MRX_ERR_INVALID_ARG;
    if (dtype != MRX_F32 && dtype != MRX_BF16) return dtype == MRX_C64 ? MRX_ERR_UNSUPPORTED : MRX_ERR_INVALID_ARG;
    if (done_dtype != MRX_DONE_U8 && done_dtype != MRX_DONE_F32) return MRX_ERR_INVALID_ARG;
    if (done_dtype == MRX_DONE_F32 && !aligned(done, 4)) return MRX_ERR_INVALID_ARG;
    const size_t ea = dtype == MRX_BF16 ? 2 : 4;  // z, h~, h, g, dz, dh~ in `dtype`; the carries in float32
    for (const void *p : {z, h_tilde, h, g, (const void *)dz, (const void *)dh_tilde})
        if (!aligned(p, ea)) return MRX_ERR_INVALID_ARG;
    for (const void *p : {h0, g_last, (const void *)dh0})
        if (!aligned(p, 4)) return MRX_ERR_INVALID_ARG;
    if (dtype == MRX_BF16)
        return launch_bwd<float, true, __bf16>((hipStream_t)stream, z, h_tilde, h, done, done_dtype, h0, g, g_last, dz,
                                               dh_tilde, dh0, B, T, D, 0);
    return launch_bwd<float, true>((hipStream_t)stream, z, h_tilde, h, done, done_dtype, h0, g, g_last, dz, dh_tilde,
                                   dh0, B, T, D, 0);
}
