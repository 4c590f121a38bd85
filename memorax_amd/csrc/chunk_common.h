// Building blocks of the chunked linear-attention / delta-rule kernels (gfx950).
//
// One workgroup = NW waves = one (batch, head) sequence, head dim 64, walking the
// time axis in chunks of C rows.  Every matrix product is executed with 16x16 MFMA
// tiles (bf16: v_mfma_f32_16x16x32_bf16, fp32: v_mfma_f32_16x16x4_f32) on two LDS
// tiles with fp32 accumulation:
//     D[m][n] = sum_k X(m, k) * Y(n, k)
// Each operand tile is stored once, in its natural orientation, and read either
//   ROWK: tile[row][k], k contiguous  -> one 16-byte read per lane, or
//   KROW: tile[k][row], row contiguous -> gfx950 transpose reads (ds_read_b64_tr_b16)
//         for bf16, four 4-byte reads for fp32,
// so no transposed copy of any tile is ever written.
// A wave lane (i = lane % 16, g = lane / 16) holds, for a 16x16 accumulator tile, the
// four elements D[4g + v][i], v = 0..3: four consecutive m-indices per lane, hence a
// result is stored with one 8/16-byte write per lane as the matrix dst[n][m].
#pragma once
#include "common.h"
#include "hd.h"

namespace mrx {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also drains the
// vector-memory counter, which would make every barrier wait for the next chunk's
// global prefetch; the compiler still inserts the vmcnt wait where a prefetched
// register is first consumed.
__device__ __forceinline__ void sync_lds()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Head dim (d_k = d_v) of the chunked and single-step kernels: 64, or 32 in the library's second build
// of these sources (hd.h).
constexpr int HD = MRX_HD;
static_assert(HD == 64 || HD == 32, "tile maps exist for head dims 64 and 32");

// Time steps per chunk of the bf16 kernels.  Linear attention: 64 (two workgroups per CU fit at 64
// and larger chunks amortise the per-chunk staging of S).  Delta rule: 32 -- the backward's fifteen
// LDS tiles fit twice per CU only at 32 (72 KB), and two resident workgroups hide each other's
// barrier and LDS latencies (measured: backward 261 -> 199 us, forward 157 -> 148 us on
// B=64, H=8, T=1024), and the triangular inverse shrinks to one off-diagonal block.
#ifndef MRX_LA_BF16_CHUNK
#define MRX_LA_BF16_CHUNK 64
#endif
#ifndef MRX_DELTA_BF16_CHUNK
#define MRX_DELTA_BF16_CHUNK 32
#endif
constexpr int LA_BF16_CHUNK = MRX_LA_BF16_CHUNK, DELTA_BF16_CHUNK = MRX_DELTA_BF16_CHUNK;

// Plain and normalised linear attention: the backward call walks the state back from chunk to chunk
// (S_c = S_{c+1} - V_c^T K_c in fp32) instead of reading a checkpoint per chunk.  Every step of that walk
// rounds at the magnitude of the late, large state, so its error relative to an early, small state grows
// with the number of chunks walked (about eps N^1.5 for a state that grows linearly).  The forward
// call therefore writes the exact fp32 state every walk_anchor() chunks as well (besides the chunks
// with resets) and the walk starts afresh there: 32 chunks keep fp32 at 1e-5 of the early states,
// bf16 inputs (tolerance 2e-2, rounding 4e-3) are re-anchored every 128.  Extra traffic: one 16 KB
// slot per 32 (128) chunks of 32 KB each way.
template <typename T> constexpr int walk_anchor() { return sizeof(T) == 2 ? 128 : 32; }

// Bounds of the screen that lets the delta-rule kernels do all episodes of a chunk in one unit (template flag
// MERGE): with |q|, |k|, |v|, |beta|, |dout| and the entries of the triangular factor at most 2^6 and the
// entries of the state and of its gradient at most 2^20, the largest intermediate of a 32-row chunk at
// head dim 64 stays below 2^123 (forward: the output, 2^5 x 2^18 x 2^50 and its state term; backward: the
// row dots behind dbeta, 2^6 x 2^6 x 2^110), inside the float32 range.
constexpr float MERGE_IN_MAX = 64.f, MERGE_STATE_MAX = 1048576.f;

// A 16-byte global load of data that no later kernel reads again (the residuals a backward call consumes):
// non-temporal, so that it does not displace what the next kernels will read -- inputs, and the residuals the
// forward call has just written -- from the last-level cache.  Row stores of results take the same hint
// (tile_rows_to_global).  Measured on the delta rule at 64 x 1024 x 8: forward + backward 0.266 -> 0.260 ms;
// the same hint on the loads of q, k, v costs the forward 3 % there (it reads k right after the factor
// kernel has), and on the stores of the residuals it costs the backward what it saves the forward.
template <typename F, typename P> __device__ __forceinline__ F load_once(const P *p)
{
    return __builtin_nontemporal_load(reinterpret_cast<const F *>(p));
}
enum OpMode { ROWK = 0, KROW = 1 };

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
        // Two packed conversions on whole words: element-wise conversions compile to four single
        // converts and two byte permutes.
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
        u32x2 w;
        w[0] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));
        w[1] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{c, d}, bf16x2));
        return __builtin_bit_cast(pack4, w);
    }
    static __device__ __forceinline__ frag ones()
    {
        frag r;
#pragma unroll
        for (int e = 0; e < 8; ++e) r[e] = (__bf16)1.f;
        return r;
    }
    // 16 rows r0.., k block k0..k0+31; lane (i, g) gets k = k0 + 8g + 0..7 of row r0 + i
    template <int MODE>
    static __device__ __forceinline__ frag load(const __bf16 *tile, int ld, int r0, int k0, int lane)
    {
        const int i = lane & 15, g = lane >> 4;
        if (MODE == ROWK) return *reinterpret_cast<const frag *>(tile + (r0 + i) * ld + k0 + 8 * g);
        // Transpose read: within a 16-lane group, source lane s addresses the 4 elements
        // tile[kk + (s >> 2)][r0 + 4 (s & 3) ..+3]; destination lane i receives
        // tile[kk + e][r0 + i], e = 0..3.
        typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
        const __bf16 *p = tile + (k0 + 8 * g + (i >> 2)) * ld + r0 + 4 * (i & 3);
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)p);
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(p + 4 * ld));
        union {
            s16x4 h[2];
            frag f;
        } u;
        u.h[0] = lo;
        u.h[1] = hi;
        return u.f;
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
    static __device__ __forceinline__ frag ones() { return frag{1.f, 1.f, 1.f, 1.f}; }
    template <int MODE>
    static __device__ __forceinline__ frag load(const float *tile, int ld, int r0, int k0, int lane)
    {
        const int i = lane & 15, g = lane >> 4;
        if (MODE == ROWK) return *reinterpret_cast<const frag *>(tile + (r0 + i) * ld + k0 + 4 * g);
        frag f;
#pragma unroll
        for (int s = 0; s < 4; ++s) f[s] = tile[(k0 + 4 * g + s) * ld + r0 + i];
        return f;
    }
};

// 16-byte LDS row padding (in elements) keeps 16-lane fragment reads conflict free.
template <typename T> constexpr int pad_of() { return 16 / (int)sizeof(T); }

// Which 16x16 tiles of an M x N result a wave owns: slot j -> (mt, nt).  A wave owns a block of
// MBW x NBW tiles, so that one k-step of a product reads MBW + NBW operand fragments from LDS
// for MBW * NBW MFMAs: 2 x 2 blocks (four or more tiles per wave) halve the LDS traffic of a
// 1 x 2 row of tiles.
constexpr int default_mbw(int M, int N, int NW)
{
    const int mt = M / 16, nt = N / 16, tpw = mt * nt / NW;
    return (tpw >= 4 && tpw % 2 == 0 && mt % 2 == 0 && nt % (tpw / 2) == 0 && (mt / 2) * (nt / (tpw / 2)) == NW) ? 2 : 1;
}
template <int M, int N, int NW, int MBW_ = 0> struct TileMap {
    static constexpr int MT = M / 16, NT = N / 16;
    static constexpr int TPW = MT * NT / NW;
    static constexpr int MBW = MBW_ > 0 ? MBW_ : default_mbw(M, N, NW);
    static constexpr int NBW = TPW / MBW;
    static constexpr int WM = MT / MBW, WN = NT / NBW;  // wave grid
    static_assert(MT * NT % NW == 0 && TPW >= 1 && TPW % MBW == 0, "tiles must divide over the waves");
    static_assert(MT % MBW == 0 && NT % NBW == 0 && WM * WN == NW, "wave grid must tile the result");
    static __device__ __forceinline__ int mt(int w, int j) { return (w % WM) * MBW + j / NBW; }
    static __device__ __forceinline__ int nt(int w, int j) { return (w / WM) * NBW + j % NBW; }
};

struct NoHook {
    template <typename F> __device__ __forceinline__ void operator()(int, int, F &) const {}
};

#ifdef MRX_PHASE_CLOCKS
// Measurement build (libmemorax_amd_clk.so): every matrix product is bracketed by reads of the shader
// clock -- from before its first operand fragment is requested until its accumulators are in hand --
// and the cycles are summed per workgroup here.  A kernel that reports them (delta_bwd_kernel) clears the
// sum at its start and adds it to its device-wide totals at its end.  The brackets serialise a product
// against what follows it, so this build is for the ratio of the two clocks only, never for timing.
static __shared__ unsigned long long wg_product_clocks;
#endif

// acc[j] += sum_k X(mt_j rows, k) * Y(nt_j rows, k), k = 0..K-1.
// hx(mi, kb, fragment) / hy(ni, kb, fragment) see every operand fragment as it is loaded, so that
// a rank-one by-product (a row or column sum, a product with one more vector) costs MFMAs only;
// a hook may also rewrite the fragment (scale it along k) before it is used.  Element e of a
// fragment belongs to k = kb * KB + KP * (lane / 16) + e in both operand modes.
template <typename T, int M, int N, int K, int XM, int YM, int NW, int MBW_ = 0, typename HX = NoHook, typename HY = NoHook>
__device__ __forceinline__ void gemm(f32x4 *acc, const T *X, int ldx, const T *Y, int ldy, int w, int lane,
                                     HX hx = HX(), HY hy = HY())
{
    using TM = TileMap<M, N, NW, MBW_>;
    using F = typename TT<T>::frag;
    constexpr int KB = TT<T>::KB;
    static_assert(K % KB == 0, "K must be a multiple of the fragment k extent");
#ifdef MRX_PHASE_CLOCKS
    const long long clk0 = clock64();
#endif
#pragma unroll
    for (int kb = 0; kb < K / KB; ++kb) {
        F a[TM::MBW];
#pragma unroll
        for (int mi = 0; mi < TM::MBW; ++mi)
        {
            a[mi] = TT<T>::template load<XM>(X, ldx, TM::mt(w, mi * TM::NBW) * 16, kb * KB, lane);
            hx(mi, kb, a[mi]);
        }
#pragma unroll
        for (int ni = 0; ni < TM::NBW; ++ni) {
            F b = TT<T>::template load<YM>(Y, ldy, TM::nt(w, ni) * 16, kb * KB, lane);
            hy(ni, kb, b);
#pragma unroll
            for (int mi = 0; mi < TM::MBW; ++mi)
                acc[mi * TM::NBW + ni] = TT<T>::mma(a[mi], b, acc[mi * TM::NBW + ni]);
        }
    }
#ifdef MRX_PHASE_CLOCKS
    float sink = 0.f;  // an ordinary read of every tile: the matrix pipe has delivered before the second clock
#pragma unroll
    for (int j = 0; j < TM::TPW; ++j) sink += acc[j][0] + acc[j][3];
    asm volatile("" ::"v"(sink));
    const long long clk1 = clock64();
    if (lane == 0) atomicAdd(&wg_product_clocks, (unsigned long long)(clk1 - clk0));
#endif
}

template <int N> __device__ __forceinline__ void zero_acc(f32x4 *acc)
{
#pragma unroll
    for (int j = 0; j < N; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
}

// Store an accumulator tile set as dst[n][m] (type T), f(m, n, x) applied per element.
template <typename T, int M, int N, int NW, typename Fn, int MBW_ = 0>
__device__ __forceinline__ void store_acc_f(const f32x4 *acc, T *dst, int ld, int w, int lane, Fn f)
{
    using TM = TileMap<M, N, NW, MBW_>;
    using P = typename TT<T>::pack4;
    const int i = lane & 15, g = lane >> 4;
#pragma unroll
    for (int j = 0; j < TM::TPW; ++j) {
        const int m = TM::mt(w, j) * 16 + 4 * g, n = TM::nt(w, j) * 16 + i;
        *reinterpret_cast<P *>(dst + n * ld + m) =
            TT<T>::pack(f(m, n, acc[j][0]), f(m + 1, n, acc[j][1]), f(m + 2, n, acc[j][2]), f(m + 3, n, acc[j][3]));
    }
}

template <typename T, int M, int N, int NW>
__device__ __forceinline__ void store_acc(const f32x4 *acc, T *dst, int ld, int w, int lane)
{
    store_acc_f<T, M, N, NW>(acc, dst, ld, w, lane, [](int, int, float x) { return x; });
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

// ---- global <-> register <-> LDS movement of one [R][COLS] tile ------------------
// A tile is R rows of COLS T = R * SEGS 16-byte segments; thread tid owns segment
// (tid % SEGS) of rows (tid / SEGS) + p * RPP, p = 0..PASSES-1.
template <typename T, int R, int NTHR, int COLS = HD> struct TileIO {
    static constexpr int KP = TT<T>::KP;
    static constexpr int SEGS = COLS / KP;
    static constexpr int RPP = NTHR / SEGS;
    static constexpr int PASSES = (R + RPP - 1) / RPP;
    static constexpr bool FULL = R % RPP == 0;  // otherwise the threads past the last row idle
    static_assert(NTHR % SEGS == 0 && (FULL || PASSES == 1), "a tile is whole passes, or less than one");
    using F = typename TT<T>::frag;
    struct Regs {
        F v[PASSES];
    };

    // rows t0.. of an array with COLS-wide rows `row_stride` apart starting at `base`; rows >= Tlen read as 0
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

    // zero the rows for which keep(row) is false (select, not multiply)
    template <typename KeepF> static __device__ __forceinline__ void mask_rows(Regs &r, int tid, KeepF keep)
    {
        const int r0 = tid / SEGS;
#pragma unroll
        for (int p = 0; p < PASSES; ++p)
            if (!keep(r0 + p * RPP)) {
#pragma unroll
                for (int e = 0; e < KP; ++e) r.v[p][e] = (T)0.f;
            }
    }

    // multiply row p of the thread's tile slice by f[p]
    static __device__ __forceinline__ void scale_rows(Regs &r, const float *f)
    {
#pragma unroll
        for (int p = 0; p < PASSES; ++p)
#pragma unroll
            for (int e = 0; e < KP; ++e) r.v[p][e] = (T)((float)r.v[p][e] * f[p]);
    }

    static __device__ __forceinline__ int row_of(int tid, int p) { return tid / SEGS + p * RPP; }

    static __device__ __forceinline__ void zero(Regs &r)
    {
#pragma unroll
        for (int p = 0; p < PASSES; ++p)
#pragma unroll
            for (int e = 0; e < KP; ++e) r.v[p][e] = (T)0.f;
    }

    // dst[row][col], row-major with leading dim ld
    static __device__ __forceinline__ void to_lds(const Regs &r, T *dst, int ld, int tid)
    {
        const int seg = tid % SEGS, r0 = tid / SEGS;
#pragma unroll
        for (int p = 0; p < PASSES; ++p)
            if (FULL || r0 + p * RPP < R) *reinterpret_cast<F *>(dst + (r0 + p * RPP) * ld + seg * KP) = r.v[p];
    }
};

// Sum over the SEGS consecutive lanes that share a tile row (4, 8 or 16), by data-parallel
// primitives; every lane of the group ends with the total.
template <int SEGS> __device__ __forceinline__ float seg_sum(float x)
{
    static_assert(SEGS == 4 || SEGS == 8 || SEGS == 16, "a row is 4, 8 or 16 segments");
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, true));   // quad_perm [1,0,3,2]
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x4E, 0xF, 0xF, true));   // quad_perm [2,3,0,1]
    if (SEGS >= 8)
        x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x141, 0xF, 0xF, true));  // row_half_mirror
    if (SEGS == 16)
        x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x140, 0xF, 0xF, true));  // row_mirror
    return x;
}

// The prologue's two scalar functions on the hardware reciprocal / reciprocal square root (1 ulp): a
// full-precision division is some ten instructions, and these sit in every thread's staging path.
__device__ __forceinline__ float sigmoidf(float x) { return __builtin_amdgcn_rcpf(1.f + __expf(-x)); }
// 1 / max(|k|, 1e-12) from the row's sum of squares
__device__ __forceinline__ float inv_norm(float ss) { return __builtin_amdgcn_rsqf(fmaxf(ss, 1e-24f)); }

// Rows of an LDS tile [C][64] to a (B,T,H,64) array, 16 bytes per thread: eight (sixteen) threads
// write one whole row, so a wave instruction covers full 128-byte lines -- against the four-feature
// pieces (16 rows x 32 bytes per instruction) of a store from accumulators.  `g` points at row 0 of
// the chunk.
// ncols: width of the rows in memory when it is less than the tile's (narrow heads: the tile's further columns are padding).
template <typename T, int C, int NTHR, typename KeepF>
__device__ __forceinline__ void tile_rows_to_global(const T *tile, int ld, T *g, int64_t rs, int t0, int Tlen, int tid,
                                                    KeepF keep, int ncols = HD)
{
    using IO = TileIO<T, C, NTHR>;
    const int seg = tid % IO::SEGS;
    if (seg * IO::KP >= ncols) return;
#pragma unroll
    for (int p = 0; p < IO::PASSES; ++p) {
        const int r = IO::row_of(tid, p);
        if ((IO::FULL || r < C) && t0 + r < Tlen && keep(r))  // results are not read again by these kernels: non-temporal
            __builtin_nontemporal_store(*reinterpret_cast<const typename IO::F *>(tile + r * ld + seg * IO::KP),
                                        reinterpret_cast<typename IO::F *>(g + (int64_t)r * rs + seg * IO::KP));
    }
}

// Which (batch, head) sequence a workgroup walks.  The device hands workgroup i to XCD i % 8, each XCD
// with an L2 of its own, and the heads of one batch row interleave in memory ((B,T,H,64): 128-byte
// rows, H of them per time step).  Giving each XCD whole batch rows -- consecutive workgroups of one
// XCD take the heads of one row -- keeps the reads and write-backs of a page on one L2 (measured:
// linear attention at 256 x 4096 x 8, which is bound by memory, 2.62 -> 2.54 ms; the other shapes
// level or 1 % better).  Batch sizes that are no multiple of 8 keep the plain order.
__device__ __forceinline__ int sequence_of_block(int i, int nblocks, int H)
{
    const int Bn = nblocks / H;
    if (Bn % 8 != 0) return i;
    const int x = i & 7, j = i >> 3;
    return ((j / H) * 8 + x) * H + (j % H);
}

// ---- per-chunk reset bookkeeping ------------------------------------------------
// dmask has bit r set when row r of the chunk starts a new episode.  episode_of(r)
// counts the resets at rows <= r; rows interact iff they have the same count.
__device__ __forceinline__ int episode_of(unsigned long long dmask, int r)
{
    return __popcll(dmask & ((2ull << r) - 1ull));
}

// ---- inverse of a unit lower-triangular matrix (fp32 arithmetic) -----------------
// X = (I + A)^-1 for A = tril(diag(beta) K K^T, -1), C x C, in 16x16 blocks.
//
// tri_diag_block: the wave that owns the accumulator tile (b, b) of K K^T inverts
//   diagonal block b straight from those registers by repeated squaring: with N = -A_bb
//   (N^16 = 0), (I+A_bb)^-1 = (I+N)(I+N^2)(I+N^4)(I+N^8).  A 16x16 product P = X Y on the
//   fp32 MFMA takes X^T and Y both in accumulator layout (lane (i,g) holds Z[4g+v][i]),
//   so each matrix is carried together with its transpose and nothing goes through LDS.
//   The result is written as fp32 into the diagonal block of sA (A-operand of other
//   waves) and, rounded to T, into sX; it is also returned in accumulator layout.
// tri_block_column: after a workgroup barrier, the same wave computes the rest of block
//   column c by forward substitution, X_bc = -X_bb sum_{k=c}^{b-1} A_bk X_kc; its own
//   earlier blocks stay in registers (the accumulator layout is the B-operand layout),
//   only A_bk (strictly lower blocks of sA) and the diagonal inverses are read from LDS.
// Blocks above the block diagonal of sX are never written (the caller zeroes them once).
__device__ __forceinline__ f32x4 mm16(const f32x4 &xt, const f32x4 &y, f32x4 c)
{
#pragma unroll
    for (int s = 0; s < 4; ++s) c = __builtin_amdgcn_mfma_f32_16x16x4f32(xt[s], y[s], c, 0, 0, 0);
    return c;
}

// A 16x16 matrix in accumulator layout prepared as an operand of such a product.  fp32 kernels take
// the exact fp32 MFMAs.  bf16 kernels run the product on the bf16 pipe with each operand split
// once into a high and a low bf16 half (x = xh + xl up to 2^-16): Xh Yh + Xl Yh + Xh Yl as three
// 16x16x16 MFMAs whose operands are those halves as they are (slot (g, e) of the 16 k-slots is
// contraction index 4 g + e, so the fp32 accumulator layout is the operand layout and nothing moves
// between lanes); a matrix is converted once however many products use it, and the dropped Xl Yl
// term is 2^-16 of a result that is rounded to bf16 in the end.  The low halves are needed: with
// keys correlated 0.9 from step to step the repeated squaring cancels, and high halves alone leave
// an error of 0.19 in a factor whose entries are of order one (2e-3 with the split).
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
template <typename T> struct Op16;
template <> struct Op16<float> {
    f32x4 x;
    static __device__ __forceinline__ Op16 of(const f32x4 &z) { return Op16{z}; }
    // c + P^T Q for P, Q the matrices whose accumulator layouts were prepared
    static __device__ __forceinline__ f32x4 mm(const Op16 &p, const Op16 &q, f32x4 c) { return mm16(p.x, q.x, c); }
};
template <> struct Op16<__bf16> {
    bf16x4 h, l;
    static __device__ __forceinline__ Op16 of(const f32x4 &z)
    {
        // pairs, so that each conversion is one packed instruction; the high half is widened
        // again with a shift or a mask of the packed word
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
        u32x2 hw, lw;  // whole words: element-wise access would undo the packed conversions
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const f32x2 x = {z[2 * p], z[2 * p + 1]};
            const uint32_t w = __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2));
            const f32x2 rest = {x[0] - __uint_as_float(w << 16), x[1] - __uint_as_float(w & 0xffff0000u)};
            hw[p] = w;
            lw[p] = __builtin_bit_cast(uint32_t, __builtin_convertvector(rest, bf16x2));
        }
        Op16 o;
        o.h = __builtin_bit_cast(bf16x4, hw);
        o.l = __builtin_bit_cast(bf16x4, lw);
        return o;
    }
    static __device__ __forceinline__ f32x4 mm(const Op16 &p, const Op16 &q, f32x4 c)
    {
        c = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(p.h, q.h, c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(p.l, q.h, c, 0, 0, 0);
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(p.h, q.l, c, 0, 0, 0);
    }
};

// kk[v] = (K K^T)[16b + i][16b + 4g + v] (symmetric); sBeta indexed by chunk row
template <typename T>
__device__ __forceinline__ f32x4 tri_diag_block(const f32x4 &kk, const float *sBeta, int b, float *sA, int lda,
                                                T *sX, int ldx, int lane)
{
    using P4 = typename TT<T>::pack4;
    const int i = lane & 15, g = lane >> 4;
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    const float beta_i = sBeta[16 * b + i];
    const f32x4 beta_r = *reinterpret_cast<const f32x4 *>(sBeta + 16 * b + 4 * g);
    f32x4 M, Mt, R, Rt;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int r = 4 * g + v;
        M[v] = (i < r) ? -beta_r[v] * kk[v] : 0.f;   // N[r][i] = -beta_r KK[r][i], strictly lower
        Mt[v] = (r < i) ? -beta_i * kk[v] : 0.f;     // N^T[r][i] = N[i][r] = -beta_i KK[i][r]
        R[v] = M[v] + (r == i ? 1.f : 0.f);
        Rt[v] = Mt[v] + (r == i ? 1.f : 0.f);
    }
    using Op = Op16<T>;
    Op oM = Op::of(M), oMt = Op::of(Mt);
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        const f32x4 M2 = Op::mm(oMt, oM, zero);       // N^2  : X = M,  Y = M
        const Op oRt = Op::of(Rt), oM2 = Op::of(M2);
        R = Op::mm(oRt, oM2, R);                      // R + R M2
        Rt = Op::mm(oM2, oRt, Rt);                    // R^T + M2^T R^T
        if (k < 2) oMt = Op::of(Op::mm(oM, oMt, zero));  // (N^2)^T = M^T M^T
        oM = oM2;
    }
    float *blk = sA + (16 * b) * lda + 16 * b;
#pragma unroll
    for (int v = 0; v < 4; ++v) blk[(4 * g + v) * lda + i] = R[v];
    // Rt[v] = X[i][4g+v]: four consecutive columns of row i
    *reinterpret_cast<P4 *>(sX + (16 * b + i) * ldx + 16 * b + 4 * g) = TT<T>::pack(Rt[0], Rt[1], Rt[2], Rt[3]);
    return R;
}

template <int C, typename T>
__device__ __forceinline__ void tri_block_column(const float *sA, int lda, T *sX, int ldx, int c, const f32x4 &Xcc,
                                                 int lane)
{
    constexpr int NB = C / 16;
    const int i = lane & 15, g = lane >> 4;
    const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
    f32x4 Xc[NB];  // Xc[r] = X_{c+r, c} in accumulator layout
    Xc[0] = Xcc;
#pragma unroll
    for (int r = 1; r < NB; ++r) {
        const int b = c + r;
        if (b < NB) {
            f32x4 part[NB - 1];
#pragma unroll
            for (int kk = 0; kk < r; ++kk) {  // k = c + kk
                const f32x4 a4 = *reinterpret_cast<const f32x4 *>(sA + (16 * b + i) * lda + 16 * (c + kk) + 4 * g);
                part[kk] = Op16<T>::mm(Op16<T>::of(a4), Op16<T>::of(Xc[kk]), zero);
            }
            f32x4 tmp = part[0];
#pragma unroll
            for (int kk = 1; kk < r; ++kk) tmp += part[kk];
            const f32x4 d4 = *reinterpret_cast<const f32x4 *>(sA + (16 * b + i) * lda + 16 * b + 4 * g);
            Xc[r] = -Op16<T>::mm(Op16<T>::of(d4), Op16<T>::of(tmp), zero);
#pragma unroll
            for (int v = 0; v < 4; ++v) sX[(16 * b + 4 * g + v) * ldx + 16 * c + i] = (T)Xc[r][v];
        }
    }
}

}  // namespace mrx
