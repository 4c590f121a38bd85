/* memorax_amd.h — C ABI of the MI355X (gfx950) sequence-model kernels.
 *
 * The reference (memory-rl/memorax) is pure Python/JAX and has no FFI for this
 * path; each entry point below replaces the arithmetic that the cited
 * reference code performs through jax.lax.associative_scan, and is what an
 * XLA-FFI / ctypes binding for that code would bind.
 *
 * Common rules
 *  - Every pointer is a DEVICE pointer owned by the caller; outputs are
 *    pre-allocated by the caller.  Nothing here allocates, frees, copies to the
 *    host or synchronises: a call validates its arguments on the host, enqueues
 *    kernels on `stream` (a hipStream_t passed as void*, NULL = default stream)
 *    and returns.
 *  - Return value: MRX_OK (0) or a negative mrx_status; never throws.
 *    mrx_status_string() names a code.  Arguments are checked before any launch;
 *    the status of a launch is the launch call's own return code (the runtime's
 *    sticky last-error state is not consulted; only the record of a launch that
 *    was itself refused, and reported as MRX_ERR_LAUNCH, is cleared).  An entry point that
 *    enqueues two kernels (mrx_delta_rule_fwd with the chunk-parallel factors)
 *    may return MRX_ERR_LAUNCH after the first has been enqueued.
 *  - The library keeps no state between calls apart from what mrx_init() sets up
 *    once per device (below); calls are re-entrant and may be captured in a HIP
 *    graph once the device has been set up.
 *  - Layouts are the reference's: time on axis 1, features last, row-major,
 *    densely packed.  `done` is (B,T); nonzero at (b,t) clears the carried state
 *    before step t consumes its input (select semantics, memoroid.py:79-83).
 *  - Recurrent state (S, h, P) is always fp32 (or complex64 for MRX_C64 scans).
 */
#ifndef MEMORAX_AMD_H
#define MEMORAX_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    MRX_OK = 0,
    MRX_ERR_INVALID_ARG = -1, /* null pointer, non-positive size, bad enum, misalignment */
    MRX_ERR_UNSUPPORTED = -2, /* valid request the kernels do not cover (e.g. a head dim the kernels are not built for) */
    MRX_ERR_LAUNCH = -3,      /* the HIP runtime rejected the launch */
    MRX_ERR_SCRATCH = -4      /* the problem exceeds the library's static scratch buffer (mrx_delta_rule_fwd_noalloc) */
} mrx_status;

typedef enum {
    MRX_F32 = 0,  /* float32 */
    MRX_BF16 = 1, /* bfloat16 inputs/outputs, fp32 state and accumulation */
    MRX_C64 = 2   /* complex64 (interleaved re,im); diagonal scan only */
} mrx_dtype;

typedef enum {
    MRX_DONE_U8 = 0, /* bool / uint8 */
    MRX_DONE_F32 = 1 /* float32, nonzero = reset (memoroid.py:67 casts done to float) */
} mrx_done_dtype;

typedef enum {
    MRX_FMAP_NONE = 0,
    MRX_FMAP_ELU1 = 1 /* phi(x) = elu(x) + 1 applied to q and k (linear_attention.py:58-60) */
} mrx_feature_map;

/* How mrx_delta_rule_fwd / mrx_deltanet_fwd obtain the per-chunk triangular factors. */
typedef enum {
    MRX_FACTORS_AUTO = 0,     /* chunk-parallel kernel iff a buffer is given and (float32, or B*H <= 2 x compute units) */
    MRX_FACTORS_PARALLEL = 1, /* chunk-parallel kernel whenever a buffer is given */
    MRX_FACTORS_INLINE = 2    /* inverted inside the sequential kernel */
} mrx_factor_path;

/* How the delta-rule kernels treat a chunk that holds episode resets.
 * MRX_RESETS_PASSES: one unit of work per episode of the chunk, the rows of the other episodes replaced by
 *   zeros by select -- exact whatever the data (a NaN or Inf of one episode never reaches another).
 * MRX_RESETS_MERGED: one unit per chunk, the episodes kept apart by masks inside it.  A masked zero then
 *   multiplies values of other episodes, which is exact while those are finite; the kernels therefore screen
 *   every such chunk first (|q|, |k|, |v|, |beta|, |dout| and the factor's entries <= 2^6, the state's and its
 *   gradient's <= 2^20: bounds under which no intermediate can leave the float32 range) and fall back to
 *   the units per episode for a chunk that fails, so the results are those of MRX_RESETS_PASSES for any data.
 *   For callers whose episodes end every hundred steps or so (ppo.py:181-190): a chunk with a reset
 *   then costs what a chunk without one costs (measured, B=64 T=1024 H=8 bf16 at one reset per hundred steps:
 *   backward 197 -> 169 us; at one per five hundred the two are level, without resets the merged instance
 *   is 5 % behind).  The forward call merges where it takes the chunk-parallel factor kernel
 *   (mrx_factor_path), the backward call always; head dim 64 at full width, 32-row chunks -- elsewhere the
 *   argument is accepted and the units per episode run.  The two calls of a pair need not agree.
 * MRX_RESETS_AUTO: MRX_RESETS_PASSES. */
typedef enum {
    MRX_RESETS_AUTO = 0,
    MRX_RESETS_PASSES = 1,
    MRX_RESETS_MERGED = 2
} mrx_reset_path;

const char *mrx_status_string(int status);

/* Per-device set-up: raises the dynamic-LDS limit of every kernel that needs more than the
 * default, caches the device's compute-unit count and resolves the address of the library's
 * static scratch array on that device.  Idempotent and thread-safe; the caller's current device
 * is left as it was.  Calling it is optional -- the first launch on a device does the same --
 * but a caller that captures its first call on a device into a HIP graph must call it before
 * the capture begins (the set-up calls are not stream operations).  No counterpart in the
 * reference (which has no native code). */
int mrx_init(int device);

/* Library version, major*10000 + minor*100 + patch. */
int mrx_version(void);

/* Time-chunk length the (gated) linear-attention kernels use for `dtype`; fixes the layout
 * of the per-chunk state checkpoints S_chk: (B, H, ceil(T/chunk), dv, dk).
 *
 * State checkpoints.  The backward calls need the state entering every chunk.  Where the chunk's
 * update can be undone cheaply (plain and normalised linear attention: S_c = S_{c+1} - V_c^T K_c)
 * they walk it back in fp32 from the forward call's S_last, which is
 * then an INPUT of the backward call, and S_chk is a float32 buffer that the forward call writes
 * SPARSELY: only the slots of chunks that contain a reset -- whose entering state the leaving one does
 * not determine -- are written and read; the other slots keep whatever the buffer held.  The gated
 * kernels (whose decayed update is not undone) and the delta rule (where the walk would need U' as a
 * further residual and one more product per chunk: measured slower) keep one checkpoint per chunk
 * in `dtype`. */
int64_t mrx_chunk_size(int dtype);

/* The same for the delta-rule kernels (S_chk and Tm_chk of mrx_delta_rule_fwd/_bwd). */
int64_t mrx_delta_chunk_size(int dtype);

/* ---- diagonal linear recurrence --------------------------------------------
 * Replaces Memoroid.scan_fn (memoroid.py:60-91) driven by the diagonal algebra
 * binary_operator of lru.py:92-95 / s5.py:133-136 / mamba.py:119-122:
 *     h_t = done_t ? b_t : a_t * h_{t-1} + b_t
 *     P_t = done_t ? a_t : a_t * P_{t-1}          (cumulative-decay leaf)
 * a: (B,T,D), or (D,) when a_time_invariant != 0 (LRU/S5 broadcast lambda,
 * lru.py:86, never materialised here).  b,h: (B,T,D).  h0,P0 (nullable: 0 and 1),
 * h_last,P_last (nullable: not written): (B,D).  dtype: MRX_F32, MRX_C64, or MRX_BF16: the (B,T,D) arrays
 * (and a) in bfloat16, the arithmetic and the (B,D) carries in float32. */
int mrx_linear_scan_fwd(void *stream, const void *a, const void *b,
                        const void *done, const void *h0, const void *P0,
                        void *h, void *h_last, void *P_last, int64_t B,
                        int64_t T, int64_t D, int dtype, int done_dtype,
                        int a_time_invariant);

/* Reverse scan of the same recurrence (what JAX autodiff of memoroid.py:87 yields):
 *     lam_t = g_t + conj(abar_{t+1}) lam_{t+1},  abar_t = done_t ? 0 : a_t
 *     db_t = lam_t ;  da_t = done_t ? 0 : lam_t conj(h_{t-1}) ;  dh0 = conj(abar_0) lam_0
 * (conj is the identity for MRX_F32; for MRX_C64 cotangents follow the
 * torch.autograd convention, the complex conjugate of JAX's).
 * h is the forward output; g = dL/dh (B,T,D); g_last = dL/dh_last (B,D, nullable).
 * da is per step (B,T,D), also when a is time-invariant (a_time_invariant = 1: the caller reduces);
 * with a_time_invariant = MRX_A_TIME_INVARIANT_SUM_DA the kernel sums the per-step terms over the
 * sequence itself and da is (B,D) -- the gradient of the broadcast lambda of lru.py:86 / s5.py is then
 * its sum over B, and the (B,T,D) array is neither written nor read back (MRX_BF16: this summed da is
 * float32, like the carries). */
#define MRX_A_TIME_INVARIANT_SUM_DA 2
int mrx_linear_scan_bwd(void *stream, const void *a, const void *h,
                        const void *done, const void *h0, const void *g,
                        const void *g_last, void *da, void *db, void *dh0,
                        int64_t B, int64_t T, int64_t D, int dtype,
                        int done_dtype, int a_time_invariant);

/* ---- causal linear attention, chunked ---------------------------------------
 * Replaces LinearAttentionCell.__call__ / binary_operator / read numerator
 * (linear_attention.py:62-86,105) scanned by memoroid.py:60-91, without
 * materialising the per-step state:
 *     S_t = (done_t ? 0 : S_{t-1}) + v_t phi(k_t)^T ;   o_t = S_t phi(q_t)
 * q,k: (B,T,H,dk); v,o: (B,T,H,dv) in `dtype` (MRX_F32 or MRX_BF16).
 * S0 (nullable = 0), S_last (nullable): (B,H,dv,dk) fp32.
 * S_chk (nullable): (B,H,ceil(T/chunk),dv,dk) float32, sparse (see mrx_chunk_size): receives the
 * state entering each chunk that contains a reset; required by the backward call together with
 * S_last.  dk = dv = 64 or dk = dv = 32 (here and in every chunked and single-step entry point below;
 * the library holds a build of those kernels for either width; mrx_delta_rule_fwd_noalloc: 64 only).
 * Narrow heads: every chunked and single-step entry point but mrx_delta_rule_fwd_noalloc also takes any
 * dk <= 64 and dv <= 64, independent of one another, whose rows are a whole number of 16-byte segments
 * (multiples of 4 in float32, of 8 in bfloat16; the reference's guides use head_dim = 16).  Every array
 * keeps its dense (.., dv, dk) / (.., dk) / (.., dv) layout at those widths; the kernels pad on the fly
 * (the 32-wide build when both widths are at most 32, else the 64-wide one). */
int mrx_linear_attn_fwd(void *stream, const void *q, const void *k,
                        const void *v, const void *done, const void *S0,
                        void *o, void *S_last, void *S_chk, int64_t B,
                        int64_t T, int64_t H, int64_t dk, int64_t dv, int dtype,
                        int done_dtype, int feature_map);

/* Gradients of the above w.r.t. q,k,v (pre-feature-map) and S0, given
 * dout = dL/do (B,T,H,dv) and dS_last = dL/dS_last (nullable).
 * S_chk, S_last: as the forward call on the same inputs left them.
 * dq,dk,dv in `dtype`; dS0 (nullable) fp32. */
int mrx_linear_attn_bwd(void *stream, const void *q, const void *k,
                        const void *v, const void *done, const void *S_chk,
                        const float *S_last, const void *dout, const void *dS_last, void *dq,
                        void *dk_out, void *dv_out, void *dS0, int64_t B,
                        int64_t T, int64_t H, int64_t dk, int64_t dv, int dtype,
                        int done_dtype, int feature_map);

/* ---- the same function cut along time: one workgroup per chunk -------------------
 * mrx_linear_attn_fwd / _bwd give every (batch, head) sequence one workgroup that walks its chunks
 * in order; with fewer sequences than the device has room for, most of it idles behind that walk.
 * The state of linear attention is additive (memoroid.py:60-91 scanning the operator of
 * linear_attention.py:82-86), so the pair below first forms every chunk's own contribution to the
 * state in parallel, sums those per sequence, and then treats every chunk of every sequence as an
 * independent workgroup.  Same arguments, results and accuracy class as the pair above, except:
 *   S_chk (required): (B,H,ceil(T/chunk),dv,dk) float32, dense: the forward call leaves the state
 *     entering every chunk in it, and the backward call reads all of it (the two calls of a pair must
 *     be of the same kind: the sequential backward call does not take these, and vice versa);
 *   workspace (backward, required): (B,H,ceil(T/chunk),dv,dk) float32 scratch, overwritten;
 *   S_last is not an input of the backward call.
 * mrx_linear_attn_chunk_parallel_pays: 1 when the library's own rule (at most one sequence per two
 * compute units of the current device and at least eight chunks each) prefers this pair, else 0. */
int mrx_linear_attn_fwd_chunk_parallel(void *stream, const void *q, const void *k,
                                       const void *v, const void *done, const void *S0,
                                       void *o, void *S_last, float *S_chk, int64_t B,
                                       int64_t T, int64_t H, int64_t dk, int64_t dv, int dtype,
                                       int done_dtype, int feature_map);
int mrx_linear_attn_bwd_chunk_parallel(void *stream, const void *q, const void *k,
                                       const void *v, const void *done, const float *S_chk,
                                       const void *dout, const void *dS_last, void *dq,
                                       void *dk_out, void *dv_out, void *dS0, float *workspace,
                                       int64_t B, int64_t T, int64_t H, int64_t dk, int64_t dv,
                                       int dtype, int done_dtype, int feature_map);
int mrx_linear_attn_chunk_parallel_pays(int64_t B, int64_t T, int64_t H, int dtype);

/* ---- linear attention with the normalised read-out fused ----------------------
 * Replaces, in addition to the above, LinearAttentionCell.read's denominator and
 * divide (linear_attention.py:107-110) and the z leaf of the carry
 * (linear_attention.py:62-86):
 *     z_t = (done_t ? 0 : z_{t-1}) + phi(k_t) ;  den_t = max(phi(q_t) . z_t, eps)
 *     o_t = S_t phi(q_t) / den_t
 * z0 (nullable = 0), z_last (nullable): (B,H,dk) fp32.  den: (B,H,T) fp32 (contiguous in time per
 * sequence: a residual, written and read back a chunk at a time), the clamped denominators, and
 * z_chk (nullable): (B,H,ceil(T/chunk),dk) fp32, z entering each chunk, are residuals of the backward call together with o and S_chk.
 * ss (nullable): (B,H,T) fp32, ss_t = sum over the dv value features of o_t^2 (o as stored, i.e. rounded to
 *   the I/O type), taken from the output tile before it leaves the kernel.  It is what the RMS norm over
 *   all heads that follows the divide (linear_attention.py:114, `self.norm(output)` over H*dv) needs from
 *   each head: mean square = sum_h ss[b,h,t] / (H dv), so the caller's side of the norm is one rescale of o
 *   instead of a reduction pass plus a rescale. */
int mrx_linear_attn_norm_fwd(void *stream, const void *q, const void *k,
                             const void *v, const void *done, const void *S0,
                             const float *z0, void *o, float *den, float *ss, void *S_last,
                             float *z_last, void *S_chk, float *z_chk, int64_t B,
                             int64_t T, int64_t H, int64_t dk, int64_t dv,
                             int dtype, int done_dtype, int feature_map, float eps);

/* Gradients of the above w.r.t. q,k,v (pre-feature-map), S0 and z0, given
 * dout = dL/do (gradient of the normalised output), dS_last and dz_last (nullable).
 * Where the clamp is active (den == eps) the denominator passes no gradient.
 * d_ss (nullable = 0): (B,H,T) fp32, dL/dss of the forward call's sums of squares; the kernel adds
 *   2 d_ss_t o_t to dout_t as it stages the chunk. */
int mrx_linear_attn_norm_bwd(void *stream, const void *q, const void *k,
                             const void *v, const void *done, const void *S_chk,
                             const float *S_last, const float *z_chk, const void *o, const float *den,
                             const void *dout, const float *d_ss, const void *dS_last,
                             const float *dz_last, void *dq, void *dk_out,
                             void *dv_out, void *dS0, float *dz0, int64_t B,
                             int64_t T, int64_t H, int64_t dk, int64_t dv,
                             int dtype, int done_dtype, int feature_map, float eps);

/* ---- DeltaNet delta rule, chunked WY/UT form --------------------------------
 * No counterpart in the reference; written in its cell idiom it would be a
 * MemoroidCellBase scanned by memoroid.py:60-91 with elements
 * (beta v k^T, I - beta k k^T):
 *     S' = done_t ? 0 : S_{t-1} ;  S_t = S'(I - beta_t k_t k_t^T) + beta_t v_t k_t^T ;
 *     o_t = S_t q_t
 * beta: (B,T,H) in `dtype`; other arguments as for linear attention.
 * Tm_chk (nullable): (B,H,ceil(T/chunk),chunk,chunk) in `dtype` (chunk = mrx_delta_chunk_size), receives each
 * chunk's unit-lower-triangular factor (I + tril(diag(beta) K K^T, -1))^-1, block
 * diagonal by episode; like S_chk it is a residual the backward call requires.
 * It may be given without S_chk: the forward call also works through it.  With the buffer and
 * B*H <= 2 x the device's compute units the factors of all chunks are computed by a chunk-parallel
 * kernel first and the sequential kernel reads them (up to a third faster while the device is not
 * full); otherwise the sequential kernel inverts in place.  Both ways fill Tm_chk with the same
 * factors up to rounding.  factor_path (mrx_factor_path) overrides the rule:
 * MRX_FACTORS_PARALLEL takes the chunk-parallel kernel whenever the buffer is given (on a full
 * device that is level with the default when episodes end every hundred steps or so, and slower
 * when resets are rare), MRX_FACTORS_INLINE never does.
 * S_chk: (B,H,ceil(T/chunk),dv,dk) in `dtype`, one checkpoint per chunk (dense; see mrx_chunk_size). */
int mrx_delta_rule_fwd(void *stream, const void *q, const void *k,
                       const void *v, const void *beta, const void *done,
                       const void *S0, void *o, void *S_last, void *S_chk,
                       void *Tm_chk, int64_t B, int64_t T, int64_t H, int64_t dk,
                       int64_t dv, int dtype, int done_dtype, int factor_path, int reset_path);

/* mrx_delta_rule_fwd without residuals for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): the triangular
 * factors, which mrx_delta_rule_fwd keeps in the caller's Tm_chk buffer, go to a static device
 * array inside the library instead (MRX_NOALLOC_SCRATCH_BYTES per device, held until the process
 * ends), and the chunk-parallel factor kernel always runs.  No counterpart in the reference.
 * Same results as mrx_delta_rule_fwd(..., S_chk = NULL, Tm_chk = buffer, MRX_FACTORS_PARALLEL).
 * Limit: B * H * ceil(T / 32) * 32 * 32 * sizeof(element) <= MRX_NOALLOC_SCRATCH_BYTES, i.e. 16384
 * chunks of bf16 or 8192 of fp32 (B=64, H=8, T=1024 in bf16 fits exactly); beyond it the call
 * returns MRX_ERR_SCRATCH and launches nothing.  The call allocates and frees nothing.  All calls
 * on one device share that device's array: calls that overlap in time on one device (different
 * streams, or graphs replayed concurrently) race; calls ordered on one stream do not.  Nothing in
 * the array needs clearing between calls: every factor a call reads, it has written itself. */
#define MRX_NOALLOC_SCRATCH_BYTES (32u << 20)
int mrx_delta_rule_fwd_noalloc(void *stream, const void *q, const void *k,
                               const void *v, const void *beta, const void *done,
                               const void *S0, void *o, void *S_last, int64_t B,
                               int64_t T, int64_t H, int64_t dk, int64_t dv, int dtype,
                               int done_dtype);

/* Gradients w.r.t. q,k,v,beta (in `dtype`) and S0 (fp32, nullable).  S_chk and
 * Tm_chk are the residuals written by mrx_delta_rule_fwd on the same inputs. */
int mrx_delta_rule_bwd(void *stream, const void *q, const void *k,
                       const void *v, const void *beta, const void *done,
                       const void *S_chk, const void *Tm_chk, const void *dout,
                       const void *dS_last, void *dq, void *dk_out, void *dv_out,
                       void *dbeta, void *dS0, int64_t B, int64_t T, int64_t H,
                       int64_t dk, int64_t dv, int dtype, int done_dtype, int reset_path);

/* ---- DeltaNet cell recurrence with its prologue fused -------------------------
 * As mrx_delta_rule_fwd / _bwd, but on the raw projections: inside the kernels
 *     k_t <- k_t / max(|k_t|, 1e-12)  (fp32, then rounded to `dtype`) ;  beta_t = sigmoid(beta_raw_t)
 * so that the normalised keys and the gates are never written to memory, and the backward
 * call returns the gradients w.r.t. the raw k and beta_raw.  Like the delta rule itself this
 * has no counterpart in the reference; it is the prologue a DeltaNet cell written in the
 * reference's cell idiom (projections -> elements, memoroid.py:20-33) would run per step.
 * Residuals as for mrx_delta_rule_*. */
int mrx_deltanet_fwd(void *stream, const void *q, const void *k, const void *v,
                     const void *beta_raw, const void *done, const void *S0, void *o,
                     void *S_last, void *S_chk, void *Tm_chk, int64_t B, int64_t T,
                     int64_t H, int64_t dk, int64_t dv, int dtype, int done_dtype,
                     int factor_path, int reset_path);

int mrx_deltanet_bwd(void *stream, const void *q, const void *k, const void *v,
                     const void *beta_raw, const void *done, const void *S_chk,
                     const void *Tm_chk, const void *dout, const void *dS_last, void *dq,
                     void *dk_out, void *dv_out, void *dbeta_raw, void *dS0, int64_t B,
                     int64_t T, int64_t H, int64_t dk, int64_t dv, int dtype,
                     int done_dtype, int reset_path);

/* Final state only, one decay per `a_group` consecutive channels: h_T of
 *     h_t = done_t ? b_t : a_t h_{t-1} + b_t ,  a: (B,T,D/a_group), b: (B,T,D), h0 (nullable), h_last: (B,D).
 * The sensitivity propagation of real-time recurrent learning, Memoroid._propagate_sensitivities
 * (memoroid.py:114-141): there a = where(done, 0, repeat(decay, param_size)), b = the local
 * Jacobians (B,T,H*param_size), h0 = the carried sensitivity and only last(state) is kept; here the
 * repeated decay and the per-step states are never materialised (a_group = param_size).
 * dtype: MRX_F32 or MRX_C64. */
int mrx_linear_scan_last(void *stream, const void *a, const void *b,
                         const void *done, const void *h0, void *h_last, int64_t B,
                         int64_t T, int64_t D, int64_t a_group, int dtype,
                         int done_dtype);

/* ---- RMS norm over the last axis -------------------------------------------------
 * y = x * rsqrt(mean(x^2) + eps) * scale -- flax.linen.RMSNorm with its defaults: the norm of the cells'
 * read-outs (linear_attention.py:109-115) and of PreNorm blocks built with it (blocks/normalization.py:10-35).
 * x, dx: (rows, D) in x_dtype; y in y_dtype, dy in dy_dtype (each MRX_F32 or MRX_BF16; arithmetic in float32);
 * scale (nullable: ones), dscale (nullable: not formed): (D) float32.  D a multiple of 4, at most 2048.
 * The backward recomputes the statistics from x, so the forward leaves nothing behind for it.
 * dx_add (nullable, like x; not dx itself): added to dx -- the gradient that reaches x along the residual branch
 * around a pre-norm block (blocks/residual.py:23-26 around normalization.py:30-31), which would otherwise
 * cost a pass of its own.
 * workspace (required with dscale): MRX_RMS_NORM_PARTS * D floats, overwritten -- per-workgroup partial sums
 * of dscale, added up in a fixed order (the result does not depend on the run). */
#define MRX_RMS_NORM_PARTS 1024
int mrx_rms_norm_fwd(void *stream, const void *x, const float *scale, void *y, int64_t rows,
                     int64_t D, int x_dtype, int y_dtype, float eps);
int mrx_rms_norm_bwd(void *stream, const void *x, const float *scale, const void *dy,
                     const void *dx_add, void *dx, float *dscale, float *workspace, int64_t rows,
                     int64_t D, int x_dtype, int dy_dtype, float eps);

/* Layer norm over the last axis: y = (x - mean(x)) * rsqrt(var(x) + eps) * scale + bias -- flax.linen.LayerNorm with
 * its defaults (eps 1e-6), the default norm of PreNorm / PostNorm (blocks/normalization.py:10-65).  Arguments as
 * mrx_rms_norm_*; bias, dbias: (D) float32 (bias nullable: zeros); dscale and dbias both or neither; workspace
 * (required with them): 2 * MRX_RMS_NORM_PARTS * D floats. */
int mrx_layer_norm_fwd(void *stream, const void *x, const float *scale, const float *bias, void *y,
                       int64_t rows, int64_t D, int x_dtype, int y_dtype, float eps);
int mrx_layer_norm_bwd(void *stream, const void *x, const float *scale, const void *dy,
                       const void *dx_add, void *dx, float *dscale, float *dbias, float *workspace,
                       int64_t rows, int64_t D, int x_dtype, int dy_dtype, float eps);

/* ---- gating product ----------------------------------------------------------------
 * y = h * silu(g): activation(gate) * value of the reference's GLU block (blocks/ffn.py:108-121) with silu as
 * the activation, one read of the operands per direction.  Backward: dh = dy * silu(g),
 * dg = dy * h * d silu(g).  All arrays n elements of `dtype` (MRX_F32 or MRX_BF16; arithmetic in float32),
 * 16-byte aligned. */
int mrx_silu_gate_fwd(void *stream, const void *h, const void *g, void *y, int64_t n, int dtype);
int mrx_silu_gate_bwd(void *stream, const void *h, const void *g, const void *dy, void *dh, void *dg,
                      int64_t n, int dtype);

/* ---- mLSTM: the stabiliser of the cell's gates ---------------------------------
 * mLSTMCell's elements (C, log_f, n, m) combine by the max-stabilised gated sum of mlstm.py:190-206
 * (m = max(m_a + log_f_b, m_b), both sides rescaled by exp(. - m)) under Memoroid.scan_fn's select-reset
 * operator (memoroid.py:60-91).  Unrolled over time the stabiliser is
 *     m_t = done_t ? log_i_t : max(m_{t-1} + log_f_t, log_i_t)
 * and C and n follow the gated linear recurrence that mrx_gated_linear_attn_* / mrx_linear_scan_* compute,
 * with log-decay and key weight
 *     g_t = done_t ? 0 : max(log_f_t + m_{t-1} - m_t, g_floor)   (<= 0) ,   w_t = exp(log_i_t - m_t)   (<= 1).
 * These two calls produce m, g, w from the gate pre-activations in one pass per (b, h), and take the gradients
 * back: dm (what the read-out's exp(-m) and the carried m contribute), dg, dw in (any of them nullable),
 * dlog_i, dlog_f and dm0 (nullable) out.  log_i, log_f, m, g, w and their gradients: (B,T,H) float32;
 * m0 (nullable: the cell's initial -1e9), dm0: (B,H); g_floor <= 0 (a decay below e^g_floor multiplies a state
 * next to a new term of weight one: the cell passes -60). */
int mrx_mlstm_gates_fwd(void *stream, const float *log_i, const float *log_f, const void *done,
                        const float *m0, float *m, float *g, float *w, int64_t B, int64_t T,
                        int64_t H, int done_dtype, float g_floor);

int mrx_mlstm_gates_bwd(void *stream, const float *log_i, const float *log_f, const void *done,
                        const float *m0, const float *m, const float *dm, const float *dg,
                        const float *dw, float *dlog_i, float *dlog_f, float *dm0, int64_t B,
                        int64_t T, int64_t H, int done_dtype, float g_floor);

/* ---- MinGRU: the diagonal scan with the cell's gate arithmetic inside ----
 * MinGRUCell (min_gru.py:49-78) maps the step's two projections z and h~ to the elements
 * (log sigma(z) + log g(h~), log sigma(-z)), g(x) = x + 0.5 (x >= 0) | sigma(x), scans them with the
 * log-space operator (logaddexp(decay_j + state_i, state_j), decay_i + decay_j) through
 * Memoroid.scan_fn (memoroid.py:60-91) and reads exp(state).  In linear space that is
 *     h_t = done_t ? b_t : a_t h_{t-1} + b_t ,   a_t = sigma(-z_t),  b_t = sigma(z_t) g(h~_t),
 * which these entry points compute from z and h~ directly: a and b are never written to memory,
 * and the backward call returns dL/dz and dL/dh~ instead of dL/da and dL/db.
 * z, h_tilde, h, g, dz, dh_tilde: (B,T,D) in `dtype`, MRX_F32 or MRX_BF16 (bfloat16 in memory, float32 in
 * the kernels: half the traffic of a kernel bound by it).  h0, P0 (nullable), h_last, P_last (nullable),
 * g_last (nullable), dh0 (nullable): (B,D) fp32 whatever `dtype` is, linear space: h0 = exp(carried log state) (0 for
 * the cell's initial -inf), P = the cumulative decay since the last reset, whose log is the carry's
 * second leaf (a product below the fp32 range underflows to 0, i.e. a log of -inf; the leaf never
 * reaches h).  No counterpart as one function in the reference (which leaves the fusion to XLA). */
int mrx_mingru_scan_fwd(void *stream, const void *z, const void *h_tilde, const void *done,
                        const void *h0, const void *P0, void *h, void *h_last, void *P_last,
                        int64_t B, int64_t T, int64_t D, int dtype, int done_dtype);

/* h: the states the forward call wrote (all of them, although a large call -- more than 600 MB through it --
 * reads only one row in eight and forms the others again from z and h_tilde).  dz, dh_tilde: gradients with
 * respect to the projections. */
int mrx_mingru_scan_bwd(void *stream, const void *z, const void *h_tilde, const void *h,
                        const void *done, const void *h0, const void *g, const void *g_last,
                        void *dz, void *dh_tilde, void *dh0, int64_t B, int64_t T, int64_t D,
                        int dtype, int done_dtype);

/* ---- Gated linear attention: linear attention with a scalar decay per step and head ----
 * The Mamba cell's algebra (mamba.py:109-122: elements (h_t = (B_t dt_t) (x) x_t, decay_t =
 * exp(dt_t A)), binary_operator (decay_j h_i + h_j, decay_j decay_i), read y_t = C_t . h_t), scanned
 * by memoroid.py:60-91, with k = B dt, v = x, q = C and the state kept as (d_v, d_k):
 *     S' = done_t ? 0 : exp(g_t) S_{t-1} ;  S_t = S' + v_t phi(k_t)^T ;  o_t = S_t phi(q_t)
 * g: (B,T,H) float32 log-decay (<= 0 for a contracting state).  Other arguments as for
 * mrx_linear_attn_fwd; S_chk is the residual for the backward call. */
int mrx_gated_linear_attn_fwd(void *stream, const void *q, const void *k,
                              const void *v, const void *g, const void *done,
                              const void *S0, void *o, void *S_last, void *S_chk,
                              int64_t B, int64_t T, int64_t H, int64_t dk, int64_t dv,
                              int dtype, int done_dtype, int feature_map);

/* Gradients w.r.t. q,k,v (pre-feature-map, in `dtype`), S0 (fp32, nullable) and the log-decay:
 * dg: (B,T,H) float32.  With edot_t = phi(q_t) . dphi(q)_t - phi(k_t) . dphi(k)_t,
 *     dg_t = done_t ? 0 : sum over i >= t of t's episode of edot_i  (+ <S_last, dS_last> when the
 *     episode reaches the end),
 * summed inside the kernel, which walks the time axis from the end.  S_last: the forward call's
 * output, read only when dS_last is given (nullable otherwise). */
int mrx_gated_linear_attn_bwd(void *stream, const void *q, const void *k,
                              const void *v, const void *g, const void *done,
                              const void *S_chk, const float *S_last, const void *dout,
                              const void *dS_last, void *dq, void *dk_out, void *dv_out,
                              float *dg, void *dS0, int64_t B, int64_t T, int64_t H, int64_t dk,
                              int64_t dv, int dtype, int done_dtype, int feature_map);

/* ---- Single time step (rollout / acting) ------------------------------------
 * What Memoroid.__call__ (memoroid.py:93-109) computes when T = 1, as PPO's rollout
 * does once per environment step (algorithms/ppo.py:105-143): one update of the
 * carry fused with the read-out, without the chunk machinery.
 *   q,k: (B,1,H,dk) = (B,H,dk), v,o: (B,H,dv) in `dtype` (head dims as for mrx_linear_attn_fwd);
 *   done: (B,) ; S_in/S_out: (B,H,dv,dk) fp32.
 * S_in may be NULL (zero state) and may equal S_out (update in place).
 *
 * Linear attention (linear_attention.py:62-117):
 *     S' = (done ? 0 : S) + v phi(k)^T ;  o = S' phi(q)
 * and, when z_out is given (z_in/z_out: (B,H,dk) fp32, z_in nullable, may alias), the
 * normaliser of LinearAttentionCell.read (linear_attention.py:100-110):
 *     z' = (done ? 0 : z) + phi(k) ;  o = S' phi(q) / max(phi(q) . z', eps). */
int mrx_linear_attn_step(void *stream, const void *q, const void *k,
                         const void *v, const void *done, const float *S_in,
                         const float *z_in, void *o, float *S_out, float *z_out,
                         int64_t B, int64_t H, int64_t dk, int64_t dv, int dtype,
                         int done_dtype, int feature_map, float eps);

/* Gated linear attention, the T = 1 case of mrx_gated_linear_attn_fwd (the Mamba cell's step,
 * mamba.py:109-135, and the mLSTM cell's in its stabilised units, mlstm.py:163-229):
 *     S' = (done ? 0 : exp(g) S) + v phi(k)^T ;  o = S' phi(q)
 * g: (B,H) float32, the log-decay of the step. */
int mrx_gated_linear_attn_step(void *stream, const void *q, const void *k,
                               const void *v, const float *g, const void *done,
                               const float *S_in, void *o, float *S_out, int64_t B,
                               int64_t H, int64_t dk, int64_t dv, int dtype,
                               int done_dtype, int feature_map);

/* Delta rule (no counterpart in the reference; the T = 1 case of mrx_delta_rule_fwd):
 *     S0 = done ? 0 : S ;  u = beta (v - S0 k) ;  S' = S0 + u k^T ;  o = S' q
 * beta: (B,H) in `dtype`. */
int mrx_delta_rule_step(void *stream, const void *q, const void *k,
                        const void *v, const void *beta, const void *done,
                        const float *S_in, void *o, float *S_out, int64_t B,
                        int64_t H, int64_t dk, int64_t dv, int dtype,
                        int done_dtype);

#ifdef __cplusplus
}
#endif
#endif /* MEMORAX_AMD_H */
