// Chunk-parallel linear attention: the two small kernels that take the state off the sequential path.
//
// The state of linear attention is additive, S_t = r_t S_{t-1} + v_t k_t^T, so the state entering
// chunk c is a sum of per-chunk terms that do not depend on one another.  When there are too few
// (batch, head) sequences to fill the device with one workgroup each, the work is cut along time
// instead:
//   1. chunk_states: every chunk of every sequence, one workgroup each, forms its own contribution
//        forward   KV_c  = sum over the rows j of the chunk's last episode of v_j phi(k_j)^T
//        backward  QdO_c = sum over the rows i of the chunk's first episode of do_i phi(q_i)^T
//      (fp32 [dv][dk], the layout of S0 / S_last), into slot c of a (B,H,NC,64,64) buffer;
//   2. state_scan: per sequence, an exclusive running sum over the slots, in place --
//        forward   slot c <- state entering chunk c,           S <- (chunk c has a reset ? 0 : S) + KV_c
//        backward  slot c <- gradient of the state leaving c,  dS <- (chunk c has a reset ? 0 : dS) + QdO_c
//      walking c upwards (forward) or downwards (backward); the final value is S_last (dS0);
//   3. the chunk kernels proper (chunk_fwd.hip, chunk_bwd.hip) run with one workgroup per chunk, each
//      taking its entering state (and the gradient of its leaving state) from its slot.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "hd.h"

namespace mrx {
inline namespace MRX_HD_NS {

// slots[B][H][NC][dv][dk] fp32 <- per-chunk contributions.  x: keys (forward) or queries (backward),
// (B,T,H,dk), y: values (forward) or output gradients (backward), (B,T,H,dv), of `dtype`; fmap: elu+1 on x.
// dk, dv: the build's head dim, or less in whole 16-byte segments (narrow heads).
// C is the chunk length of the linear-attention kernels for `dtype`.  Returns an MRX_* status.
int launch_la_chunk_states(hipStream_t st, const void *x, const void *y, const void *done, int done_f32, float *slots,
                           int64_t B, int64_t Tlen, int64_t H, int dtype, bool fmap, bool backward, int64_t dk, int64_t dv);

// In-place exclusive scan over the slots of every sequence (see above).  init: (B,H,dv,dk) fp32 or
// null (zero); fin: (B,H,dv,dk) fp32 or null.  C: chunk length the slots were formed with.
int launch_la_state_scan(hipStream_t st, float *slots, const float *init, float *fin, const void *done, int done_f32,
                         int64_t B, int64_t Tlen, int64_t H, int C, bool backward, int64_t dk, int64_t dv);

}  // namespace MRX_HD_NS
}  // namespace mrx
