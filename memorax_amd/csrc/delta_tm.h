// The delta rule's triangular factors, one wave per chunk, before the sequential kernel runs.
//
// Tm = (I + tril(diag(beta) K K^T, -1))^-1 of a 32-row chunk depends on the chunk's keys and gates
// only, yet inside the forward kernel its chain of small dependent products sat in the middle of
// the per-chunk sequence and took half of it with one or two of four waves busy.  Here every chunk
// of every sequence is an independent task for one wave and nothing but registers is used:
//   * the K tile is loaded straight into MFMA operand fragments (16 bytes per lane),
//   * K K^T: the two diagonal 16x16 tiles and both off-diagonal ones,
//   * per episode of the chunk ("pass"; rows of other episodes removed by select): the two diagonal
//     blocks by repeated squaring, interleaved, then X_10 = -X_11 A_10 X_00, computed transposed so
//     that a lane ends up with four consecutive columns of a row,
//   * rows of the pass's episode -> Tm_chk (row-major 32x32 per chunk), which is what the forward
//     and the backward kernel read.
// The 16x16 products of the bf16 kernels run on the bf16 pipe with each operand split once into a
// high and a low bf16 half (x = xh + xl up to 2^-16): Xh Yh + Xl Yh + Xh Yl as three 16x16x16
// MFMAs whose operands are those halves as they are, so a matrix is converted once however many
// products use it.  The vector ALU, not the matrix pipe, bounds this kernel.
// PRO: keys L2-normalised and gates passed through a sigmoid exactly as the kernels that stage
// them do (same summation tree for the norm, same rounding), so all three see the same k_n, beta.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "hd.h"

namespace mrx {
inline namespace MRX_HD_NS {

// Longest sequence the launch covers: four chunks per workgroup, 65535 workgroups along the grid's y.
constexpr int64_t DELTA_TM_MAX_T = 4ll * 65535 * 32;

// Fills Tm_chk[B][H][ceil(T / 32)][32][32] (dtype: MRX_F32 or MRX_BF16) from the keys [B][T][H][dk],
// the gates [B][T][H] and the reset flags [B][T].  prologue: keys are L2-normalised and gates go
// through a sigmoid first.  dk: the build's head dim, or less in whole 16-byte segments (narrow heads).
// Returns an MRX_* status (MRX_ERR_INVALID_ARG beyond DELTA_TM_MAX_T steps).
int launch_delta_tm(hipStream_t st, const void *k, const void *beta, const void *done, int done_f32, void *Tm_chk,
                    int64_t B, int64_t Tlen, int64_t H, int dtype, bool prologue, int64_t dk);

}  // namespace MRX_HD_NS
}  // namespace mrx
