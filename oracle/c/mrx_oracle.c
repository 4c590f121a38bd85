/* Plain-C sequential restatement of the memorax sequence-model hot path
 * (forward + analytic backward).
 *
 * TEST INFRASTRUCTURE ONLY: loaded by tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py as the checker / timed CPU baseline.  The product
 * library never links or loads it.
 *
 * Each function is pinned (tests/test_oracle_c.py) against the NumPy fp64
 * restatement in oracle/memoroid.py and the torch-fp64 autograd gradients in
 * oracle/grad.py, which are themselves pinned by closed forms and independent
 * formulations; the reference ships no vectors for this path.
 *
 * _f64 entry points keep the running state in double (parity checker);
 * _f32 entry points keep it in float (what a CPU implementation would ship;
 * used as the timed baseline).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)

#define REAL double
#define FN(name) CAT(name, _f64)
#include "mrx_oracle_core.inc"
#undef REAL
#undef FN

#define REAL float
#define FN(name) CAT(name, _f32)
#include "mrx_oracle_core.inc"
#undef REAL
#undef FN

#ifdef _OPENMP
#include <omp.h>
int orc_num_threads(void) { return omp_get_max_threads(); }
void orc_set_num_threads(int n) { omp_set_num_threads(n); }
#else
int orc_num_threads(void) { return 1; }
void orc_set_num_threads(int n) { (void)n; }
#endif
