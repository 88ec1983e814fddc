/* C restatement of the reference's CTC-Transducer arithmetic, in float and in
 * double.  TEST INFRASTRUCTURE ONLY: used by tests/, the smoke check and the
 * cpu_baseline leg of bench.py; the shipped library never links or loads it.
 *
 * Exported (each in an _f32 and an _f64 flavour, see ctct_lattice.inc):
 *   oracle_ctct_loss_fwd_*    mirror of _C.ctct_loss_fwd   (csrc/binding.cpp:31-100)
 *   oracle_ctct_loss_dense_*  gather + lattice + dense gradient of ctct_loss
 *                             (warp_ctct/__init__.py:88-147 and its autograd)
 *   oracle_log_matmul_*       log-semiring matmul (csrc/logmatmul.cu:44-146)
 *   oracle_num_threads        OpenMP threads the loops above will use
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define REAL float
#define SUF f32
#define R_EXP expf
#define R_LOG logf
#define R_LOG1P log1pf
#include "ctct_lattice.inc"
#undef REAL
#undef SUF
#undef R_EXP
#undef R_LOG
#undef R_LOG1P

#define REAL double
#define SUF f64
#define R_EXP exp
#define R_LOG log
#define R_LOG1P log1p
#include "ctct_lattice.inc"
#undef REAL
#undef SUF
#undef R_EXP
#undef R_LOG
#undef R_LOG1P

int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void oracle_set_num_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}
