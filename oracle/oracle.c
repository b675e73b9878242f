/* CPU oracle: the reference's algorithms restated in plain C.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker that tests/, the
 * smoke check and the benchmark's CPU-baseline leg compare the HIP path
 * against.  The shipped library never links, loads or calls it.
 *
 * Built twice over by the preprocessor: every op exists as name_f32 (float
 * arithmetic with the float libm routines, i.e. what the reference computes in
 * device code) and name_f64 (double).  Compile with contraction off so each
 * statement rounds exactly as written.
 */
#include <math.h>
#include <stddef.h>
#include <omp.h>

#define REAL float
#define SUFFIX _f32
#define R_EXP expf
#define R_SIN sinf
#define R_COS cosf
#define R_SQRT sqrtf
#define R_ABS fabsf
#include "oracle_ops.inc"
#undef REAL
#undef SUFFIX
#undef R_EXP
#undef R_SIN
#undef R_COS
#undef R_SQRT
#undef R_ABS

#define REAL double
#define SUFFIX _f64
#define R_EXP exp
#define R_SIN sin
#define R_COS cos
#define R_SQRT sqrt
#define R_ABS fabs
#include "oracle_ops.inc"
#undef REAL
#undef SUFFIX
#undef R_EXP
#undef R_SIN
#undef R_COS
#undef R_SQRT
#undef R_ABS

int oracle_max_threads(void) { return omp_get_max_threads(); }
void oracle_set_threads(int n) { if (n > 0) omp_set_num_threads(n); }
