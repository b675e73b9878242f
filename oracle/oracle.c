/* CPU oracle: the reference's algorithms restated in plain C.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker that tests/, the
 * smoke check and the benchmark's CPU-baseline leg compare the HIP path
 * against.  The shipped library never links, loads or calls it.
 *
 * What pins each part (tests/test_oracle_*.py, tests/test_accumulate_oracle.py);
 * no function here is left unpinned:
 *   per-op rules (oracle_ops.inc)  formulas written independently in numpy, central
 *       differences in fp64, reverse-mode autodiff of every op written once more as
 *       a differentiable expression, the guards and special cases of the reference's
 *       op tests;
 *   chain (oracle_chain_*)         the reference's own evaluation of the graph at the
 *       points of tests/golden/chain_reference_vector.json, a closed form without a
 *       matrix inverse, reverse-mode autodiff of an independent statement, central
 *       differences;
 *   accumulation sums              a bincount formulation and the reference's exact
 *       counting pattern (tests/test_parallel_gradient_accumulation.cu:94-99);
 *   least squares (oracle_linreg.c) hand-computed gradients at the reference's test
 *       points, a closed form, central differences, one-step and schedule closed forms;
 *   Adam (oracle_adam.c) and the renderer (oracle_splat.inc): the reference's tests
 *       hold no expected values for either (parity with the reference is unpinned
 *       in that sense); pinned by closed forms, an fp64 recurrence, a brute-force
 *       renderer, invariance to listing order, central differences of the loss, and
 *       an independently written renderer whose gradients come from reverse-mode
 *       autodiff (image, loss and all nine gradients of a single-tile scene).
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
