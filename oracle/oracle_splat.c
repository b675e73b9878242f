/* CPU oracle of the tile-binned splatting step.  TEST INFRASTRUCTURE ONLY.
 * See oracle_splat.inc for the model and for which parts follow the reference. */
#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <omp.h>

#define REAL float
#define SUFFIX _f32
#define R_SQRT sqrtf
#define R_FLOOR floorf
#include "oracle_splat.inc"
#undef REAL
#undef SUFFIX
#undef R_SQRT
#undef R_FLOOR

#define REAL double
#define SUFFIX _f64
#define R_SQRT sqrt
#define R_FLOOR floor
#include "oracle_splat.inc"
