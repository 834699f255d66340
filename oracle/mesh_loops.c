/*
 * TEST INFRASTRUCTURE ONLY.  Builds the brute-force loop restatement of the
 * reference's mesh ops (see mesh_loops.inc) in two precisions:
 *   *_f32  reference precision, sequential summation order
 *   *_f64  double precision, the answer parity is measured against
 * Only tests, the smoke check and the benchmark's CPU-baseline leg may load
 * the resulting shared object; the product never does.
 */
#include <math.h>
#include <stdlib.h>

#define REAL float
#define SUFFIX f32
#include "mesh_loops.inc"
#undef REAL
#undef SUFFIX

#define REAL double
#define SUFFIX f64
#include "mesh_loops.inc"
#undef REAL
#undef SUFFIX
