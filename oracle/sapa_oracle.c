/* Brute-force CPU oracle for SAPA's operators, in plain C.
 *
 * TEST INFRASTRUCTURE ONLY: used by tests/, by __graft_entry__.smoke() and by
 * bench.py's cpu_baseline leg as the checker.  The product never links it.
 *
 * Three arithmetic modes are generated from sapa_oracle_body.inc, which
 * transcribes the index math and loop order of the reference's kernels
 * (file:line cited at each function there):
 *   oracle_f32_*     float storage, float FMA accumulation in the kernels'
 *                    order: the reference's own fp32 arithmetic
 *   oracle_f64_*     everything in double
 *   oracle_f32a64_*  float inputs, coordinates and weights in float as the
 *                    kernels compute them, sums in double, double output:
 *                    the value fp32 results are measured against
 *                    (forward functions only)
 */
#include <math.h>
#include <stddef.h>

#define IN_T float
#define OUT_T float
#define ACC_T float
#define FMA fmaf
#define FLOOR floorf
#define EXP expf
#define NAME(x) oracle_f32_##x
#include "sapa_oracle_body.inc"
#undef IN_T
#undef OUT_T
#undef ACC_T
#undef FMA
#undef FLOOR
#undef EXP
#undef NAME

#define IN_T double
#define OUT_T double
#define ACC_T double
#define FMA fma
#define FLOOR floor
#define EXP exp
#define NAME(x) oracle_f64_##x
#include "sapa_oracle_body.inc"
#undef IN_T
#undef OUT_T
#undef ACC_T
#undef FMA
#undef FLOOR
#undef EXP
#undef NAME

#define ORACLE_FORWARD_ONLY
#define IN_T float
#define OUT_T double
#define ACC_T double
#define FMA fma
#define FLOOR floorf
#define EXP exp
#define NAME(x) oracle_f32a64_##x
#include "sapa_oracle_body.inc"
