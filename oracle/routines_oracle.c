/* CPU restatement of the reference's dense routines for float32, float64 and float16 operands.  TEST INFRASTRUCTURE ONLY: the
 * product never links or calls this file; it is the checker the GPU kernels are compared with.
 *
 * Every function follows the loop structure of the reference's CPU implementation and keeps its arithmetic:
 * scalars are doubles (JavaScript numbers), typed-array stores round to the element type (Float32Array,
 * Float16Array; a Float64Array keeps the double).  Built with -ffp-contract=off so that no multiply-add is fused.
 * The bodies are in routines_body.h, included once per element type: the float32 functions keep their plain
 * names, the others end in _f64 and _f16 (float16 values travel as uint16_t bit patterns).
 *
 *   ro_triangular_solve  src/routine.ts:298-336
 *   ro_cholesky          src/routine.ts:338-362
 *   ro_lu                src/routine.ts:364-420
 *   ro_jacobi_eigh       src/routine.ts:422-543
 *   ro_fft               src/routine.ts:545-640
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "half.h"

static double js_max(double a, double b) { return (a != a || b != b) ? NAN : (a > b ? a : b); }

#define RO_T float
#define RO_LD(x) ((double)(x))
#define RO_ST(v) ((float)(v))
#define RO_NAME(f) f
#include "routines_body.h"
#undef RO_T
#undef RO_LD
#undef RO_ST
#undef RO_NAME

#define RO_T double
#define RO_LD(x) (x)
#define RO_ST(v) ((double)(v))
#define RO_NAME(f) f##_f64
#include "routines_body.h"
#undef RO_T
#undef RO_LD
#undef RO_ST
#undef RO_NAME

#define RO_T uint16_t
#define RO_LD(x) half_to_double(x)
#define RO_ST(v) double_to_half(v)
#define RO_NAME(f) f##_f16
#include "routines_body.h"
#undef RO_T
#undef RO_LD
#undef RO_ST
#undef RO_NAME
