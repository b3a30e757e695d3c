/* C restatement of the reference's OpenMP CPU path for evaluate_inversed (forward, backward, and the
 * box-culled variants).  TEST INFRASTRUCTURE ONLY: parity checker for tests/ and the timed CPU baseline of
 * bench.py; the product never links or loads it.  The algorithm text lives in cpu_ref_impl.h, instantiated
 * here for float and double.  Build: see Makefile in this directory. */
#include <math.h>
#include <stddef.h>
#include <string.h>

#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)

#define SCALAR float
#define FN(name) CAT(name, _f32)
#define SQRT sqrtf
#define EXP expf
#include "cpu_ref_impl.h"
#undef SCALAR
#undef FN
#undef SQRT
#undef EXP

#define SCALAR double
#define FN(name) CAT(name, _f64)
#define SQRT sqrt
#define EXP exp
#include "cpu_ref_impl.h"
#undef SCALAR
#undef FN
#undef SQRT
#undef EXP

#ifdef _OPENMP
#include <omp.h>
int cpu_ref_max_threads(void) { return omp_get_max_threads(); }
#else
int cpu_ref_max_threads(void) { return 1; }
#endif
