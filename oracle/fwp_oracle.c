/*
 * TEST INFRASTRUCTURE ONLY.  CPU oracle of the fast-weight update operators in
 * plain C, float and double.  Only tests, the smoke check and the benchmark's
 * CPU-baseline leg may load this library; no product code path does.
 * The algorithm and the reference lines it follows are in fwp_oracle_impl.h.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

#define REAL float
#define SUFFIX _f32
#define EXP expf
#define TANH tanhf
#include "fwp_oracle_impl.h"
#undef REAL
#undef SUFFIX
#undef EXP
#undef TANH

#define REAL double
#define SUFFIX _f64
#define EXP exp
#define TANH tanh
#include "fwp_oracle_impl.h"
#undef REAL
#undef SUFFIX
#undef EXP
#undef TANH

#ifdef _OPENMP
#include <omp.h>
int fwp_oracle_threads(void) { return omp_get_max_threads(); }
void fwp_oracle_set_threads(int n) { if (n > 0) omp_set_num_threads(n); }
#else
int fwp_oracle_threads(void) { return 1; }
void fwp_oracle_set_threads(int n) { (void)n; }
#endif
