/* TEST INFRASTRUCTURE ONLY -- see dk_oracle.h.  Instantiates the restatement
 * in dk_oracle_impl.h for float and double. */
#include "dk_oracle.h"

#include <math.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define REAL float
#define SUFFIX _f32
#include "dk_oracle_impl.h"
#undef REAL
#undef SUFFIX

#define REAL double
#define SUFFIX _f64
#include "dk_oracle_impl.h"
#undef REAL
#undef SUFFIX

int dko_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void dko_set_threads(int n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}
