/*
 * TEST INFRASTRUCTURE ONLY -- see d2c_oracle.h.  Instantiates the restatement
 * in d2c_oracle_impl.h for float and double.
 */
#include "d2c_oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* dconv_gpu_common.h:13-15 get_output_size */
int oracle_output_size(int in, int k, int stride, int pad, int dil)
{
    return (in + 2 * pad - (dil * (k - 1) + 1)) / stride + 1;
}

int oracle_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

#define T float
#define SUFFIX f32
#define FLOOR floorf
#define FMA fmaf
#define FABS fabsf
#include "d2c_oracle_impl.h"
#undef T
#undef SUFFIX
#undef FLOOR
#undef FMA
#undef FABS

#define T double
#define SUFFIX f64
#define FLOOR floor
#define FMA fma
#define FABS fabs
#include "d2c_oracle_impl.h"
