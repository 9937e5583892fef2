/*
 * TEST INFRASTRUCTURE -- CPU oracle for the CGT native CNN hot path.
 *
 * A plain-C, single-threaded restatement of what the reference computes in
 * include/im2col.h, include/pooling.h, include/lrn.cuh and the Mul22 /
 * BatchedMul22 / Transpose op bodies of cgt/core.py.  It exists to check the
 * HIP library and to be timed as the CPU baseline; the product never calls it.
 * Build: `make -C oracle` (gcc, no -march flags, fp contraction off so that
 * the add order written here is the add order executed).
 */
#include <float.h>
#include <math.h>
#include <stddef.h>

#define REAL float
#define FN(x) x##_f32
#define FN_POW powf
#include "cgt_oracle_impl.h"
#undef REAL
#undef FN
#undef FN_POW

#define REAL double
#define FN(x) x##_f64
#define FN_POW pow
#include "cgt_oracle_impl.h"
#undef REAL
#undef FN
#undef FN_POW

/* Pooled extent: ceil((H + 2*pad - k) / stride), no "+1"
 * (/root/reference/cgt/nn_ops/max_pool_2d.py:40-41, cgt/api.py:145-146). */
long oracle_pool_outsize(long H, int k, int pad, int stride)
{
    long num = H + 2 * pad - k;
    if (num <= 0) return 0;
    return (num + stride - 1) / stride;
}

/* im2col extent: (H + 2*pad - k) / stride + 1
 * (/root/reference/cgt/nn_ops/im2col.py:39-40). */
long oracle_conv_outsize(long H, int k, int pad, int stride)
{
    return (H + 2 * pad - k) / stride + 1;
}
