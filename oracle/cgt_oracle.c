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

/* ------------------------------------------------------------------ conv-layer glue
 * Elementwise ops as the reference's native CPU templates evaluate them: the
 * C expression of UNARY_INFO / BINARY_INFO (/root/reference/cgt/core.py:1118-1152)
 * applied to operands of their own C type (float, or int8_t for "i1"), the
 * usual arithmetic conversions, result cast to the output type
 * (core.py:1206-1218, 1336-1349).  math.h functions therefore run in double. */

enum { UN_ABS, UN_COS, UN_EXP, UN_LOG, UN_NEG, UN_SIGN, UN_SIN, UN_SQUARE, UN_SQRT, UN_TANH, UN_SIGMOID };
enum { BIN_MUL, BIN_ADD, BIN_SUB, BIN_DIV, BIN_LT, BIN_GT, BIN_LE, BIN_GE, BIN_POW, BIN_EQ, BIN_NE };

int oracle_elwise_unary_f32(int op, long n, const float *in, float *out)
{
    for (long i = 0; i < n; ++i) {
        float x = in[i];
        switch (op) {
        case UN_ABS: out[i] = fabs(x); break;
        case UN_COS: out[i] = cos(x); break;
        case UN_EXP: out[i] = exp(x); break;
        case UN_LOG: out[i] = log(x); break;
        case UN_NEG: out[i] = (-x); break;
        case UN_SIGN: out[i] = 2 * (x > 0) - 1; break;
        case UN_SIN: out[i] = sin(x); break;
        case UN_SQUARE: out[i] = x * x; break;
        case UN_SQRT: out[i] = sqrt(x); break;
        case UN_TANH: out[i] = tanh(x); break;
        case UN_SIGMOID: out[i] = 1.0 / (1.0 + exp(-x)); break;
        default: return 1;
        }
    }
    return 0;
}

#define ORACLE_BINARY(NAME, TX, TY, TZ, TCMP)                                              \
    int NAME(int op, long n, const TX *in0, int s0, const TY *in1, int s1, void *outv)     \
    {                                                                                      \
        TZ *out = (TZ *)outv;                                                              \
        TCMP *outc = (TCMP *)outv;                                                         \
        float *outf = (float *)outv;                                                       \
        for (long i = 0; i < n; ++i) {                                                     \
            TX x = in0[s0 ? 0 : i];                                                        \
            TY y = in1[s1 ? 0 : i];                                                        \
            switch (op) {                                                                  \
            case BIN_MUL: out[i] = x * y; break;                                           \
            case BIN_ADD: out[i] = x + y; break;                                           \
            case BIN_SUB: out[i] = x - y; break;                                           \
            case BIN_DIV: outf[i] = (x + 0.0) / y; break;                                  \
            case BIN_POW: out[i] = pow(x, y); break;                                       \
            case BIN_LT: outc[i] = x < y; break;                                           \
            case BIN_GT: outc[i] = x > y; break;                                           \
            case BIN_LE: outc[i] = x <= y; break;                                          \
            case BIN_GE: outc[i] = x >= y; break;                                          \
            case BIN_EQ: outc[i] = x == y; break;                                          \
            case BIN_NE: outc[i] = x != y; break;                                          \
            default: return 1;                                                             \
            }                                                                              \
        }                                                                                  \
        return 0;                                                                          \
    }
/* output: comparisons int8, "/" float, otherwise the promoted operand type */
ORACLE_BINARY(oracle_elwise_binary_ff, float, float, float, signed char)
ORACLE_BINARY(oracle_elwise_binary_fb, float, signed char, float, signed char)
ORACLE_BINARY(oracle_elwise_binary_bf, signed char, float, float, signed char)
ORACLE_BINARY(oracle_elwise_binary_bb, signed char, signed char, signed char, signed char)

/* Repeat (/root/reference/cgt/core.py:1528-1546): write.at(i0..) = read.at(i0.. with 0 on
 * the repeated axes).  Element size in bytes. */
int oracle_repeat(const void *x, int itemsize, int ndim, const long *oshape, const int *repeated, void *out)
{
    long n = 1, xstride[8], idx[8];
    if (ndim > 8) return 1;
    long acc = 1;
    for (int a = ndim - 1; a >= 0; --a) {
        xstride[a] = repeated[a] ? 0 : acc;
        if (!repeated[a]) acc *= oshape[a];
        n *= oshape[a];
        idx[a] = 0;
    }
    for (long o = 0; o < n; ++o) {
        long src = 0;
        for (int a = 0; a < ndim; ++a) src += idx[a] * xstride[a];
        for (int b = 0; b < itemsize; ++b)
            ((char *)out)[o * itemsize + b] = ((const char *)x)[src * itemsize + b];
        for (int a = ndim - 1; a >= 0; --a) {
            if (++idx[a] < oshape[a]) break;
            idx[a] = 0;
        }
    }
    return 0;
}

/* Sum over axes, keepdims (gen_reduction_code, /root/reference/cgt/core.py:1663-1685):
 * out initialised to 0, then one pass over the input in row-major order, each element
 * added to its output cell in the array's own type. */
#define ORACLE_SUM(NAME, T)                                                                \
    int NAME(const T *x, int ndim, const long *shape, const int *reduced, T *out)          \
    {                                                                                      \
        long n = 1, nout = 1, ostride[8], idx[8];                                          \
        if (ndim > 8) return 1;                                                            \
        long acc = 1;                                                                      \
        for (int a = ndim - 1; a >= 0; --a) {                                              \
            ostride[a] = reduced[a] ? 0 : acc;                                             \
            if (!reduced[a]) acc *= shape[a];                                              \
            n *= shape[a];                                                                 \
            idx[a] = 0;                                                                    \
        }                                                                                  \
        nout = acc;                                                                        \
        for (long o = 0; o < nout; ++o) out[o] = 0;                                        \
        for (long i = 0; i < n; ++i) {                                                     \
            long dst = 0;                                                                  \
            for (int a = 0; a < ndim; ++a) dst += idx[a] * ostride[a];                     \
            out[dst] = out[dst] + x[i];                                                    \
            for (int a = ndim - 1; a >= 0; --a) {                                          \
                if (++idx[a] < shape[a]) break;                                            \
                idx[a] = 0;                                                                \
            }                                                                              \
        }                                                                                  \
        return 0;                                                                          \
    }
ORACLE_SUM(oracle_sum_f32, float)
ORACLE_SUM(oracle_sum_f64, double)
