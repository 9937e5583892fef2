// TEST INFRASTRUCTURE -- thin extern "C" wrappers around the REFERENCE's own
// CPU code, compiled in place from /root/reference (include/im2col.h,
// include/pooling.h, include/cgt_common.h, src/cgt_common.cpp).  Nothing from
// the reference is copied: this file only names its templates and classes.
// The result (oracle/_ref/libcgt_ref.so) is used to validate the restatement
// in cgt_oracle.c and to write the golden vectors under tests/golden/.
//
// im2col_cpu / col2im_cpu take their geometry as template constants
// (im2col.h:5,29), so the wrappers dispatch over a fixed table of geometries.
#include "cgt_common.h"
#include "im2col.h"
#include "pooling.h"

// (kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w)
#define REF_GEOMS(X) \
    X(4, 4, 0, 0, 1, 1)   \
    X(3, 3, 1, 1, 2, 2)   \
    X(3, 3, 1, 1, 3, 3)   \
    X(3, 3, 1, 1, 1, 1)   \
    X(3, 3, 0, 0, 1, 1)   \
    X(5, 5, 2, 2, 1, 1)   \
    X(11, 11, 0, 0, 4, 4) \
    X(4, 7, 3, 6, 1, 1)   \
    X(2, 3, 0, 1, 3, 2)   \
    X(1, 1, 0, 0, 1, 1)   \
    X(2, 2, 0, 0, 2, 2)   \
    X(3, 2, 1, 0, 2, 1)   \
    X(5, 3, 2, 1, 2, 3)   \
    X(2, 2, 1, 1, 1, 1)

template <typename T>
static int im2col_dispatch(const T* im, long B, long C, long H, long W,
                           int kh, int kw, int ph, int pw, int sh, int sw, T* col) {
    long m = (H + 2 * ph - kh) / sh + 1, n = (W + 2 * pw - kw) / sw + 1;
    long istride = C * H * W, ostride = m * n * C * kh * kw;
#define X(KH, KW, PH, PW, SH, SW)                                                      \
    if (kh == KH && kw == KW && ph == PH && pw == PW && sh == SH && sw == SW) {        \
        for (long b = 0; b < B; ++b)                                                   \
            im2col_cpu<T, KH, KW, PH, PW, SH, SW>(im + b * istride, C, H, W,           \
                                                  col + b * ostride);                  \
        return 0;                                                                      \
    }
    REF_GEOMS(X)
#undef X
    return -1;
}

template <typename T>
static int col2im_dispatch(const T* col, long B, long C, long H, long W,
                           int kh, int kw, int ph, int pw, int sh, int sw, T* im) {
    long m = (H + 2 * ph - kh) / sh + 1, n = (W + 2 * pw - kw) / sw + 1;
    long istride = C * H * W, ostride = m * n * C * kh * kw;
#define X(KH, KW, PH, PW, SH, SW)                                                      \
    if (kh == KH && kw == KW && ph == PH && pw == PW && sh == SH && sw == SW) {        \
        for (long b = 0; b < B; ++b)                                                   \
            col2im_cpu<T, KH, KW, PH, PW, SH, SW>(col + b * ostride, C, H, W,          \
                                                  im + b * istride);                   \
        return 0;                                                                      \
    }
    REF_GEOMS(X)
#undef X
    return -1;
}

template <typename T> struct dtype_of;
template <> struct dtype_of<float> { static const cgtDtype v = cgt_f4; };
template <> struct dtype_of<double> { static const cgtDtype v = cgt_f8; };

template <typename T>
static void pool_fwd(const T* bottom, long N, long C, long H, long W,
                     int kh, int kw, int ph, int pw, int sh, int sw,
                     long PH, long PW, T* top, int* mask) {
    conv_closure cl = {kh, kw, ph, pw, sh, sw};
    long bs[4] = {N, C, H, W}, ts[4] = {N, C, PH, PW};
    IRC<cgtArray> b(new cgtArray(4, bs, dtype_of<T>::v, cgtCPU, (void*)bottom, false));
    IRC<cgtArray> t(new cgtArray(4, ts, dtype_of<T>::v, cgtCPU, (void*)top, false));
    IRC<cgtArray> m(new cgtArray(4, ts, cgt_i4, cgtCPU, (void*)mask, false));
    max_pool<T>(&cl, b.get(), t.get(), m.get());
}

template <typename T>
static void pool_bwd(const int* mask, const T* top_diff, long N, long C, long H, long W,
                     long PH, long PW, T* bottom_diff) {
    long bs[4] = {N, C, H, W}, ts[4] = {N, C, PH, PW};
    // max_pool_pullback only reads shapes from `bottom` and `top`
    // (pooling.h:84-89); bottom_diff stands in for bottom, top_diff for top.
    IRC<cgtArray> bd(new cgtArray(4, bs, dtype_of<T>::v, cgtCPU, (void*)bottom_diff, false));
    IRC<cgtArray> td(new cgtArray(4, ts, dtype_of<T>::v, cgtCPU, (void*)top_diff, false));
    IRC<cgtArray> m(new cgtArray(4, ts, cgt_i4, cgtCPU, (void*)mask, false));
    max_pool_pullback<T>(bd.get(), td.get(), m.get(), td.get(), bd.get());
}

extern "C" {
__attribute__((visibility("default"))) int ref_im2col_f32(const float* im, long B, long C, long H, long W, int kh, int kw, int ph, int pw, int sh, int sw, float* col) { return im2col_dispatch<float>(im, B, C, H, W, kh, kw, ph, pw, sh, sw, col); }
__attribute__((visibility("default"))) int ref_im2col_f64(const double* im, long B, long C, long H, long W, int kh, int kw, int ph, int pw, int sh, int sw, double* col) { return im2col_dispatch<double>(im, B, C, H, W, kh, kw, ph, pw, sh, sw, col); }
__attribute__((visibility("default"))) int ref_col2im_f32(const float* col, long B, long C, long H, long W, int kh, int kw, int ph, int pw, int sh, int sw, float* im) { return col2im_dispatch<float>(col, B, C, H, W, kh, kw, ph, pw, sh, sw, im); }
__attribute__((visibility("default"))) int ref_col2im_f64(const double* col, long B, long C, long H, long W, int kh, int kw, int ph, int pw, int sh, int sw, double* im) { return col2im_dispatch<double>(col, B, C, H, W, kh, kw, ph, pw, sh, sw, im); }
__attribute__((visibility("default"))) void ref_max_pool_f32(const float* bottom, long N, long C, long H, long W, int kh, int kw, int ph, int pw, int sh, int sw, long PH, long PW, float* top, int* mask) { pool_fwd<float>(bottom, N, C, H, W, kh, kw, ph, pw, sh, sw, PH, PW, top, mask); }
__attribute__((visibility("default"))) void ref_max_pool_f64(const double* bottom, long N, long C, long H, long W, int kh, int kw, int ph, int pw, int sh, int sw, long PH, long PW, double* top, int* mask) { pool_fwd<double>(bottom, N, C, H, W, kh, kw, ph, pw, sh, sw, PH, PW, top, mask); }
__attribute__((visibility("default"))) void ref_max_pool_pullback_f32(const int* mask, const float* top_diff, long N, long C, long H, long W, long PH, long PW, float* bottom_diff) { pool_bwd<float>(mask, top_diff, N, C, H, W, PH, PW, bottom_diff); }
__attribute__((visibility("default"))) void ref_max_pool_pullback_f64(const int* mask, const double* top_diff, long N, long C, long H, long W, long PH, long PW, double* bottom_diff) { pool_bwd<double>(mask, top_diff, N, C, H, W, PH, PW, bottom_diff); }
}
