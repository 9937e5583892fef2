// TEST INFRASTRUCTURE -- the REFERENCE's own cross-channel LRN kernels
// (include/lrn.cuh: LRNFillScale, LRNComputeOutput, LRNComputeDiff), compiled
// in place from /root/reference with hipcc and launched exactly as the
// reference's op bodies launch them (cgt/nn_ops/cross_channel_lrn.py:27-39,
// 72-84, with the launch geometry of cgt_get_bt, include/cgt_cuda.h:46-63,
// restated below because cgt_cuda.h itself needs the CUDA toolkit headers).
// The reference has no CPU LRN; this is the only executable form of it.
// Nothing is copied: this file only includes lrn.cuh and names its kernels.
// The result (oracle/_ref/liblrn_ref.so) runs on the GPU box as a checker for
// oracle/cgt_oracle.c and for the product kernels; the product never loads it.
#include <hip/hip_runtime.h>
#include "lrn.cuh"

static void get_bt(size_t size, int& num_blocks, int& num_threads) {
    num_threads = size <= 32 ? 32 : size <= 64 ? 64 : size <= 128 ? 128 : size <= 256 ? 256 : size <= 512 ? 512 : 1024;
    num_blocks = (int)((size + num_threads - 1) / num_threads);
    if (num_blocks < 0 || 128 < num_blocks) num_blocks = 128;
}

template <typename T>
static int lrn_fwd(int num_img, int channels, int height, int width, int localsize, double alpha,
                   double beta, const T* X, T* top, T* scale) {
    int size = num_img * height * width, nblocks, nthreads;
    get_bt(size, nblocks, nthreads);
    LRNFillScale<T><<<nblocks, nthreads, 0>>>(size, X, num_img, channels, height, width, localsize,
                                              (T)(alpha / localsize), scale);
    size = num_img * channels * width * height;
    get_bt(size, nblocks, nthreads);
    LRNComputeOutput<T><<<nblocks, nthreads, 0>>>(size, X, scale, (T)(-beta), top);
    return (int)hipDeviceSynchronize();
}

template <typename T>
static int lrn_bwd(int num_img, int channels, int height, int width, int localsize, double alpha,
                   double beta, const T* X, const T* top, const T* scale, const T* top_diff,
                   T* bottom_diff) {
    int size = num_img * width * height, nblocks, nthreads;
    get_bt(size, nblocks, nthreads);
    LRNComputeDiff<T><<<nblocks, nthreads, 0>>>(size, X, top, scale, top_diff, num_img, channels,
                                                height, width, localsize, (T)(-beta),
                                                (T)(2. * alpha * beta / localsize), bottom_diff);
    return (int)hipDeviceSynchronize();
}

#define EXPORT extern "C" __attribute__((visibility("default")))
// all pointers are device pointers
EXPORT int ref_lrn_fwd_f32(int n, int c, int h, int w, int size, double alpha, double beta, const float* X, float* top, float* scale) { return lrn_fwd<float>(n, c, h, w, size, alpha, beta, X, top, scale); }
EXPORT int ref_lrn_fwd_f64(int n, int c, int h, int w, int size, double alpha, double beta, const double* X, double* top, double* scale) { return lrn_fwd<double>(n, c, h, w, size, alpha, beta, X, top, scale); }
EXPORT int ref_lrn_bwd_f32(int n, int c, int h, int w, int size, double alpha, double beta, const float* X, const float* top, const float* scale, const float* td, float* bd) { return lrn_bwd<float>(n, c, h, w, size, alpha, beta, X, top, scale, td, bd); }
EXPORT int ref_lrn_bwd_f64(int n, int c, int h, int w, int size, double alpha, double beta, const double* X, const double* top, const double* scale, const double* td, double* bd) { return lrn_bwd<double>(n, c, h, w, size, alpha, beta, X, top, scale, td, bd); }
