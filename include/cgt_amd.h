/*
 * cgt_amd -- C ABI of the MI355X (gfx950) implementation of CGT's native CNN
 * hot path: im2col / col2im, the Mul22 / BatchedMul22 fp32 GEMM, max-pool
 * forward / pullback with argmax, cross-channel LRN forward / backward.
 *
 * These are the device-side launchers a CGT op body calls after it has
 * unpacked its cgtArray arguments, the role `launchker_$function(raw
 * pointers, ints...)` plays in the reference's two-translation-unit GPU ops
 * (cgt/nn_ops/cross_channel_lrn.py:24-55).  Plain pointers and sizes only.
 *
 * Conventions
 *   - every data pointer is DEVICE memory, fp32 contiguous row-major unless
 *     noted; argmax masks are int32; sizes are `long` as in cgtArray::shape().
 *   - `stream` is a hipStream_t passed as void*; NULL is the default stream.
 *     Launches are asynchronous; nothing here synchronises.
 *   - return value: CGT_AMD_OK or an error code; cgt_amd_last_error() gives
 *     the message for the calling thread.  (The reference's CUDA_CHECK only
 *     prints, include/cgt_cuda.h:11-21; a status is returned here instead.)
 *   - outputs are fully overwritten on every call: the interpreter reuses
 *     output buffers between calls without clearing them
 *     (src/execution.cpp:260-263).
 */
#ifndef CGT_AMD_H
#define CGT_AMD_H

#ifdef __cplusplus
extern "C" {
#endif

#define CGT_AMD_OK 0
#define CGT_AMD_ERR_ARG 1     /* bad shape / geometry / null pointer      */
#define CGT_AMD_ERR_HIP 2     /* a HIP runtime call failed                */
#define CGT_AMD_ERR_NOMEM 3   /* workspace allocation failed              */
#define CGT_AMD_ERR_NODEVICE 4

/* devtype values of cgt_amd_memcpy, numerically equal to the reference's
 * cgtDevtype { cgtCPU, cgtGPU } (include/cgt_common.h:68-71). */
#define CGT_AMD_CPU 0
#define CGT_AMD_GPU 1

/* ---------------------------------------------------------------- runtime */

/* Library version (major*100 + minor). */
int cgt_amd_version(void);

/* Message of the last error on the calling thread ("" if none). */
const char *cgt_amd_last_error(void);

/* Number of visible HIP devices (0 if none / no driver); never fails. */
int cgt_amd_device_count(void);

/* Device name of the current device, e.g. "gfx950..." into buf. */
int cgt_amd_device_name(char *buf, int buflen);

/* Device allocation for cgtGPU arrays.  Replaces the cudaMalloc / cudaFree
 * branches of cgt_alloc / cgt_free (src/cgt_common.cpp:110-136).
 * cgt_amd_alloc returns NULL on failure. */
void *cgt_amd_alloc(long nbytes);
int cgt_amd_free(void *ptr);

/* Free and total device memory of the current device in bytes (no counterpart in
 * the reference; lets a host size its batches and lets the tests watch the
 * library's workspaces). */
int cgt_amd_mem_info(long *free_bytes, long *total_bytes);

/* Synchronous copy between host and device memory.  Replaces the cudaMemcpy
 * branch of cgt_memcpy (src/cgt_common.cpp:138-153). */
int cgt_amd_memcpy(int dest_devtype, int src_devtype, void *dest, const void *src, long nbytes);

/* The same copy issued to `stream` without waiting for it: device-to-device
 * copies are ordered with the kernels of that stream (the interpreter's
 * Transport between two device buffers and the write-back of a parameter
 * update use it); a copy that touches pageable host memory may still block the
 * caller until the host side has been staged. */
int cgt_amd_memcpy_async(int dest_devtype, int src_devtype, void *dest, const void *src, long nbytes,
                         void *stream);

/* The device-to-device case of that copy as a kernel of this library (the D2D
 * branch of cgt_memcpy, src/cgt_common.cpp:146-150, without the runtime's copy
 * engine path): each workgroup streams its own contiguous region with several
 * 16-byte loads in flight per lane and non-temporal stores; any alignment and
 * size, the ranges must not overlap.  It is also the yardstick the measurement
 * script prices the bandwidth-bound kernels against.  cgt_amd_stream_copy_tune
 * sets the region per workgroup (a multiple of 4096 bytes) and the loads in
 * flight per lane (4, 8 or 16) for all later calls. */
int cgt_amd_stream_copy(void *dest, const void *src, long nbytes, void *stream);
int cgt_amd_stream_copy_tune(long bytes_per_workgroup, int loads_in_flight);

/* Asynchronous fill of `count` 32-bit words with `value` (a fill kernel, safe
 * to capture in a HIP graph). */
int cgt_amd_fill_u32(void *dst, unsigned int value, long count, void *stream);

/* Block the host until `stream` (NULL: the whole device) has drained. */
int cgt_amd_synchronize(void *stream);

/* Stream and event helpers so a host without its own HIP binding can time
 * launches on the stream they were issued to. */
int cgt_amd_stream_create(void **stream);
int cgt_amd_stream_destroy(void *stream);
int cgt_amd_event_create(void **event);
int cgt_amd_event_destroy(void *event);
int cgt_amd_event_record(void *event, void *stream);
/* Work issued to `stream` after this call starts only once the work recorded
 * in `event` is done: lets a host run independent branches of the backward
 * graph (weight gradient | data gradient + col2im) on two streams. */
int cgt_amd_stream_wait_event(void *stream, void *event);
int cgt_amd_event_elapsed_ms(void *start, void *stop, float *ms); /* waits for stop */

/* HIP graph of a fixed launch sequence: between capture_begin and capture_end
 * every launch issued to `stream` (a created stream, not NULL) by the calling
 * thread is recorded instead of run; graph_launch replays the recording.  For
 * launch-bound sequences (the MNIST / CIFAR sized layers: a dozen kernels of a
 * few microseconds).  Everything in this library can be captured except the
 * first call that grows a workspace (split-K GEMM, sum): run the sequence once
 * on the same stream before capturing it.  Device pointers are baked into the
 * graph. */
int cgt_amd_graph_capture_begin(void *stream);
int cgt_amd_graph_capture_end(void *stream, void **graph_exec);
int cgt_amd_graph_launch(void *graph_exec, void *stream);
int cgt_amd_graph_destroy(void *graph_exec);

/* ---------------------------------------------------------------- conv-layer glue
 *
 * The ops either side of the GEMM path in a SpatialConvolution training step:
 * bias add (broadcast "+"), ReLU = x * (x >= 0), their gradients, the scalar
 * loss and the bias gradient.  In the reference these are code-generated per
 * op from expression tables; here one entry point per op family takes the op
 * code. */

/* Element types, numbered like cgtDtype / numpy type numbers
 * (include/cgt_common.h:21-35): int8 "i1" and float32 "f4". */
#define CGT_AMD_I8 1
#define CGT_AMD_F32 11

/* Unary ops, y[i] = f(x[i]), fp32.  Replaces the generated kernel of
 * ElwiseUnary (cgt/core.py:1160-1241; expressions UNARY_INFO 1118-1134).
 * SIGN is 2*(x>0)-1 as in the reference's native template (sign(0) = -1). */
#define CGT_AMD_UN_ABS 0
#define CGT_AMD_UN_COS 1
#define CGT_AMD_UN_EXP 2
#define CGT_AMD_UN_LOG 3
#define CGT_AMD_UN_NEG 4
#define CGT_AMD_UN_SIGN 5
#define CGT_AMD_UN_SIN 6
#define CGT_AMD_UN_SQUARE 7
#define CGT_AMD_UN_SQRT 8
#define CGT_AMD_UN_TANH 9
#define CGT_AMD_UN_SIGMOID 10
int cgt_amd_elwise_unary_f32(int op, long n, const float *x, float *y, void *stream);

/* Binary ops, z[i] = f(x[i or 0], y[i or 0]).  Replaces the generated kernel
 * of ElwiseBinary (cgt/core.py:1243-1378; expressions BINARY_INFO 1139-1152).
 * Operand types are CGT_AMD_F32 or CGT_AMD_I8; a scalar operand is a
 * one-element device array (`*_is_scalar` != 0), as under the reference's
 * scalar_mask.  Output type, as typ_apply gives it: comparisons -> i1,
 * DIV -> f4, otherwise f4 if either operand is f4, else i1.  `n` is the
 * element count of the non-scalar operand(s) and of z. */
#define CGT_AMD_BIN_MUL 0
#define CGT_AMD_BIN_ADD 1
#define CGT_AMD_BIN_SUB 2
#define CGT_AMD_BIN_DIV 3
#define CGT_AMD_BIN_LT 4
#define CGT_AMD_BIN_GT 5
#define CGT_AMD_BIN_LE 6
#define CGT_AMD_BIN_GE 7
#define CGT_AMD_BIN_POW 8
#define CGT_AMD_BIN_EQ 9
#define CGT_AMD_BIN_NE 10
int cgt_amd_elwise_binary(int op, int xdtype, int ydtype, long n, const void *x, int x_is_scalar,
                          const void *y, int y_is_scalar, void *z, void *stream);

/* Repeat: `out` (shape outshape[ndim]) = x broadcast along the axes with
 * repeated[a] != 0, where x has extent 1.  Replaces the nested at<>() loops of
 * Repeat (cgt/core.py:1511-1557, cpu-only there).  itemsize 4 or 1, ndim <= 8. */
int cgt_amd_repeat(const void *x, int itemsize, int ndim, const long *outshape, const int *repeated,
                   void *out, void *stream);

/* Sum over the axes with reduced[a] != 0, keepdims: out has extent 1 there.
 * Replaces the reduction loop of Sum (cgt/core.py:1663-1709, cpu-only there).
 * The summation order differs from the reference's single running sum (lanes,
 * then a fixed tree, then partials in order) but is fixed: same input, same
 * bits.  ndim <= 8. */
int cgt_amd_sum_f32(const float *x, int ndim, const long *shape, const int *reduced, float *out,
                    void *stream);

/* Fill with an fp32 value (Fill op, cgt/core.py:966-1007, cpu-only there). */
int cgt_amd_fill_f32(float *dst, float value, long count, void *stream);

/* ---------------------------------------------------------------- im2col / col2im */

/* Patch extraction.  im [B,C,H,W] -> col [B,m,n,Z], Z = C*kh*kw ordered
 * (channel, kernel row, kernel col), m = (H+2*ph-kh)/sh + 1, n likewise;
 * taps outside the image are 0.  Bit-exact copy.
 * Replaces im2col_cpu (include/im2col.h:6-28) and the per-image loop of the
 * Im2Col op body (cgt/nn_ops/im2col.py:50-61). */
int cgt_amd_im2col_f32(const float *im, long B, long C, long H, long W,
                       int kh, int kw, int ph, int pw, int sh, int sw,
                       float *col, void *stream);

/* Adjoint of im2col.  col [B,m,n,Z] -> im [B,C,H,W]; every pixel is the sum of
 * its taps taken in ascending Z order starting from +0, which is the order
 * the reference's sequential loop produces, so results are bit-identical.
 * Replaces col2im_cpu (include/im2col.h:30-50) and the Col2Im op body
 * (cgt/nn_ops/im2col.py:80-92). */
int cgt_amd_col2im_f32(const float *col, long B, long C, long H, long W,
                       int kh, int kw, int ph, int pw, int sh, int sw,
                       float *im, void *stream);

/* ---------------------------------------------------------------- max pooling */

/* Pooled extent of the MaxPool op: ceil((H + 2*pad - k) / stride), no "+1"
 * (cgt/nn_ops/max_pool_2d.py:40-41).  Returns 0 when the window does not fit. */
long cgt_amd_pool_outsize(long H, int k, int pad, int stride);

/* Host-side query, no launch: planes per workgroup the LDS-staged pooling kernel
 * (backward != 0: the generic pullback kernel) would take for planes of H x W
 * pooled to PH x PW, or 0 when the launcher falls back to the direct kernel --
 * planes that do not fit LDS, or index ranges beyond what the staged kernels'
 * reciprocal-multiply index split handles exactly (2^21). */
int cgt_amd_pool_staged_planes(int backward, long H, long W, long PH, long PW);

/* Max pooling with argmax.  bottom [N,C,H,W] -> top, mask [N,C,PH,PW].
 * Window rows/cols outside the image are skipped; the first maximum in
 * (h, w) scan order wins (strict >, starting from -FLT_MAX); mask holds
 * h*W + w within the (n,c) plane, or -1 if no cell exceeded -FLT_MAX.
 * Replaces max_pool<float> (include/pooling.h:24-71). */
int cgt_amd_max_pool_f32(const float *bottom, long N, long C, long H, long W,
                         int kh, int kw, int ph, int pw, int sh, int sw,
                         long PH, long PW, float *top, int *mask, void *stream);

/* Pool pullback.  bottom_diff [N,C,H,W] = 0, then += top_diff at the cell each
 * mask entry names; cells named by several windows add in ascending (ph, pw)
 * order, bit-identical to the reference's sequential loop.  `mask` must be the
 * output of cgt_amd_max_pool_f32 for the same geometry (each entry lies inside
 * its own window); entries of -1 contribute nothing.
 * Replaces max_pool_pullback<float> (include/pooling.h:73-106). */
int cgt_amd_max_pool_pullback_f32(const int *mask, const float *top_diff,
                                  long N, long C, long H, long W,
                                  int kh, int kw, int ph, int pw, int sh, int sw,
                                  long PH, long PW, float *bottom_diff, void *stream);

/* ---------------------------------------------------------------- cross-channel LRN */

/* scale[n,c,h,w] = k + (alpha/size) * sum_{c' in [c-pre, c+post]} x^2 with
 * pre = (size-1)/2, post = size-pre-1, window clipped to [0,C);
 * top = x * scale^(-beta).  k = 1 is the reference (it has no k parameter).
 * Requires 1 <= size <= C, as the reference kernel does.
 * scale == NULL: the scale array is not stored (for callers that only keep top,
 * as cross_channel_lrn() does, cgt/nn_ops/cross_channel_lrn.py:106-108; the
 * gradient then comes from cgt_amd_lrn_bwd_from_x_f32).
 * Replaces LRNFillScale + LRNComputeOutput (include/lrn.cuh:3-52) and
 * launchker of CrossChannelLRNForward (cgt/nn_ops/cross_channel_lrn.py:27-39). */
int cgt_amd_lrn_fwd_f32(const float *x, long N, long C, long H, long W,
                        int size, double alpha, double beta, double k,
                        float *top, float *scale, void *stream);

/* bottom_diff = top_diff * scale^(-beta)
 *             - (2*alpha*beta/size) * x * sum_{c' in [c-pre', c+post']} top_diff*top/scale
 * with pre' = size-(size+1)/2, post' = size-pre'-1.
 * Replaces LRNComputeDiff (include/lrn.cuh:54-114) and launchker of
 * CrossChannelLRNBackward (cgt/nn_ops/cross_channel_lrn.py:72-84). */
int cgt_amd_lrn_bwd_f32(const float *x, const float *top, const float *scale,
                        const float *top_diff, long N, long C, long H, long W,
                        int size, double alpha, double beta,
                        float *bottom_diff, void *stream);

/* The same without the `top` operand: top = x * scale^(-beta) is formed again
 * from x and scale with the forward kernels' own operations, so for the
 * (top, scale) pair cgt_amd_lrn_fwd_f32 wrote the result has the bits of
 * cgt_amd_lrn_bwd_f32 while one array less is streamed from memory (four
 * instead of five).  What CrossChannelLRNBackward's closure calls: its `top`
 * input is always the forward op's output. */
int cgt_amd_lrn_bwd_recompute_f32(const float *x, const float *scale, const float *top_diff,
                                  long N, long C, long H, long W, int size, double alpha,
                                  double beta, float *bottom_diff, void *stream);

/* The same from x and top_diff alone: scale = k + (alpha/size) * window sum of
 * x^2 and top = x * scale^(-beta) are formed again inside the kernel, so three
 * arrays are streamed (x, top_diff, bottom_diff) instead of five.  Equal to
 * cgt_amd_lrn_bwd_f32 on the forward's outputs up to rounding (the window sum
 * may be taken in another order than the forward kernel took it).  `k` is the
 * forward's additive constant.  What the gradient of nn.cross_channel_lrn
 * calls when the scale array was not stored. */
int cgt_amd_lrn_bwd_from_x_f32(const float *x, const float *top_diff, long N, long C, long H,
                               long W, int size, double alpha, double beta, double k,
                               float *bottom_diff, void *stream);

/* ---------------------------------------------------------------- GEMM */

/* Row-major C[M,N] = op(A) . op(B), alpha = 1, beta = 0, true fp32 (MFMA
 * v_mfma_f32_32x32x2_f32, no reduced-precision inputs).  tA/tB select the
 * transposed operand; lda/ldb/ldc are the stored row lengths.
 * Replaces the cblas_sgemm / cublasSgemm_v2 call of the Mul22 op body
 * (cgt/core.py:2194-2224).  May use a split-K workspace owned by the library
 * (one per stream); the reduction order is fixed, so results are
 * deterministic.  Limits: M, N, K < 2^31 - 128; ldc < 2^27 unless M <= 4
 * (CGT_AMD_ERR_ARG otherwise); lda / ldb of 2^23 floats and more are accepted
 * and take a slower, fully bounds-tested load path.  Operands need 4-byte
 * alignment only. */
int cgt_amd_sgemm(int tA, int tB, long M, long N, long K,
                  const float *A, long lda, const float *B, long ldb,
                  float *C, long ldc, void *stream);

/* cgt_amd_sgemm for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has
 * no counterpart in the reference.  Same arguments, same kernels, same split
 * plan and therefore bit-identical results; the split-K partials and tail
 * pieces go to a 64 MiB device array that is part of the library's code object
 * (one copy per GPU, held until the process ends) instead of a workspace that
 * cgt_amd_sgemm grows with hipMalloc.  No hipMalloc / hipFree is ever called.
 * A product whose plan needs more than 64 MiB of partials (e.g. a weight
 * gradient with M*N*splits > 16 M floats) is refused with CGT_AMD_ERR_ARG and a
 * message naming both sizes.  All calls on one GPU share the array: calls that
 * overlap in time on different streams of the same GPU race on it -- issue them
 * on one stream, or order them with events. */
int cgt_amd_sgemm_noalloc(int tA, int tB, long M, long N, long K,
                          const float *A, long lda, const float *B, long ldb,
                          float *C, long ldc, void *stream);

/* P independent products at A + p*strideA, B + p*strideB, C + p*strideC.
 * Replaces the cblas_sgemm loop of BatchedMul22 (cgt/core.py:2272-2285);
 * the reference has no GPU implementation of it.  A stride of 0 shares one
 * operand between all products.  P < 65536; other limits as cgt_amd_sgemm. */
int cgt_amd_sgemm_batched(int tA, int tB, long P, long M, long N, long K,
                          const float *A, long lda, long strideA,
                          const float *B, long ldb, long strideB,
                          float *C, long ldc, long strideC, void *stream);

/* ---------------------------------------------------------------- convolution without a column buffer
 *
 * conv2d with stride 1 and pad = (kernel - 1) / 2 (odd kernels), forward and
 * both gradients, as GEMMs that read the image operand straight from a
 * zero-padded copy of the image: no im2col / col2im pass and no [B,m,n,Z]
 * column buffer.  They take the place, for the geometries they cover, of the
 * reference's fused GPU convolution ops CudnnConvForward / BackwardData /
 * BackwardFilter (cgt/nn_ops/cudnn_ops.py:58-143, include/cudnn_support.h:
 * 135-215), and compute what nn.conv2d's im2col -> Mul22 composition computes
 * (cgt/nn.py:95-100) to GEMM accuracy; the sums run over (tap, channel) instead
 * of (channel, tap), so results agree with that composition to rounding, not
 * bit for bit.
 *
 * Padded layout: `planes` planes of cgt_amd_conv_same_padded_size(1,...) -
 * tail floats each, pixel (h, w) at pw + (h + ph) * (W + pw) + w (the pw zeros
 * that end a row are the left padding of the next one), zeros elsewhere, plus
 * a zeroed tail; cgt_amd_conv_same_pad_f32 writes all of it. */

/* 1 if the three entry points below cover this layer: stride 1, odd kernel,
 * pad = (kernel - 1) / 2, C and L multiples of 16 (the products walk the
 * channels in blocks of 16; tiles are whole when L and C are multiples of 128,
 * 96 or 64 and padded otherwise).  Otherwise use im2col + cgt_amd_sgemm +
 * col2im. */
int cgt_amd_conv_same_supported(long C, long L, int kh, int kw, int ph, int pw, int sh, int sw);

/* 1 if, besides that, the extents of this batch of images are inside what the
 * three entry points index (padded plane below 2^21 floats, the channels of one
 * padded image below 2^30 floats, pixel tiles of the batch below 2^31): a host
 * that finds 0 here builds the layer from im2col and the column-buffer products
 * or cgt_amd_sgemm instead.  No counterpart in the reference (its cuDNN branch
 * takes any descriptor, cgt/nn_ops/cudnn_ops.py:58-143). */
int cgt_amd_conv_same_fits(long B, long C, long H, long W, long L, int kh, int kw);

/* Floats in the padded copy of `planes` planes of H x W (tail included); -1 on bad arguments. */
long cgt_amd_conv_same_padded_size(long planes, long H, long W, int kh, int kw);

/* x [planes][H][W] -> xpad (padded layout above; 16-byte aligned). */
int cgt_amd_conv_same_pad_f32(const float *x, long planes, long H, long W, int kh, int kw,
                              float *xpad, void *stream);

/* gypad = pad(relu_mask * max_pool_pullback(mask, top_diff)) in one pass: the
 * padded cotangent of a convolution whose result went through a max pool
 * (cgt_amd_max_pool_pullback_f32, bit for bit, written in the padded layout
 * instead of [planes][H][W]), optionally multiplied by the int8 mask of a
 * rectify in between ((float)mask * value, as the Op graph's mask * gy;
 * relu_mask may be NULL).  Pool geometry and PH, PW as for
 * cgt_amd_max_pool_pullback_f32; kh, kw are the convolution's kernel. */
int cgt_amd_conv_same_pad_pool_pullback_f32(const int *mask, const float *top_diff,
                                            const signed char *relu_mask, long planes, long H, long W,
                                            int pool_kh, int pool_kw, int pool_ph, int pool_pw,
                                            int pool_sh, int pool_sw, long PH, long PW,
                                            int kh, int kw, float *gypad, void *stream);

/* y [B,L,H,W] = conv(x, f), f [L,C,kh,kw], from the padded x.  `bias` (L floats,
 * may be NULL) is added per channel and, if relu != 0, the result is replaced by
 * v * (v >= 0) -- the bias add and rectify of SpatialConvolution + nn.rectify
 * (cgt/nn.py:44-45, 231-233) applied while the result is written, with the same
 * fp32 operations as the separate ops.  `mask` (int8 [B,L,H,W], may be NULL)
 * receives (v >= 0) of the value before the rectify: the factor of the
 * rectify's gradient.  Uses workspaces owned by the library. */
int cgt_amd_conv_same_fwd_f32(const float *xpad, const float *f, const float *bias, int relu,
                              long B, long C, long H, long W, long L, int kh, int kw,
                              float *y, signed char *mask, void *stream);

/* The pieces the three products are made of, one kernel each (plus the GEMM's
 * own reduce kernel), for a host that keeps the intermediate buffers itself:
 *   filter   f [L,C,kh,kw] -> fk in the K order of the product (block of 16
 *            channels, tap, channel in the block): [L][C/16][tap][16] (flipped = 0:
 *            forward) or [C][L/16][flipped tap][16] (flipped = 1: the data
 *            gradient's filter bank)
 *   product  out [B,N,H,W] = sum_{c,tap} fk[n][c/16][tap][c%16] * imgpad[b][c][q + tapoff]
 *            (+ bias[n], rectify), written in NCHW by the GEMM itself
 *   wgrad    gfk [L][tap][C] from the two padded arrays; transpose4 {0,3,1,2}
 *            of it viewed [L,kh,kw,C] is gf [L,C,kh,kw] */
int cgt_amd_conv_same_filter_f32(const float *f, long L, long C, int kh, int kw, int flipped,
                                 float *fk, void *stream);
int cgt_amd_conv_same_product_f32(const float *imgpad, const float *fk, const float *bias, int relu,
                                  long B, long Cin, long H, long W, long N, int kh, int kw,
                                  float *out, signed char *mask, void *stream);
int cgt_amd_conv_same_wgrad_f32(const float *gypad, const float *xpad, long B, long C, long H, long W,
                                long L, int kh, int kw, float *gfk, void *stream);

/* gx [B,C,H,W] from the padded cotangent gypad (L planes per image). */
int cgt_amd_conv_same_bwd_data_f32(const float *gypad, const float *f, long B, long C, long H, long W,
                                   long L, int kh, int kw, float *gx, void *stream);

/* gf [L,C,kh,kw] from the padded cotangent and the padded input (the wgrad product above, its
 * split-K reduce kernel storing the filters' layout: no separate transpose). */
int cgt_amd_conv_same_bwd_filter_f32(const float *gypad, const float *xpad, long B, long C, long H,
                                     long W, long L, int kh, int kw, float *gf, void *stream);

/* ---------------------------------------------------------------- convolution over the column buffer
 *
 * conv2d of any geometry as the reference composes it on the CPU -- im2col,
 * one GEMM, reshape, Transpose{0,3,1,2} (cgt/nn.py:95-100), and for the
 * gradients Transpose{0,2,3,1} followed by the NN / TN GEMMs that autodiff
 * derives (cgt/core.py:2143-2175) -- with the [B*m*n, L] intermediates and
 * both transposes folded into the GEMMs: each product reads or writes the
 * NCHW array in place.  Same sums in the same order of z as the composition
 * (results agree with it to GEMM accuracy; the split of the weight gradient's
 * K axis differs).  In all three: col [B*P][Z] is cgt_amd_im2col_f32's
 * result (P = m*n output pixels per image, Z = C*kh*kw), f [L][Z] is the
 * filter bank [L,C,kh,kw] as it is stored, y / gy are [B,L,m,n]. */

/* 1 if the extents are inside what these products index (B*P pixels below
 * 2^31, a filter bank of fewer than 2^29 floats, and -- for the forward
 * product's NCHW epilogue -- about L*P below 2^29); otherwise build the layer
 * from cgt_amd_sgemm and cgt_amd_transpose4_f32.  The weight gradient takes any
 * batch size: beyond 256 MiB of per-image partial sums it runs in groups of
 * images whose results are added in order. */
int cgt_amd_conv_col_fits(long B, long P, long Z, long L);

/* y = conv(x, f) from col.  bias / relu / mask as in cgt_amd_conv_same_fwd_f32. */
int cgt_amd_conv_col_fwd_f32(const float *col, const float *f, const float *bias, int relu,
                             long B, long P, long Z, long L, float *y, signed char *mask,
                             void *stream);

/* gcol [B*P][Z] (the argument of cgt_amd_col2im_f32) from the cotangent gy. */
int cgt_amd_conv_col_bwd_data_f32(const float *gy, const float *f, long B, long P, long Z, long L,
                                  float *gcol, void *stream);

/* gf [L,C,kh,kw] from the cotangent gy and col.  Uses a workspace owned by
 * the library (one partial sum per image, or per piece of an image). */
int cgt_amd_conv_col_bwd_filter_f32(const float *gy, const float *col, long B, long P, long Z, long L,
                                    float *gf, void *stream);

/* The forward product and the weight gradient of the same composition without
 * the column buffer: the element col[b*P + p][z] is read from x where
 * cgt_amd_im2col_f32 would have copied it from (zero outside the image) while
 * the GEMM loads its operand tile.  Any kernel, padding and stride; results
 * agree with the products over col to rounding (same sums, same order of z;
 * the forward product bit for bit, the weight gradient bit for bit when both
 * take the same tile shape and therefore cut K into the same pieces).  x [B,C,H,W], f / gf [L,C,kh,kw], y / gy
 * [B,L,m,n] with m = (H + 2 ph - kh) / sh + 1.  The data gradient keeps the
 * column buffer (cgt_amd_conv_col_bwd_data_f32 + cgt_amd_col2im_f32). */

/* 1 if the two entry points below take this layer (m*n < 2^21, extents and
 * kernel < 32768, B*C*H*W < 2^29: byte offsets into x are 32-bit). */
int cgt_amd_conv_patch_supported(long B, long C, long H, long W, int kh, int kw, int ph, int pw,
                                 int sh, int sw);
int cgt_amd_conv_patch_fwd_f32(const float *x, const float *f, const float *bias, int relu,
                               long B, long C, long H, long W, long L, int kh, int kw, int ph,
                               int pw, int sh, int sw, float *y, signed char *mask, void *stream);
int cgt_amd_conv_patch_bwd_filter_f32(const float *gy, const float *x, long B, long C, long H,
                                      long W, long L, int kh, int kw, int ph, int pw, int sh,
                                      int sw, float *gf, void *stream);

/* ---------------------------------------------------------------- conv glue */

/* out[i0,i1,i2,i3] = in[...] with out.shape[d] = in.shape[axes[d]].
 * Replaces the Transpose op's CPU loop (cgt/core.py:1578-1594), which conv2d
 * applies as {0,3,1,2} after the GEMM and its pullback as {0,2,3,1}. */
int cgt_amd_transpose4_f32(const float *in, const long *inshape, const int *axes,
                           float *out, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* CGT_AMD_H */
