/*
 * TEST INFRASTRUCTURE -- not part of the product path.
 *
 * Body of the CPU oracle, included twice by cgt_oracle.c with
 *   REAL   = float / double
 *   FN(x)  = x##_f32 / x##_f64
 * Every function restates, in plain C and single-threaded, what the reference
 * computes for the native CNN hot path.  Loop order and arithmetic order follow
 * the reference where the result depends on it (col2im, pool pullback, LRN
 * running sums), because those are compared bit-for-bit or to 1e-4.
 *
 * Only tests, the smoke check and the cpu_baseline leg of the benchmark may
 * link or call this file.
 */

/* Patch extraction, one image.  Follows /root/reference/include/im2col.h:6-28:
 * outer loop over the column channel z = (c_im*kh + ho)*kw + wo, inner loops
 * over output rows/cols; the column buffer is channels-last [m, n, Z] and
 * out-of-bounds taps store 0. */
static void FN(im2col_one)(const REAL *im, long C, long H, long W,
                           int kh, int kw, int ph, int pw, int sh, int sw,
                           REAL *col)
{
    long m = (H + 2 * ph - kh) / sh + 1;
    long n = (W + 2 * pw - kw) / sw + 1;
    long Z = C * kh * kw;
    for (long z = 0; z < Z; ++z) {
        long wo = z % kw;
        long ho = (z / kw) % kh;
        long c = z / kh / kw;
        for (long h = 0; h < m; ++h) {
            for (long w = 0; w < n; ++w) {
                long hp = h * sh - ph + ho;
                long wp = w * sw - pw + wo;
                REAL v = 0;
                if (hp >= 0 && hp < H && wp >= 0 && wp < W)
                    v = im[(c * H + hp) * W + wp];
                col[(h * n + w) * Z + z] = v;
            }
        }
    }
}

/* Batched im2col: the per-image loop of the Im2Col op body,
 * /root/reference/cgt/nn_ops/im2col.py:50-61; output shape rule :36-41. */
void FN(oracle_im2col)(const REAL *im, long B, long C, long H, long W,
                       int kh, int kw, int ph, int pw, int sh, int sw,
                       REAL *col)
{
    long m = (H + 2 * ph - kh) / sh + 1;
    long n = (W + 2 * pw - kw) / sw + 1;
    long Z = C * kh * kw;
    for (long b = 0; b < B; ++b)
        FN(im2col_one)(im + b * C * H * W, C, H, W, kh, kw, ph, pw, sh, sw,
                       col + b * m * n * Z);
}

/* Adjoint of im2col, one image.  Follows /root/reference/include/im2col.h:30-50:
 * zero-fill, then for z outer / h / w inner add col[h,w,z] into the image.  A
 * given pixel therefore receives its addends in ascending z order, which is
 * what fixes the fp rounding. */
static void FN(col2im_one)(const REAL *col, long C, long H, long W,
                           int kh, int kw, int ph, int pw, int sh, int sw,
                           REAL *im)
{
    long m = (H + 2 * ph - kh) / sh + 1;
    long n = (W + 2 * pw - kw) / sw + 1;
    long Z = C * kh * kw;
    for (long i = 0; i < C * H * W; ++i) im[i] = 0;
    for (long z = 0; z < Z; ++z) {
        long wo = z % kw;
        long ho = (z / kw) % kh;
        long c = z / kh / kw;
        for (long h = 0; h < m; ++h) {
            for (long w = 0; w < n; ++w) {
                long hp = h * sh - ph + ho;
                long wp = w * sw - pw + wo;
                if (hp >= 0 && hp < H && wp >= 0 && wp < W)
                    im[(c * H + hp) * W + wp] += col[(h * n + w) * Z + z];
            }
        }
    }
}

/* Batched col2im: Col2Im op body, /root/reference/cgt/nn_ops/im2col.py:80-92
 * (B, C, H, W arrive as four host-side int64 scalars there). */
void FN(oracle_col2im)(const REAL *col, long B, long C, long H, long W,
                       int kh, int kw, int ph, int pw, int sh, int sw,
                       REAL *im)
{
    long m = (H + 2 * ph - kh) / sh + 1;
    long n = (W + 2 * pw - kw) / sw + 1;
    long Z = C * kh * kw;
    for (long b = 0; b < B; ++b)
        FN(col2im_one)(col + b * m * n * Z, C, H, W, kh, kw, ph, pw, sh, sw,
                       im + b * C * H * W);
}

/* Max pooling with argmax.  Follows /root/reference/include/pooling.h:24-71:
 * top starts at -FLT_MAX (also in the double build: the reference writes
 * Dtype(-FLT_MAX)), mask at -1; the window end is clipped BEFORE the start is
 * clamped to 0; cells are scanned h then w and replace the running maximum
 * only on strict '>'; the mask is the index h*W+w inside the (n,c) plane.
 * The pooled size PH x PW is an input here; the op's shape rule
 * (/root/reference/cgt/nn_ops/max_pool_2d.py:35-43) is oracle_pool_outsize. */
void FN(oracle_max_pool)(const REAL *bottom, long N, long C, long H, long W,
                         int kh, int kw, int ph, int pw, int sh, int sw,
                         long PH, long PW, REAL *top, int *mask)
{
    long cnt = N * C * PH * PW;
    for (long i = 0; i < cnt; ++i) { top[i] = (REAL)(-FLT_MAX); mask[i] = -1; }
    for (long nc = 0; nc < N * C; ++nc) {
        const REAL *bp = bottom + nc * H * W;
        REAL *tp = top + nc * PH * PW;
        int *mp = mask + nc * PH * PW;
        for (long y = 0; y < PH; ++y) {
            for (long x = 0; x < PW; ++x) {
                long hs = y * sh - ph, ws = x * sw - pw;
                long he = hs + kh < H ? hs + kh : H;
                long we = ws + kw < W ? ws + kw : W;
                if (hs < 0) hs = 0;
                if (ws < 0) ws = 0;
                long pi = y * PW + x;
                for (long h = hs; h < he; ++h)
                    for (long w = ws; w < we; ++w) {
                        long idx = h * W + w;
                        if (bp[idx] > tp[pi]) { tp[pi] = bp[idx]; mp[pi] = (int)idx; }
                    }
            }
        }
    }
}

/* Pool pullback.  Follows /root/reference/include/pooling.h:73-106: zero-fill
 * the bottom gradient, then walk (n,c,ph,pw) ascending and add top_diff into
 * the cell the mask names.  Overlapping windows that share an argmax add in
 * that order.  The reference would write out of bounds for mask == -1 (a
 * window with no cell above -FLT_MAX); here such entries are skipped. */
void FN(oracle_max_pool_pullback)(const int *mask, const REAL *top_diff,
                                  long N, long C, long H, long W,
                                  long PH, long PW, REAL *bottom_diff)
{
    for (long i = 0; i < N * C * H * W; ++i) bottom_diff[i] = 0;
    for (long nc = 0; nc < N * C; ++nc) {
        REAL *bd = bottom_diff + nc * H * W;
        const REAL *td = top_diff + nc * PH * PW;
        const int *mp = mask + nc * PH * PW;
        for (long i = 0; i < PH * PW; ++i)
            if (mp[i] >= 0) bd[mp[i]] += td[i];
    }
}

/* Cross-channel LRN forward.  The reference has no CPU implementation; this
 * walks /root/reference/include/lrn.cuh:3-52 per pixel exactly as one GPU
 * thread does: a running sum of squares over the channel axis (add the head,
 * subtract the tail, both in REAL), scale = k + accum*(alpha/size) evaluated
 * in double and rounded to REAL (lrn.cuh:27 writes `1. + ...`, i.e. k = 1 and
 * a double literal), then top = x * pow(scale, -beta) (lrn.cuh:51, launched
 * with negative_beta = -beta cast to REAL, cross_channel_lrn.py:37).
 * pre_pad = (size-1)/2, post_pad = size-pre_pad-1 (lrn.cuh:15-16).
 * `k` is an extension (the reference fixes it at 1).  Requires C >= size. */
void FN(oracle_lrn_fwd)(const REAL *x, long N, long C, long H, long W,
                        int size, double alpha, double beta, double k,
                        REAL *top, REAL *scale)
{
    long step = H * W;
    REAL aos = (REAL)(alpha / size);          /* kernel parameter is Dtype */
    REAL nbeta = (REAL)(-beta);
    int pre = (size - 1) / 2, post = size - pre - 1;
    (void)pre;
    for (long n = 0; n < N; ++n)
        for (long p = 0; p < step; ++p) {
            const REAL *in = x + n * C * step + p;
            REAL *sc = scale + n * C * step + p;
            long head = 0;
            REAL acc = 0;
            while (head < post) { acc += in[head * step] * in[head * step]; ++head; }
            while (head < size) {
                acc += in[head * step] * in[head * step];
                sc[(head - post) * step] = (REAL)(k + acc * aos);
                ++head;
            }
            while (head < C) {
                acc += in[head * step] * in[head * step];
                acc -= in[(head - size) * step] * in[(head - size) * step];
                sc[(head - post) * step] = (REAL)(k + acc * aos);
                ++head;
            }
            while (head < C + post) {
                acc -= in[(head - size) * step] * in[(head - size) * step];
                sc[(head - post) * step] = (REAL)(k + acc * aos);
                ++head;
            }
        }
    for (long i = 0; i < N * C * step; ++i)
        top[i] = x[i] * FN_POW(scale[i], nbeta);
}

/* Cross-channel LRN backward.  Walks /root/reference/include/lrn.cuh:54-114:
 * running sum of top_diff*top/scale over the transposed window
 * pre_pad = size-(size+1)/2, post_pad = size-pre_pad-1 (lrn.cuh:75-76), and
 * bottom_diff = top_diff*pow(scale,-beta) - cache_ratio*x*accum with
 * cache_ratio = 2*alpha*beta/size (cross_channel_lrn.py:81). */
void FN(oracle_lrn_bwd)(const REAL *x, const REAL *top, const REAL *scale,
                        const REAL *top_diff, long N, long C, long H, long W,
                        int size, double alpha, double beta,
                        REAL *bottom_diff)
{
    long step = H * W;
    REAL nbeta = (REAL)(-beta);
    REAL ratio = (REAL)(2. * alpha * beta / size);
    int pre = size - (size + 1) / 2, post = size - pre - 1;
    (void)pre;
    for (long n = 0; n < N; ++n)
        for (long p = 0; p < step; ++p) {
            long off = n * C * step + p;
            const REAL *bx = x + off, *tp = top + off, *sc = scale + off, *td = top_diff + off;
            REAL *bd = bottom_diff + off;
            long head = 0;
            REAL acc = 0;
#define LRN_TERM(i) (td[(i) * step] * tp[(i) * step] / sc[(i) * step])
#define LRN_EMIT(i) bd[(i) * step] = td[(i) * step] * FN_POW(sc[(i) * step], nbeta) - ratio * bx[(i) * step] * acc
            while (head < post) { acc += LRN_TERM(head); ++head; }
            while (head < size) { acc += LRN_TERM(head); LRN_EMIT(head - post); ++head; }
            while (head < C) {
                acc += LRN_TERM(head);
                acc -= LRN_TERM(head - size);
                LRN_EMIT(head - post);
                ++head;
            }
            while (head < C + post) { acc -= LRN_TERM(head - size); LRN_EMIT(head - post); ++head; }
#undef LRN_TERM
#undef LRN_EMIT
        }
}

/* Row-major C[M,N] = op(A) . op(B), alpha = 1, beta = 0, with the argument
 * mapping of the Mul22 CPU body, /root/reference/cgt/core.py:2196-2205:
 * M = C.shape[0], N = C.shape[1], K = A.shape[tA ? 0 : 1], leading dimensions
 * are the stored row lengths.  The reference hands this to OpenBLAS 0.2.14
 * (not vendored); its own tests pin the result to the textbook product
 * (cgt/tests/test_affine.py:346-354), so the oracle is the textbook triple
 * loop with a double accumulator. */
void FN(oracle_gemm)(int tA, int tB, long M, long N, long K,
                     const REAL *A, long lda, const REAL *B, long ldb,
                     REAL *Cm, long ldc)
{
    for (long i = 0; i < M; ++i)
        for (long j = 0; j < N; ++j) {
            double s = 0;
            for (long k = 0; k < K; ++k) {
                double a = tA ? A[k * lda + i] : A[i * lda + k];
                double b = tB ? B[j * ldb + k] : B[k * ldb + j];
                s += a * b;
            }
            Cm[i * ldc + j] = (REAL)s;
        }
}

/* BatchedMul22 CPU body, /root/reference/cgt/core.py:2272-2285: P independent
 * products at data + i*stride(0) for each of A, B, C. */
void FN(oracle_gemm_batched)(int tA, int tB, long P, long M, long N, long K,
                             const REAL *A, long lda, long strideA,
                             const REAL *B, long ldb, long strideB,
                             REAL *Cm, long ldc, long strideC)
{
    for (long p = 0; p < P; ++p)
        FN(oracle_gemm)(tA, tB, M, N, K, A + p * strideA, lda, B + p * strideB, ldb,
                        Cm + p * strideC, ldc);
}

/* 4-d axis permutation, the Transpose op's CPU body
 * (/root/reference/cgt/core.py:1578-1594): out[i0,i1,i2,i3] = in[j...] with
 * out.shape[d] = in.shape[axes[d]]. */
void FN(oracle_transpose4)(const REAL *in, const long *inshape, const int *axes, REAL *out)
{
    long os[4], istr[4], st = 1;
    for (int d = 3; d >= 0; --d) { istr[d] = st; st *= inshape[d]; }
    for (int d = 0; d < 4; ++d) os[d] = inshape[axes[d]];
    long o = 0;
    for (long i0 = 0; i0 < os[0]; ++i0)
        for (long i1 = 0; i1 < os[1]; ++i1)
            for (long i2 = 0; i2 < os[2]; ++i2)
                for (long i3 = 0; i3 < os[3]; ++i3)
                    out[o++] = in[i0 * istr[axes[0]] + i1 * istr[axes[1]] +
                                  i2 * istr[axes[2]] + i3 * istr[axes[3]]];
}
