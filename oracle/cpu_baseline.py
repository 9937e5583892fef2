"""TEST INFRASTRUCTURE -- the CPU path timed beside the GPU figures.

The reference's CPU conv path is im2col (single thread) -> OpenBLAS
cblas_sgemm -> Transpose, with pooling.h for pooling; its OpenBLAS 0.2.14 is
fetched at build time and is not in the reference tree, so scipy's bundled
OpenBLAS stands in for it, called row-major with the reference's argument
mapping (cgt/core.py:2196-2205) and at most 16 threads (CMakeLists.txt:51).
The single-threaded stages are the reference's own loops where they exist as
C++ and were compiled here (oracle/_ref/libcgt_ref.so: im2col_cpu / col2im_cpu
with the geometry as template constants, max_pool / max_pool_pullback), else
the oracle's (oracle/cgt_oracle.c: transposes, LRN, geometries that were not
instantiated).  Only bench.py's cpu_baseline leg uses this module.
"""
import ctypes
import glob
import os
import time

import numpy as np

from . import oracle as O
from . import ref as R

_BLAS = None


def conv_impl(kernel, pad, stride):
    """(module with im2col / col2im, "reference" | "port") for a geometry."""
    if R.available() and tuple(kernel) + tuple(pad) + tuple(stride) in R.GEOMS:
        return R, "reference"
    return O, "port"


def pool_impl():
    return (R, "reference") if R.available() else (O, "port")


def blas():
    global _BLAS
    if _BLAS is None:
        import scipy
        pat = os.path.join(os.path.dirname(scipy.__file__), "..", "scipy.libs", "libscipy_openblas*.so")
        paths = sorted(glob.glob(pat))
        if not paths:
            raise RuntimeError("scipy's bundled OpenBLAS not found")
        _BLAS = ctypes.CDLL(paths[0])
        _BLAS.scipy_openblas_get_config.restype = ctypes.c_char_p
    return _BLAS


def blas_config():
    return blas().scipy_openblas_get_config().decode()


def set_threads(n):
    blas().scipy_openblas_set_num_threads(int(n))
    return int(blas().scipy_openblas_get_num_threads())


def host_cores():
    try:
        return len(os.sched_getaffinity(0))
    except AttributeError:
        return os.cpu_count() or 1


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def sgemm(A, B, tA=False, tB=False):
    """Mul22 on the CPU: cblas_sgemm(CblasRowMajor, tA+111, tB+111, M, N, K, 1, A, lda, B, ldb, 0, C, ldc)."""
    A = np.ascontiguousarray(A, np.float32)
    B = np.ascontiguousarray(B, np.float32)
    M = A.shape[1] if tA else A.shape[0]
    K = A.shape[0] if tA else A.shape[1]
    N = B.shape[0] if tB else B.shape[1]
    C = np.empty((M, N), np.float32)
    ci, cf, vp = ctypes.c_int, ctypes.c_float, ctypes.c_void_p
    blas().scipy_cblas_sgemm(ci(101), ci(111 + int(tA)), ci(111 + int(tB)), ci(M), ci(N), ci(K), cf(1.0),
                             vp(A.ctypes.data), ci(A.shape[1]), vp(B.ctypes.data), ci(B.shape[1]), cf(0.0),
                             vp(C.ctypes.data), ci(N))
    return C


def conv2d_fwd_bwd(x, f, gy, pad, stride):
    """conv2d forward + both gradients the way the reference's CPU graph runs them."""
    L, K, r, c = f.shape
    I, _ = conv_impl((r, c), pad, stride)
    col = I.im2col(x, (r, c), pad, stride)
    B, m, n, Z = col.shape
    f_LZ = f.reshape(L, Z)
    y = O.transpose4(sgemm(col.reshape(B * m * n, Z), f_LZ, False, True).reshape(B, m, n, L), (0, 3, 1, 2))
    gc = O.transpose4(gy, (0, 2, 3, 1)).reshape(B * m * n, L)
    gcol = sgemm(gc, f_LZ, False, False)
    gx = I.col2im(gcol.reshape(B, m, n, Z), x.shape, (r, c), pad, stride)
    gf = sgemm(gc, col.reshape(B * m * n, Z), True, False).reshape(f.shape)
    return y, gx, gf


def timed(fn, min_seconds=2.0, max_reps=50):
    """Best-of wall time of fn(), repeated until min_seconds have elapsed."""
    best, total, reps = float("inf"), 0.0, 0
    while reps < 1 or (total < min_seconds and reps < max_reps):
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
        best = min(best, dt)
        total += dt
        reps += 1
    return best, reps


def stage_times(x, f, gy, pad, stride, pool=None, lrn=None, min_seconds=0.5):
    """Best-of wall time of each CPU stage of the layer on the sample, in the
    order the reference's graph runs them: {stage: (seconds, bytes or flops)}."""
    L, K, r, c = f.shape
    out = {}
    I, _ = conv_impl((r, c), pad, stride)
    P, _ = pool_impl()
    col = I.im2col(x, (r, c), pad, stride)
    B, m, n, Z = col.shape
    col2, f_LZ = col.reshape(B * m * n, Z), f.reshape(L, Z)
    io = 4 * (x.size + col.size)
    flops = 2 * B * m * n * L * Z
    out["im2col"] = (timed(lambda: I.im2col(x, (r, c), pad, stride), min_seconds, 5)[0], io)
    out["gemm_fwd_NT"] = (timed(lambda: sgemm(col2, f_LZ, False, True), min_seconds, 5)[0], flops)
    y2 = sgemm(col2, f_LZ, False, True).reshape(B, m, n, L)
    out["transpose_0312"] = (timed(lambda: O.transpose4(y2, (0, 3, 1, 2)), min_seconds, 5)[0], 8 * y2.size)
    y = O.transpose4(y2, (0, 3, 1, 2))
    act = y
    if lrn:
        size, alpha, beta, k = lrn
        out["lrn_fwd"] = (timed(lambda: O.lrn_fwd(y, size, alpha, beta, k), min_seconds, 5)[0], 12 * y.size)
        act, scale = O.lrn_fwd(y, size, alpha, beta, k)
    g = gy
    if pool:
        pk, pp, ps = pool
        out["max_pool_fwd"] = (timed(lambda: P.max_pool(act, pk, pp, ps), min_seconds, 5)[0], None)
        pooled, mask = P.max_pool(act, pk, pp, ps)
        out["max_pool_fwd"] = (out["max_pool_fwd"][0], 4 * (act.size + 2 * pooled.size))
        gp = np.ones_like(pooled)
        out["max_pool_bwd"] = (timed(lambda: P.max_pool_pullback(act.shape, mask, gp), min_seconds, 5)[0],
                               4 * (2 * pooled.size + act.size))
        g = P.max_pool_pullback(act.shape, mask, gp)
    if lrn:
        out["lrn_bwd"] = (timed(lambda: O.lrn_bwd(y, act, scale, g, size, alpha, beta), min_seconds, 5)[0], 20 * y.size)
    out["transpose_0231"] = (timed(lambda: O.transpose4(g, (0, 2, 3, 1)), min_seconds, 5)[0], 8 * y.size)
    gc = O.transpose4(g, (0, 2, 3, 1)).reshape(B * m * n, L)
    out["gemm_dgrad_NN"] = (timed(lambda: sgemm(gc, f_LZ, False, False), min_seconds, 5)[0], flops)
    gcol = sgemm(gc, f_LZ, False, False).reshape(B, m, n, Z)
    out["col2im"] = (timed(lambda: I.col2im(gcol, x.shape, (r, c), pad, stride), min_seconds, 5)[0], io)
    out["gemm_wgrad_TN"] = (timed(lambda: sgemm(gc, col2, True, False), min_seconds, 5)[0], flops)
    return out
