"""TEST INFRASTRUCTURE -- the CPU path timed beside the GPU figures.

The reference's CPU conv path is im2col (single thread) -> OpenBLAS
cblas_sgemm -> Transpose, with pooling.h for pooling; its OpenBLAS 0.2.14 is
fetched at build time and is not in the reference tree, so scipy's bundled
OpenBLAS stands in for it, called row-major with the reference's argument
mapping (cgt/core.py:2196-2205) and at most 16 threads (CMakeLists.txt:51).
The single-threaded stages are the oracle's (oracle/cgt_oracle.c).  Only
bench.py's cpu_baseline leg uses this module.
"""
import ctypes
import glob
import os
import time

import numpy as np

from . import oracle as O

_BLAS = None


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
    col = O.im2col(x, (r, c), pad, stride)
    B, m, n, Z = col.shape
    f_LZ = f.reshape(L, Z)
    y = O.transpose4(sgemm(col.reshape(B * m * n, Z), f_LZ, False, True).reshape(B, m, n, L), (0, 3, 1, 2))
    gc = O.transpose4(gy, (0, 2, 3, 1)).reshape(B * m * n, L)
    gcol = sgemm(gc, f_LZ, False, False)
    gx = O.col2im(gcol.reshape(B, m, n, Z), x.shape, (r, c), pad, stride)
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
