"""TEST INFRASTRUCTURE -- numpy front end of oracle/_ref/libcgt_ref.so, the
reference's own im2col.h / pooling.h compiled in place (see ref_shim.cpp).

``available()`` is False where the library has not been built (it can only be
built where the reference tree is present).  Same call shapes as oracle.py.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PATH = os.path.join(_HERE, "_ref", "libcgt_ref.so")
_LIB = None

# geometries instantiated in ref_shim.cpp: (kh, kw, ph, pw, sh, sw)
GEOMS = [
    (4, 4, 0, 0, 1, 1), (3, 3, 1, 1, 2, 2), (3, 3, 1, 1, 3, 3), (3, 3, 1, 1, 1, 1),
    (3, 3, 0, 0, 1, 1), (5, 5, 2, 2, 1, 1), (11, 11, 0, 0, 4, 4), (4, 7, 3, 6, 1, 1),
    (2, 3, 0, 1, 3, 2), (1, 1, 0, 0, 1, 1), (2, 2, 0, 0, 2, 2), (3, 2, 1, 0, 2, 1),
    (5, 3, 2, 1, 2, 3), (2, 2, 1, 1, 1, 1),
]


def available():
    return os.path.exists(_PATH)


def lib():
    global _LIB
    if _LIB is None:
        _LIB = ctypes.CDLL(_PATH)
    return _LIB


def _sfx(dtype):
    return {np.dtype(np.float32): "_f32", np.dtype(np.float64): "_f64"}[np.dtype(dtype)]


def _p(a):
    return ctypes.c_void_p(a.ctypes.data)


def _L(*v):
    return [ctypes.c_long(int(i)) for i in v]


def _I(*v):
    return [ctypes.c_int(int(i)) for i in v]


def im2col(x, kernel, pad, stride):
    x = np.ascontiguousarray(x)
    B, C, H, W = x.shape
    m = (H + 2 * pad[0] - kernel[0]) // stride[0] + 1
    n = (W + 2 * pad[1] - kernel[1]) // stride[1] + 1
    col = np.empty((B, m, n, C * kernel[0] * kernel[1]), x.dtype)
    fn = getattr(lib(), "ref_im2col" + _sfx(x.dtype))
    fn.restype = ctypes.c_int
    rc = fn(_p(x), *_L(B, C, H, W), *_I(*kernel, *pad, *stride), _p(col))
    if rc != 0:
        raise ValueError("geometry not instantiated in ref_shim.cpp")
    return col


def col2im(col, imshape, kernel, pad, stride):
    col = np.ascontiguousarray(col)
    B, C, H, W = imshape
    im = np.empty(imshape, col.dtype)
    fn = getattr(lib(), "ref_col2im" + _sfx(col.dtype))
    fn.restype = ctypes.c_int
    rc = fn(_p(col), *_L(B, C, H, W), *_I(*kernel, *pad, *stride), _p(im))
    if rc != 0:
        raise ValueError("geometry not instantiated in ref_shim.cpp")
    return im


def max_pool(x, kernel, pad, stride):
    x = np.ascontiguousarray(x)
    N, C, H, W = x.shape
    PH = max(0, -(-(H + 2 * pad[0] - kernel[0]) // stride[0]))
    PW = max(0, -(-(W + 2 * pad[1] - kernel[1]) // stride[1]))
    top = np.empty((N, C, PH, PW), x.dtype)
    mask = np.empty((N, C, PH, PW), np.int32)
    fn = getattr(lib(), "ref_max_pool" + _sfx(x.dtype))
    fn.restype = None
    fn(_p(x), *_L(N, C, H, W), *_I(*kernel, *pad, *stride), *_L(PH, PW), _p(top), _p(mask))
    return top, mask


def max_pool_pullback(xshape, mask, gtop):
    mask = np.ascontiguousarray(mask, np.int32)
    gtop = np.ascontiguousarray(gtop)
    N, C, H, W = xshape
    PH, PW = mask.shape[2:]
    gb = np.empty(xshape, gtop.dtype)
    fn = getattr(lib(), "ref_max_pool_pullback" + _sfx(gtop.dtype))
    fn.restype = None
    fn(_p(mask), _p(gtop), *_L(N, C, H, W, PH, PW), _p(gb))
    return gb
