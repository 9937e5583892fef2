"""TEST INFRASTRUCTURE -- front end of oracle/_ref/liblrn_ref.so: the
reference's own LRN device kernels (include/lrn.cuh) compiled in place with
hipcc (see ref_lrn_shim.hip).  Needs a GPU; takes and returns numpy arrays.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PATH = os.path.join(_HERE, "_ref", "liblrn_ref.so")
_LIB = None


def available():
    return os.path.exists(_PATH)


def lib():
    global _LIB
    if _LIB is None:
        _LIB = ctypes.CDLL(_PATH)
    return _LIB


def _sfx(dtype):
    return {np.dtype(np.float32): "_f32", np.dtype(np.float64): "_f64"}[np.dtype(dtype)]


def _args(shape, size, alpha, beta):
    n, c, h, w = shape
    return [ctypes.c_int(n), ctypes.c_int(c), ctypes.c_int(h), ctypes.c_int(w), ctypes.c_int(size),
            ctypes.c_double(alpha), ctypes.c_double(beta)]


def lrn_fwd(x, size, alpha, beta):
    from cgt_amd.gpuarray import empty, to_gpu
    x = np.ascontiguousarray(x)
    dx = to_gpu(x)
    top, scale = empty(x.shape, x.dtype), empty(x.shape, x.dtype)
    fn = getattr(lib(), "ref_lrn_fwd" + _sfx(x.dtype))
    rc = fn(*_args(x.shape, size, alpha, beta), ctypes.c_void_p(dx.ptr), ctypes.c_void_p(top.ptr), ctypes.c_void_p(scale.ptr))
    assert rc == 0, "reference LRN forward kernel failed (hip error %d)" % rc
    return top.get(), scale.get()


def lrn_bwd(x, top, scale, gtop, size, alpha, beta):
    from cgt_amd.gpuarray import empty, to_gpu
    x = np.ascontiguousarray(x)
    d = [to_gpu(np.ascontiguousarray(a, dtype=x.dtype)) for a in (x, top, scale, gtop)]
    gb = empty(x.shape, x.dtype)
    fn = getattr(lib(), "ref_lrn_bwd" + _sfx(x.dtype))
    rc = fn(*_args(x.shape, size, alpha, beta), *[ctypes.c_void_p(a.ptr) for a in d], ctypes.c_void_p(gb.ptr))
    assert rc == 0, "reference LRN backward kernel failed (hip error %d)" % rc
    return gb.get()
