"""TEST INFRASTRUCTURE -- numpy front end of the CPU oracle (liboracle.so).

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the product path never does.

Each function mirrors one reference Op of the native CNN hot path and returns
fresh numpy arrays.  The arithmetic lives in ``cgt_oracle.c``; the shape rules
and the conv2d composition (reference ``cgt/nn.py:95-100`` and the backward
graph its autodiff derives) are restated here in numpy.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

_c_long = ctypes.c_long
_c_int = ctypes.c_int
_c_double = ctypes.c_double
_vp = ctypes.c_void_p


def build():
    """Compile liboracle.so (and oracle/_ref when the reference tree exists)."""
    subprocess.check_call(["make", "-C", _HERE, "all"], stdout=subprocess.DEVNULL)


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        _LIB = ctypes.CDLL(path)
        _LIB.oracle_pool_outsize.restype = _c_long
        _LIB.oracle_pool_outsize.argtypes = [_c_long, _c_int, _c_int, _c_int]
        _LIB.oracle_conv_outsize.restype = _c_long
        _LIB.oracle_conv_outsize.argtypes = [_c_long, _c_int, _c_int, _c_int]
    return _LIB


def _sfx(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "_f32"
    if dtype == np.float64:
        return "_f64"
    raise TypeError("oracle supports float32/float64, got %s" % dtype)


def _p(a):
    return _vp(a.ctypes.data)


def _c(a, dtype=None):
    return np.ascontiguousarray(a, dtype=dtype)


def _call(name, dtype, *args):
    fn = getattr(lib(), name + _sfx(dtype))
    fn.restype = None
    fn(*args)


def _geom(kernel, pad, stride):
    (kh, kw), (ph, pw), (sh, sw) = kernel, pad, stride
    return [_c_int(int(v)) for v in (kh, kw, ph, pw, sh, sw)]


def conv_outsize(H, k, pad, stride):
    """im2col extent, reference cgt/nn_ops/im2col.py:39-40."""
    return (H + 2 * pad - k) // stride + 1


def pool_outsize(H, k, pad, stride):
    """pooled extent ceil((H+2p-k)/s) with no +1, reference max_pool_2d.py:40-41."""
    return int(lib().oracle_pool_outsize(H, k, pad, stride))


def im2col(x, kernel, pad, stride):
    x = _c(x)
    B, C, H, W = x.shape
    m = conv_outsize(H, kernel[0], pad[0], stride[0])
    n = conv_outsize(W, kernel[1], pad[1], stride[1])
    col = np.empty((B, m, n, C * kernel[0] * kernel[1]), x.dtype)
    _call("oracle_im2col", x.dtype, _p(x), _c_long(B), _c_long(C), _c_long(H), _c_long(W),
          *_geom(kernel, pad, stride), _p(col))
    return col


def col2im(col, imshape, kernel, pad, stride):
    col = _c(col)
    B, C, H, W = imshape
    im = np.empty((B, C, H, W), col.dtype)
    _call("oracle_col2im", col.dtype, _p(col), _c_long(B), _c_long(C), _c_long(H), _c_long(W),
          *_geom(kernel, pad, stride), _p(im))
    return im


def max_pool(x, kernel, pad, stride):
    x = _c(x)
    N, C, H, W = x.shape
    PH = pool_outsize(H, kernel[0], pad[0], stride[0])
    PW = pool_outsize(W, kernel[1], pad[1], stride[1])
    top = np.empty((N, C, PH, PW), x.dtype)
    mask = np.empty((N, C, PH, PW), np.int32)
    _call("oracle_max_pool", x.dtype, _p(x), _c_long(N), _c_long(C), _c_long(H), _c_long(W),
          *_geom(kernel, pad, stride), _c_long(PH), _c_long(PW), _p(top), _p(mask))
    return top, mask


def max_pool_pullback(xshape, mask, gtop):
    mask = _c(mask, np.int32)
    gtop = _c(gtop)
    N, C, H, W = xshape
    PH, PW = mask.shape[2:]
    gb = np.empty((N, C, H, W), gtop.dtype)
    _call("oracle_max_pool_pullback", gtop.dtype, _p(mask), _p(gtop), _c_long(N), _c_long(C),
          _c_long(H), _c_long(W), _c_long(PH), _c_long(PW), _p(gb))
    return gb


def lrn_fwd(x, size, alpha, beta, k=1.0):
    x = _c(x)
    N, C, H, W = x.shape
    assert C >= size, "reference kernel reads head < size unguarded (lrn.cuh:25)"
    top = np.empty_like(x)
    scale = np.empty_like(x)
    _call("oracle_lrn_fwd", x.dtype, _p(x), _c_long(N), _c_long(C), _c_long(H), _c_long(W),
          _c_int(size), _c_double(alpha), _c_double(beta), _c_double(k), _p(top), _p(scale))
    return top, scale


def lrn_bwd(x, top, scale, gtop, size, alpha, beta):
    x, top, scale, gtop = (_c(a) for a in (x, top, scale, gtop))
    N, C, H, W = x.shape
    gb = np.empty_like(x)
    _call("oracle_lrn_bwd", x.dtype, _p(x), _p(top), _p(scale), _p(gtop), _c_long(N), _c_long(C),
          _c_long(H), _c_long(W), _c_int(size), _c_double(alpha), _c_double(beta), _p(gb))
    return gb


def mul22(A, B, tA=False, tB=False):
    """Mul22 with the reference's argument mapping (cgt/core.py:2196-2205)."""
    A, B = _c(A), _c(B)
    M = A.shape[1] if tA else A.shape[0]
    K = A.shape[0] if tA else A.shape[1]
    N = B.shape[0] if tB else B.shape[1]
    C = np.empty((M, N), A.dtype)
    _call("oracle_gemm", A.dtype, _c_int(tA), _c_int(tB), _c_long(M), _c_long(N), _c_long(K),
          _p(A), _c_long(A.shape[1]), _p(B), _c_long(B.shape[1]), _p(C), _c_long(N))
    return C


def batched_mul22(A, B, tA=False, tB=False):
    """BatchedMul22 (cgt/core.py:2272-2285)."""
    A, B = _c(A), _c(B)
    P = A.shape[0]
    M = A.shape[2] if tA else A.shape[1]
    K = A.shape[1] if tA else A.shape[2]
    N = B.shape[1] if tB else B.shape[2]
    C = np.empty((P, M, N), A.dtype)
    _call("oracle_gemm_batched", A.dtype, _c_int(tA), _c_int(tB), _c_long(P), _c_long(M),
          _c_long(N), _c_long(K), _p(A), _c_long(A.shape[2]), _c_long(A.shape[1] * A.shape[2]),
          _p(B), _c_long(B.shape[2]), _c_long(B.shape[1] * B.shape[2]),
          _p(C), _c_long(N), _c_long(M * N))
    return C


def transpose4(x, axes):
    x = _c(x)
    out = np.empty(tuple(x.shape[a] for a in axes), x.dtype)
    shp = (ctypes.c_long * 4)(*x.shape)
    ax = (ctypes.c_int * 4)(*axes)
    _call("oracle_transpose4", x.dtype, _p(x), shp, ax, _p(out))
    return out


def rectify(x):
    """x * (x >= 0), reference cgt/nn.py:44-45."""
    return x * (x >= 0).astype(x.dtype)


def conv2d(x, f, pad=(0, 0), stride=(1, 1)):
    """conv2d forward on the CPU path, reference cgt/nn.py:95-100:
    im2col -> [B*m*n, Z] -> Mul22(False, True) with f reshaped [L, Z] ->
    [B, m, n, L] -> Transpose{0,3,1,2}."""
    L, K, r, c = f.shape
    col = im2col(x, (r, c), pad, stride)
    B, m, n, Z = col.shape
    out = mul22(col.reshape(B * m * n, Z), _c(f).reshape(L, Z), False, True)
    return transpose4(out.reshape(B, m, n, L), (0, 3, 1, 2))


def conv2d_pullback(x, f, gy, pad=(0, 0), stride=(1, 1)):
    """Gradients of conv2d as the reference's autodiff derives them:
    Transpose{0,2,3,1} of gy (core.py:1569-1570), then for Mul22(F,T)
    (core.py:2160-2162) GA = Mul22(F,F)[GC, f_LZ] -> Col2Im, and
    GB = Mul22(T,F)[GC, col].  Returns (gx, gf)."""
    L, K, r, c = f.shape
    col = im2col(x, (r, c), pad, stride)
    B, m, n, Z = col.shape
    gc = transpose4(gy, (0, 2, 3, 1)).reshape(B * m * n, L)
    gcol = mul22(gc, _c(f).reshape(L, Z), False, False)
    gx = col2im(gcol.reshape(B, m, n, Z), x.shape, (r, c), pad, stride)
    gf = mul22(gc, col.reshape(B * m * n, Z), True, False).reshape(f.shape)
    return gx, gf


def conv_same_padded(x, kernel, total):
    """x [B,C,H,W] in the zero-padded plane layout that the library's products without a
    column buffer read (a layout of this library, no reference counterpart; a copy, so the
    bar is bit-exact): per plane pw zeros, then H + 2 ph rows of W + pw floats (W pixels, pw
    zeros -- the zeros that end a row are the left padding of the next), rounded up past 16
    zero floats to a multiple of 16; `total` floats in all, the rest zero."""
    B, C, H, W = x.shape
    ph, pw = (kernel[0] - 1) // 2, (kernel[1] - 1) // 2
    Hp, Wp = H + 2 * ph, W + pw
    plane = (pw + Hp * Wp + 16 + 15) // 16 * 16
    ref = np.zeros(total, x.dtype)
    img = np.zeros((B * C, Hp, Wp), x.dtype)
    img[:, ph:ph + H, :W] = x.reshape(B * C, H, W)
    ref[:B * C * plane].reshape(B * C, plane)[:, pw:pw + Hp * Wp] = img.reshape(B * C, -1)
    return ref


# ---------------------------------------------------------------- conv-layer glue

UNARY_OPS = ["abs", "cos", "exp", "log", "neg", "sign", "sin", "square", "sqrt", "tanh", "sigmoid"]
BINARY_OPS = ["*", "+", "-", "/", "<", ">", "<=", ">=", "**", "==", "!="]


def elwise_unary(opname, x):
    """ElwiseUnary on float32 (reference cgt/core.py:1160-1218)."""
    x = _c(x, np.float32)
    out = np.empty_like(x)
    rc = lib().oracle_elwise_unary_f32(_c_int(UNARY_OPS.index(opname)), _c_long(x.size), _p(x), _p(out))
    assert rc == 0
    return out


def elwise_binary_out_dtype(opname, xdtype, ydtype):
    """typ_apply of ElwiseBinary (reference cgt/core.py:1319-1333)."""
    if opname in ("<", ">", "<=", ">=", "==", "!="):
        return np.dtype(np.int8)
    if opname == "/":
        return np.dtype(np.float32)
    return np.dtype(np.float32) if np.float32 in (np.dtype(xdtype), np.dtype(ydtype)) else np.dtype(np.int8)


def elwise_binary(opname, x, y):
    """ElwiseBinary on float32 / int8 operands; a 0-d operand is the scalar side
    (scalar_mask, reference cgt/core.py:1243-1349)."""
    x, y = (a if a.ndim == 0 else np.ascontiguousarray(a) for a in (np.asarray(x), np.asarray(y)))
    assert x.dtype in (np.float32, np.int8) and y.dtype in (np.float32, np.int8)
    sx, sy = x.ndim == 0, y.ndim == 0
    shape = y.shape if sx else x.shape
    if not sx and not sy:
        assert x.shape == y.shape, "no implicit broadcasting"
    out = np.empty(shape, elwise_binary_out_dtype(opname, x.dtype, y.dtype))
    fn = getattr(lib(), "oracle_elwise_binary_%s%s" % ("f" if x.dtype == np.float32 else "b",
                                                        "f" if y.dtype == np.float32 else "b"))
    rc = fn(_c_int(BINARY_OPS.index(opname)), _c_long(out.size), _p(x), _c_int(sx), _p(y), _c_int(sy), _p(out))
    assert rc == 0
    return out


def repeat(x, axes, reps):
    """Repeat(axes) with repeat counts `reps` (reference cgt/core.py:1511-1557)."""
    x = np.ascontiguousarray(x)
    oshape = list(x.shape)
    flags = [0] * x.ndim
    for ax, rep in zip(axes, reps):
        assert x.shape[ax] == 1
        oshape[ax] = int(rep)
        flags[ax] = 1
    out = np.empty(oshape, x.dtype)
    rc = lib().oracle_repeat(_p(x), _c_int(x.dtype.itemsize), _c_int(x.ndim), (ctypes.c_long * max(x.ndim, 1))(*oshape),
                             (ctypes.c_int * max(x.ndim, 1))(*flags), _p(out))
    assert rc == 0
    return out


def sum_keepdims(x, axes):
    """Sum(axes), keepdims (reference cgt/core.py:1663-1709): sequential, in the array's dtype."""
    x = _c(x)
    flags = [1 if a in axes else 0 for a in range(x.ndim)]
    oshape = [1 if f else s for s, f in zip(x.shape, flags)]
    out = np.empty(oshape, x.dtype)
    fn = lib().oracle_sum_f32 if x.dtype == np.float32 else lib().oracle_sum_f64
    rc = fn(_p(x), _c_int(x.ndim), (ctypes.c_long * max(x.ndim, 1))(*x.shape), (ctypes.c_int * max(x.ndim, 1))(*flags), _p(out))
    assert rc == 0
    return out
