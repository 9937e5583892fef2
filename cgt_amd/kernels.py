"""Direct calls of the C ABI on device arrays -- one function per hot-path op.

These apply the same shape rules as the reference Ops (cited per function) and
hand raw pointers to libcgt_amd.so.  Outputs may be passed in (`out=`) to be
reused across calls, as the reference interpreter reuses them
(src/execution.cpp:260-263); every kernel overwrites its output fully.
"""
import ctypes

import numpy as np

from . import capi
from .gpuarray import GpuArray, empty


def _geom(kernel, pad, stride):
    (kh, kw), (ph, pw), (sh, sw) = kernel, pad, stride
    return [int(v) for v in (kh, kw, ph, pw, sh, sw)]


def _out(out, shape, dtype=np.float32):
    if out is None:
        return empty(shape, dtype)
    if out.shape != tuple(shape) or out.dtype != np.dtype(dtype):
        raise ValueError("out has shape %s dtype %s, expected %s %s" % (out.shape, out.dtype, tuple(shape), dtype))
    return out


def _f32(*arrays):
    for a in arrays:
        if a.dtype != np.float32:
            raise TypeError("expected float32 device array, got %s" % a.dtype)


def conv_outsize(H, k, pad, stride):
    """(H + 2*pad - k) // stride + 1 (reference cgt/nn_ops/im2col.py:39-40)."""
    return (H + 2 * pad - k) // stride + 1


def pool_outsize(H, k, pad, stride):
    """ceil((H + 2*pad - k) / stride), no +1 (reference cgt/nn_ops/max_pool_2d.py:40-41)."""
    return int(capi.lib().cgt_amd_pool_outsize(H, k, pad, stride))


def im2col(x, kernel, pad, stride, out=None, stream=None):
    """Im2Col op (reference cgt/nn_ops/im2col.py:25-62): [B,C,H,W] -> [B,m,n,C*kh*kw]."""
    _f32(x)
    B, C, H, W = x.shape
    g = _geom(kernel, pad, stride)
    m, n = conv_outsize(H, g[0], g[2], g[4]), conv_outsize(W, g[1], g[3], g[5])
    col = _out(out, (B, m, n, C * g[0] * g[1]))
    capi.check(capi.lib().cgt_amd_im2col_f32(x.ptr, B, C, H, W, *g, col.ptr, stream))
    return col


def col2im(col, imshape, kernel, pad, stride, out=None, stream=None):
    """Col2Im op (reference cgt/nn_ops/im2col.py:64-93): adjoint of im2col."""
    _f32(col)
    B, C, H, W = (int(s) for s in imshape)
    g = _geom(kernel, pad, stride)
    m, n = conv_outsize(H, g[0], g[2], g[4]), conv_outsize(W, g[1], g[3], g[5])
    if col.shape != (B, m, n, C * g[0] * g[1]):
        raise ValueError("col has shape %s, expected %s" % (col.shape, (B, m, n, C * g[0] * g[1])))
    im = _out(out, (B, C, H, W))
    capi.check(capi.lib().cgt_amd_col2im_f32(col.ptr, B, C, H, W, *g, im.ptr, stream))
    return im


def max_pool(x, kernel, pad, stride, out=None, stream=None):
    """MaxPool op (reference cgt/nn_ops/max_pool_2d.py:22-53): returns (pool, int32 mask)."""
    _f32(x)
    N, C, H, W = x.shape
    g = _geom(kernel, pad, stride)
    PH, PW = pool_outsize(H, g[0], g[2], g[4]), pool_outsize(W, g[1], g[3], g[5])
    top = _out(out[0] if out else None, (N, C, PH, PW))
    mask = _out(out[1] if out else None, (N, C, PH, PW), np.int32)
    capi.check(capi.lib().cgt_amd_max_pool_f32(x.ptr, N, C, H, W, *g, PH, PW, top.ptr, mask.ptr, stream))
    return top, mask


def max_pool_pullback(xshape, mask, gtop, kernel, pad, stride, out=None, stream=None):
    """MaxPoolPullback op (reference cgt/nn_ops/max_pool_2d.py:55-72)."""
    _f32(gtop)
    if mask.dtype != np.int32:
        raise TypeError("mask must be int32")
    N, C, H, W = (int(s) for s in xshape)
    g = _geom(kernel, pad, stride)
    PH, PW = mask.shape[2:]
    if mask.shape != gtop.shape or mask.shape[:2] != (N, C):
        raise ValueError("mask %s / gtop %s do not match x %s" % (mask.shape, gtop.shape, xshape))
    gb = _out(out, (N, C, H, W))
    capi.check(capi.lib().cgt_amd_max_pool_pullback_f32(mask.ptr, gtop.ptr, N, C, H, W, *g, PH, PW,
                                                        gb.ptr, stream))
    return gb


def lrn_fwd(x, size, alpha, beta, k=1.0, out=None, stream=None, want_scale=True):
    """CrossChannelLRNForward op (reference cgt/nn_ops/cross_channel_lrn.py:15-63):
    returns (top, scale).  k=1 is the reference; other k is an extension.
    want_scale=False: the scale array is not stored and only top is returned."""
    _f32(x)
    N, C, H, W = x.shape
    if not want_scale:
        top = _out(out, x.shape)
        capi.check(capi.lib().cgt_amd_lrn_fwd_f32(x.ptr, N, C, H, W, int(size), float(alpha), float(beta),
                                                  float(k), top.ptr, None, stream))
        return top
    top = _out(out[0] if out else None, x.shape)
    scale = _out(out[1] if out else None, x.shape)
    capi.check(capi.lib().cgt_amd_lrn_fwd_f32(x.ptr, N, C, H, W, int(size), float(alpha), float(beta),
                                              float(k), top.ptr, scale.ptr, stream))
    return top, scale


def lrn_bwd_from_x(x, gtop, size, alpha, beta, k=1.0, out=None, stream=None):
    """The LRN gradient from x and the cotangent alone (scale and top are formed again in the kernel)."""
    _f32(x, gtop)
    N, C, H, W = x.shape
    if gtop.shape != x.shape:
        raise ValueError("LRN backward operands must be float32 arrays of x's shape")
    gb = _out(out, x.shape)
    capi.check(capi.lib().cgt_amd_lrn_bwd_from_x_f32(x.ptr, gtop.ptr, N, C, H, W, int(size), float(alpha), float(beta),
                                                     float(k), gb.ptr, stream))
    return gb


def lrn_bwd(x, top, scale, gtop, size, alpha, beta, out=None, stream=None):
    """CrossChannelLRNBackward op (reference cgt/nn_ops/cross_channel_lrn.py:65-104).
    top=None: top = x * scale^-beta is formed again inside the kernel (the bits lrn_fwd wrote)."""
    _f32(x, scale, gtop)
    N, C, H, W = x.shape
    for a in (scale, gtop) + (() if top is None else (top,)):
        if a.shape != x.shape or a.dtype != np.float32:
            raise ValueError("LRN backward operands must be float32 arrays of x's shape")
    gb = _out(out, x.shape)
    if top is None:
        capi.check(capi.lib().cgt_amd_lrn_bwd_recompute_f32(x.ptr, scale.ptr, gtop.ptr, N, C, H, W, int(size),
                                                            float(alpha), float(beta), gb.ptr, stream))
    else:
        capi.check(capi.lib().cgt_amd_lrn_bwd_f32(x.ptr, top.ptr, scale.ptr, gtop.ptr, N, C, H, W, int(size),
                                                  float(alpha), float(beta), gb.ptr, stream))
    return gb


def mul22(A, B, tA=False, tB=False, out=None, stream=None):
    """Mul22 op (reference cgt/core.py:2129-2229): C = op(A) . op(B); M, N, K and
    leading dimensions as in its op body (2196-2205)."""
    _f32(A, B)
    if A.ndim != 2 or B.ndim != 2:
        raise ValueError("Mul22 takes matrices")
    M = A.shape[1] if tA else A.shape[0]
    K = A.shape[0] if tA else A.shape[1]
    N = B.shape[0] if tB else B.shape[1]
    Kb = B.shape[1] if tB else B.shape[0]
    if K != Kb:
        raise ValueError("shape mismatch at matrix-matrix multiplication: %s %s" % (A.shape, B.shape))
    C = _out(out, (M, N))
    capi.check(capi.lib().cgt_amd_sgemm(int(tA), int(tB), M, N, K, A.ptr, A.shape[1], B.ptr, B.shape[1],
                                        C.ptr, N, stream))
    return C


def batched_mul22(A, B, tA=False, tB=False, out=None, stream=None):
    """BatchedMul22 op (reference cgt/core.py:2231-2288)."""
    _f32(A, B)
    if A.ndim != 3 or B.ndim != 3 or A.shape[0] != B.shape[0]:
        raise ValueError("BatchedMul22 takes [P,.,.] arrays with equal P")
    P = A.shape[0]
    M = A.shape[2] if tA else A.shape[1]
    K = A.shape[1] if tA else A.shape[2]
    N = B.shape[1] if tB else B.shape[2]
    Kb = B.shape[2] if tB else B.shape[1]
    if K != Kb:
        raise ValueError("shape mismatch at batched matrix multiplication: %s %s" % (A.shape, B.shape))
    C = _out(out, (P, M, N))
    capi.check(capi.lib().cgt_amd_sgemm_batched(int(tA), int(tB), P, M, N, K,
                                                A.ptr, A.shape[2], A.shape[1] * A.shape[2],
                                                B.ptr, B.shape[2], B.shape[1] * B.shape[2],
                                                C.ptr, N, M * N, stream))
    return C


def transpose4(x, axes, out=None, stream=None):
    """Transpose op for 4-d arrays (reference cgt/core.py:1559-1594)."""
    _f32(x)
    axes = tuple(int(a) for a in axes)
    res = _out(out, tuple(x.shape[a] for a in axes))
    shp = (ctypes.c_long * 4)(*x.shape)
    ax = (ctypes.c_int * 4)(*axes)
    capi.check(capi.lib().cgt_amd_transpose4_f32(x.ptr, shp, ax, res.ptr, stream))
    return res


# ---------------------------------------------------------------- conv-layer glue

UNARY_OPS = ["abs", "cos", "exp", "log", "neg", "sign", "sin", "square", "sqrt", "tanh", "sigmoid"]
BINARY_OPS = ["*", "+", "-", "/", "<", ">", "<=", ">=", "**", "==", "!="]
_DTYPE_CODE = {np.dtype(np.float32): 11, np.dtype(np.int8): 1}    # cgtDtype / numpy type numbers


def binary_out_dtype(opname, xdtype, ydtype):
    """typ_apply of ElwiseBinary (reference cgt/core.py:1319-1333): comparisons
    give i1, "/" gives floatX, everything else the promoted operand type."""
    if opname in ("<", ">", "<=", ">=", "==", "!="):
        return np.dtype(np.int8)
    if opname == "/":
        return np.dtype(np.float32)
    return np.dtype(np.float32) if np.dtype(np.float32) in (np.dtype(xdtype), np.dtype(ydtype)) else np.dtype(np.int8)


def elwise_unary(opname, x, out=None, stream=None):
    """ElwiseUnary (reference cgt/core.py:1160-1241), float32."""
    _f32(x)
    y = _out(out, x.shape)
    capi.check(capi.lib().cgt_amd_elwise_unary_f32(UNARY_OPS.index(opname), x.size, x.ptr, y.ptr, stream))
    return y


def elwise_binary(opname, x, y, out=None, stream=None):
    """ElwiseBinary (reference cgt/core.py:1243-1378).  A 0-d operand is the
    scalar side; otherwise shapes must agree (no implicit broadcasting)."""
    sx, sy = x.ndim == 0, y.ndim == 0
    if not sx and not sy and x.shape != y.shape:
        raise ValueError("mismatched shapes %s %s: implicit broadcasting is not allowed, use broadcast(...)"
                         % (x.shape, y.shape))
    if x.dtype not in _DTYPE_CODE or y.dtype not in _DTYPE_CODE:
        raise TypeError("elementwise ops take float32 / int8 device arrays, got %s, %s" % (x.dtype, y.dtype))
    shape = y.shape if sx else x.shape
    z = _out(out, shape, binary_out_dtype(opname, x.dtype, y.dtype))
    capi.check(capi.lib().cgt_amd_elwise_binary(BINARY_OPS.index(opname), _DTYPE_CODE[x.dtype], _DTYPE_CODE[y.dtype],
                                                z.size, x.ptr, int(sx), y.ptr, int(sy), z.ptr, stream))
    return z


def repeat(x, axes, reps, out=None, stream=None):
    """Repeat(axes) (reference cgt/core.py:1511-1557): x has extent 1 on `axes`."""
    oshape = list(x.shape)
    flags = [0] * x.ndim
    for ax, rep in zip(axes, reps):
        if x.shape[ax] != 1:
            raise ValueError("Repeat: axis %d has extent %d, not 1" % (ax, x.shape[ax]))
        oshape[ax] = int(rep)
        flags[ax] = 1
    res = _out(out, tuple(oshape), x.dtype)
    nd = max(x.ndim, 1)
    capi.check(capi.lib().cgt_amd_repeat(x.ptr, x.dtype.itemsize, x.ndim, (ctypes.c_long * nd)(*oshape),
                                         (ctypes.c_int * nd)(*flags), res.ptr, stream))
    return res


def sum_keepdims(x, axes, out=None, stream=None):
    """Sum(axes), keepdims (reference cgt/core.py:1687-1709)."""
    _f32(x)
    flags = [1 if a in axes else 0 for a in range(x.ndim)]
    oshape = tuple(1 if f else s for s, f in zip(x.shape, flags))
    res = _out(out, oshape)
    nd = max(x.ndim, 1)
    capi.check(capi.lib().cgt_amd_sum_f32(x.ptr, x.ndim, (ctypes.c_long * nd)(*x.shape), (ctypes.c_int * nd)(*flags),
                                          res.ptr, stream))
    return res


def fill(value, shape, out=None, stream=None):
    """Fill(value) (reference cgt/core.py:966-1007), float32."""
    res = _out(out, tuple(int(s) for s in shape))
    capi.check(capi.lib().cgt_amd_fill_f32(res.ptr, float(value), res.size, stream))
    return res


def conv2d(x, f, pad=(0, 0), stride=(1, 1), stream=None, keep=None):
    """conv2d forward as the reference composes it on its CPU path
    (cgt/nn.py:95-100): im2col -> [B*m*n, Z] -> Mul22(False, True) with the
    filters as [L, Z] -> [B, m, n, L] -> Transpose{0,3,1,2}.
    `keep`, if a dict, receives the column buffer for the backward pass."""
    L, K, r, c = f.shape
    col = im2col(x, (r, c), pad, stride, stream=stream)
    B, m, n, Z = col.shape
    y = mul22(col.reshape(B * m * n, Z), f.reshape(L, Z), False, True, stream=stream)
    if keep is not None:
        keep["col"] = col
    return transpose4(y.reshape(B, m, n, L), (0, 3, 1, 2), stream=stream)


def conv2d_pullback(x, f, gy, pad=(0, 0), stride=(1, 1), col=None, stream=None):
    """Gradients (gx, gf) of conv2d, following the graph the reference's autodiff
    derives: Transpose{0,2,3,1} of gy (cgt/core.py:1569-1570); for Mul22(F,T)
    (core.py:2160-2162) gcol = Mul22(F,F)[gc, f_LZ] -> Col2Im (im2col.py:34-35)
    and gf = Mul22(T,F)[gc, col]."""
    L, K, r, c = f.shape
    if col is None:
        col = im2col(x, (r, c), pad, stride, stream=stream)
    B, m, n, Z = col.shape
    gc = transpose4(gy, (0, 2, 3, 1), stream=stream).reshape(B * m * n, L)
    gcol = mul22(gc, f.reshape(L, Z), False, False, stream=stream)
    gx = col2im(gcol.reshape(B, m, n, Z), x.shape, (r, c), pad, stride, stream=stream)
    gf = mul22(gc, col.reshape(B * m * n, Z), True, False, stream=stream).reshape(f.shape)
    return gx, gf


# ---------------------------------------------------------------- convolution without a column buffer

def conv_same_supported(C, L, kernel, pad, stride):
    """Whether the im2col-free path covers a layer (stride 1, odd kernel, pad = (kernel-1)/2,
    channel / filter counts its GEMM tiles fit)."""
    return bool(capi.lib().cgt_amd_conv_same_supported(int(C), int(L), *_geom(kernel, pad, stride)))


def conv_same_fits(xshape, L, kernel):
    """Whether a batch of images of this shape is inside what the products over the padded image index."""
    B, C, H, W = (int(v) for v in xshape)
    return bool(capi.lib().cgt_amd_conv_same_fits(B, C, H, W, int(L), int(kernel[0]), int(kernel[1])))


def conv_col_fits(xshape, L, kernel, pad, stride):
    """Whether the products over the column buffer of this layer are inside what they index."""
    B, C, H, W = (int(v) for v in xshape)
    g = _geom(kernel, pad, stride)
    m, n = conv_outsize(H, g[0], g[2], g[4]), conv_outsize(W, g[1], g[3], g[5])
    return bool(capi.lib().cgt_amd_conv_col_fits(B, m * n, C * g[0] * g[1], int(L)))


def conv_same_padded_size(planes, H, W, kernel):
    n = capi.lib().cgt_amd_conv_same_padded_size(int(planes), int(H), int(W), int(kernel[0]), int(kernel[1]))
    if n < 0:
        raise ValueError("conv_same: bad geometry")
    return n


def conv_same_pad(x, kernel, out=None, stream=None):
    """Zero-padded copy of x [B,C,H,W] in the layout the im2col-free products read (a flat array)."""
    _f32(x)
    B, C, H, W = x.shape
    res = _out(out, (conv_same_padded_size(B * C, H, W, kernel),))
    capi.check(capi.lib().cgt_amd_conv_same_pad_f32(x.ptr, B * C, H, W, int(kernel[0]), int(kernel[1]), res.ptr, stream))
    return res


def conv_same_pad_pool_pullback(xshape, mask, gtop, pool_kernel, pool_pad, pool_stride, kernel, relu_mask=None,
                                out=None, stream=None):
    """conv_same_pad(relu_mask * max_pool_pullback(xshape, mask, gtop, ...), kernel) in one pass,
    bit for bit; relu_mask is an int8 array of shape xshape or None."""
    _f32(gtop)
    B, C, H, W = xshape
    if mask.dtype != np.int32 or tuple(mask.shape) != tuple(gtop.shape) or tuple(mask.shape[:2]) != (B, C):
        raise ValueError("mask %s / cotangent %s do not fit an input of shape %s" % (tuple(mask.shape), tuple(gtop.shape), tuple(xshape)))
    if relu_mask is not None and (relu_mask.dtype != np.int8 or tuple(relu_mask.shape) != tuple(xshape)):
        raise ValueError("the rectify mask must be an int8 array of the input's shape")
    res = _out(out, (conv_same_padded_size(B * C, H, W, kernel),))
    capi.check(capi.lib().cgt_amd_conv_same_pad_pool_pullback_f32(
        mask.ptr, gtop.ptr, None if relu_mask is None else relu_mask.ptr, B * C, H, W, *_geom(pool_kernel, pool_pad, pool_stride),
        mask.shape[2], mask.shape[3], int(kernel[0]), int(kernel[1]), res.ptr, stream))
    return res


def conv_same_fwd(xpad, f, xshape, bias=None, relu=False, out=None, mask=None, stream=None):
    """conv2d (stride 1, same padding) from the padded input; optional fused bias add and
    rectify; `mask` (int8 array of the output's shape) receives (pre-activation >= 0)."""
    _f32(xpad, f)
    B, C, H, W = xshape
    L, C2, kh, kw = f.shape
    if C2 != C:
        raise ValueError("filter channels %d != input channels %d" % (C2, C))
    y = _out(out, (B, L, H, W))
    capi.check(capi.lib().cgt_amd_conv_same_fwd_f32(xpad.ptr, f.ptr, None if bias is None else bias.ptr, int(bool(relu)),
                                                    B, C, H, W, L, kh, kw, y.ptr, None if mask is None else mask.ptr, stream))
    return y


def conv_same_bwd_data(gypad, f, xshape, out=None, stream=None):
    _f32(gypad, f)
    B, C, H, W = xshape
    L, _, kh, kw = f.shape
    gx = _out(out, (B, C, H, W))
    capi.check(capi.lib().cgt_amd_conv_same_bwd_data_f32(gypad.ptr, f.ptr, B, C, H, W, L, kh, kw, gx.ptr, stream))
    return gx


def conv_same_bwd_filter(gypad, xpad, xshape, fshape, out=None, stream=None):
    _f32(gypad, xpad)
    B, C, H, W = xshape
    L, _, kh, kw = fshape
    gf = _out(out, tuple(fshape))
    capi.check(capi.lib().cgt_amd_conv_same_bwd_filter_f32(gypad.ptr, xpad.ptr, B, C, H, W, L, kh, kw, gf.ptr, stream))
    return gf


def conv_col_fwd(col, f, bias=None, relu=False, out=None, mask=None, stream=None):
    """y [B,L,m,n] = conv2d from the column buffer col [B,m,n,Z] and the filters f [L,C,kh,kw]
    (Z = C*kh*kw), written in NCHW by the product itself; optional fused bias add and rectify."""
    _f32(col, f)
    B, m, n, Z = col.shape
    L = f.shape[0]
    if int(np.prod(f.shape[1:])) != Z:
        raise ValueError("filters %s do not match patches of %d" % (tuple(f.shape), Z))
    y = _out(out, (B, L, m, n))
    capi.check(capi.lib().cgt_amd_conv_col_fwd_f32(col.ptr, f.ptr, None if bias is None else bias.ptr, int(bool(relu)),
                                                   B, m * n, Z, L, y.ptr, None if mask is None else mask.ptr, stream))
    return y


def conv_col_bwd_data(gy, f, out=None, stream=None):
    """gcol [B,m,n,Z] from the NCHW cotangent gy [B,L,m,n] and the filters."""
    _f32(gy, f)
    B, L, m, n = gy.shape
    if f.shape[0] != L:
        raise ValueError("cotangent has %d channels, the filter bank %d filters" % (L, f.shape[0]))
    Z = int(np.prod(f.shape[1:]))
    gcol = _out(out, (B, m, n, Z))
    capi.check(capi.lib().cgt_amd_conv_col_bwd_data_f32(gy.ptr, f.ptr, B, m * n, Z, L, gcol.ptr, stream))
    return gcol


def conv_col_bwd_filter(gy, col, fshape, out=None, stream=None):
    """gf [L,C,kh,kw] from the NCHW cotangent gy [B,L,m,n] and the column buffer."""
    _f32(gy, col)
    B, L, m, n = gy.shape
    Z = col.shape[3]
    if tuple(col.shape[:3]) != (B, m, n) or int(np.prod(fshape)) != L * Z:
        raise ValueError("cotangent %s, columns %s and filters %s do not match" % (tuple(gy.shape), tuple(col.shape), tuple(fshape)))
    gf = _out(out, tuple(fshape))
    capi.check(capi.lib().cgt_amd_conv_col_bwd_filter_f32(gy.ptr, col.ptr, B, m * n, Z, L, gf.ptr, stream))
    return gf


def conv_patch_supported(xshape, kernel, pad, stride):
    B, C, H, W = (int(s) for s in xshape)
    return bool(capi.lib().cgt_amd_conv_patch_supported(B, C, H, W, *_geom(kernel, pad, stride)))


def conv_patch_fwd(x, f, pad, stride, bias=None, relu=False, out=None, mask=None, stream=None):
    """y [B,L,m,n] = conv2d(x, f) with the patches gathered from x inside the product (no column
    buffer); optional fused bias add and rectify as in conv_col_fwd."""
    _f32(x, f)
    B, C, H, W = x.shape
    L, C2, kh, kw = f.shape
    if C2 != C:
        raise ValueError("filter channels %d != input channels %d" % (C2, C))
    g = _geom((kh, kw), pad, stride)
    m, n = conv_outsize(H, g[0], g[2], g[4]), conv_outsize(W, g[1], g[3], g[5])
    y = _out(out, (B, L, m, n))
    capi.check(capi.lib().cgt_amd_conv_patch_fwd_f32(x.ptr, f.ptr, None if bias is None else bias.ptr, int(bool(relu)),
                                                     B, C, H, W, L, *g, y.ptr, None if mask is None else mask.ptr, stream))
    return y


def conv_patch_bwd_filter(gy, x, fshape, pad, stride, out=None, stream=None):
    """gf [L,C,kh,kw] from the NCHW cotangent gy and the image x (no column buffer)."""
    _f32(gy, x)
    B, C, H, W = x.shape
    L, C2, kh, kw = (int(s) for s in fshape)
    g = _geom((kh, kw), pad, stride)
    m, n = conv_outsize(H, g[0], g[2], g[4]), conv_outsize(W, g[1], g[3], g[5])
    if C2 != C or tuple(gy.shape) != (B, L, m, n):
        raise ValueError("cotangent %s does not fit x %s and filters %s" % (tuple(gy.shape), tuple(x.shape), tuple(fshape)))
    gf = _out(out, (L, C, kh, kw))
    capi.check(capi.lib().cgt_amd_conv_patch_bwd_filter_f32(gy.ptr, x.ptr, B, C, H, W, L, *g, gf.ptr, stream))
    return gf
