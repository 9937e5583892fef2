"""cgt.nn front end of the CNN hot path (reference cgt/nn.py:85-111).

The reference's CPU path composes conv2d as
    im2col -> reshape -> Mul22(False, True) -> reshape -> transpose{0,3,1,2}
and its devtype == "gpu" branch switches to fused convolution ops (cuDNN,
cgt/nn.py:88-93).  This build's GPU branch switches to its own fused ops:
  * stride 1, pad = (kernel - 1) / 2, channel and filter counts in multiples
    of 16: products that read a zero-padded copy of the image, no column
    buffer (nn_ops/conv_same.py);
  * layers with few input channels (the first layer of a network: 1 or 3
    channels, any stride): products that gather their patches from the image
    and write / read the NCHW arrays themselves -- no column buffer for the
    forward product and the weight gradient, no transposes (nn_ops/conv_col.py,
    ConvPatch*);
  * every other layer: Im2Col, then the same products over the column
    buffer (nn_ops/conv_col.py, ConvCol*) -- conv_algo("col") uses these for
    every layer;
conv_algo("im2col") keeps the literal composition, every op on the GPU.
"""
from . import core
from .nn_ops import conv_col, conv_same
from .nn_ops import cross_channel_lrn as _lrn
from .nn_ops.cross_channel_lrn import cross_channel_lrn  # noqa: F401
from .nn_ops.im2col import im2col
from .nn_ops.max_pool_2d import MaxPool, PoolInfo


_CONV_ALGO = "auto"


def conv_algo(name=None):
    """Select how conv2d is built: "auto" (the fused ops without a column buffer where
    they apply, those over the column buffer elsewhere), "col" (always the fused ops over
    the column buffer) or "im2col" (always the literal im2col -> Mul22 -> transpose
    composition).  Returns the previous setting."""
    global _CONV_ALGO
    old = _CONV_ALGO
    if name is not None:
        assert name in ("auto", "col", "im2col")
        _CONV_ALGO = name
    return old


def _check_geometry(x, channels, kernelshape, pad, stride):
    """The reference's shape rule, (H + 2p - k) // s + 1 (cgt/nn_ops/im2col.py:36-41), goes to zero or
    below when the kernel does not fit the padded image; say so here instead of failing in an allocation."""
    B, K, H, W = x.shape
    if K != channels:
        raise ValueError("conv2d: the image has %d channels, the filters take %d" % (K, channels))
    if min(stride) < 1 or min(pad) < 0 or min(kernelshape) < 1:
        raise ValueError("conv2d: bad geometry kernel=%s pad=%s stride=%s" % (kernelshape, pad, stride))
    if H + 2 * pad[0] < kernelshape[0] or W + 2 * pad[1] < kernelshape[1]:
        raise ValueError("conv2d: the %dx%d kernel is larger than the %dx%d image padded by %s"
                         % (kernelshape[0], kernelshape[1], H, W, tuple(pad)))


def conv2d(x_BKRC, f_LKrc, kernelshape, pad=(0, 0), stride=(1, 1)):
    x_BKRC, f_LKrc = core.as_node(x_BKRC), core.as_node(f_LKrc)
    L, K, r, c = f_LKrc.shape
    assert tuple(kernelshape) == (r, c), "kernelshape must match the filter's last two axes"
    _check_geometry(x_BKRC, K, tuple(kernelshape), tuple(pad), tuple(stride))
    if _CONV_ALGO == "auto" and conv_same.supported(x_BKRC, f_LKrc, kernelshape, pad, stride):
        return conv_same.conv_same(x_BKRC, f_LKrc, kernelshape)
    # extents beyond what the fused products index fall through: padded-image products ->
    # products over a column buffer -> the literal composition, which takes any size
    fits_col = conv_col.col_supported(x_BKRC, f_LKrc, kernelshape, pad, stride)
    if _CONV_ALGO == "auto" and fits_col and conv_col.patch_supported(x_BKRC, kernelshape, pad, stride):
        return conv_col.conv_patch(x_BKRC, f_LKrc, kernelshape, pad, stride)
    col_BmnZ = im2col(x_BKRC, kernelshape, pad, stride)
    if _CONV_ALGO != "im2col" and fits_col:
        return conv_col.conv_col(col_BmnZ, f_LKrc)
    f_LZ = f_LKrc.reshape([L, K * r * c])
    B, m, n, Z = col_BmnZ.shape
    col_Bmn_Z = col_BmnZ.reshape([B * m * n, Z])
    col_Bmn_L = core.Result(core.Mul22(False, True), [col_Bmn_Z, f_LZ])
    return col_Bmn_L.reshape([B, m, n, L]).transpose([0, 3, 1, 2])


_CONV_FUSION = True


def conv_fusion(on=None):
    """Whether the fusions around the layer's ops are built (default) or every op stays the
    reference's: SpatialConvolution's bias add and a rectify that follows a fused convolution
    in the convolution's epilogue, a pool pullback written straight into the padded cotangent,
    and cross_channel_lrn without a stored scale array.  Returns the previous setting."""
    global _CONV_FUSION
    old = _CONV_FUSION
    if on is not None:
        _CONV_FUSION = bool(on)
        conv_same.FUSE_POOL_PULLBACK = bool(on)
        _lrn.STORE_TOP_ONLY = bool(on)
    return old


def rectify(x):
    """ReLU as the reference builds it: x * (x >= 0) (cgt/nn.py:44-45).  On the result of a
    fused convolution it becomes part of that op (same values, same gradient)."""
    x = core.as_node(x)
    if (_CONV_FUSION and isinstance(x.op, (conv_same.ConvForward, conv_col.ConvColForward, conv_col.ConvPatchForward))
            and not x.op.relu):
        # the same inputs run again with the rectify in the epilogue.  Nodes are evaluated as
        # they are built, so this costs a second product while the graph is traced; a compiled
        # function replays only the fused one (the plain result is no longer reachable from
        # the outputs)
        return core.Result(x.op.with_relu(), x.parents)[0]
    return x * (x >= 0)


class SpatialConvolution(object):
    """conv2d plus a per-channel bias [1, L, 1, 1] (reference cgt/nn.py:216-233).
    Weights and bias are device-resident leaf nodes."""

    def __init__(self, input_channels, output_channels, kernelshape, pad, stride=(1, 1), name=None,
                 weight_init=None, bias_init=None):
        import numpy as np
        input_channels, output_channels = int(input_channels), int(output_channels)
        self.kernelshape = tuple(map(int, kernelshape))
        self.pad = tuple(map(int, pad))
        self.stride = tuple(map(int, stride))
        self.name = "unnamed" if name is None else name
        wshape = (output_channels, input_channels) + self.kernelshape
        w = np.zeros(wshape, np.float32) if weight_init is None else np.asarray(weight_init, np.float32).reshape(wshape)
        b = np.zeros((1, output_channels, 1, 1), np.float32) if bias_init is None else \
            np.asarray(bias_init, np.float32).reshape(1, output_channels, 1, 1)
        self.weight = core.constant(w)
        self.bias = core.constant(b)

    def __call__(self, x):
        x = core.as_node(x)
        _check_geometry(x, self.weight.shape[1], self.kernelshape, self.pad, self.stride)
        if (_CONV_FUSION and _CONV_ALGO == "auto"
                and conv_same.supported(x, self.weight, self.kernelshape, self.pad, self.stride)):
            return conv_same.conv_same(x, self.weight, self.kernelshape, bias=self.bias)
        fits_col = conv_col.col_supported(x, self.weight, self.kernelshape, self.pad, self.stride)
        if (_CONV_FUSION and _CONV_ALGO == "auto" and fits_col
                and conv_col.patch_supported(x, self.kernelshape, self.pad, self.stride)):
            return conv_col.conv_patch(x, self.weight, self.kernelshape, self.pad, self.stride, bias=self.bias)
        if _CONV_FUSION and _CONV_ALGO != "im2col" and fits_col:
            col = im2col(x, self.kernelshape, self.pad, self.stride)
            return conv_col.conv_col(col, self.weight, bias=self.bias)
        tmp = conv2d(x, self.weight, self.kernelshape, self.pad, self.stride)
        return core.broadcast("+", tmp, self.bias, "xxxx,1x11")


class Affine(object):
    """x.dot(W) + b with W [input_size, output_size], b [1, output_size] (reference cgt/nn.py:198-213): the
    fully connected layer that ends the reference's convolutional examples.  Weights default to zero as there."""

    def __init__(self, input_size, output_size, name=None, weight_init=None, bias_init=None):
        import numpy as np
        input_size, output_size = int(input_size), int(output_size)
        self.name = "unnamed" if name is None else name
        w = np.zeros((input_size, output_size), np.float32) if weight_init is None else \
            np.asarray(weight_init, np.float32).reshape(input_size, output_size)
        b = np.zeros((1, output_size), np.float32) if bias_init is None else np.asarray(bias_init, np.float32).reshape(1, output_size)
        self.weight = core.constant(w)
        self.bias = core.constant(b)

    def __call__(self, x):
        return core.broadcast("+", core.dot(core.as_node(x), self.weight), self.bias, "xx,1x")


def softmax(x, axis=1):
    """exp(x) / sum(exp(x), axis) for a matrix, without the shift by the row maximum -- as the
    reference computes it (cgt/nn.py:55-59)."""
    out = core.exp(core.as_node(x))
    return core.broadcast("/", out, core.sum(out, axis=axis, keepdims=True), "xx,x1" if axis == 1 else "xx,1x")


def logsoftmax(x, axis=1):
    """log(softmax(x)) (cgt/nn.py:61-62)."""
    return core.log(softmax(x, axis=axis))


def max_pool_2d(x, kernelshape, pad=(0, 0), stride=(1, 1)):
    kernel_h, kernel_w = kernelshape
    pad_h, pad_w = pad
    stride_h, stride_w = stride
    info = PoolInfo(kernel_h, kernel_w, pad_h, pad_w, stride_h, stride_w)
    return core.Result(MaxPool(info), [x])[0]


def sgd(cost, params, learning_rate):
    """Stochastic gradient descent updates, param := param - learning_rate * gradient
    (reference cgt/nn.py:240-262): a list of (param, new_param) for function(..., updates=)."""
    grads = core.grad(cost, params)
    return [(param, param - learning_rate * g) for param, g in zip(params, grads)]
