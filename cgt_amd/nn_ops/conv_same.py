"""Fused convolution ops for stride 1 and pad = (kernel - 1) / 2: forward, data
gradient and weight gradient without a column buffer.

They stand where the reference's GPU branch of nn.conv2d puts its fused ops --
CudnnConvForward with its pullback made of CudnnConvBackwardData /
CudnnConvBackwardFilter (cgt/nn_ops/cudnn_ops.py:58-143, cgt/nn.py:88-93) --
with this library's own kernels behind them instead of cuDNN.  The image
operand of each product is the zero-padded copy made by ConvPad, which the
forward op and both gradients share.
"""
import ctypes
from collections import namedtuple

from .. import core

ConvSameInfo = namedtuple("ConvSameInfo", ["kernel_h", "kernel_w"])


def info2closure(info):
    return [("kernel_h", ctypes.c_int, info.kernel_h), ("kernel_w", ctypes.c_int, info.kernel_w)]


def padded_size(planes, H, W, info):
    """Floats in the padded copy of `planes` planes (cgt_amd_conv_same_padded_size), as a
    shape expression."""
    pw = (info.kernel_w - 1) // 2
    Hp, Wp = H + 2 * ((info.kernel_h - 1) // 2), W + pw
    plane = (pw + Hp * Wp + 16 + 15) // 16 * 16
    tail = (256 + info.kernel_h * Wp + 3) // 4 * 4
    return planes * plane + tail


class ConvPad(core.Op):
    """x [B,C,H,W] -> flat zero-padded copy, the layout the products read."""
    available_impls = ("native_gpu",)

    def __init__(self, info):
        self.info = info

    def get_diff(self, _):
        return [False]          # gradients reach x through ConvForward's own pullback

    def shp_apply(self, inputs):
        B, C, H, W = core.shape(inputs[0])
        return [padded_size(B * C, H, W, self.info)]

    def typ_apply(self, input_types):
        assert input_types[0].ndim == 4 and input_types[0].dtype == "f4"
        return core.TensorType("f4", 1)

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu"
        code = r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtArray* write) {
                cgtArray* x = reads[0];
                const long* s = x->shape();
                long need = cgt_amd_conv_same_padded_size(s[0] * s[1], s[2], s[3], cl->kernel_h, cl->kernel_w);
                cgt_check(write->size() == need, "ConvPad: output has %ld floats, the geometry needs %ld", write->size(), need);
                if (cgtGlobalStatus != cgtStatusOK) return;
                int rc = cgt_amd_conv_same_pad_f32((const float*)x->data(), s[0] * s[1], s[2], s[3],
                    cl->kernel_h, cl->kernel_w, (float*)write->data(), cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "ConvPad: %s", cgt_amd_last_error());
            }"""
        return core.NativeCompileInfo(code, includes=["cgt_amd.h"], closure_triples=info2closure(self.info),
                                      gpu_deref_mask=(True,))


# Whether the padded cotangent of a convolution that feeds (a rectify and) a max pool is written
# by the pool's pullback itself (ConvPadPoolPullback) instead of MaxPoolPullback -> (mask *) -> ConvPad
FUSE_POOL_PULLBACK = True


class ConvPadPoolPullback(core.Op):
    """inputs [x, pool, mask, gpool] (+ [relu_mask]) -> ConvPad(relu_mask * MaxPoolPullback(x, pool, mask, gpool))
    in one pass, bit for bit: the inputs are MaxPoolPullback's own (cgt/nn_ops/max_pool_2d.py:55-72,
    only mask and gpool are read), x gives the shape."""
    available_impls = ("native_gpu",)

    def __init__(self, info, poolinfo, has_relu=False):
        self.info, self.poolinfo, self.has_relu = info, poolinfo, bool(has_relu)

    def get_diff(self, n):
        return [False] * n

    def shp_apply(self, inputs):
        B, C, H, W = core.shape(inputs[0])
        return [padded_size(B * C, H, W, self.info)]

    def typ_apply(self, input_types):
        return core.TensorType("f4", 1)

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu"
        from .max_pool_2d import info2closure as pool_closure
        code = r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtArray* write) {
                cgtArray *x = reads[0], *mask = reads[2], *gpool = reads[3], *rmask = cl->has_relu ? reads[4] : NULL;
                const long* s = x->shape();
                long need = cgt_amd_conv_same_padded_size(s[0] * s[1], s[2], s[3], cl->conv_kernel_h, cl->conv_kernel_w);
                cgt_check(write->size() == need, "ConvPadPoolPullback: output has %ld floats, the geometry needs %ld", write->size(), need);
                cgt_check(gpool->size() == mask->size() && mask->shape()[0] == s[0] && mask->shape()[1] == s[1] &&
                          (!rmask || (rmask->size() == x->size() && rmask->dtype() == cgt_i1)),
                          "ConvPadPoolPullback: mask, cotangent or rectify mask do not fit the input's shape");
                if (cgtGlobalStatus != cgtStatusOK) return;
                int rc = cgt_amd_conv_same_pad_pool_pullback_f32((const int*)mask->data(), (const float*)gpool->data(),
                    rmask ? (const signed char*)rmask->data() : NULL, s[0] * s[1], s[2], s[3],
                    cl->kernel_h, cl->kernel_w, cl->pad_h, cl->pad_w, cl->stride_h, cl->stride_w,
                    mask->shape()[2], mask->shape()[3], cl->conv_kernel_h, cl->conv_kernel_w,
                    (float*)write->data(), cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "ConvPadPoolPullback: %s", cgt_amd_last_error());
            }"""
        triples = pool_closure(self.poolinfo) + [("conv_kernel_h", ctypes.c_int, self.info.kernel_h),
                                                 ("conv_kernel_w", ctypes.c_int, self.info.kernel_w),
                                                 ("has_relu", ctypes.c_int, int(self.has_relu))]
        return core.NativeCompileInfo(code, includes=["cgt_amd.h"], closure_triples=triples,
                                      gpu_deref_mask=(False, False, True, True) + ((True,) if self.has_relu else ()))


_CHECK_PADDED = r"""
                long need = cgt_amd_conv_same_padded_size(%s, H, W, cl->kernel_h, cl->kernel_w);
                cgt_check(%s->size() == need, "%s: padded operand has %%ld floats, the geometry needs %%ld", %s->size(), need);
"""


class ConvForward(core.Op):
    """inputs [x, xpad, f] (+ [bias] when has_bias) -> y [B,L,H,W]; with relu, the tuple
    (y, mask): y = pre * (pre >= 0) and mask = (pre >= 0) as int8, pre = conv + bias.

    x gives the shape and receives the gradient; the product reads xpad = ConvPad(x).  The
    bias add and the rectify are the SpatialConvolution bias (cgt/nn.py:231-233) and
    nn.rectify (cgt/nn.py:44-45) applied in the product's epilogue with the same fp32
    operations, and the pullback is built from the same ops the unfused graph would use
    (mask * gy, Sum over (0, 2, 3) for the bias), so values and gradients have the bits of
    the unfused graph."""
    available_impls = ("native_gpu",)

    def __init__(self, info, has_bias=False, relu=False):
        self.info, self.has_bias, self.relu = info, bool(has_bias), bool(relu)

    def with_relu(self):
        return ConvForward(self.info, self.has_bias, True)

    def get_diff(self, _):
        return [True, False, True] + ([True] if self.has_bias else [])

    def shp_apply(self, inputs):
        B, _, H, W = core.shape(inputs[0])
        shp = [B, core.size(inputs[2], 0), H, W]
        return (shp, list(shp)) if self.relu else shp

    def typ_apply(self, input_types):
        t = core.TensorType("f4", 4)
        return core.TupleType(t, core.TensorType("i1", 4)) if self.relu else t

    def pullback(self, inputs, output, goutput):
        return self.pullback_wanted(inputs, output, goutput, self.get_diff(len(inputs)))

    def pullback_wanted(self, inputs, output, goutput, wanted):
        from .max_pool_2d import MaxPoolPullback
        x, xpad, f = inputs[:3]
        gz = goutput[0] if self.relu else goutput
        mask = core.unpack(output)[1] if self.relu else None
        want_bias = self.has_bias and wanted[3]
        # the cotangent comes out of a max pool and nothing but the padded copy needs it: the
        # pool's pullback writes the padded copy itself (rectify mask applied on the way)
        fuse_pool = FUSE_POOL_PULLBACK and isinstance(gz.op, MaxPoolPullback) and not want_bias
        gy = None
        if not fuse_pool:
            # what x * (x >= 0) hands back: (x >= 0) * gz
            gy = core.elwise_binary("*", mask, gz) if self.relu else gz
        gbias = None
        if want_bias:
            gbias = core.sum(gy, axis=(0, 2, 3), keepdims=True)  # the pullback of the bias' Repeat
        gx = gf = None
        if wanted[0] or wanted[2]:
            if fuse_pool:
                gypad = core.Result(ConvPadPoolPullback(self.info, gz.op.info, self.relu),
                                    list(gz.parents) + ([mask] if self.relu else []))
            else:
                gypad = core.Result(ConvPad(self.info), [gy])
            gx = core.Result(ConvBackwardData(self.info), [gypad, f, x]) if wanted[0] else None
            gf = core.Result(ConvBackwardFilter(self.info), [gypad, xpad, f, x]) if wanted[2] else None
        return [gx, None, gf] + ([gbias] if self.has_bias else [])

    def get_closure(self):
        return info2closure(self.info) + [("has_bias", ctypes.c_int, int(self.has_bias)), ("relu", ctypes.c_int, int(self.relu))]

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu"
        head = (r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtTuple* out) {
                cgtArray* write = static_cast<cgtArray*>(out->getitem(0));
                cgtArray* mask = static_cast<cgtArray*>(out->getitem(1));
                cgt_check(mask->size() == write->size() && mask->dtype() == cgt_i1, "ConvForward: the mask must be an int8 array of the output's shape");
""" if self.relu else r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtArray* write) {
                cgtArray* mask = NULL;
""")
        code = head + r"""
                cgtArray *x = reads[0], *xpad = reads[1], *f = reads[2], *bias = cl->has_bias ? reads[3] : NULL;
                long B = x->shape()[0], C = x->shape()[1], H = x->shape()[2], W = x->shape()[3], L = f->shape()[0];
                cgt_check(f->ndim() == 4 && f->shape()[1] == C && f->shape()[2] == cl->kernel_h && f->shape()[3] == cl->kernel_w
                          && write->size() == B * L * H * W && (!bias || bias->size() == L),
                          "ConvForward: filters, bias or output do not fit the input");
""" + _CHECK_PADDED % ("B * C", "xpad", "ConvForward", "xpad") + r"""
                if (cgtGlobalStatus != cgtStatusOK) return;
                int rc = cgt_amd_conv_same_fwd_f32((const float*)xpad->data(), (const float*)f->data(),
                    bias ? (const float*)bias->data() : NULL, cl->relu, B, C, H, W, L, cl->kernel_h, cl->kernel_w,
                    (float*)write->data(), mask ? (signed char*)mask->data() : NULL, cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "ConvForward: %s", cgt_amd_last_error());
            }"""
        return core.NativeCompileInfo(code, includes=["cgt_amd.h"], closure_triples=self.get_closure(),
                                      gpu_deref_mask=(False, True, True) + ((True,) if self.has_bias else ()))


class ConvBackwardData(core.Op):
    """inputs [gypad, f, x] -> gx (x gives the shape only)."""
    available_impls = ("native_gpu",)

    def __init__(self, info):
        self.info = info

    def shp_apply(self, inputs):
        return core.shape(inputs[2])

    def typ_apply(self, input_types):
        return core.TensorType("f4", 4)

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu"
        code = r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtArray* write) {
                cgtArray *gypad = reads[0], *f = reads[1], *x = reads[2];
                long B = x->shape()[0], C = x->shape()[1], H = x->shape()[2], W = x->shape()[3], L = f->shape()[0];
                cgt_check(f->ndim() == 4 && f->shape()[1] == C && f->shape()[2] == cl->kernel_h && f->shape()[3] == cl->kernel_w
                          && write->size() == x->size(), "ConvBackwardData: filters or output do not fit the input");
""" + _CHECK_PADDED % ("B * L", "gypad", "ConvBackwardData", "gypad") + r"""
                if (cgtGlobalStatus != cgtStatusOK) return;
                int rc = cgt_amd_conv_same_bwd_data_f32((const float*)gypad->data(), (const float*)f->data(),
                    B, C, H, W, L, cl->kernel_h, cl->kernel_w, (float*)write->data(), cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "ConvBackwardData: %s", cgt_amd_last_error());
            }"""
        return core.NativeCompileInfo(code, includes=["cgt_amd.h"], closure_triples=info2closure(self.info),
                                      gpu_deref_mask=(True, True, False))


class ConvBackwardFilter(core.Op):
    """inputs [gypad, xpad, f, x] -> gf (f and x give shapes only)."""
    available_impls = ("native_gpu",)

    def __init__(self, info):
        self.info = info

    def shp_apply(self, inputs):
        return core.shape(inputs[2])

    def typ_apply(self, input_types):
        return core.TensorType("f4", 4)

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu"
        code = r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtArray* write) {
                cgtArray *gypad = reads[0], *xpad = reads[1], *f = reads[2], *x = reads[3];
                long B = x->shape()[0], C = x->shape()[1], H = x->shape()[2], W = x->shape()[3], L = f->shape()[0];
                cgt_check(f->ndim() == 4 && f->shape()[1] == C && f->shape()[2] == cl->kernel_h && f->shape()[3] == cl->kernel_w
                          && write->size() == f->size(), "ConvBackwardFilter: output does not fit the filters");
""" + _CHECK_PADDED % ("B * L", "gypad", "ConvBackwardFilter", "gypad") + _CHECK_PADDED.replace("long need", "need") % ("B * C", "xpad", "ConvBackwardFilter", "xpad") + r"""
                if (cgtGlobalStatus != cgtStatusOK) return;
                int rc = cgt_amd_conv_same_bwd_filter_f32((const float*)gypad->data(), (const float*)xpad->data(),
                    B, C, H, W, L, cl->kernel_h, cl->kernel_w, (float*)write->data(), cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "ConvBackwardFilter: %s", cgt_amd_last_error());
            }"""
        return core.NativeCompileInfo(code, includes=["cgt_amd.h"], closure_triples=info2closure(self.info),
                                      gpu_deref_mask=(True, True, False, False))


def supported(x, f, kernelshape, pad, stride):
    """Whether these ops cover the layer (see cgt_amd_conv_same_supported)."""
    from .. import kernels
    return (kernels.conv_same_supported(core.size(x, 1), core.size(f, 0), kernelshape, pad, stride)
            and kernels.conv_same_fits(core.shape(x), core.size(f, 0), kernelshape))


def conv_same(x, f, kernelshape, bias=None, relu=False):
    """conv2d (+ per-channel bias [1,L,1,1]) (+ rectify) through the fused ops."""
    x, f = core.as_node(x), core.as_node(f)
    info = ConvSameInfo(int(kernelshape[0]), int(kernelshape[1]))
    xpad = core.Result(ConvPad(info), [x])
    parents = [x, xpad, f] + ([core.as_node(bias)] if bias is not None else [])
    out = core.Result(ConvForward(info, bias is not None, relu), parents)
    return out[0] if relu else out
