"""conv2d over the column buffer of Im2Col, for every layer geometry, with the NCHW
side read and written by the products themselves.

The reference's CPU path composes conv2d from im2col -> reshape -> Mul22(F,T) ->
reshape -> Transpose{0,3,1,2} (cgt/nn.py:95-100), and its autodiff answers with
Transpose{0,2,3,1} -> Mul22(F,F) -> Col2Im and Mul22(T,F) (cgt/core.py:2143-2175,
1569-1570).  Its GPU branch puts one fused op with a pullback made of two more in that
place (cgt/nn.py:88-93, cgt/nn_ops/cudnn_ops.py:58-143).  These ops keep Im2Col / Col2Im
as they are and fuse the rest: the forward product writes [B,L,m,n] itself and the two
gradient products read the NCHW cotangent itself, so the [B*m*n, L] matrices and both
transposes are never materialised.
"""
import ctypes

from .. import core


class ConvColForward(core.Op):
    """inputs [col, f] (+ [bias] when has_bias) -> y [B,L,m,n]; with relu, the tuple
    (y, mask): y = pre * (pre >= 0) and mask = (pre >= 0) as int8, pre = conv + bias.

    col [B,m,n,Z] is Im2Col's result, f [L,C,kh,kw] with C*kh*kw = Z.  Bias add and rectify
    are the SpatialConvolution bias (cgt/nn.py:231-233) and nn.rectify (cgt/nn.py:44-45)
    applied in the product's epilogue with the same fp32 operations; the pullback is built
    from the ops the unfused graph would use for them (mask * gy, Sum over (0, 2, 3))."""
    available_impls = ("native_gpu",)

    def __init__(self, has_bias=False, relu=False):
        self.has_bias, self.relu = bool(has_bias), bool(relu)

    def with_relu(self):
        return ConvColForward(self.has_bias, True)

    def get_diff(self, _):
        return [True, True] + ([True] if self.has_bias else [])

    def shp_apply(self, inputs):
        B, m, n, _ = core.shape(inputs[0])
        shp = [B, core.size(inputs[1], 0), m, n]
        return (shp, list(shp)) if self.relu else shp

    def typ_apply(self, input_types):
        assert input_types[0].ndim == 4 and input_types[1].ndim == 4
        t = core.TensorType("f4", 4)
        return core.TupleType(t, core.TensorType("i1", 4)) if self.relu else t

    def pullback(self, inputs, output, goutput):
        return self.pullback_wanted(inputs, output, goutput, self.get_diff(len(inputs)))

    def pullback_wanted(self, inputs, output, goutput, wanted):
        col, f = inputs[:2]
        if self.relu:
            _y, mask = core.unpack(output)
            gy = core.elwise_binary("*", mask, goutput[0])     # what x * (x >= 0) hands back: (x >= 0) * gz
        else:
            gy = goutput
        gbias = None
        if self.has_bias and wanted[2]:
            gbias = core.sum(gy, axis=(0, 2, 3), keepdims=True)  # the pullback of the bias' Repeat
        gcol = core.Result(ConvColBackwardData(), [gy, f, col]) if wanted[0] else None
        gf = core.Result(ConvColBackwardFilter(), [gy, col, f]) if wanted[1] else None
        return [gcol, gf] + ([gbias] if self.has_bias else [])

    def get_closure(self):
        return [("has_bias", ctypes.c_int, int(self.has_bias)), ("relu", ctypes.c_int, int(self.relu))]

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu"
        head = (r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtTuple* out) {
                cgtArray* write = static_cast<cgtArray*>(out->getitem(0));
                cgtArray* mask = static_cast<cgtArray*>(out->getitem(1));
                cgt_check(mask->size() == write->size() && mask->dtype() == cgt_i1, "ConvColForward: the mask must be an int8 array of the output's shape");
""" if self.relu else r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtArray* write) {
                cgtArray* mask = NULL;
""")
        code = head + r"""
                cgtArray *col = reads[0], *f = reads[1], *bias = cl->has_bias ? reads[2] : NULL;
                long B = col->shape()[0], P = col->shape()[1] * col->shape()[2], Z = col->shape()[3], L = f->shape()[0];
                cgt_check(col->ndim() == 4 && f->size() == L * Z && write->size() == B * L * P && (!bias || bias->size() == L),
                          "ConvColForward: filters, bias or output do not fit the column buffer");
                if (cgtGlobalStatus != cgtStatusOK) return;
                int rc = cgt_amd_conv_col_fwd_f32((const float*)col->data(), (const float*)f->data(),
                    bias ? (const float*)bias->data() : NULL, cl->relu, B, P, Z, L,
                    (float*)write->data(), mask ? (signed char*)mask->data() : NULL, cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "ConvColForward: %s", cgt_amd_last_error());
            }"""
        return core.NativeCompileInfo(code, includes=["cgt_amd.h"], closure_triples=self.get_closure(),
                                      gpu_deref_mask=(True, True) + ((True,) if self.has_bias else ()))


class ConvColBackwardData(core.Op):
    """inputs [gy, f, col] -> gcol, the cotangent of the column buffer (col gives the shape only)."""
    available_impls = ("native_gpu",)

    def shp_apply(self, inputs):
        return core.shape(inputs[2])

    def typ_apply(self, input_types):
        return core.TensorType("f4", 4)

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu"
        code = r"""
            CGT_EXPORT_C void $function(void* cl, cgtArray** reads, cgtArray* write) {
                cgtArray *gy = reads[0], *f = reads[1], *col = reads[2];
                long B = col->shape()[0], P = col->shape()[1] * col->shape()[2], Z = col->shape()[3], L = f->shape()[0];
                cgt_check(gy->size() == B * L * P && f->size() == L * Z && write->size() == col->size(),
                          "ConvColBackwardData: cotangent, filters or output do not fit the column buffer");
                if (cgtGlobalStatus != cgtStatusOK) return;
                int rc = cgt_amd_conv_col_bwd_data_f32((const float*)gy->data(), (const float*)f->data(), B, P, Z, L,
                    (float*)write->data(), cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "ConvColBackwardData: %s", cgt_amd_last_error());
            }"""
        return core.NativeCompileInfo(code, includes=["cgt_amd.h"], gpu_deref_mask=(True, True, False))


class ConvColBackwardFilter(core.Op):
    """inputs [gy, col, f] -> gf (f gives the shape only)."""
    available_impls = ("native_gpu",)

    def shp_apply(self, inputs):
        return core.shape(inputs[2])

    def typ_apply(self, input_types):
        return core.TensorType("f4", 4)

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu"
        code = r"""
            CGT_EXPORT_C void $function(void* cl, cgtArray** reads, cgtArray* write) {
                cgtArray *gy = reads[0], *col = reads[1], *f = reads[2];
                long B = col->shape()[0], P = col->shape()[1] * col->shape()[2], Z = col->shape()[3], L = f->shape()[0];
                cgt_check(gy->size() == B * L * P && f->size() == L * Z && write->size() == f->size(),
                          "ConvColBackwardFilter: cotangent or output do not fit the column buffer and the filters");
                if (cgtGlobalStatus != cgtStatusOK) return;
                int rc = cgt_amd_conv_col_bwd_filter_f32((const float*)gy->data(), (const float*)col->data(), B, P, Z, L,
                    (float*)write->data(), cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "ConvColBackwardFilter: %s", cgt_amd_last_error());
            }"""
        return core.NativeCompileInfo(code, includes=["cgt_amd.h"], gpu_deref_mask=(True, True, False))


def conv_col(col, f, bias=None, relu=False):
    """conv2d (+ per-channel bias [1,L,1,1]) (+ rectify) from the column buffer."""
    col, f = core.as_node(col), core.as_node(f)
    parents = [col, f] + ([core.as_node(bias)] if bias is not None else [])
    out = core.Result(ConvColForward(bias is not None, relu), parents)
    return out[0] if relu else out


# ---- the same fused op without the column buffer: the forward product and the weight gradient
# gather their patches from x while the GEMM loads its operand tile.  The data gradient still goes
# through a column buffer (its cotangent) and Im2Col's own pullback, Col2Im.

_PATCH_GEOM = "cl->kernel_h, cl->kernel_w, cl->pad_h, cl->pad_w, cl->stride_h, cl->stride_w"


def _out_hw(H, W, info):
    return ((H + 2 * info.pad_h - info.kernel_h) // info.stride_h + 1,
            (W + 2 * info.pad_w - info.kernel_w) // info.stride_w + 1)


class ConvPatchForward(core.Op):
    """inputs [x, f] (+ [bias] when has_bias) -> y [B,L,m,n] = conv2d(x, f) (+ bias) (rectified: the
    tuple (y, mask)), as ConvColForward computes it from Im2Col(x) -- bit for bit -- with the
    patches read from x inside the product.  info is Im2Col's (kernel, pad, stride)."""
    available_impls = ("native_gpu",)

    def __init__(self, info, has_bias=False, relu=False):
        self.info, self.has_bias, self.relu = info, bool(has_bias), bool(relu)

    def with_relu(self):
        return ConvPatchForward(self.info, self.has_bias, True)

    def get_diff(self, _):
        return [True, True] + ([True] if self.has_bias else [])

    def shp_apply(self, inputs):
        B, _, H, W = core.shape(inputs[0])
        m, n = _out_hw(H, W, self.info)
        shp = [B, core.size(inputs[1], 0), m, n]
        return (shp, list(shp)) if self.relu else shp

    def typ_apply(self, input_types):
        assert input_types[0].ndim == 4 and input_types[1].ndim == 4
        t = core.TensorType("f4", 4)
        return core.TupleType(t, core.TensorType("i1", 4)) if self.relu else t

    def pullback(self, inputs, output, goutput):
        return self.pullback_wanted(inputs, output, goutput, self.get_diff(len(inputs)))

    def pullback_wanted(self, inputs, output, goutput, wanted):
        from .im2col import Col2Im
        x, f = inputs[:2]
        if self.relu:
            _y, mask = core.unpack(output)
            gy = core.elwise_binary("*", mask, goutput[0])     # what x * (x >= 0) hands back: (x >= 0) * gz
        else:
            gy = goutput
        gbias = None
        if self.has_bias and wanted[2]:
            gbias = core.sum(gy, axis=(0, 2, 3), keepdims=True)
        gx = None
        if wanted[0]:
            gcol = core.Result(ConvPatchBackwardData(self.info), [gy, f, x])
            gx = core.Result(Col2Im(self.info), [gcol] + core.shape(x))
        gf = core.Result(ConvPatchBackwardFilter(self.info), [gy, x, f]) if wanted[1] else None
        return [gx, gf] + ([gbias] if self.has_bias else [])

    def get_closure(self):
        from .im2col import info2closure
        return info2closure(self.info) + [("has_bias", ctypes.c_int, int(self.has_bias)), ("relu", ctypes.c_int, int(self.relu))]

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu"
        head = (r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtTuple* out) {
                cgtArray* write = static_cast<cgtArray*>(out->getitem(0));
                cgtArray* mask = static_cast<cgtArray*>(out->getitem(1));
                cgt_check(mask->size() == write->size() && mask->dtype() == cgt_i1, "ConvPatchForward: the mask must be an int8 array of the output's shape");
""" if self.relu else r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtArray* write) {
                cgtArray* mask = NULL;
""")
        code = head + r"""
                cgtArray *x = reads[0], *f = reads[1], *bias = cl->has_bias ? reads[2] : NULL;
                const long* s = x->shape();
                long L = f->shape()[0];
                long m = (s[2] + 2*cl->pad_h - cl->kernel_h) / cl->stride_h + 1,
                     n = (s[3] + 2*cl->pad_w - cl->kernel_w) / cl->stride_w + 1;
                cgt_check(x->ndim() == 4 && f->ndim() == 4 && f->shape()[1] == s[1] && f->shape()[2] == cl->kernel_h &&
                          f->shape()[3] == cl->kernel_w && write->size() == s[0] * L * m * n && (!bias || bias->size() == L),
                          "ConvPatchForward: filters, bias or output do not fit the input");
                if (cgtGlobalStatus != cgtStatusOK) return;
                int rc = cgt_amd_conv_patch_fwd_f32((const float*)x->data(), (const float*)f->data(),
                    bias ? (const float*)bias->data() : NULL, cl->relu, s[0], s[1], s[2], s[3], L, """ + _PATCH_GEOM + r""",
                    (float*)write->data(), mask ? (signed char*)mask->data() : NULL, cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "ConvPatchForward: %s", cgt_amd_last_error());
            }"""
        return core.NativeCompileInfo(code, includes=["cgt_amd.h"], closure_triples=self.get_closure(),
                                      gpu_deref_mask=(True, True) + ((True,) if self.has_bias else ()))


class ConvPatchBackwardData(core.Op):
    """inputs [gy, f, x] -> gcol [B,m,n,Z], the cotangent of the column buffer Im2Col(x) would be (x gives
    the shape only); Col2Im takes it to gx."""
    available_impls = ("native_gpu",)

    def __init__(self, info):
        self.info = info

    def shp_apply(self, inputs):
        B, C, H, W = core.shape(inputs[2])
        m, n = _out_hw(H, W, self.info)
        return [B, m, n, C * self.info.kernel_w * self.info.kernel_h]

    def typ_apply(self, input_types):
        return core.TensorType("f4", 4)

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu"
        code = r"""
            CGT_EXPORT_C void $function(void* cl, cgtArray** reads, cgtArray* write) {
                cgtArray *gy = reads[0], *f = reads[1];
                long B = gy->shape()[0], L = gy->shape()[1], P = gy->shape()[2] * gy->shape()[3];
                long Z = L ? f->size() / L : 0;
                cgt_check(gy->ndim() == 4 && f->shape()[0] == L && f->size() == L * Z && write->size() == B * P * Z,
                          "ConvPatchBackwardData: cotangent, filters or output do not fit");
                if (cgtGlobalStatus != cgtStatusOK) return;
                int rc = cgt_amd_conv_col_bwd_data_f32((const float*)gy->data(), (const float*)f->data(), B, P, Z, L,
                    (float*)write->data(), cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "ConvPatchBackwardData: %s", cgt_amd_last_error());
            }"""
        return core.NativeCompileInfo(code, includes=["cgt_amd.h"], gpu_deref_mask=(True, True, False))


class ConvPatchBackwardFilter(core.Op):
    """inputs [gy, x, f] -> gf (f gives the shape only): ConvColBackwardFilter's sums with the patches read
    from x (equal to it to rounding; bit for bit when both products take the same tile shape)."""
    available_impls = ("native_gpu",)

    def __init__(self, info):
        self.info = info

    def shp_apply(self, inputs):
        return core.shape(inputs[2])

    def typ_apply(self, input_types):
        return core.TensorType("f4", 4)

    def get_closure(self):
        from .im2col import info2closure
        return info2closure(self.info)

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu"
        code = r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtArray* write) {
                cgtArray *gy = reads[0], *x = reads[1], *f = reads[2];
                const long* s = x->shape();
                long L = gy->shape()[1];
                long m = (s[2] + 2*cl->pad_h - cl->kernel_h) / cl->stride_h + 1,
                     n = (s[3] + 2*cl->pad_w - cl->kernel_w) / cl->stride_w + 1;
                cgt_check(gy->ndim() == 4 && gy->shape()[0] == s[0] && gy->shape()[2] == m && gy->shape()[3] == n &&
                          f->size() == L * s[1] * cl->kernel_h * cl->kernel_w && write->size() == f->size(),
                          "ConvPatchBackwardFilter: cotangent or output do not fit the input and the filters");
                if (cgtGlobalStatus != cgtStatusOK) return;
                int rc = cgt_amd_conv_patch_bwd_filter_f32((const float*)gy->data(), (const float*)x->data(),
                    s[0], s[1], s[2], s[3], L, """ + _PATCH_GEOM + r""", (float*)write->data(), cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "ConvPatchBackwardFilter: %s", cgt_amd_last_error());
            }"""
        return core.NativeCompileInfo(code, includes=["cgt_amd.h"], closure_triples=self.get_closure(),
                                      gpu_deref_mask=(True, True, False))


def col_supported(x, f, kernelshape, pad, stride):
    """Whether the products over the column buffer cover a layer of these extents
    (cgt_amd_conv_col_fits); the literal composition has no such limits."""
    from .. import kernels
    return kernels.conv_col_fits(core.shape(x), core.size(f, 0), kernelshape, pad, stride)


def patch_supported(x, kernelshape, pad, stride):
    """Whether the layer is one for the patch-gather products: few input channels (the image is small
    and re-read from cache, and a patch row is a long enough run to gather) and extents the
    32-bit offsets of the gather cover (cgt_amd_conv_patch_supported)."""
    from .. import kernels
    shp = [int(v) for v in core.shape(x)]
    return shp[1] < 16 and kernels.conv_patch_supported(shp, kernelshape, pad, stride)      # (filter count: see nn.conv2d)


def conv_patch(x, f, kernelshape, pad, stride, bias=None, relu=False):
    """conv2d (+ per-channel bias [1,L,1,1]) (+ rectify) with the patches gathered inside the products."""
    from .im2col import Im2ColInfo
    x, f = core.as_node(x), core.as_node(f)
    info = Im2ColInfo(*(tuple(kernelshape) + tuple(pad) + tuple(stride)))
    parents = [x, f] + ([core.as_node(bias)] if bias is not None else [])
    out = core.Result(ConvPatchForward(info, bias is not None, relu), parents)
    return out[0] if relu else out
