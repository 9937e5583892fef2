"""Cross-channel LRN ops (reference cgt/nn_ops/cross_channel_lrn.py).

The closure keeps the reference's fields (localsize, alpha, beta) and adds
`k`, the additive constant of the scale, which the reference fixes at 1
(include/lrn.cuh:27); k = 1 is therefore reference behaviour.
"""
import ctypes
from collections import namedtuple

from .. import core

LRNInfo = namedtuple("LRNInfo", ["localsize", "alpha", "beta"])


def make_closure(info, k=1.0):
    return [
        ("localsize", ctypes.c_int, info.localsize),
        ("alpha", ctypes.c_double, info.alpha),
        ("beta", ctypes.c_double, info.beta),
        ("k", ctypes.c_double, k),
    ]


class CrossChannelLRNForward(core.Op):
    available_impls = ("native_gpu",)

    def __init__(self, info, k=1.0):
        assert isinstance(info, LRNInfo)
        self.info = info
        self.k = float(k)

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu" and input_types[0].dtype == "f4"
        code = r"""
            CGT_EXPORT_C void $function($closure* cldata, cgtArray** reads, cgtTuple* write) {
                cgtArray* X = reads[0];
                long num_img = X->shape()[0],
                     channels = X->shape()[1],
                     height = X->shape()[2],
                     width = X->shape()[3];
                cgtArray* top = (cgtArray*)write->getitem(0);
                cgtArray* scale = (cgtArray*)write->getitem(1);
                int rc = cgt_amd_lrn_fwd_f32((const float*)X->data(), num_img, channels, height, width,
                    cldata->localsize, cldata->alpha, cldata->beta, cldata->k,
                    (float*)top->data(), (float*)scale->data(), cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "CrossChannelLRNForward: %s", cgt_amd_last_error());
            }"""
        return core.NativeCompileInfo(code, closure_triples=make_closure(self.info, self.k),
                                      includes=["cgt_amd.h"], gpu_deref_mask=(True,))

    def shp_apply(self, inputs):
        return (core.shape(inputs[0]), core.shape(inputs[0]))

    def typ_apply(self, input_types):
        return core.TupleType(input_types[0], input_types[0])

    def pullback(self, inputs, output, gout):
        top, scaling = core.unpack(output)
        gtop, _ = gout
        return [core.Result(CrossChannelLRNBackward(self.info), [inputs[0], top, scaling, gtop])]


class CrossChannelLRNBackward(core.Op):
    available_impls = ("native_gpu",)

    def __init__(self, info):
        self.info = info

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu" and input_types[0].dtype == "f4"
        code = r"""
            CGT_EXPORT_C void $function($closure* cldata, cgtArray** reads, cgtArray* bottom_diff) {
                // reads[1], the forward op's `top`, is not read: top = X * scaling^-beta is formed
                // again from X and scaling with the forward kernel's own operations (same bits)
                cgtArray *X=reads[0], *scaling=reads[2], *top_diff=reads[3];
                long num_img = X->shape()[0],
                     channels = X->shape()[1],
                     height = X->shape()[2],
                     width = X->shape()[3];
                cgt_check(scaling->size() == X->size() && top_diff->size() == X->size() && bottom_diff->size() == X->size(),
                          "CrossChannelLRNBackward: operands do not share the input's shape");
                if (cgtGlobalStatus != cgtStatusOK) return;
                int rc = cgt_amd_lrn_bwd_recompute_f32((const float*)X->data(),
                    (const float*)scaling->data(), (const float*)top_diff->data(),
                    num_img, channels, height, width, cldata->localsize, cldata->alpha, cldata->beta,
                    (float*)bottom_diff->data(), cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "CrossChannelLRNBackward: %s", cgt_amd_last_error());
            }"""
        return core.NativeCompileInfo(code, closure_triples=make_closure(self.info),
                                      includes=["cgt_amd.h"], gpu_deref_mask=(True, False, True, True))

    def shp_apply(self, inputs):
        return core.shape(inputs[0])

    def typ_apply(self, _inputs):
        return core.TensorType(core.floatX, 4)


class CrossChannelLRNTop(core.Op):
    """top of CrossChannelLRNForward alone.  cross_channel_lrn() hands out only `top`
    (reference cgt/nn_ops/cross_channel_lrn.py:106-108), so the scale array has no reader but the
    gradient, which forms it again from X (CrossChannelLRNBackwardFromX): a third of the
    forward's traffic and two fifths of the backward's are not moved."""
    available_impls = ("native_gpu",)

    def __init__(self, info, k=1.0):
        assert isinstance(info, LRNInfo)
        self.info = info
        self.k = float(k)

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu" and input_types[0].dtype == "f4"
        code = r"""
            CGT_EXPORT_C void $function($closure* cldata, cgtArray** reads, cgtArray* top) {
                cgtArray* X = reads[0];
                cgt_check(top->size() == X->size(), "CrossChannelLRNTop: the output does not have the input's shape");
                if (cgtGlobalStatus != cgtStatusOK) return;
                int rc = cgt_amd_lrn_fwd_f32((const float*)X->data(), X->shape()[0], X->shape()[1], X->shape()[2], X->shape()[3],
                    cldata->localsize, cldata->alpha, cldata->beta, cldata->k, (float*)top->data(), NULL, cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "CrossChannelLRNTop: %s", cgt_amd_last_error());
            }"""
        return core.NativeCompileInfo(code, closure_triples=make_closure(self.info, self.k),
                                      includes=["cgt_amd.h"], gpu_deref_mask=(True,))

    def shp_apply(self, inputs):
        return core.shape(inputs[0])

    def typ_apply(self, input_types):
        return input_types[0]

    def pullback(self, inputs, output, gout):
        return [core.Result(CrossChannelLRNBackwardFromX(self.info, self.k), [inputs[0], gout])]


class CrossChannelLRNBackwardFromX(core.Op):
    """CrossChannelLRNBackward from X and the cotangent alone."""
    available_impls = ("native_gpu",)

    def __init__(self, info, k=1.0):
        self.info = info
        self.k = float(k)

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu" and input_types[0].dtype == "f4"
        code = r"""
            CGT_EXPORT_C void $function($closure* cldata, cgtArray** reads, cgtArray* bottom_diff) {
                cgtArray *X=reads[0], *top_diff=reads[1];
                cgt_check(top_diff->size() == X->size() && bottom_diff->size() == X->size(),
                          "CrossChannelLRNBackwardFromX: operands do not share the input's shape");
                if (cgtGlobalStatus != cgtStatusOK) return;
                int rc = cgt_amd_lrn_bwd_from_x_f32((const float*)X->data(), (const float*)top_diff->data(),
                    X->shape()[0], X->shape()[1], X->shape()[2], X->shape()[3], cldata->localsize, cldata->alpha,
                    cldata->beta, cldata->k, (float*)bottom_diff->data(), cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "CrossChannelLRNBackwardFromX: %s", cgt_amd_last_error());
            }"""
        return core.NativeCompileInfo(code, closure_triples=make_closure(self.info, self.k),
                                      includes=["cgt_amd.h"], gpu_deref_mask=(True, True))

    def shp_apply(self, inputs):
        return core.shape(inputs[0])

    def typ_apply(self, _inputs):
        return core.TensorType(core.floatX, 4)


# True: cross_channel_lrn() builds CrossChannelLRNTop; False: the reference's tuple-valued op
STORE_TOP_ONLY = True


def cross_channel_lrn(X, localsize, alpha, beta, k=1.0):
    X = core.as_node(X)
    assert X.ndim == 4
    info = LRNInfo(localsize, alpha, beta)
    if STORE_TOP_ONLY:
        return core.Result(CrossChannelLRNTop(info, k), [X])
    return core.Result(CrossChannelLRNForward(info, k), [X])[0]
