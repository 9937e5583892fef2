"""cgt_amd: the native CNN hot path of CGT (im2col/col2im, Mul22/BatchedMul22,
max-pool with argmax, cross-channel LRN) on an MI355X, behind CGT's Op API.

    import cgt_amd as cgt
    from cgt_amd import nn
    y = nn.conv2d(cgt.constant(x), cgt.constant(f), kernelshape=(3, 3), pad=(1, 1))
    gx, gf = cgt.grad(y, [x_node, f_node], goutput=gy)

There is no CPU fallback: the HIP library must be built (python -m cgt_amd.build)
and a GPU visible, or calls raise.
"""
from . import capi  # noqa: F401
from .core import (BatchedMul22, ElwiseBinary, ElwiseUnary, Fill, MethodNotDefined, Mul22,  # noqa: F401
                   NativeCallable, NativeCompileInfo, Node, Op, Repeat, Reshape, Result, SrcFile, Sum,
                   TensorType, Transport, Transpose, TupleType, abs, as_node, batched_matmul, broadcast,
                   constant, cos, dot, elwise_binary, exp, fill, floatX, grad, greater_equal, log, mean,
                   neg, ones, ones_like, power, reshape, shape, sigmoid, sign, sin, size, sqrt, square,
                   sum, tanh, to_device, transpose, unpack, zeros, zeros_like)
from .function import Function, function  # noqa: F401
from .gpuarray import GpuArray, empty, to_gpu  # noqa: F401

__all__ = ["nn", "core", "capi", "kernels", "compilation", "rt"]
