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
from .core import (BatchedMul22, MethodNotDefined, Mul22, NativeCallable, NativeCompileInfo, Node, Op,  # noqa: F401
                   Reshape, Result, SrcFile, TensorType, Transport, Transpose, TupleType, as_node,
                   batched_matmul, constant, dot, floatX, grad, reshape, shape, size, to_device,
                   transpose, unpack)
from .gpuarray import GpuArray, empty, to_gpu  # noqa: F401

__all__ = ["nn", "core", "capi", "kernels", "compilation", "rt"]
