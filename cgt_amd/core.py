"""The Op API of CGT for the native CNN hot path, on an MI355X.

Mirrors the parts of the reference's cgt/core.py the hot path stands on:
  * Op (393-489): available_impls, return_type, shp_apply, typ_apply,
    pullback, get_native_compile_info;
  * NativeCompileInfo / SrcFile / NativeCallable (734-855);
  * the dense-contraction ops Mul22 (2129-2229) and BatchedMul22 (2231-2288),
    Transpose (1559-1594), Reshape (1432-1465) and Transport (1596-1612).

What is NOT here is the symbolic array language around them (graph
simplifier, shape algebra, the other ~40 ops).  Nodes are evaluated as they
are built -- `Result(op, parents)` fires the op's compiled closure at once and
returns a Node holding the device array -- and each Node remembers its op and
parents, so `grad` can walk back through the ops' own `pullback` rules
exactly as the reference's autodiff does (core.py:633-705).

Every op here is `native_gpu`: its closure is C++ host code compiled by the
native-compile step (compilation.py) that unpacks cgtArray arguments and calls
the HIP library through the C ABI of include/cgt_amd.h.
"""
import ctypes
from collections import namedtuple

import numpy as np

from . import rt
from .gpuarray import GpuArray, empty, to_gpu

floatX = "f4"

np2c = {"i1": "int8_t", "i2": "int16_t", "i4": "int32_t", "i8": "int64_t",
        "f4": "float", "f8": "double"}


class MethodNotDefined(Exception):
    pass


# ================================================================ types

class TensorType(object):
    def __init__(self, dtype, ndim):
        self.dtype = np.dtype(dtype).str[1:] if not isinstance(dtype, str) or dtype[0] in "<>=|" else dtype
        self.ndim = int(ndim)

    def __repr__(self):
        return "Tensor{%s,%d}" % (self.dtype, self.ndim)

    def __eq__(self, other):
        return isinstance(other, TensorType) and (self.dtype, self.ndim) == (other.dtype, other.ndim)

    def __hash__(self):
        return hash((self.dtype, self.ndim))


class TupleType(object):
    def __init__(self, *eltypes):
        self.eltypes = tuple(eltypes)

    def __len__(self):
        return len(self.eltypes)

    def __getitem__(self, i):
        return self.eltypes[i]

    def __repr__(self):
        return "Tup(%s)" % ",".join(map(repr, self.eltypes))

    def __eq__(self, other):
        return isinstance(other, TupleType) and self.eltypes == other.eltypes

    def __hash__(self):
        return hash(self.eltypes)


# ================================================================ nodes

class Node(object):
    """A value together with how it was made (op, parents)."""

    def __init__(self, typ, op, parents, value, name=None):
        self.typ, self.op, self.parents, self.value, self.name = typ, op, list(parents), value, name

    @property
    def ndim(self):
        return self.typ.ndim

    @property
    def dtype(self):
        return self.typ.dtype

    @property
    def shape(self):
        return tuple(self.value.shape)

    @property
    def devtype(self):
        return "gpu" if isinstance(self.value, GpuArray) else "cpu"

    def get(self):
        """Value as numpy (device arrays are copied back, synchronously)."""
        v = self.value
        if isinstance(v, tuple):
            return tuple(x.get() if isinstance(x, GpuArray) else np.asarray(x) for x in v)
        return v.get() if isinstance(v, GpuArray) else np.asarray(v)

    def reshape(self, shp):
        return reshape(self, shp)

    def transpose(self, axes):
        return transpose(self, axes)

    def __getitem__(self, i):
        if isinstance(self.typ, TupleType):
            return unpack(self)[i]
        raise TypeError("only tuple-valued nodes can be indexed")

    def __repr__(self):
        return "Node(%s, op=%s)" % (self.typ, self.op)


def _value_type(value):
    if isinstance(value, tuple):
        return TupleType(*map(_value_type, value))
    return TensorType(np.dtype(value.dtype).str[1:], len(value.shape))


def constant(value, devtype=None):
    """A leaf node.  float arrays go to the GPU, integer scalars (shape operands)
    stay on the host, as the reference's device placement keeps them
    (cgt/compilation.py:45-80)."""
    if isinstance(value, Node):
        return value
    if isinstance(value, GpuArray):
        return Node(_value_type(value), None, [], value)
    arr = np.asarray(value)
    if arr.dtype.kind == "f":
        if devtype == "cpu":
            return Node(TensorType("f4", arr.ndim), None, [], arr.astype(np.float32))
        return Node(TensorType("f4", arr.ndim), None, [], to_gpu(arr, np.float32))
    arr = arr.astype(np.int64)
    return Node(TensorType("i8", arr.ndim), None, [], arr)


as_node = constant
to_device = constant


def shape(x):
    """Shape as a list of python ints (the reference returns symbolic scalars)."""
    return [int(s) for s in as_node(x).shape]


def size(x, axis):
    return shape(x)[axis]


# ================================================================ Op base

class Op(object):
    """Describes an operation performed on some data (reference core.py:393-489)."""
    return_type = "byref"        # or "byval"
    writes_to_input = -1
    available_impls = ()         # python, native_cpu, native_gpu
    is_data_op = False
    is_random_op = False

    def shp_apply(self, parents):
        """Output shape(s) as a function of the input nodes."""
        raise NotImplementedError

    def typ_apply(self, parent_types):
        """Output type as a function of the input types."""
        raise NotImplementedError

    def get_diff(self, num_inputs):
        return [True] * num_inputs

    def get_name(self):
        return type(self).__name__

    def get_hash(self):
        return repr(sorted(self.__dict__.items())) + self.__class__.__name__

    def pullback(self, inputs, output, goutput):
        """grad wrt each input given the gradient of the output (J^T g)."""
        raise MethodNotDefined

    def get_native_compile_info(self, input_types, devtype):
        """Returns NativeCompileInfo."""
        raise MethodNotDefined

    def get_py_func(self, input_types):
        raise MethodNotDefined

    def __repr__(self):
        return type(self).__name__


# ================================================================ compilation records

class NativeCompileInfo(object):
    """Everything needed to build a NativeCallable (reference core.py:734-767).

    func_code       code of the exported function, with $function / $closure /
                    $setup / $teardown placeholders
    closure_triples list of (fieldname, ctypes class, value) -> the closure struct
    includes        headers to include after cgt_common.h
    link_flags      extra link flags
    setup/teardown  whether $setup / $teardown functions exist
    gpu_deref_mask  which inputs are dereferenced on the GPU (None: host-only op)
    extra_srcs      list of SrcFile(lang, code), lang in {"c++", "hip"}
    """

    def __init__(self, func_code, closure_triples=None, includes=(), link_flags="",
                 setup=False, teardown=False, gpu_deref_mask=None, store_objects=(), extra_srcs=()):
        self.op_str = None
        self.return_type = None
        self.n_in = None
        self.func_code = func_code
        self.closure_triples = closure_triples
        self.includes = list(includes)
        self.link_flags = link_flags
        self.setup = setup
        self.teardown = teardown
        self.gpu_deref_mask = gpu_deref_mask
        self.store_objects = store_objects
        self.extra_srcs = list(extra_srcs)

    def involves_gpu(self):
        return self.gpu_deref_mask is not None


SrcFile = namedtuple("SrcFile", ["lang", "code"])


class NativeCallable(object):
    """A compiled closure: function pointer + closure struct (reference core.py:816-855)."""

    def __init__(self, n_in, return_type, op_str, fptr, cldata=None, store_objects=None,
                 setup_fptr=None, teardown_fptr=None):
        self._n_in, self._return_type, self._op_str = n_in, return_type, op_str
        self.fptr = fptr
        self.cldata = cldata
        self.store_objects = store_objects
        self.setup_fptr, self.teardown_fptr = setup_fptr, teardown_fptr
        self._kind = "native"
        if setup_fptr is not None:
            setup_fptr(self._cl_ref())

    def _cl_ref(self):
        return ctypes.byref(self.cldata) if self.cldata is not None else None

    def __del__(self):
        if getattr(self, "teardown_fptr", None) is not None:
            self.teardown_fptr(self._cl_ref())

    n_in = property(lambda self: self._n_in)
    return_type = property(lambda self: self._return_type)
    op_str = property(lambda self: self._op_str)
    kind = property(lambda self: self._kind)

    @property
    def fptr_address(self):
        return ctypes.cast(self.fptr, ctypes.c_void_p).value

    @property
    def closure_address(self):
        return ctypes.addressof(self.cldata) if self.cldata is not None else None

    def call(self, inputs, output):
        if self._return_type != "byref":
            raise NotImplementedError("by-value native ops are applied by the interpreter only")
        rt.apply_byref(self.fptr_address, self.cldata, inputs, output)


# ================================================================ evaluation

_CALLABLES = {}


def get_callable(op, input_types, devtype="gpu"):
    """Compile (or fetch) the op's closure (reference cgt/compilation.py:251-283)."""
    from . import compilation
    key = (op.get_hash(), tuple(input_types), devtype)
    if key not in _CALLABLES:
        if "native_" + devtype not in op.available_impls:
            raise MethodNotDefined("%s has no native_%s implementation" % (op, devtype))
        nci = op.get_native_compile_info(list(input_types), devtype)
        nci.op_str, nci.return_type, nci.n_in = str(op), op.return_type, len(input_types)
        _CALLABLES[key] = compilation.nci2callable(nci)
    return _CALLABLES[key]


def _alloc(typ, shp):
    if isinstance(typ, TupleType):
        return tuple(_alloc(t, s) for t, s in zip(typ.eltypes, shp))
    return empty(tuple(int(s) for s in shp), np.dtype(typ.dtype))


def Result(op, parents):
    """Apply `op` to `parents` now and return the Node that holds the result.
    (In the reference this only builds the graph node, core.py:511-517; the
    Alloc + ReturnByRef pair that runs it comes from the compilation pipeline.)"""
    parents = [as_node(p) for p in parents]
    input_types = [p.typ for p in parents]
    typ = op.typ_apply(input_types)
    if "python" in op.available_impls and "native_gpu" not in op.available_impls:
        value = op.get_py_func(input_types)([p.value for p in parents])
    else:
        out = _alloc(typ, op.shp_apply(parents))
        get_callable(op, input_types, "gpu").call([p.value for p in parents], out)
        value = out
    return Node(typ, op, parents, value)


class TupleIndex(Op):
    """Member of a tuple-valued node (reference core.py:2420-2442)."""
    available_impls = ("python",)

    def __init__(self, idx):
        self.idx = idx

    def typ_apply(self, input_types):
        return input_types[0][self.idx]

    def get_py_func(self, input_types):
        return lambda reads: reads[0][self.idx]

    def pullback(self, inputs, output, goutput):
        raise MethodNotDefined("tuple members are differentiated through their producer")


def unpack(node):
    return [Result(TupleIndex(i), [node]) for i in range(len(node.typ))]


# ================================================================ autodiff

def grad(output, wrt, goutput):
    """Gradients of <output, goutput> with respect to the nodes in `wrt`, by
    walking back through each op's pullback (the reference's `grad`,
    core.py:633-728, takes a scalar cost; here the cotangent of `output` is
    given explicitly because the elementwise/reduction ops that would build a
    scalar cost are outside the hot path)."""
    order, seen = [], set()

    def visit(n):
        if id(n) in seen:
            return
        seen.add(id(n))
        for p in n.parents:
            visit(p)
        order.append(n)

    visit(output)
    gmap = {id(output): as_node(goutput)}
    for node in reversed(order):
        if node.op is None:
            continue
        if isinstance(node.op, TupleIndex):
            # route the member's gradient to the producing tuple node
            parent = node.parents[0]
            slot = gmap.setdefault(id(parent), [None] * len(parent.typ))
            g = gmap.get(id(node))
            if g is not None:
                slot[node.op.idx] = g if slot[node.op.idx] is None else add(slot[node.op.idx], g)
            continue
        g = gmap.get(id(node))
        if g is None:
            continue
        gins = node.op.pullback(node.parents, node, g)
        for p, gp, d in zip(node.parents, gins, node.op.get_diff(len(node.parents))):
            if gp is None or not d:
                continue
            gmap[id(p)] = gp if id(p) not in gmap else add(gmap[id(p)], gp)
    return [gmap.get(id(w)) for w in wrt]


def add(a, b):
    raise MethodNotDefined("a node feeding several consumers needs the elementwise add op, "
                           "which is outside the CNN hot path")


# ================================================================ ops

class Mul22(Op):
    """C = op(A) . op(B) on matrices (reference core.py:2129-2229)."""
    available_impls = ("native_gpu",)

    def __init__(self, tA, tB):
        self.tA, self.tB = bool(tA), bool(tB)

    def pullback(self, inputs, output, goutput):
        A, B = inputs
        GC = goutput
        v = (self.tA, self.tB)
        if v == (False, False):
            return [Result(Mul22(False, True), [GC, B]), Result(Mul22(True, False), [A, GC])]
        if v == (False, True):
            return [Result(Mul22(False, False), [GC, B]), Result(Mul22(True, False), [GC, A])]
        if v == (True, False):
            return [Result(Mul22(False, True), [B, GC]), Result(Mul22(False, False), [A, GC])]
        return [Result(Mul22(True, True), [B, GC]), Result(Mul22(True, True), [GC, A])]

    def shp_apply(self, inputs):
        return [size(inputs[0], 1 if self.tA else 0), size(inputs[1], 0 if self.tB else 1)]

    def typ_apply(self, input_types):
        assert input_types[0].dtype == floatX and input_types[1].dtype == floatX
        return input_types[0]

    def get_closure(self):
        return [("tA", ctypes.c_bool, self.tA), ("tB", ctypes.c_bool, self.tB), ("handle", ctypes.c_void_p, 0)]

    def get_native_compile_info(self, input_types, devtype):
        if input_types[0].dtype != "f4":
            raise MethodNotDefined("Dtype %s not supported by this GEMM" % input_types[0].dtype)
        assert devtype == "gpu"
        code = r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** AB, cgtArray* C) {
                cgtArray *A=AB[0], *B=AB[1];
                long lda = A->shape()[1], ldb = B->shape()[1], ldc = C->shape()[1];
                long M = C->shape()[0];
                long N = C->shape()[1];
                long K = A->shape()[cl->tA ? 0 : 1];
                long Kb = B->shape()[cl->tB ? 1 : 0];
                cgt_check(K == Kb && A->shape()[cl->tA ? 1 : 0] == M && B->shape()[cl->tB ? 0 : 1] == N,
                    "shape mismatch at matrix-matrix multiplication");
                if (K != Kb) return;
                int rc = cgt_amd_sgemm(cl->tA, cl->tB, M, N, K, (const float*)A->data(), lda,
                    (const float*)B->data(), ldb, (float*)C->data(), ldc, cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "Mul22: %s", cgt_amd_last_error());
            }
            """
        return NativeCompileInfo(code, includes=["cgt_amd.h"], closure_triples=self.get_closure(),
                                 gpu_deref_mask=(True, True))

    def __repr__(self):
        return "Mul22{%s,%s}" % ("T" if self.tA else "N", "T" if self.tB else "N")


class BatchedMul22(Op):
    """P independent products (reference core.py:2231-2288; no GPU impl exists there)."""
    available_impls = ("native_gpu",)

    def __init__(self, tA, tB):
        self.tA, self.tB = bool(tA), bool(tB)

    def pullback(self, inputs, output, goutput):
        A, B = inputs
        GC = goutput
        v = (self.tA, self.tB)
        if v == (False, False):
            return [Result(BatchedMul22(False, True), [GC, B]), Result(BatchedMul22(True, False), [A, GC])]
        if v == (False, True):
            return [Result(BatchedMul22(False, False), [GC, B]), Result(BatchedMul22(True, False), [GC, A])]
        if v == (True, False):
            return [Result(BatchedMul22(False, True), [B, GC]), Result(BatchedMul22(False, False), [A, GC])]
        return [Result(BatchedMul22(True, True), [B, GC]), Result(BatchedMul22(True, True), [GC, A])]

    def shp_apply(self, inputs):
        return [size(inputs[0], 0), size(inputs[0], 2 if self.tA else 1), size(inputs[1], 1 if self.tB else 2)]

    def typ_apply(self, input_types):
        return input_types[0]

    def get_closure(self):
        return [("tA", ctypes.c_bool, self.tA), ("tB", ctypes.c_bool, self.tB)]

    def get_native_compile_info(self, input_types, devtype):
        if input_types[0].dtype != "f4":
            raise MethodNotDefined("Dtype %s not supported by this GEMM" % input_types[0].dtype)
        assert devtype == "gpu"
        code = r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** AB, cgtArray* C) {
                cgtArray *A=AB[0], *B=AB[1];
                long P = A->shape()[0];
                long lda = A->shape()[2], ldb = B->shape()[2], ldc = C->shape()[2];
                long M = C->shape()[1];
                long N = C->shape()[2];
                long K = A->shape()[1+(cl->tA ? 0 : 1)];
                cgt_check(B->shape()[0] == P && C->shape()[0] == P && B->shape()[1+(cl->tB ? 1 : 0)] == K,
                    "shape mismatch at batched matrix multiplication");
                if (cgtGlobalStatus != cgtStatusOK) return;
                int rc = cgt_amd_sgemm_batched(cl->tA, cl->tB, P, M, N, K,
                    (const float*)A->data(), lda, A->stride(0), (const float*)B->data(), ldb, B->stride(0),
                    (float*)C->data(), ldc, C->stride(0), cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "BatchedMul22: %s", cgt_amd_last_error());
            }
            """
        return NativeCompileInfo(code, includes=["cgt_amd.h"], closure_triples=self.get_closure(),
                                 gpu_deref_mask=(True, True))

    def __repr__(self):
        return "BatchedMul22{%s,%s}" % ("T" if self.tA else "N", "T" if self.tB else "N")


class Transpose(Op):
    """Axis permutation of a 4-d array (reference core.py:1559-1594, cpu-only there)."""
    available_impls = ("native_gpu",)

    def __init__(self, axes):
        self.axes = tuple(int(a) for a in axes)

    def get_diff(self, _):
        return [True]

    def pullback(self, inputs, output, goutput):
        inv = [0] * len(self.axes)
        for i, a in enumerate(self.axes):
            inv[a] = i
        return [transpose(goutput, inv)]

    def shp_apply(self, inputs):
        inshape = shape(inputs[0])
        return [inshape[ax] for ax in self.axes]

    def typ_apply(self, input_types):
        return input_types[0]

    def __repr__(self):
        return "Transpose{%s}" % ",".join(map(str, self.axes))

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu" and input_types[0].ndim == 4 and input_types[0].dtype == "f4"
        triples = [("a%d" % i, ctypes.c_int, a) for i, a in enumerate(self.axes)]
        code = r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtArray* write) {
                cgtArray* in = reads[0];
                int axes[4] = {cl->a0, cl->a1, cl->a2, cl->a3};
                int rc = cgt_amd_transpose4_f32((const float*)in->data(), in->shape(), axes,
                    (float*)write->data(), cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "Transpose: %s", cgt_amd_last_error());
            }"""
        return NativeCompileInfo(code, includes=["cgt_amd.h"], closure_triples=triples, gpu_deref_mask=(True,))


class Reshape(Op):
    """Zero-copy view with a new shape (reference core.py:1432-1465, a by-value op
    whose result shares the input's data)."""
    available_impls = ("python",)
    return_type = "byval"

    def get_diff(self, num_inputs):
        return [True] + [False] * (num_inputs - 1)

    def typ_apply(self, input_types):
        return TensorType(input_types[0].dtype, len(input_types) - 1)

    def get_py_func(self, input_types):
        def f(reads):
            return reads[0].reshape(tuple(int(np.asarray(s)) for s in reads[1:]))
        return f

    def pullback(self, inputs, _out, gout):
        return [reshape(gout, shape(inputs[0]))] + [None] * (len(inputs) - 1)


class Transport(Op):
    """Copy between host and device (reference core.py:1596-1612: cgt_copy_object)."""
    available_impls = ("python",)

    def __init__(self, dev):
        assert dev in ("cpu", "gpu")
        self.dev = dev

    def typ_apply(self, input_types):
        return input_types[0]

    def get_py_func(self, input_types):
        def f(reads):
            v = reads[0]
            if self.dev == "gpu":
                return v if isinstance(v, GpuArray) else to_gpu(v)
            return v.get() if isinstance(v, GpuArray) else v
        return f

    def pullback(self, inputs, _out, gout):
        return [Result(Transport(as_node(inputs[0]).devtype), [gout])]


def reshape(x, shp):
    return Result(Reshape(), [x] + [int(s) for s in shp])


def transpose(x, axes):
    return Result(Transpose(axes), [x])


def dot(a, b):
    return Result(Mul22(False, False), [a, b])


def batched_matmul(a, b):
    return Result(BatchedMul22(False, False), [a, b])
