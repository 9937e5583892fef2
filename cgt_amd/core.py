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


# ================================================================ symbolic extents

class ShapeInt(int):
    """An array extent that remembers how it was computed.

    The reference derives every shape symbolically (Size ops and integer
    arithmetic over them, cgt/core.py:1614-1640 and the shp_apply rules), so a
    compiled function serves any batch size.  Nodes here are evaluated while
    they are built, so an extent is a concrete python int -- this subclass --
    that also carries its expression:
        ("const", v) | ("size", node, axis) | (op, a, b) with op in + - * // ceildiv | ("neg", a)
    `function` turns the expressions that depend on its arguments into
    Size / integer-op instructions; everywhere else a ShapeInt is just an int.
    """

    def __new__(cls, value, expr=None):
        self = int.__new__(cls, value)
        self.expr = ("const", int(value)) if expr is None else expr
        return self

    @staticmethod
    def _expr(v):
        return v.expr if isinstance(v, ShapeInt) else ("const", int(v))

    def _bin(self, other, op, value, swap=False):
        if not isinstance(other, (int, np.integer)) or isinstance(other, bool):
            return NotImplemented
        a, b = (ShapeInt._expr(other), self.expr) if swap else (self.expr, ShapeInt._expr(other))
        if a[0] == "const" and b[0] == "const":
            return ShapeInt(value)
        return ShapeInt(value, (op, a, b))

    def __add__(self, o):
        return self._bin(o, "+", int(self) + int(o)) if isinstance(o, (int, np.integer)) else NotImplemented

    def __radd__(self, o):
        return self._bin(o, "+", int(o) + int(self), True) if isinstance(o, (int, np.integer)) else NotImplemented

    def __sub__(self, o):
        return self._bin(o, "-", int(self) - int(o)) if isinstance(o, (int, np.integer)) else NotImplemented

    def __rsub__(self, o):
        return self._bin(o, "-", int(o) - int(self), True) if isinstance(o, (int, np.integer)) else NotImplemented

    def __mul__(self, o):
        return self._bin(o, "*", int(self) * int(o)) if isinstance(o, (int, np.integer)) else NotImplemented

    def __rmul__(self, o):
        return self._bin(o, "*", int(o) * int(self), True) if isinstance(o, (int, np.integer)) else NotImplemented

    def __floordiv__(self, o):
        return self._bin(o, "//", int(self) // int(o)) if isinstance(o, (int, np.integer)) else NotImplemented

    def __rfloordiv__(self, o):
        return self._bin(o, "//", int(o) // int(self), True) if isinstance(o, (int, np.integer)) else NotImplemented

    def __neg__(self):
        return ShapeInt(-int(self), None if self.expr[0] == "const" else ("neg", self.expr))

    def is_constant(self):
        return self.expr[0] == "const"

    @staticmethod
    def _lift(v):
        return v if isinstance(v, ShapeInt) else ShapeInt(int(v))

    def __reduce__(self):
        return (int, (int(self),))


def ceil_divide(x, y):
    """max(0, iceil(x / y)), the pooled-extent rule (reference cgt/api.py:145-146 as
    MaxPool.shp_apply uses it), symbolic when an operand is."""
    v = max(0, -((-int(x)) // int(y)))
    a, b = ShapeInt._expr(x), ShapeInt._expr(y)
    if a[0] == "const" and b[0] == "const":
        return ShapeInt(v)
    return ShapeInt(v, ("ceildiv", a, b))


def shape_depends_on(expr, out=None):
    """The nodes whose extents a shape expression reads."""
    out = [] if out is None else out
    if expr[0] == "size":
        out.append(expr[1])
    elif expr[0] != "const":
        for sub in expr[1:]:
            shape_depends_on(sub, out)
    return out


# ================================================================ nodes

class Node(object):
    """A value together with how it was made (op, parents)."""

    def __init__(self, typ, op, parents, value, name=None, shape_sym=None, scalar_expr=None):
        self.typ, self.op, self.parents, self.value, self.name = typ, op, list(parents), value, name
        # extents as ShapeInts (a tuple of such lists for a tuple-valued node); None: taken
        # from the value, each extent then reads "size of this node along that axis"
        self.shape_sym = shape_sym
        # for an int64 scalar leaf that stands for an extent: the expression it came from
        self.scalar_expr = scalar_expr
        # a constant whose VALUE was computed from an extent (e.g. the 1/n of a mean): a
        # compiled function that contains it is tied to the shapes it was traced with
        self.shape_baked = False

    @property
    def ndim(self):
        return self.typ.ndim

    @property
    def dtype(self):
        return self.typ.dtype

    @property
    def shape(self):
        """Extents as ShapeInts (plain ints to every consumer that does not care)."""
        if self.shape_sym is not None and not isinstance(self.typ, TupleType):
            return tuple(self.shape_sym)
        if isinstance(self.typ, TupleType):
            raise TypeError("a tuple-valued node has no single shape")
        return tuple(ShapeInt(d, ("size", self, i)) for i, d in enumerate(self.value.shape))

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

    # arithmetic and comparisons build ElwiseBinary / ElwiseUnary results
    # (reference core.py:204-262)
    def __neg__(self):
        return Result(ElwiseUnary("neg"), [self])

    def __add__(self, other):
        return elwise_binary("+", self, other)

    def __sub__(self, other):
        return elwise_binary("-", self, other)

    def __mul__(self, other):
        return elwise_binary("*", self, other)

    def __truediv__(self, other):
        return elwise_binary("/", self, other)

    def __pow__(self, other):
        return elwise_binary("**", self, other)

    def __radd__(self, other):
        return elwise_binary("+", other, self)

    def __rsub__(self, other):
        return elwise_binary("-", other, self)

    def __rmul__(self, other):
        return elwise_binary("*", other, self)

    def __rtruediv__(self, other):
        return elwise_binary("/", other, self)

    def __lt__(self, other):
        return elwise_binary("<", self, other)

    def __le__(self, other):
        return elwise_binary("<=", self, other)

    def __gt__(self, other):
        return elwise_binary(">", self, other)

    def __ge__(self, other):
        return elwise_binary(">=", self, other)

    def sum(self, axis=None, keepdims=False):
        return sum(self, axis=axis, keepdims=keepdims)

    __hash__ = object.__hash__

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
    if isinstance(value, ShapeInt):
        # an extent used as an operand (Reshape / Col2Im / Repeat / Fill take their shape
        # operands as int64 host scalars): the node remembers the expression
        return Node(TensorType("i8", 0), None, [], np.array(int(value), np.int64), scalar_expr=value.expr)
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
    """Shape as a list of ShapeInts: python ints that remember the expression they came
    from (the reference returns symbolic scalar nodes)."""
    return list(as_node(x).shape)


def size(x, axis):
    return shape(x)[axis]


def scalar_extent(node):
    """The extent an int64 scalar operand stands for, with its expression."""
    node = as_node(node)
    return ShapeInt(int(np.asarray(node.value)), node.scalar_expr)


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

    def pullback_wanted(self, inputs, output, goutput, wanted):
        """pullback, told which inputs' gradients will be used.  Nodes are
        evaluated as they are built, so an op whose gradient expressions are
        separate kernels overrides this to launch only the wanted ones."""
        return self.pullback(inputs, output, goutput)

    def get_native_compile_info(self, input_types, devtype):
        """Returns NativeCompileInfo."""
        raise MethodNotDefined

    def get_gpu_deref_mask(self, input_types):
        """Which inputs the op's GPU closure dereferences on the device: the
        gpu_deref_mask of its NativeCompileInfo (all of them if it declares none)."""
        mask = self.get_native_compile_info(list(input_types), "gpu").gpu_deref_mask
        return tuple(mask) if mask is not None else (True,) * len(input_types)

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


_DEREF_MASKS = {}


def determine_device(op, parents):
    """Device an op's result lives on (the rule of the reference's determine_devices,
    cgt/compilation.py:45-80, for this build's ops): by-value views and Transport follow
    their definition, every computing op is native_gpu; int64 scalars never reach here --
    they are leaves and stay on the host."""
    if isinstance(op, Transport):
        return op.dev
    if op.return_type == "byval":
        return parents[0].devtype
    return "gpu" if "native_gpu" in op.available_impls else "cpu"


def add_transports(op, parents, devtype):
    """The parents `op` will actually read: a parent that lives on another device than
    the op is replaced by a Transport of it -- but only if the op dereferences that input
    on its own device, which is what its gpu_deref_mask says (reference
    cgt/compilation.py:285-304 ships EVERY cross-device parent and carries the note
    "look at native compilation info, gpu deref mask"; core.py:748 declares the mask).
    Shape operands and repeat counts (mask False) are read in place on the host.  One
    Transport per (node, device), shared by all its consumers, as the reference's
    dev2copy does."""
    if isinstance(op, Transport) or devtype != "gpu":
        return parents
    key = (op.get_hash(), tuple(p.typ for p in parents))
    if key not in _DEREF_MASKS:
        _DEREF_MASKS[key] = op.get_gpu_deref_mask([p.typ for p in parents])
    nci_mask = _DEREF_MASKS[key]
    placed = []
    for p, deref in zip(parents, nci_mask):
        if deref and p.devtype != devtype and not isinstance(p.typ, TupleType):
            copies = p.__dict__.setdefault("_transports", {})
            if devtype not in copies:
                copies[devtype] = Result(Transport(devtype), [p])
            p = copies[devtype]
        placed.append(p)
    return placed


def Result(op, parents):
    """Apply `op` to `parents` now and return the Node that holds the result.
    (In the reference this only builds the graph node, core.py:511-517; device
    placement, the Transports and the Alloc + ReturnByRef pair that runs it come
    from the compilation pipeline.  Here placement happens as the node is built,
    by the same rules, so that the traced graph `function` compiles already has
    its Transport nodes.)"""
    parents = [as_node(p) for p in parents]
    parents = add_transports(op, parents, determine_device(op, parents))
    input_types = [p.typ for p in parents]
    typ = op.typ_apply(input_types)
    shp = op.shp_apply(parents)
    if "python" in op.available_impls and (op.return_type == "byval" or "native_gpu" not in op.available_impls
                                           or isinstance(op, Transport)):
        value = op.get_py_func(input_types)([p.value for p in parents])
    else:
        out = _alloc(typ, shp)
        get_callable(op, input_types, "gpu").call([p.value for p in parents], out)
        value = out
    if isinstance(typ, TupleType):
        shape_sym = tuple([ShapeInt._lift(d) for d in s] for s in shp)
    else:
        shape_sym = [ShapeInt._lift(d) for d in shp]
    return Node(typ, op, parents, value, shape_sym=shape_sym)


class TupleIndex(Op):
    """Member of a tuple-valued node (reference core.py:2420-2442).  Evaluated in
    python while nodes are built; the native by-value closure is what a compiled
    `function` replays."""
    available_impls = ("python", "native_cpu", "native_gpu")
    return_type = "byval"

    def __init__(self, idx):
        self.idx = idx

    def get_native_compile_info(self, input_types, devtype):
        code = r"""
            CGT_EXPORT_C cgtObject* $function($closure* cldata, cgtTuple** reads) {
                return reads[0]->getitem(cldata->idx);
            }"""
        return NativeCompileInfo(code, closure_triples=[("idx", ctypes.c_int, self.idx)])

    def typ_apply(self, input_types):
        return input_types[0][self.idx]

    def shp_apply(self, inputs):
        return list(inputs[0].shape_sym[self.idx])

    def get_py_func(self, input_types):
        return lambda reads: reads[0][self.idx]

    def pullback(self, inputs, output, goutput):
        raise MethodNotDefined("tuple members are differentiated through their producer")


def unpack(node):
    return [Result(TupleIndex(i), [node]) for i in range(len(node.typ))]


# ================================================================ autodiff

def grad(output, wrt, goutput=None):
    """Gradients of <output, goutput> with respect to the nodes in `wrt`, by
    walking back through each op's pullback (the reference's `grad`,
    core.py:633-728).  With `goutput` omitted, `output` must be a scalar cost,
    as in the reference, and its cotangent is 1."""
    if goutput is None:
        output = as_node(output)
        if output.value.size != 1:
            raise ValueError("grad of a non-scalar needs its cotangent (goutput=...)")
        goutput = fill(1.0, shape(output))
    order, seen = [], set()

    def visit(n):
        if id(n) in seen:
            return
        seen.add(id(n))
        for p in n.parents:
            visit(p)
        order.append(n)

    visit(output)
    # nodes whose value depends differentiably on a `wrt` node: only they need a
    # gradient (the reference's differentiably_influenced_by, core.py:620-631)
    active = set(id(w) for w in wrt)
    for node in order:
        if node.op is None:
            continue
        diff = [True] * len(node.parents) if isinstance(node.op, TupleIndex) else node.op.get_diff(len(node.parents))
        if any(d and id(p) in active for p, d in zip(node.parents, diff)):
            active.add(id(node))
    gmap = {id(output): as_node(goutput)}
    for node in reversed(order):
        if node.op is None or id(node) not in active:
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
        wanted = [bool(d) and id(p) in active for p, d in zip(node.parents, node.op.get_diff(len(node.parents)))]
        gins = node.op.pullback_wanted(node.parents, node, g, wanted)
        for p, gp, w in zip(node.parents, gins, wanted):
            if gp is None or not w:
                continue
            gmap[id(p)] = gp if id(p) not in gmap else add(gmap[id(p)], gp)
    return [gmap.get(id(w)) for w in wrt]


def add(a, b):
    """Sum of the gradients reaching a node that feeds several consumers."""
    return elwise_binary("+", a, b)


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
                if (cgtGlobalStatus != cgtStatusOK) return;     // no launch on operands that do not fit
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
                cgt_check(B->shape()[0] == P && C->shape()[0] == P && B->shape()[1+(cl->tB ? 1 : 0)] == K &&
                          A->shape()[1+(cl->tA ? 1 : 0)] == M && B->shape()[1+(cl->tB ? 0 : 1)] == N,
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
    """Axis permutation of an array of up to four axes (reference core.py:1559-1594, cpu-only and of
    any rank there; the conv path transposes 4-d arrays, fewer axes ride along as leading extents of 1)."""
    available_impls = ("native_gpu",)

    def __init__(self, axes):
        self.axes = tuple(int(a) for a in axes)
        if sorted(self.axes) != list(range(len(self.axes))):
            raise ValueError("Transpose: %s is not a permutation of the axes" % (self.axes,))
        if len(self.axes) > 4:
            raise NotImplementedError("Transpose: arrays of more than four axes are not supported on the device")

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
        assert devtype == "gpu" and input_types[0].dtype == "f4"
        if input_types[0].ndim != len(self.axes):
            raise ValueError("Transpose%s applied to an array of %d axes" % (self.axes, input_types[0].ndim))
        triples = [("a%d" % i, ctypes.c_int, a) for i, a in enumerate(self.axes + (0,) * (4 - len(self.axes)))]
        triples.append(("nd", ctypes.c_int, len(self.axes)))
        code = r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtArray* write) {
                cgtArray* in = reads[0];
                const int given[4] = {cl->a0, cl->a1, cl->a2, cl->a3};
                const int nd = cl->nd, lead = 4 - nd;
                cgt_check(in->ndim() == nd && write->size() == in->size(), "Transpose: operand rank or size does not fit");
                if (cgtGlobalStatus != cgtStatusOK) return;
                long shape4[4];
                int axes4[4];
                for (int i = 0; i < 4; ++i) {       // fewer than four axes: leading extents of 1 that stay in place
                    shape4[i] = i < lead ? 1 : in->shape()[i - lead];
                    axes4[i] = i < lead ? i : given[i - lead] + lead;
                }
                int rc = cgt_amd_transpose4_f32((const float*)in->data(), shape4, axes4,
                    (float*)write->data(), cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "Transpose: %s", cgt_amd_last_error());
            }"""
        return NativeCompileInfo(code, includes=["cgt_amd.h"], closure_triples=triples, gpu_deref_mask=(True,))


class Reshape(Op):
    """Zero-copy view with a new shape (reference core.py:1432-1465, a by-value op
    whose result shares the input's data).  Evaluated in python while nodes are
    built; the native by-value closure is what a compiled `function` replays."""
    available_impls = ("python", "native_cpu", "native_gpu")
    return_type = "byval"

    def get_native_compile_info(self, input_types, devtype):
        # the view borrows the input's storage (kept alive by its storage slot);
        # shape operands are host integers
        code = r"""
            CGT_EXPORT_C cgtObject* $function($closure* cldata, cgtArray** reads) {
                cgtArray* in = reads[0];
                long newshape[16];
                long n = 1;
                for (int i = 0; i < cldata->ndim; ++i) {
                    newshape[i] = static_cast<long*>(reads[i + 1]->data())[0];
                    n *= newshape[i];
                }
                cgt_check(n == in->size(), "Reshape: size mismatch (%ld vs %ld)", n, in->size());
                cgtArray* view = new cgtArray(cldata->ndim, newshape, in->dtype(), in->devtype(), in->data(), false);
                view->set_base(in);     // the view keeps the array it shows alive
                return view;
            }"""
        return NativeCompileInfo(code, closure_triples=[("ndim", ctypes.c_int, len(input_types) - 1)],
                                 gpu_deref_mask=(False,) * len(input_types))

    def get_diff(self, num_inputs):
        return [True] + [False] * (num_inputs - 1)

    def typ_apply(self, input_types):
        return TensorType(input_types[0].dtype, len(input_types) - 1)

    def shp_apply(self, inputs):
        return [scalar_extent(s) for s in inputs[1:]]

    def get_py_func(self, input_types):
        def f(reads):
            return reads[0].reshape(tuple(int(np.asarray(s)) for s in reads[1:]))
        return f

    def pullback(self, inputs, _out, gout):
        return [reshape(gout, shape(inputs[0]))] + [None] * (len(inputs) - 1)


class Transport(Op):
    """Copy to another device (reference core.py:1596-1612: cgt_copy_object).  Evaluated
    in python while nodes are built; a compiled `function` replays the native closure
    into an array Alloc'ed on the target device."""
    available_impls = ("python", "native_cpu", "native_gpu")

    def __init__(self, dev):
        assert dev in ("cpu", "gpu")
        self.dev = dev

    def get_hash(self):
        return "Transport"          # one closure serves both directions

    def typ_apply(self, input_types):
        return input_types[0]

    def shp_apply(self, inputs):
        return shape(inputs[0])

    def get_native_compile_info(self, _input_types, _devtype):
        # only ever placed between two different devices (there are no no-op transports)
        code = r"""
            CGT_EXPORT_C void $function(void* cldata, cgtObject** reads, cgtObject* write) {
                cgt_copy_object(write, reads[0]);
            }
            """
        return NativeCompileInfo(code)

    def get_py_func(self, input_types):
        def f(reads):
            v = reads[0]
            if self.dev == "gpu":
                return v if isinstance(v, GpuArray) else to_gpu(v)
            return v.get() if isinstance(v, GpuArray) else v
        return f

    def __repr__(self):
        return "Transport{%s}" % self.dev

    def pullback(self, inputs, _out, gout):
        return [Result(Transport(as_node(inputs[0]).devtype), [gout])]


def reshape(x, shp):
    return Result(Reshape(), [x] + list(shp))


def transpose(x, axes):
    return Result(Transpose(axes), [x])


def dot(a, b):
    return Result(Mul22(False, False), [a, b])


def batched_matmul(a, b):
    return Result(BatchedMul22(False, False), [a, b])


# ================================================================ conv-layer glue ops
#
# The ops either side of conv2d in a training step -- bias add, ReLU, the
# scalar loss, the bias gradient -- as the reference spells them: ElwiseUnary /
# ElwiseBinary over expression tables, Repeat for broadcasting, Sum for
# reductions, Fill for constants.  One compiled closure per op class; the op
# code travels in the closure struct and the closure calls the HIP library.

UnaryInfo = namedtuple("UnaryInfo", ("short", "diff", "gradexpr"))

# reference UNARY_INFO (core.py:1118-1134), the float -> float entries
UNARY_INFO = {
    "abs": UnaryInfo("abs", True, lambda x, y, gy: gy * sign(x)),
    "cos": UnaryInfo("cos", True, lambda x, y, gy: -gy * sin(x)),
    "exp": UnaryInfo("exp", True, lambda x, y, gy: gy * exp(x)),
    "log": UnaryInfo("log", True, lambda x, y, gy: gy / x),
    "neg": UnaryInfo("negative", True, lambda x, y, gy: -gy),
    "sign": UnaryInfo("sign", False, None),
    "sin": UnaryInfo("sin", True, lambda x, y, gy: gy * cos(x)),
    "square": UnaryInfo("square", True, lambda x, y, gy: 2.0 * gy * x),
    "sqrt": UnaryInfo("sqrt", True, lambda x, y, gy: gy / (2.0 * y)),
    "tanh": UnaryInfo("tanh", True, lambda x, y, gy: gy * (1 - square(y))),
    "sigmoid": UnaryInfo("sigmoid", True, lambda x, y, gy: gy * y * (1 - y)),
}
UNARY_CODES = ["abs", "cos", "exp", "log", "neg", "sign", "sin", "square", "sqrt", "tanh", "sigmoid"]

BinaryInfo = namedtuple("BinaryInfo", ("short", "diff", "typeinfo", "gradexpr"))

# reference BINARY_INFO (core.py:1139-1152)
BINARY_INFO = {
    "*": BinaryInfo("multiply", (True, True), "p", lambda x, y, z, gz: [y * gz, x * gz]),
    "+": BinaryInfo("add", (True, True), "p", lambda x, y, z, gz: [gz, gz]),
    "-": BinaryInfo("subtract", (True, True), "p", lambda x, y, z, gz: [gz, -gz]),
    "/": BinaryInfo("divide", (True, True), "f", lambda x, y, z, gz: [gz / y, -gz * z / y]),
    "<": BinaryInfo("less", (False, False), "i1", None),
    ">": BinaryInfo("greater", (False, False), "i1", None),
    "<=": BinaryInfo("less_equal", (False, False), "i1", None),
    ">=": BinaryInfo("greater_equal", (False, False), "i1", None),
    "**": BinaryInfo("power", (True, True), "p", lambda x, y, z, gz: [gz * y * power(x, y - 1), gz * z * log(x)]),
    "==": BinaryInfo("equal", (False, False), "i1", None),
    "!=": BinaryInfo("not_equal", (False, False), "i1", None),
}
BINARY_CODES = ["*", "+", "-", "/", "<", ">", "<=", ">=", "**", "==", "!="]


class ElwiseUnary(Op):
    """Elementwise unary operation (reference core.py:1160-1241)."""
    available_impls = ("native_gpu",)

    def __init__(self, opname):
        self.opname = opname
        self.info = UNARY_INFO[opname]

    def get_diff(self, _):
        return [self.info.diff]

    def __repr__(self):
        return self.info.short

    def pullback(self, inputs, y, gy):
        return [self.info.gradexpr(inputs[0], y, gy)]

    def shp_apply(self, inputs):
        return shape(inputs[0])

    def typ_apply(self, input_types):
        assert input_types[0].dtype == "f4", "unary ops take float32 here"
        return TensorType(floatX, input_types[0].ndim)

    def get_closure(self):
        return [("op", ctypes.c_int, UNARY_CODES.index(self.opname))]

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu"
        code = r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtArray* write) {
                cgtArray* read = reads[0];
                int rc = cgt_amd_elwise_unary_f32(cl->op, read->size(), (const float*)read->data(),
                    (float*)write->data(), cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "ElwiseUnary: %s", cgt_amd_last_error());
            }"""
        return NativeCompileInfo(code, includes=["cgt_amd.h"], closure_triples=self.get_closure(),
                                 gpu_deref_mask=(True,))


def _promote(d0, d1):
    return "f4" if "f4" in (d0, d1) else "i1"


class ElwiseBinary(Op):
    """Elementwise binary operation; scalar_mask says which operand is a 0-d
    array (reference core.py:1243-1378)."""
    available_impls = ("native_gpu",)

    def __init__(self, opname, scalar_mask):
        assert opname in BINARY_INFO
        self.opname = opname
        self.info = BINARY_INFO[opname]
        self.scalar_mask = tuple(bool(m) for m in scalar_mask)

    def get_diff(self, _):
        return list(self.info.diff)

    def __repr__(self):
        return self.info.short

    def pullback(self, inputs, z, gz):
        return self.pullback_wanted(inputs, z, gz, [True, True])

    def pullback_wanted(self, inputs, z, gz, wanted):
        x, y = inputs
        # the table's expressions, one operand at a time so that only the wanted one runs
        exprs = {
            "*": (lambda: y * gz, lambda: x * gz),
            "+": (lambda: gz, lambda: gz),
            "-": (lambda: gz, lambda: -gz),
            "/": (lambda: gz / y, lambda: -gz * z / y),
            "**": (lambda: gz * y * power(x, y - 1), lambda: gz * z * log(x)),
        }[self.opname]
        gin = [e() if w else None for e, w in zip(exprs, wanted)]
        return [None if gv is None else (sum(gv) if (v.ndim == 0 and gv.ndim > 0) else gv)
                for v, gv in zip([x, y], gin)]

    def shp_apply(self, inputs):
        ind4shape = 1 if self.scalar_mask[0] else 0
        if self.scalar_mask == (False, False) and shape(inputs[0]) != shape(inputs[1]):
            raise ValueError("mismatched shapes %s %s. Note that implicit broadcasting isn't allowed. "
                             "Use the broadcast(...) function" % (shape(inputs[0]), shape(inputs[1])))
        return shape(inputs[ind4shape])

    def typ_apply(self, input_types):
        assert ((input_types[0].ndim == 0) == self.scalar_mask[0]) and ((input_types[1].ndim == 0) == self.scalar_mask[1])
        if self.scalar_mask == (False, False):
            assert input_types[0].ndim == input_types[1].ndim
        for t in input_types:
            assert t.dtype in ("f4", "i1"), "elementwise ops take f4 / i1 arrays here, got %s" % t.dtype
        typeinfo = self.info.typeinfo
        if typeinfo == "p":
            out_dtype = _promote(input_types[0].dtype, input_types[1].dtype)
        elif typeinfo == "f":
            out_dtype = floatX
        else:
            out_dtype = typeinfo
        ind4shape = 1 if self.scalar_mask[0] else 0
        return TensorType(out_dtype, input_types[ind4shape].ndim)

    def get_closure(self):
        return [("op", ctypes.c_int, BINARY_CODES.index(self.opname)),
                ("scalar0", ctypes.c_int, int(self.scalar_mask[0])),
                ("scalar1", ctypes.c_int, int(self.scalar_mask[1]))]

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu"
        code = r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtArray* write) {
                long n = reads[cl->scalar0 ? 1 : 0]->size();
                cgt_check(write->size() == n && (cl->scalar0 || cl->scalar1 || reads[1]->size() == n),
                    "Shape error in elementwise binary operation. You might be missing a call to cgt.broadcast(...)");
                if (cgtGlobalStatus != cgtStatusOK) return;     // no launch on operands that do not fit
                int rc = cgt_amd_elwise_binary(cl->op, (int)reads[0]->dtype(), (int)reads[1]->dtype(), n,
                    reads[0]->data(), cl->scalar0, reads[1]->data(), cl->scalar1, write->data(), cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "ElwiseBinary: %s", cgt_amd_last_error());
            }"""
        return NativeCompileInfo(code, includes=["cgt_amd.h"], closure_triples=self.get_closure(),
                                 gpu_deref_mask=(True, True))


class ExtentAsFloat(Op):
    """An int64 host scalar (an extent, or integer arithmetic over extents) as a 0-d float32
    device array.  The reference's cgt.size is a symbolic i8 scalar that elementwise ops
    promote (cgt/core.py:1319-1333, 1614-1640), so `x / cgt.size(x, 0)` is right at any
    shape; here extents are python ints that carry their expression, and this op keeps
    that expression alive inside a compiled function instead of freezing the traced value
    into a constant.  The scalar is read on the host (like the shape operands of Reshape
    and Fill) and written by the fill kernel."""
    available_impls = ("native_gpu",)

    def get_diff(self, num_inputs):
        return [False] * num_inputs

    def __repr__(self):
        return "ExtentAsFloat"

    def pullback(self, inputs, output, goutput):
        raise MethodNotDefined("an extent is not differentiable")

    def shp_apply(self, inputs):
        return []

    def typ_apply(self, input_types):
        assert len(input_types) == 1 and input_types[0].dtype == "i8" and input_types[0].ndim == 0, \
            "ExtentAsFloat takes one integer scalar"
        return TensorType(floatX, 0)

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu"
        code = r"""
            CGT_EXPORT_C void $function(void* cl, cgtArray** reads, cgtArray* write) {
                int rc = cgt_amd_fill_f32((float*)write->data(), (float)reads[0]->at<long>(0), 1, cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "ExtentAsFloat: %s", cgt_amd_last_error());
            }"""
        return NativeCompileInfo(code, includes=["cgt_amd.h"], gpu_deref_mask=(False,))


def extent_as_float(n):
    """float32 scalar node holding the extent `n`; a plain constant when `n` does not depend
    on any array's shape."""
    n = ShapeInt._lift(n)
    if n.is_constant():
        return constant(np.float32(int(n)))
    return Result(ExtentAsFloat(), [constant(n)])


def _scalar_operand(v, like):
    """python numbers become 0-d device arrays of the other operand's float type; an extent
    that depends on an array's shape stays an expression (ExtentAsFloat)."""
    if isinstance(v, Node):
        return v
    if isinstance(v, ShapeInt) and not v.is_constant():
        return extent_as_float(v)
    if isinstance(v, (int, float, np.integer, np.floating)) or (isinstance(v, np.ndarray) and v.ndim == 0):
        return constant(np.float32(v))
    return as_node(v)


def elwise_binary(opname, x, y):
    """reference core.py:1380-1386"""
    x, y = _scalar_operand(x, y), _scalar_operand(y, x)
    scalar_mask = ((x.ndim == 0), (y.ndim == 0))
    if scalar_mask == (False, False):
        assert x.ndim == y.ndim
    return Result(ElwiseBinary(opname, scalar_mask), [x, y])


class Repeat(Op):
    """Blow up singleton axes: inputs (x, count per axis in `axes`), counts are
    host integers (reference core.py:1511-1557, cpu-only there)."""
    available_impls = ("native_gpu",)

    def __init__(self, axes):
        self.axes = tuple(int(a) for a in axes)

    def get_diff(self, num_inputs):
        return [True] + [False] * (num_inputs - 1)

    def __repr__(self):
        return "Repeat{%s}" % ",".join(map(str, self.axes))

    def pullback(self, inputs, output, goutput):
        return [sum(goutput, self.axes, keepdims=True)] + [None] * (len(inputs) - 1)

    def shp_apply(self, inputs):
        out = shape(inputs[0])
        for ax, rep in zip(self.axes, inputs[1:]):
            if out[ax] != 1:
                raise ValueError("Repeat: axis %d has extent %d, not 1" % (ax, out[ax]))
            out[ax] = scalar_extent(rep)
        return out

    def typ_apply(self, input_types):
        assert all(t.dtype == "i8" for t in input_types[1:])
        assert input_types[0].ndim <= 8
        return input_types[0]

    def get_closure(self):
        mask = 0
        for a in self.axes:
            mask |= 1 << a
        return [("axes_mask", ctypes.c_int, mask)]

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu"
        code = r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtArray* write) {
                cgtArray* read = reads[0];
                int nd = read->ndim();
                long oshape[8];
                int rep[8];
                for (int a = 0; a < nd; ++a) {
                    oshape[a] = write->shape()[a];
                    rep[a] = (cl->axes_mask >> a) & 1;
                    cgt_check(rep[a] ? read->shape()[a] == 1 : read->shape()[a] == oshape[a],
                        "Repeat: a repeated axis must have extent 1 and the others the output's extent");
                }
                if (cgtGlobalStatus != cgtStatusOK) return;
                int rc = cgt_amd_repeat(read->data(), cgt_itemsize(read->dtype()), nd, oshape, rep,
                    write->data(), cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "Repeat: %s", cgt_amd_last_error());
            }"""
        return NativeCompileInfo(code, includes=["cgt_amd.h"], closure_triples=self.get_closure(),
                                 gpu_deref_mask=(True,) + (False,) * (len(input_types) - 1))


class Sum(Op):
    """Sum over `axes`, keeping them with extent 1 (reference core.py:1687-1709,
    cpu-only there)."""
    available_impls = ("native_gpu",)

    def __init__(self, axes):
        self.axes = tuple(int(a) for a in axes)

    def get_diff(self, _):
        return [True]

    def __repr__(self):
        return "Sum{%s}" % ",".join(map(str, self.axes))

    def pullback(self, inputs, output, goutput):
        return [Result(Repeat(self.axes), [goutput] + [size(inputs[0], ax) for ax in self.axes])]

    def shp_apply(self, inputs):
        s = shape(inputs[0])
        return [1 if i in self.axes else s[i] for i in range(len(s))]

    def typ_apply(self, input_types):
        assert input_types[0].dtype == "f4" and input_types[0].ndim <= 8
        return input_types[0]

    def get_closure(self):
        mask = 0
        for a in self.axes:
            mask |= 1 << a
        return [("axes_mask", ctypes.c_int, mask)]

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu"
        code = r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtArray* write) {
                cgtArray* read = reads[0];
                int nd = read->ndim();
                int red[8];
                for (int a = 0; a < nd; ++a) red[a] = (cl->axes_mask >> a) & 1;
                int rc = cgt_amd_sum_f32((const float*)read->data(), nd, read->shape(), red,
                    (float*)write->data(), cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "Sum: %s", cgt_amd_last_error());
            }"""
        return NativeCompileInfo(code, includes=["cgt_amd.h"], closure_triples=self.get_closure(),
                                 gpu_deref_mask=(True,))


class Fill(Op):
    """(shape...) -> float32 array filled with `value` (reference core.py:966-1007,
    cpu-only there)."""
    available_impls = ("native_gpu",)

    def __init__(self, value):
        self.value = float(value)

    def get_diff(self, num_inputs):
        return [False] * num_inputs

    def __repr__(self):
        return "Fill{%g}" % self.value

    def pullback(self, inputs, output, goutput):
        raise MethodNotDefined("Fill is not differentiable")

    def shp_apply(self, inputs):
        return [scalar_extent(i) for i in inputs]

    def typ_apply(self, input_types):
        assert all(t.dtype == "i8" and t.ndim == 0 for t in input_types), \
            "Fill Op should have integer scalars as arguments"
        return TensorType(floatX, len(input_types))

    def get_closure(self):
        return [("value", ctypes.c_double, self.value)]

    def get_native_compile_info(self, input_types, devtype):
        assert devtype == "gpu"
        code = r"""
            CGT_EXPORT_C void $function($closure* cl, cgtArray** reads, cgtArray* write) {
                int rc = cgt_amd_fill_f32((float*)write->data(), (float)cl->value, write->size(), cgt_get_stream());
                cgt_check(rc == CGT_AMD_OK, "Fill: %s", cgt_amd_last_error());
            }"""
        return NativeCompileInfo(code, includes=["cgt_amd.h"], closure_triples=self.get_closure(),
                                 gpu_deref_mask=(False,) * len(input_types))


# ---------------------------------------------------------------- functions over the glue ops (reference cgt/api.py)

def _unary(opname):
    def f(x):
        return Result(ElwiseUnary(opname), [x])
    f.__name__ = opname
    f.__doc__ = "elementwise %s (reference cgt/api_autogen.py)" % opname
    return f


abs = _unary("abs")            # noqa: A001  (the reference exports these names)
cos = _unary("cos")
exp = _unary("exp")
log = _unary("log")
neg = _unary("neg")
sign = _unary("sign")
sin = _unary("sin")
square = _unary("square")
sqrt = _unary("sqrt")
tanh = _unary("tanh")
sigmoid = _unary("sigmoid")


def power(x, y):
    return elwise_binary("**", x, y)


def greater_equal(x, y):
    return elwise_binary(">=", x, y)


def broadcast(opname, a, b, bcpat):
    """Elementwise binary op with singleton axes expanded first; bcpat names
    them, e.g. "xxxx,1x11" for activation + bias (reference cgt/api.py:92-120)."""
    x, y = as_node(a), as_node(b)
    xpat, ypat = bcpat.split(",")
    xbcaxes, ybcaxes = [[i for i, letter in enumerate(pat) if letter == "1"] for pat in (xpat, ypat)]
    assert x.ndim == y.ndim
    if xbcaxes:
        x = Result(Repeat(xbcaxes), [x] + [size(y, ax) for ax in xbcaxes])
    if ybcaxes:
        y = Result(Repeat(ybcaxes), [y] + [size(x, ax) for ax in ybcaxes])
    return elwise_binary(opname, x, y)


def _red_axes(axis, ndim):
    if axis is None:
        return list(range(ndim))
    if isinstance(axis, int):
        return [axis]
    return list(axis)


def sum(x, axis=None, keepdims=False):      # noqa: A001
    """Like numpy.sum (reference cgt/api.py:647-659)."""
    x = as_node(x)
    axes = _red_axes(axis, x.ndim)
    if len(axes) == 0:
        return x
    out = Result(Sum(axes), [x])
    if not keepdims:
        out = reshape(out, [size(x, i) for i in range(x.ndim) if i not in axes])
    return out


def mean(x, axis=None, keepdims=False):
    """Like numpy.mean (reference cgt/api.py:470-476)."""
    x = as_node(x)
    axes = _red_axes(axis, x.ndim)
    n = 1
    for ax in axes:
        n *= size(x, ax)
    # the divisor follows the extents at every call of a compiled function
    return sum(x, axis=axes, keepdims=keepdims) / extent_as_float(n)


def fill(val, shp):
    """Array of shape `shp` filled with the scalar `val` (reference cgt/api.py:246-258)."""
    return Result(Fill(val), list(shp))


def zeros(shp):
    return fill(0.0, shp)


def ones(shp):
    return fill(1.0, shp)


def zeros_like(x):
    return zeros(shape(x))


def ones_like(x):
    return ones(shape(x))
