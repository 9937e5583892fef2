"""`function(inputs, outputs)`: the nodes that lead from `inputs` to `outputs`,
compiled into an instruction list for the C++ interpreter and replayed without
python in the per-op loop -- the role of cgt.function + the native backend in
the reference (cgt/compilation.py:17-43, 306-380; src/execution.cpp:247-292).

Storage slots follow the reference's instruction set: LoadArgument for the
inputs, Alloc + ReturnByRef for by-reference ops (BuildTup for tuple outputs),
ReturnByVal for Reshape / TupleIndex; leaves that are not inputs (weights,
constants) are bound to their slots once, by reference, so updating a weight
array in place is seen by the next call.

Shapes.  The nodes were evaluated while they were built, but every extent
remembers the expression it came from (core.ShapeInt).  Extents that depend on
an argument are recomputed at every call by Size / integer-op instructions
(by-value closures of the runtime), and Alloc reads its shape from those
slots: one compiled function serves any batch size, and Alloc allocates anew
only when a shape outgrows what it has (src/execution.cpp:251-264 re-allocates
on every change of shape).  The exception is a graph that bakes an extent into
a VALUE (the 1/n of `mean`): such a function accepts the traced shapes only,
and so does one replayed as a HIP graph.

Placement.  Transport nodes are already in the traced graph where an op
dereferences, on the GPU, a parent that lives on the host (core.add_transports
applies the ops' gpu_deref_mask); here each becomes Alloc + ReturnByRef of the
copy closure.  An input that lives on the device may be handed over as a device
array (no copy) or as a numpy array: its LoadArgument is followed by an
argument-transport instruction that passes a device array through and copies a
host one (cgt_copy_object) into a buffer it keeps.

Updates.  `updates=[(param, new)]` leaves `new` in the parameter's own storage
(the reference gives both the same memory owner, cgt/compilation.py:150-163).
The producing op writes there directly -- as the last instructions, after every
reader of the old value -- when that is safe: it is elementwise, nothing else
reads `new`, and it reads no other parameter that is being updated.  Otherwise
`new` is computed in place in the graph like any node, so its readers see the
new value, and a copy into the parameter is appended at the end.
"""
import ctypes

import numpy as np

from . import core, rt
from .gpuarray import GpuArray

_INTOPS = {"+": 0, "-": 1, "*": 2, "//": 3, "ceildiv": 4, "neg": 5}


class _SizeClosure(ctypes.Structure):
    _fields_ = [("axis", ctypes.c_int)]


class _IntOpClosure(ctypes.Structure):
    _fields_ = [("op", ctypes.c_int)]


class _RtCallable(object):
    """A closure exported by the runtime library itself (shape arithmetic)."""

    def __init__(self, symbol, cldata):
        self.fptr_address = ctypes.cast(getattr(rt.lib(), symbol), ctypes.c_void_p).value
        self.cldata = cldata
        self.closure_address = ctypes.addressof(cldata)


def _expr_key(expr):
    if expr[0] == "const":
        return expr
    if expr[0] == "size":
        return ("size", id(expr[1]), expr[2])
    return (expr[0],) + tuple(_expr_key(e) for e in expr[1:])


class _Plan(object):
    """The instruction list of a function."""

    def __init__(self, fn):
        self.steps = []
        self.n_slots = 0
        self.slot_of = {}
        self._expr_slots = {}
        self._consts = {}
        self.fn = fn
        self._build()

    def new_slot(self):
        self.n_slots += 1
        return self.n_slots - 1

    def const_slot(self, v):
        v = int(v)
        if v not in self._consts:
            self._consts[v] = self.new_slot()
            self.steps.append(("set", self._consts[v], v))
        return self._consts[v]

    def expr_slot(self, expr):
        """Slot that holds the value of a shape expression as an int64 host scalar."""
        fn = self.fn
        if expr[0] == "const":
            return self.const_slot(expr[1])
        key = _expr_key(expr)
        if key in self._expr_slots:
            return self._expr_slots[key]
        if expr[0] == "size":
            node, axis = expr[1], expr[2]
            if id(node) not in fn._input_index or not fn.shape_generic:
                s = self.const_slot(node.value.shape[axis])
            else:
                s = self.new_slot()
                call = _RtCallable("cgt_rt_op_size", _SizeClosure(axis))
                self.steps.append(("byval", call, [self.arg_slot[fn._input_index[id(node)]]], (s, rt.CPU)))
        elif not fn.shape_generic or not any(id(n) in fn._input_index for n in core.shape_depends_on(expr)):
            s = self.const_slot(_eval_expr(expr))
        else:
            reads = [(self.expr_slot(e), rt.CPU) for e in expr[1:]]
            s = self.new_slot()
            call = _RtCallable("cgt_rt_op_intop", _IntOpClosure(_INTOPS[expr[0]]))
            self.steps.append(("byval", call, reads, (s, rt.CPU)))
        self._expr_slots[key] = s
        return s

    def shape_locs(self, shape_sym):
        return [(self.expr_slot(core.ShapeInt._lift(d).expr), rt.CPU) for d in shape_sym]

    def _build(self):
        fn = self.fn
        transport = core.get_callable(core.Transport("gpu"), [core.TensorType("f4", 1)], "gpu")
        dev = lambda value: rt.GPU if isinstance(value, GpuArray) else rt.CPU      # noqa: E731
        # ---- arguments first: LoadArgument; an input that lives on the device is followed by
        #      an argument transport (a device array passes through, a host array is copied)
        self.arg_slot = {}
        for i, n in enumerate(fn.inputs):
            where = dev(n.value)
            s = (self.new_slot(), where)
            self.steps.append(("arg", i, s))
            self.arg_slot[i] = s
            if where == rt.GPU:
                w = (self.new_slot(), rt.GPU)
                self.steps.append(("argtransport", s, w))
                s = w
            self.slot_of[id(n)] = s
        # ---- the nodes
        slot_of = self.slot_of
        deferred, copies = [], []
        for n in fn._order:
            if id(n) in slot_of:
                continue
            if n.op is None:
                if n.scalar_expr is not None:
                    slot_of[id(n)] = (self.expr_slot(n.scalar_expr), rt.CPU)
                else:
                    s = self.new_slot()
                    slot_of[id(n)] = (s, dev(n.value))
                    self.steps.append(("set", s, n.value))
                continue
            reads = [slot_of[id(p)] for p in n.parents]
            types = [p.typ for p in n.parents]
            if "native_gpu" not in n.op.available_impls:
                raise core.MethodNotDefined("%s has no native implementation and cannot be part of a compiled "
                                            "function" % n.op)
            call = core.get_callable(n.op, types, "gpu")
            if n.op.return_type == "byval":
                w = (self.new_slot(), dev(n.value))
                self.steps.append(("byval", call, reads, w))
                slot_of[id(n)] = w
                continue
            tag = "transport" if isinstance(n.op, core.Transport) else "op"
            if isinstance(n.typ, core.TupleType):
                members = []
                for t, v, shp in zip(n.typ.eltypes, n.value, n.shape_sym):
                    m = (self.new_slot(), dev(v))
                    self.steps.append(("alloc", np.dtype(t.dtype), self.shape_locs(shp), m))
                    members.append(m)
                w = (self.new_slot(), members[0][1])
                self.steps.append(("tup", members, w))
            elif id(n) in fn._inplace_update:
                target = slot_of[id(fn._inplace_update[id(n)])]
                deferred.append(("byref", call, reads, target, tag))
                slot_of[id(n)] = target
                continue
            else:
                w = (self.new_slot(), dev(n.value))
                self.steps.append(("alloc", np.dtype(n.typ.dtype), self.shape_locs(n.shape_sym), w))
            self.steps.append(("byref", call, reads, w, tag))
            slot_of[id(n)] = w
        for before, after in fn._copy_updates:
            copies.append(("byref", transport, [slot_of[id(after)]], slot_of[id(before)], "update-copy"))
        self.steps.extend(deferred)
        self.steps.extend(copies)
        # ---- emit
        it = rt.Interpreter(self.n_slots)
        for step in self.steps:
            kind = step[0]
            if kind == "set":
                it.set_slot(step[1], step[2])
            elif kind == "arg":
                it.load_argument(step[1], step[2])
            elif kind == "argtransport":
                it.arg_transport(step[1], step[2])
            elif kind == "alloc":
                it.alloc(step[1], step[2], step[3])
            elif kind == "tup":
                it.build_tup(step[1], step[2])
            elif kind == "byref":
                it.return_byref(step[1], step[2], step[3])
            elif kind == "byval":
                it.return_byval(step[1], step[2], step[3])
        self.it = it
        self.out_slots = [slot_of[id(o)][0] for o in fn.outputs]
        self.n_instructions = sum(1 for s in self.steps if s[0] != "set")
        self.n_transports = sum(1 for s in self.steps if s[0] == "byref" and s[4] == "transport")
        self.n_arg_transports = sum(1 for s in self.steps if s[0] == "argtransport")
        self.n_shape_instructions = sum(1 for s in self.steps if s[0] == "byval" and isinstance(s[1], _RtCallable))


def _eval_expr(expr):
    """Value of a shape expression from the traced shapes."""
    k = expr[0]
    if k == "const":
        return expr[1]
    if k == "size":
        return int(expr[1].value.shape[expr[2]])
    a = _eval_expr(expr[1])
    if k == "neg":
        return -a
    b = _eval_expr(expr[2])
    if k == "+":
        return a + b
    if k == "-":
        return a - b
    if k == "*":
        return a * b
    if k == "//":
        return a // b
    if k == "ceildiv":
        return max(0, -((-a) // b))
    raise ValueError("unknown shape expression %r" % (k,))


class Function(object):
    def __init__(self, inputs, outputs, device_outputs=False, updates=None, use_graph=False):
        self._single = isinstance(outputs, core.Node)
        # use_graph: the instruction list is recorded once into a HIP graph (on a
        # stream of its own) and replayed with one launch per call; arguments are
        # copied into fixed staging buffers because device addresses are baked in.
        self.use_graph = use_graph
        self._graph = self._stream = None
        self._staging = None
        self.sync = True      # graph mode: wait for the replay before returning
        self.inputs = [core.as_node(i) for i in inputs]
        self.outputs = [outputs] if self._single else list(outputs)
        self.device_outputs = device_outputs
        updates = list(updates.items()) if isinstance(updates, dict) else list(updates or [])
        for before, after in updates:
            if before.op is not None:
                raise ValueError("the left-hand side of an update must be a leaf node (a parameter)")
            if after.op is None or isinstance(after.typ, core.TupleType):
                raise ValueError("the right-hand side of an update must be the result of an op")
            if tuple(after.shape) != tuple(before.shape) or after.typ != before.typ:
                raise ValueError("update changes the parameter's shape or type")
            if before.devtype != after.devtype:
                raise ValueError("update moves the parameter to another device")
        for n in self.inputs:
            if n.op is not None:
                raise ValueError("function inputs must be leaf nodes")
        order, seen = [], set()

        def visit(n):
            if id(n) in seen:
                return
            seen.add(id(n))
            for p in n.parents:
                visit(p)
            order.append(n)

        for o in self.outputs:
            visit(o)
        for before, after in updates:
            visit(before)
            visit(after)
        self._order = order
        self._input_index = {id(n): i for i, n in enumerate(self.inputs)}
        # ---- which updates may write straight into the parameter (see the module docstring)
        consumers = {}
        for n in order:
            for p in n.parents:
                consumers.setdefault(id(p), []).append(n)
        targets = {id(before) for before, _ in updates}
        self._inplace_update, self._copy_updates = {}, []
        for before, after in updates:
            elementwise = isinstance(after.op, (core.ElwiseBinary, core.ElwiseUnary))
            reads_other_target = any(id(p) in targets and p is not before for p in after.parents)
            is_output = any(o is after for o in self.outputs)
            if (elementwise and not consumers.get(id(after)) and not reads_other_target and not is_output
                    and id(after) not in self._inplace_update):
                self._inplace_update[id(after)] = before
            else:
                self._copy_updates.append((before, after))
        # ---- shape-generic unless an extent that depends on an argument was baked into a value
        self.shape_generic = not use_graph
        for n in order:
            if getattr(n, "shape_baked", False) and any(
                    id(d) in self._input_index for d in core.shape_depends_on(n.baked_expr)):
                self.shape_generic = False
        self._arg_specs = [(tuple(int(d) for d in n.value.shape), n.typ.dtype, isinstance(n.value, GpuArray))
                           for n in self.inputs]
        plan = self._plan = _Plan(self)
        self._it = plan.it
        self._out_slots = plan.out_slots
        self.n_instructions = plan.n_instructions
        self.n_transports = plan.n_transports
        self.n_arg_transports = plan.n_arg_transports
        self.n_shape_instructions = plan.n_shape_instructions

    def plan_steps(self):
        """The instruction list as (kind, ...) tuples, for inspection."""
        return list(self._plan.steps)

    def __call__(self, *args):
        if len(args) != len(self.inputs):
            raise TypeError("expected %d arguments, got %d" % (len(self.inputs), len(args)))
        vals = []
        for i, (a, (shape, dtype, on_gpu)) in enumerate(zip(args, self._arg_specs)):
            if isinstance(a, core.Node):
                a = a.value
            if not isinstance(a, GpuArray):
                # a host array: LoadArgument takes a view of it; if the input lives on the
                # device the argument transport behind it makes the copy
                a = np.require(a, dtype=np.dtype(dtype), requirements="C")
            elif not on_gpu:
                raise ValueError("argument %d lives on the device; this function was compiled for a host array" % i)
            if len(a.shape) != len(shape) or (not self.shape_generic and tuple(a.shape) != shape):
                raise ValueError("argument has shape %s; this function was compiled for %s"
                                 % (tuple(a.shape), shape if not self.shape_generic else "%d-d arrays" % len(shape)))
            vals.append(a)
        plan = self._plan
        if self.use_graph:
            from .gpuarray import to_gpu
            uploaded = [on_gpu and not isinstance(v, GpuArray) for v, (_s, _d, on_gpu) in zip(vals, self._arg_specs)]
            vals = [to_gpu(v) if up else v for v, up in zip(vals, uploaded)]
            self._run_graph(vals)
            if any(uploaded):       # the staging copies read temporaries that die with this call
                self._stream.synchronize()
        else:
            plan.it.run(vals)
        outs = [plan.it.get_array(s) for s in plan.out_slots]
        if not self.device_outputs:
            outs = [tuple(m.get() if isinstance(m, GpuArray) else m for m in o) if isinstance(o, tuple)
                    else (o.get() if isinstance(o, GpuArray) else o) for o in outs]
        return outs[0] if self._single else outs

    def _run_graph(self, vals):
        from . import capi
        from .gpuarray import GpuArray as GA, empty
        if self._stream is None:
            self._stream = capi.Stream()
            self._staging = [empty(v.shape, v.dtype) if isinstance(v, GA) else None for v in vals]
        staged = []
        for v, s in zip(vals, self._staging):
            if s is None:
                staged.append(v)              # host operand (shape integers): read at capture time
            else:
                if v.ptr != s.ptr:      # on the graph's own stream: ordered before the replay, no host wait
                    capi.check(capi.lib().cgt_amd_memcpy_async(capi.GPU, capi.GPU, s.ptr, v.ptr, s.nbytes, self._stream.handle))
                staged.append(s)
        rt.set_stream(self._stream.handle)
        try:
            if self._graph is None:
                # first call: run for real (this also grows workspaces and allocates
                # the output buffers), then record the same sequence without running it
                self._it.run(staged)
                self._stream.synchronize()
                self._graph = capi.Graph.capture(self._stream, lambda: self._it.run(staged))
            else:
                self._graph.launch()
                if self.sync:
                    self._stream.synchronize()
        finally:
            rt.set_stream(None)


def function(inputs, outputs, device_outputs=False, updates=None, use_graph=False):
    """Compile the nodes between `inputs` and `outputs` (reference cgt.function).
    Results come back as numpy arrays, like the reference's; with
    device_outputs=True they are device arrays that view the function's own
    buffers and are overwritten by its next call.  `updates` is a list of
    (parameter, new value) pairs applied in place at the end of every call.
    use_graph=True records the instruction list into a HIP graph on the first
    call and replays it with a single launch afterwards (for launch-bound graphs
    of small kernels; such a function is tied to the traced shapes)."""
    return Function(inputs, outputs, device_outputs, updates, use_graph)
