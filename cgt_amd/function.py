"""`function(inputs, outputs)`: the nodes that lead from `inputs` to `outputs`,
compiled into an instruction list for the C++ interpreter and replayed without
python in the per-op loop -- the role of cgt.function + the native backend in
the reference (cgt/compilation.py:17-43, 306-380; src/execution.cpp:247-292).

The reference derives every output shape symbolically; here the nodes were
evaluated while they were built, so shapes are those of that first evaluation
and a compiled function accepts arguments of exactly those shapes.  Storage
slots follow the reference's instruction set: LoadArgument for the inputs,
Alloc + ReturnByRef for by-reference ops (BuildTup for tuple outputs),
ReturnByVal for Reshape / TupleIndex; leaves that are not inputs (weights,
constants, shape integers) are bound to their slots once, by reference, so
updating a weight array in place is seen by the next call.  Output buffers are
reused from call to call (src/execution.cpp:260-263).
"""
import numpy as np

from . import core, rt
from .gpuarray import GpuArray, to_gpu


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
        # updates: (before, after) pairs; `after` is written straight into the
        # storage of the leaf `before` (the reference gives both the same memory
        # owner, cgt/compilation.py:150-163).  The op that produces `after` is
        # moved to the end of the list so every reader of the old value has run.
        updates = list(updates.items()) if isinstance(updates, dict) else list(updates or [])
        for before, after in updates:
            if before.op is not None:
                raise ValueError("the left-hand side of an update must be a leaf node (a parameter)")
            if after.op is None or after.op.return_type != "byref" or isinstance(after.typ, core.TupleType):
                raise ValueError("the right-hand side of an update must be the result of a by-reference op")
            if tuple(after.shape) != tuple(before.shape) or after.typ != before.typ:
                raise ValueError("update changes the parameter's shape or type")
        update_target = {id(after): before for before, after in updates}
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
        deferred = []        # the ops that write the updates, emitted last
        # ---- slot assignment
        slot_of, n_slots = {}, 0

        def new_slot():
            nonlocal n_slots
            n_slots += 1
            return n_slots - 1

        consts = {}          # shape integers, one slot per distinct value
        plan = []            # deferred emission: needs the interpreter, which needs n_slots

        def const_slot(v):
            v = int(v)
            if v not in consts:
                consts[v] = new_slot()
                plan.append(("set", consts[v], v))
            return consts[v]

        def dev(value):
            return rt.GPU if isinstance(value, GpuArray) else rt.CPU

        input_index = {id(n): i for i, n in enumerate(self.inputs)}
        self._arg_specs = [(tuple(n.shape), n.typ.dtype, isinstance(n.value, GpuArray)) for n in self.inputs]
        for n in order:
            if n.op is None:
                s = new_slot()
                slot_of[id(n)] = (s, dev(n.value))
                if id(n) in input_index:
                    plan.append(("arg", input_index[id(n)], slot_of[id(n)]))
                else:
                    plan.append(("set", s, n.value))
                continue
            reads = [slot_of[id(p)] for p in n.parents]
            types = [p.typ for p in n.parents]
            if n.op.return_type == "byval":
                if "native_gpu" not in n.op.available_impls:
                    raise core.MethodNotDefined("%s cannot be part of a compiled function" % n.op)
                w = (new_slot(), dev(n.value))
                plan.append(("byval", core.get_callable(n.op, types, "gpu"), reads, w))
                slot_of[id(n)] = w
                continue
            if "native_gpu" not in n.op.available_impls:
                raise core.MethodNotDefined("%s has no native implementation and cannot be part of a compiled "
                                            "function" % n.op)
            call = core.get_callable(n.op, types, "gpu")
            if isinstance(n.typ, core.TupleType):
                members = []
                for t, v in zip(n.typ.eltypes, n.value):
                    m = (new_slot(), dev(v))
                    plan.append(("alloc", np.dtype(t.dtype), [(const_slot(d), rt.CPU) for d in v.shape], m))
                    members.append(m)
                w = (new_slot(), members[0][1])
                plan.append(("tup", members, w))
            elif id(n) in update_target:
                deferred.append(("byref", call, reads, slot_of[id(update_target[id(n)])]))
                slot_of[id(n)] = slot_of[id(update_target[id(n)])]
                continue
            else:
                w = (new_slot(), dev(n.value))
                plan.append(("alloc", np.dtype(n.typ.dtype), [(const_slot(d), rt.CPU) for d in n.value.shape], w))
            plan.append(("byref", call, reads, w))
            slot_of[id(n)] = w
        plan.extend(deferred)
        # ---- emit
        it = rt.Interpreter(n_slots)
        for step in plan:
            kind = step[0]
            if kind == "set":
                it.set_slot(step[1], step[2])
            elif kind == "arg":
                it.load_argument(step[1], step[2])
            elif kind == "alloc":
                it.alloc(step[1], step[2], step[3])
            elif kind == "tup":
                it.build_tup(step[1], step[2])
            elif kind == "byref":
                it.return_byref(step[1], step[2], step[3])
            elif kind == "byval":
                it.return_byval(step[1], step[2], step[3])
        self._it = it
        self._out_slots = [slot_of[id(o)][0] for o in self.outputs]
        self.n_instructions = sum(1 for s in plan if s[0] != "set")

    def __call__(self, *args):
        if len(args) != len(self.inputs):
            raise TypeError("expected %d arguments, got %d" % (len(self.inputs), len(args)))
        vals = []
        for a, (shape, dtype, on_gpu) in zip(args, self._arg_specs):
            if isinstance(a, core.Node):
                a = a.value
            if not isinstance(a, GpuArray):
                a = np.asarray(a, dtype=np.dtype(dtype))
                if on_gpu:
                    a = to_gpu(a)         # what the reference's Transport instruction does
            if tuple(a.shape) != shape:
                raise ValueError("argument has shape %s; this function was compiled for %s"
                                 % (tuple(a.shape), shape))
            vals.append(a)
        if self.use_graph:
            self._run_graph(vals)
        else:
            self._it.run(vals)
        outs = [self._it.get_array(s) for s in self._out_slots]
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
                if v.ptr != s.ptr:
                    capi.check(capi.lib().cgt_amd_memcpy(capi.GPU, capi.GPU, s.ptr, v.ptr, s.nbytes))
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
    of small kernels)."""
    return Function(inputs, outputs, device_outputs, updates, use_graph)
