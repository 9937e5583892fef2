"""ctypes binding of libcgt_rt.so (include/cgt_rt.h): building the cgtArray /
cgtTuple objects a compiled closure receives, firing closures, and the C++
sequential interpreter.

Covers what the reference does in Cython (src/cycgt.pyx): python <-> cgtObject
conversion (97-141), apply_byref (439-449) and the interpreter wrapper
(338-434).
"""
import ctypes
import os

import numpy as np

from . import build as _build
from . import capi
from .gpuarray import GpuArray

c_int, c_long, c_void_p, c_char_p = ctypes.c_int, ctypes.c_long, ctypes.c_void_p, ctypes.c_char_p
LONGP = ctypes.POINTER(c_long)
INTP = ctypes.POINTER(c_int)
VOIDPP = ctypes.POINTER(c_void_p)

CPU, GPU = 0, 1
ARRAY_KIND, TUPLE_KIND = 1, 2

PROTOTYPES = {
    "cgt_rt_status": (c_int, []),
    "cgt_rt_error": (c_char_p, []),
    "cgt_rt_clear_error": (None, []),
    "cgt_get_stream": (c_void_p, []),
    "cgt_set_stream": (None, [c_void_p]),
    "cgt_rt_array_new": (c_void_p, [c_int, LONGP, c_int, c_int]),
    "cgt_rt_array_view": (c_void_p, [c_int, LONGP, c_int, c_int, c_void_p]),
    "cgt_rt_tuple_new": (c_void_p, [c_int]),
    "cgt_rt_tuple_setitem": (None, [c_void_p, c_int, c_void_p]),
    "cgt_rt_tuple_getitem": (c_void_p, [c_void_p, c_int]),
    "cgt_rt_tuple_len": (c_int, [c_void_p]),
    "cgt_rt_retain": (None, [c_void_p]),
    "cgt_rt_release": (None, [c_void_p]),
    "cgt_rt_kind": (c_int, [c_void_p]),
    "cgt_rt_array_ndim": (c_int, [c_void_p]),
    "cgt_rt_array_shape": (LONGP, [c_void_p]),
    "cgt_rt_array_dtype": (c_int, [c_void_p]),
    "cgt_rt_array_devtype": (c_int, [c_void_p]),
    "cgt_rt_array_data": (c_void_p, [c_void_p]),
    "cgt_rt_array_nbytes": (c_long, [c_void_p]),
    "cgt_rt_array_stride": (c_long, [c_void_p, c_int]),
    "cgt_rt_copy_object": (c_int, [c_void_p, c_void_p]),
    "cgt_rt_apply_byref": (c_int, [c_void_p, c_void_p, VOIDPP, c_int, c_void_p]),
    "cgt_rt_apply_byval": (c_void_p, [c_void_p, c_void_p, VOIDPP, c_int]),
    "cgt_rt_interp_new": (c_void_p, [c_long]),
    "cgt_rt_interp_free": (None, [c_void_p]),
    "cgt_rt_interp_add_load_argument": (c_int, [c_void_p, c_int, c_long, c_int]),
    "cgt_rt_interp_add_alloc": (c_int, [c_void_p, c_int, LONGP, INTP, c_int, c_long, c_int]),
    "cgt_rt_interp_add_arg_transport": (c_int, [c_void_p, c_long, c_int, c_long, c_int]),
    "cgt_rt_interp_add_build_tup": (c_int, [c_void_p, LONGP, INTP, c_int, c_long, c_int]),
    "cgt_rt_interp_add_return_byref": (c_int, [c_void_p, c_void_p, c_void_p, LONGP, INTP, c_int, c_long, c_int]),
    "cgt_rt_interp_add_return_byval": (c_int, [c_void_p, c_void_p, c_void_p, LONGP, INTP, c_int, c_long, c_int]),
    "cgt_rt_interp_set_slot": (c_int, [c_void_p, c_long, c_void_p]),
    "cgt_rt_interp_get_slot": (c_void_p, [c_void_p, c_long]),
    "cgt_rt_interp_run": (c_int, [c_void_p, VOIDPP, c_int]),
}

_LIB = None


def libpath():
    return _build.RT_LIBPATH


def lib():
    global _LIB
    if _LIB is None:
        capi.lib()  # libcgt_amd first; raises if it is not built
        path = libpath()
        if not os.path.exists(path):
            raise capi.CgtAmdError("%s not found: run `python -m cgt_amd.build`" % path)
        handle = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)  # op closures link against it
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _LIB = handle
    return _LIB


def check_status(what=""):
    L = lib()
    if L.cgt_rt_status() != 0:
        msg = L.cgt_rt_error().decode("utf-8", "replace")
        L.cgt_rt_clear_error()
        raise capi.CgtAmdError("%s: %s" % (what or "native op failed", msg))


def set_stream(stream):
    lib().cgt_set_stream(stream)


def _shape_arr(shape):
    return (c_long * max(1, len(shape)))(*shape)


class CgtObject(object):
    """Owns one reference to a runtime object and keeps alive whatever backs it."""

    def __init__(self, handle, keepalive=None):
        self.handle = handle
        self.keepalive = keepalive

    def __del__(self):
        h = getattr(self, "handle", None)
        if h and _LIB is not None:
            _LIB.cgt_rt_release(h)
            self.handle = None


def to_cgt(value):
    """Wrap a host value as a runtime object: GpuArray -> GPU view, numpy array
    or python int -> host view (ints become int64 scalars, as shape operands
    are), tuple/list -> cgtTuple.  Views, not copies (cycgt.pyx:120-141)."""
    L = lib()
    if isinstance(value, CgtObject):
        return value
    if isinstance(value, GpuArray):
        h = L.cgt_rt_array_view(value.ndim, _shape_arr(value.shape), value.dtype.num, GPU, value.ptr)
        return CgtObject(h, value)
    if isinstance(value, (tuple, list)):
        members = [to_cgt(v) for v in value]
        h = L.cgt_rt_tuple_new(len(members))
        for i, m in enumerate(members):
            L.cgt_rt_tuple_setitem(h, i, m.handle)
        return CgtObject(h, members)
    if isinstance(value, (int, np.integer)):
        value = np.array(value, dtype=np.int64)
    if isinstance(value, np.ndarray):
        arr = np.ascontiguousarray(value)
        ptr = arr.ctypes.data if arr.size else ctypes.addressof(ctypes.create_string_buffer(8))
        h = L.cgt_rt_array_view(arr.ndim, _shape_arr(arr.shape), arr.dtype.num, CPU, ptr)
        return CgtObject(h, arr)
    raise TypeError("cannot pass %r to a native op" % type(value))


def apply_byref(fptr, cldata, inputs, output):
    """Fire a compiled by-reference closure on python values (cycgt.pyx:439-449)."""
    L = lib()
    reads = [to_cgt(v) for v in inputs]
    write = to_cgt(output)
    arr = (c_void_p * max(1, len(reads)))(*[r.handle for r in reads])
    cl = ctypes.cast(ctypes.byref(cldata), c_void_p) if cldata is not None else None
    L.cgt_rt_apply_byref(fptr, cl, arr, len(reads), write.handle)
    check_status("native op")


class Interpreter(object):
    """The C++ sequential interpreter: a fixed instruction list over storage slots."""

    def __init__(self, n_slots):
        self._L = lib()
        self.handle = self._L.cgt_rt_interp_new(n_slots)
        self.n_slots = n_slots
        self._keep = []

    def __del__(self):
        if getattr(self, "handle", None) and _LIB is not None:
            _LIB.cgt_rt_interp_free(self.handle)
            self.handle = None

    @staticmethod
    def _locs(locs):
        idx = (c_long * max(1, len(locs)))(*[l[0] for l in locs])
        dev = (c_int * max(1, len(locs)))(*[l[1] for l in locs])
        return idx, dev, len(locs)

    def _ok(self, rc, what):
        if rc < 0:
            raise ValueError("interpreter: bad slot index in %s" % what)
        return rc

    def load_argument(self, arg_index, wloc):
        return self._ok(self._L.cgt_rt_interp_add_load_argument(self.handle, arg_index, wloc[0], wloc[1]), "LoadArgument")

    def alloc(self, dtype, shape_locs, wloc):
        idx, dev, n = self._locs(shape_locs)
        return self._ok(self._L.cgt_rt_interp_add_alloc(self.handle, np.dtype(dtype).num, idx, dev, n, wloc[0], wloc[1]), "Alloc")

    def arg_transport(self, rloc, wloc):
        return self._ok(self._L.cgt_rt_interp_add_arg_transport(self.handle, rloc[0], rloc[1], wloc[0], wloc[1]), "ArgTransport")

    def build_tup(self, read_locs, wloc):
        idx, dev, n = self._locs(read_locs)
        return self._ok(self._L.cgt_rt_interp_add_build_tup(self.handle, idx, dev, n, wloc[0], wloc[1]), "BuildTup")

    def return_byref(self, callable_, read_locs, wloc):
        idx, dev, n = self._locs(read_locs)
        self._keep.append(callable_)
        return self._ok(self._L.cgt_rt_interp_add_return_byref(self.handle, callable_.fptr_address, callable_.closure_address,
                                                               idx, dev, n, wloc[0], wloc[1]), "ReturnByRef")

    def return_byval(self, callable_, read_locs, wloc):
        idx, dev, n = self._locs(read_locs)
        self._keep.append(callable_)
        return self._ok(self._L.cgt_rt_interp_add_return_byval(self.handle, callable_.fptr_address, callable_.closure_address,
                                                               idx, dev, n, wloc[0], wloc[1]), "ReturnByVal")

    def set_slot(self, idx, value):
        obj = to_cgt(value)
        self._keep.append(obj)
        self._ok(self._L.cgt_rt_interp_set_slot(self.handle, idx, obj.handle), "set_slot")

    def run(self, args=()):
        objs = [to_cgt(a) for a in args]
        arr = (c_void_p * max(1, len(objs)))(*[o.handle for o in objs])
        rc = self._L.cgt_rt_interp_run(self.handle, arr, len(objs))
        if rc != 0:
            check_status("interpreter instruction %d" % (rc - 1))
            raise capi.CgtAmdError("interpreter instruction %d failed" % (rc - 1))

    def get_array(self, idx):
        """GpuArray / numpy view of what slot idx holds (device data is not copied)."""
        h = self._L.cgt_rt_interp_get_slot(self.handle, idx)
        if not h:
            return None
        return from_cgt_handle(h, owner=self)


class _Borrowed(object):
    """Device memory owned by a runtime object: holds one reference on that object (a view
    holds one on the buffer it shows), so the memory outlives later calls of the function
    that handed it out; `owner` (the interpreter) is kept alive as well."""

    def __init__(self, ptr, nbytes, owner, handle=None):
        self.ptr, self.nbytes, self.owner, self.handle = ptr, nbytes, owner, handle
        if handle:
            lib().cgt_rt_retain(handle)

    def __del__(self):
        h = getattr(self, "handle", None)
        if h and _LIB is not None:
            _LIB.cgt_rt_release(h)
            self.handle = None


def from_cgt_handle(h, owner=None):
    L = lib()
    kind = L.cgt_rt_kind(h)
    if kind == TUPLE_KIND:
        return tuple(from_cgt_handle(L.cgt_rt_tuple_getitem(h, i), owner) for i in range(L.cgt_rt_tuple_len(h)))
    ndim = L.cgt_rt_array_ndim(h)
    shp = L.cgt_rt_array_shape(h)
    shape = tuple(shp[i] for i in range(ndim))
    dtype = {11: np.float32, 5: np.int32, 7: np.int64, 12: np.float64, 1: np.int8}[L.cgt_rt_array_dtype(h)]
    data = L.cgt_rt_array_data(h)
    nbytes = L.cgt_rt_array_nbytes(h)
    if L.cgt_rt_array_devtype(h) == GPU:
        return GpuArray(shape, dtype, _buffer=_Borrowed(data, nbytes, owner, h))
    buf = (ctypes.c_char * max(1, nbytes)).from_address(data)
    return np.frombuffer(buf, dtype=dtype, count=int(np.prod(shape)) if shape else 1).reshape(shape).copy()
