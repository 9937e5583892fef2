"""Device arrays: the Python-side handle of a cgtArray with devtype GPU.

A GpuArray owns (or views) a contiguous row-major buffer in HBM, allocated
through the library's own cgt_amd_alloc -- the role cgtArray plays in the
reference with cgt_alloc (include/cgt_common.h:91-146, src/cgt_common.cpp:15-66).
Copies to and from numpy are synchronous, like the reference's cgt_memcpy.
"""
import numpy as np

from . import capi

# int8 is the reference's "i1" (what comparisons produce); float64 buffers exist
# only so tests can hand double data to checker kernels
_DTYPES = (np.dtype(np.float32), np.dtype(np.int32), np.dtype(np.int64), np.dtype(np.float64), np.dtype(np.int8))


class _Buffer(object):
    """Owns one device allocation; freed when the last array using it dies."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        self.ptr = capi.lib().cgt_amd_alloc(self.nbytes)
        if not self.ptr:
            raise capi.CgtAmdError("device allocation of %d bytes failed: %s"
                                   % (self.nbytes, capi.last_error()))

    def __del__(self):
        ptr = getattr(self, "ptr", None)
        if ptr and capi._LIB is not None:
            capi._LIB.cgt_amd_free(ptr)
            self.ptr = None


class GpuArray(object):
    def __init__(self, shape, dtype=np.float32, _buffer=None, _offset=0):
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        if self.dtype not in _DTYPES:
            raise TypeError("unsupported device dtype %s" % self.dtype)
        self.size = int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1
        self.nbytes = self.size * self.dtype.itemsize
        self._buffer = _buffer if _buffer is not None else _Buffer(self.nbytes)
        self._offset = _offset
        assert self._offset + self.nbytes <= self._buffer.nbytes

    @property
    def ndim(self):
        return len(self.shape)

    @property
    def ptr(self):
        """Device address as an int (pass to the C ABI as void*)."""
        return self._buffer.ptr + self._offset

    def reshape(self, *shape):
        """Zero-copy view with a new shape (the reference's Reshape op is a view
        too, cgt/core.py:1452-1465)."""
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = tuple(shape[0])
        n = int(np.prod(shape, dtype=np.int64)) if shape else 1
        if n != self.size:
            raise ValueError("cannot reshape %s into %s" % (self.shape, shape))
        return GpuArray(shape, self.dtype, _buffer=self._buffer, _offset=self._offset)

    def set(self, host):
        host = _contiguous(host, self.dtype)
        if host.shape != self.shape:
            raise ValueError("shape mismatch %s vs %s" % (host.shape, self.shape))
        capi.check(capi.lib().cgt_amd_memcpy(capi.GPU, capi.CPU, self.ptr, host.ctypes.data, self.nbytes))
        return self

    def get(self):
        out = np.empty(self.shape, self.dtype)
        capi.check(capi.lib().cgt_amd_memcpy(capi.CPU, capi.GPU, out.ctypes.data, self.ptr, self.nbytes))
        return out

    def fill_u32(self, word, stream=None):
        capi.check(capi.lib().cgt_amd_fill_u32(self.ptr, word, self.nbytes // 4, stream))
        return self

    def __repr__(self):
        return "GpuArray(shape=%s, dtype=%s)" % (self.shape, self.dtype)


def empty(shape, dtype=np.float32):
    return GpuArray(shape, dtype)


def _contiguous(host, dtype=None):
    """C-contiguous copy/view that keeps 0-d arrays 0-d (np.ascontiguousarray makes them 1-d)."""
    host = np.asarray(host, dtype=dtype)
    return host if host.ndim == 0 else np.ascontiguousarray(host)


def to_gpu(host, dtype=None):
    host = _contiguous(host, dtype)
    return GpuArray(host.shape, host.dtype).set(host)
