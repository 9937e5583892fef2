"""ctypes binding of libcgt_amd.so -- every symbol include/cgt_amd.h declares.

There is no fallback: if the library has not been built, or a call fails,
this raises.  Build with ``python -m cgt_amd.build``.
"""
import ctypes
import os

from . import build as _build

c_int = ctypes.c_int
c_long = ctypes.c_long
c_double = ctypes.c_double
c_void_p = ctypes.c_void_p
c_char_p = ctypes.c_char_p

OK = 0
CPU, GPU = 0, 1

# name -> (restype, argtypes); mirrors include/cgt_amd.h one to one
PROTOTYPES = {
    "cgt_amd_version": (c_int, []),
    "cgt_amd_last_error": (c_char_p, []),
    "cgt_amd_device_count": (c_int, []),
    "cgt_amd_device_name": (c_int, [c_char_p, c_int]),
    "cgt_amd_mem_info": (c_int, [ctypes.POINTER(c_long), ctypes.POINTER(c_long)]),
    "cgt_amd_alloc": (c_void_p, [c_long]),
    "cgt_amd_free": (c_int, [c_void_p]),
    "cgt_amd_memcpy": (c_int, [c_int, c_int, c_void_p, c_void_p, c_long]),
    "cgt_amd_fill_u32": (c_int, [c_void_p, ctypes.c_uint, c_long, c_void_p]),
    "cgt_amd_synchronize": (c_int, [c_void_p]),
    "cgt_amd_stream_create": (c_int, [ctypes.POINTER(c_void_p)]),
    "cgt_amd_stream_destroy": (c_int, [c_void_p]),
    "cgt_amd_event_create": (c_int, [ctypes.POINTER(c_void_p)]),
    "cgt_amd_event_destroy": (c_int, [c_void_p]),
    "cgt_amd_event_record": (c_int, [c_void_p, c_void_p]),
    "cgt_amd_stream_wait_event": (c_int, [c_void_p, c_void_p]),
    "cgt_amd_graph_capture_begin": (c_int, [c_void_p]),
    "cgt_amd_graph_capture_end": (c_int, [c_void_p, ctypes.POINTER(c_void_p)]),
    "cgt_amd_graph_launch": (c_int, [c_void_p, c_void_p]),
    "cgt_amd_graph_destroy": (c_int, [c_void_p]),
    "cgt_amd_event_elapsed_ms": (c_int, [c_void_p, c_void_p, ctypes.POINTER(ctypes.c_float)]),
    "cgt_amd_memcpy_async": (c_int, [c_int, c_int, c_void_p, c_void_p, c_long, c_void_p]),
    "cgt_amd_stream_copy": (c_int, [c_void_p, c_void_p, c_long, c_void_p]),
    "cgt_amd_stream_copy_tune": (c_int, [c_long, c_int]),
    "cgt_amd_im2col_f32": (c_int, [c_void_p] + [c_long] * 4 + [c_int] * 6 + [c_void_p, c_void_p]),
    "cgt_amd_col2im_f32": (c_int, [c_void_p] + [c_long] * 4 + [c_int] * 6 + [c_void_p, c_void_p]),
    "cgt_amd_pool_outsize": (c_long, [c_long, c_int, c_int, c_int]),
    "cgt_amd_pool_staged_planes": (c_int, [c_int, c_long, c_long, c_long, c_long]),
    "cgt_amd_max_pool_f32": (c_int, [c_void_p] + [c_long] * 4 + [c_int] * 6 + [c_long] * 2
                             + [c_void_p, c_void_p, c_void_p]),
    "cgt_amd_max_pool_pullback_f32": (c_int, [c_void_p, c_void_p] + [c_long] * 4 + [c_int] * 6
                                      + [c_long] * 2 + [c_void_p, c_void_p]),
    "cgt_amd_lrn_fwd_f32": (c_int, [c_void_p] + [c_long] * 4 + [c_int, c_double, c_double, c_double]
                            + [c_void_p, c_void_p, c_void_p]),
    "cgt_amd_lrn_bwd_f32": (c_int, [c_void_p] * 4 + [c_long] * 4 + [c_int, c_double, c_double]
                            + [c_void_p, c_void_p]),
    "cgt_amd_lrn_bwd_recompute_f32": (c_int, [c_void_p] * 3 + [c_long] * 4 + [c_int, c_double, c_double]
                                      + [c_void_p, c_void_p]),
    "cgt_amd_lrn_bwd_from_x_f32": (c_int, [c_void_p] * 2 + [c_long] * 4 + [c_int, c_double, c_double, c_double]
                                   + [c_void_p, c_void_p]),
    "cgt_amd_sgemm": (c_int, [c_int, c_int, c_long, c_long, c_long, c_void_p, c_long, c_void_p,
                              c_long, c_void_p, c_long, c_void_p]),
    "cgt_amd_sgemm_noalloc": (c_int, [c_int, c_int, c_long, c_long, c_long, c_void_p, c_long, c_void_p,
                                      c_long, c_void_p, c_long, c_void_p]),
    "cgt_amd_sgemm_batched": (c_int, [c_int, c_int, c_long, c_long, c_long, c_long,
                                      c_void_p, c_long, c_long, c_void_p, c_long, c_long,
                                      c_void_p, c_long, c_long, c_void_p]),
    "cgt_amd_conv_same_supported": (c_int, [c_long, c_long] + [c_int] * 6),
    "cgt_amd_conv_same_fits": (c_int, [c_long] * 5 + [c_int, c_int]),
    "cgt_amd_conv_col_fits": (c_int, [c_long] * 4),
    "cgt_amd_conv_same_padded_size": (c_long, [c_long, c_long, c_long, c_int, c_int]),
    "cgt_amd_conv_same_pad_f32": (c_int, [c_void_p, c_long, c_long, c_long, c_int, c_int, c_void_p, c_void_p]),
    "cgt_amd_conv_same_filter_f32": (c_int, [c_void_p, c_long, c_long, c_int, c_int, c_int, c_void_p, c_void_p]),
    "cgt_amd_conv_same_product_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_int] + [c_long] * 5 + [c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "cgt_amd_conv_same_wgrad_f32": (c_int, [c_void_p, c_void_p] + [c_long] * 5 + [c_int, c_int, c_void_p, c_void_p]),
    "cgt_amd_conv_same_fwd_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_int] + [c_long] * 5 + [c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "cgt_amd_conv_same_bwd_data_f32": (c_int, [c_void_p, c_void_p] + [c_long] * 5 + [c_int, c_int, c_void_p, c_void_p]),
    "cgt_amd_conv_same_bwd_filter_f32": (c_int, [c_void_p, c_void_p] + [c_long] * 5 + [c_int, c_int, c_void_p, c_void_p]),
    "cgt_amd_conv_same_pad_pool_pullback_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_long, c_long, c_long] + [c_int] * 6 +
                                                [c_long, c_long, c_int, c_int, c_void_p, c_void_p]),
    "cgt_amd_conv_patch_supported": (c_int, [c_long] * 4 + [c_int] * 6),
    "cgt_amd_conv_patch_fwd_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_int] + [c_long] * 5 + [c_int] * 6 + [c_void_p, c_void_p, c_void_p]),
    "cgt_amd_conv_patch_bwd_filter_f32": (c_int, [c_void_p, c_void_p] + [c_long] * 5 + [c_int] * 6 + [c_void_p, c_void_p]),
    "cgt_amd_conv_col_fwd_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_int] + [c_long] * 4 + [c_void_p, c_void_p, c_void_p]),
    "cgt_amd_conv_col_bwd_data_f32": (c_int, [c_void_p, c_void_p] + [c_long] * 4 + [c_void_p, c_void_p]),
    "cgt_amd_conv_col_bwd_filter_f32": (c_int, [c_void_p, c_void_p] + [c_long] * 4 + [c_void_p, c_void_p]),
    "cgt_amd_elwise_unary_f32": (c_int, [c_int, c_long, c_void_p, c_void_p, c_void_p]),
    "cgt_amd_elwise_binary": (c_int, [c_int, c_int, c_int, c_long, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p]),
    "cgt_amd_repeat": (c_int, [c_void_p, c_int, c_int, ctypes.POINTER(c_long), ctypes.POINTER(c_int), c_void_p, c_void_p]),
    "cgt_amd_sum_f32": (c_int, [c_void_p, c_int, ctypes.POINTER(c_long), ctypes.POINTER(c_int), c_void_p, c_void_p]),
    "cgt_amd_fill_f32": (c_int, [c_void_p, ctypes.c_float, c_long, c_void_p]),
    "cgt_amd_transpose4_f32": (c_int, [c_void_p, ctypes.POINTER(c_long), ctypes.POINTER(c_int),
                                       c_void_p, c_void_p]),
}


class CgtAmdError(RuntimeError):
    pass


_LIB = None


def libpath():
    return _build.LIBPATH


def lib():
    """The loaded library.  Raises if it is not built (no CPU fallback exists)."""
    global _LIB
    if _LIB is None:
        path = libpath()
        if not os.path.exists(path):
            raise CgtAmdError("%s not found: run `python -m cgt_amd.build` (hipcc, gfx950)" % path)
        handle = ctypes.CDLL(path)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(handle, name)  # AttributeError if the symbol is missing
            fn.restype = res
            fn.argtypes = args
        _LIB = handle
    return _LIB


def last_error():
    return lib().cgt_amd_last_error().decode("utf-8", "replace")


def check(rc):
    if rc != OK:
        raise CgtAmdError("cgt_amd error %d: %s" % (rc, last_error()))


def device_count():
    return lib().cgt_amd_device_count()


def require_gpu():
    if device_count() < 1:
        raise CgtAmdError("no HIP device visible; the cgt_amd kernels have no CPU fallback")


def device_name():
    buf = ctypes.create_string_buffer(256)
    check(lib().cgt_amd_device_name(buf, 256))
    return buf.value.decode()


def synchronize(stream=None):
    check(lib().cgt_amd_synchronize(stream))


def stream_wait_event(stream, event):
    """Later work on `stream` waits for the work recorded in `event`."""
    check(lib().cgt_amd_stream_wait_event(stream, event.handle))


class Stream(object):
    """A HIP stream at default priority."""

    def __init__(self):
        h = c_void_p()
        check(lib().cgt_amd_stream_create(ctypes.byref(h)))
        self.handle = h

    def synchronize(self):
        synchronize(self.handle)

    def __del__(self):
        if getattr(self, "handle", None) is not None and _LIB is not None:
            _LIB.cgt_amd_stream_destroy(self.handle)
            self.handle = None


class Graph(object):
    """A captured launch sequence (HIP graph).  Use:
        g = Graph.capture(stream, fn)   # fn() issues its launches to `stream`
        g.launch()
    """

    def __init__(self, handle, stream):
        self.handle, self.stream = handle, stream

    @classmethod
    def capture(cls, stream, fn):
        h = c_void_p()
        check(lib().cgt_amd_graph_capture_begin(stream.handle))
        try:
            fn()
        finally:
            rc = lib().cgt_amd_graph_capture_end(stream.handle, ctypes.byref(h))
        check(rc)
        return cls(h, stream)

    def launch(self):
        check(lib().cgt_amd_graph_launch(self.handle, self.stream.handle))

    def __del__(self):
        if getattr(self, "handle", None) is not None and _LIB is not None:
            _LIB.cgt_amd_graph_destroy(self.handle)
            self.handle = None


class Event(object):
    def __init__(self):
        h = c_void_p()
        check(lib().cgt_amd_event_create(ctypes.byref(h)))
        self.handle = h

    def record(self, stream=None):
        check(lib().cgt_amd_event_record(self.handle, stream))

    def elapsed_ms(self, stop):
        """Milliseconds from this event to `stop` (waits for `stop`)."""
        ms = ctypes.c_float()
        check(lib().cgt_amd_event_elapsed_ms(self.handle, stop.handle, ctypes.byref(ms)))
        return ms.value

    def __del__(self):
        if getattr(self, "handle", None) is not None and _LIB is not None:
            _LIB.cgt_amd_event_destroy(self.handle)
            self.handle = None
