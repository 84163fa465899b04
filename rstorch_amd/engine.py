"""Engine handle (one GPU, one stream) and the device-resident ``Array2``.

``Array2`` stands where the reference has ``ndarray::Array2<f64>`` (src/module/mod.rs:42-49):
a dense row-major f64 matrix.  Here its storage lives in HBM; ``to_numpy`` / ``from_numpy``
are the explicit host crossings.
"""
import ctypes
import os

import numpy as np

from . import _ffi


class Event:
    def __init__(self, engine):
        self._engine = engine
        h = ctypes.c_void_p()
        _ffi.check(_ffi.load().rst_event_create(engine.handle, ctypes.byref(h)))
        self.handle = h

    def record(self):
        _ffi.check(_ffi.load().rst_event_record(self.handle))
        return self

    def elapsed_ms(self, stop):
        ms = ctypes.c_double()
        _ffi.check(_ffi.load().rst_event_elapsed_ms(self.handle, stop.handle, ctypes.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            # destroying an event does not touch its engine, so this is safe after Engine.close()
            if self.handle:
                _ffi.load().rst_event_destroy(self.handle)
            self.handle = None
        except Exception:
            pass


class Engine:
    """Owns an ``rst_engine``.  Raises if the library or the GPU is not there."""

    def __init__(self, device=0):
        self.lib = _ffi.load()
        h = ctypes.c_void_p()
        _ffi.check(self.lib.rst_engine_create(int(device), ctypes.byref(h)))
        self.handle = h
        self.device = int(device)

    def close(self):
        if getattr(self, "handle", None):
            self.lib.rst_engine_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- plumbing ---------------------------------------------------------------------------
    def synchronize(self):
        _ffi.check(self.lib.rst_engine_synchronize(self.handle))

    def device_info(self):
        name = ctypes.create_string_buffer(256)
        cus = ctypes.c_int()
        mem = ctypes.c_size_t()
        _ffi.check(self.lib.rst_engine_device_info(self.handle, name, 256, ctypes.byref(cus),
                                                   ctypes.byref(mem)))
        return {"name": name.value.decode(), "compute_units": cus.value, "memory_bytes": mem.value}

    def event(self):
        return Event(self)

    def wait_event(self, event):
        """Later work on this engine starts only after ``event`` (recorded on any engine of this GPU)."""
        _ffi.check(self.lib.rst_event_wait(self.handle, event.handle))

    def malloc(self, count):
        p = ctypes.c_void_p()
        _ffi.check(self.lib.rst_malloc(self.handle, int(count), ctypes.byref(p)))
        return p.value

    def free(self, ptr):
        if ptr and self.handle:
            _ffi.check(self.lib.rst_free(self.handle, ptr))

    # -- Array2 factories -------------------------------------------------------------------
    def empty(self, rows, cols):
        return Array2(self, int(rows), int(cols))

    def zeros(self, rows, cols):
        a = Array2(self, int(rows), int(cols))
        _ffi.check(self.lib.rst_fill(self.handle, a.ptr, a.size, 0.0))
        return a

    def full(self, rows, cols, value):
        a = Array2(self, int(rows), int(cols))
        _ffi.check(self.lib.rst_fill(self.handle, a.ptr, a.size, float(value)))
        return a

    def from_numpy(self, host):
        host = np.ascontiguousarray(host, dtype=np.float64)
        if host.ndim != 2:
            raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "Array2 needs a 2-D array, got %r" % (host.shape,))
        a = Array2(self, host.shape[0], host.shape[1])
        _ffi.check(self.lib.rst_upload(self.handle, a.ptr, host.ctypes.data_as(_ffi.c_double_p),
                                       host.size))
        return a

    def uniform(self, rows, cols, seed, stream, lo=0.0, hi=1.0):
        a = Array2(self, int(rows), int(cols))
        _ffi.check(self.lib.rst_fill_uniform(self.handle, a.ptr, a.size, seed, stream, lo, hi))
        return a

    def normal(self, rows, cols, seed, stream, mean=0.0, std=1.0):
        a = Array2(self, int(rows), int(cols))
        _ffi.check(self.lib.rst_fill_normal(self.handle, a.ptr, a.size, seed, stream, mean, std))
        return a

    def one_hot(self, rows, cols, seed, stream):
        a = Array2(self, int(rows), int(cols))
        _ffi.check(self.lib.rst_fill_one_hot(self.handle, a.ptr, rows, cols, seed, stream))
        return a


class Array2:
    """Dense row-major f64 matrix in device memory.

    ``ptr`` is the device address.  Two kinds of array fill it in late: the gradient views that a
    compiled ``Sequential`` hands out (reading ``ptr`` first runs the backward pass that
    ``backward`` deferred, see ``rstorch_amd.module``) and the input gradient that ``backward``
    returns (computed only if somebody looks at it).  Every access to the contents goes through
    ``ptr``, so such an array behaves like any other."""

    def __init__(self, engine, rows, cols, ptr=None, owner=None, before_access=None, resolver=None):
        self.engine = engine
        self.rows, self.cols = int(rows), int(cols)
        self._before_access = before_access  # called before every read of ``ptr`` (or None)
        self._resolver = resolver            # called once, to produce the contents (or None)
        if resolver is not None:
            self._ptr = None
            self._owns = False
        elif ptr is None:
            self._ptr = engine.malloc(self.rows * self.cols)
            self._owns = True
        else:
            self._ptr = ptr
            self._owns = False
        self._owner = owner  # keeps the owning object alive for borrowed views

    @property
    def ptr(self):
        if self._resolver is not None:
            resolver, self._resolver = self._resolver, None
            resolver(self)
        if self._before_access is not None:
            self._before_access()
        return self._ptr

    def _materialise(self):
        """Gives a deferred array memory of its own (called by its resolver)."""
        self._ptr = self.engine.malloc(self.rows * self.cols)
        self._owns = True
        return self._ptr

    @property
    def shape(self):
        return (self.rows, self.cols)

    @property
    def size(self):
        return self.rows * self.cols

    def nrows(self):
        return self.rows

    def to_numpy(self):
        out = np.empty((self.rows, self.cols), dtype=np.float64)
        _ffi.check(self.engine.lib.rst_download(self.engine.handle,
                                                out.ctypes.data_as(_ffi.c_double_p), self.ptr,
                                                out.size))
        return out

    def assign(self, host):
        """Overwrites the device contents with a host array of the same shape."""
        host = np.ascontiguousarray(host, dtype=np.float64)
        if host.shape != self.shape:
            raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "assign %r into %r" % (host.shape, self.shape))
        _ffi.check(self.engine.lib.rst_upload(self.engine.handle, self.ptr,
                                              host.ctypes.data_as(_ffi.c_double_p), host.size))

    def clone(self):
        out = Array2(self.engine, self.rows, self.cols)
        _ffi.check(self.engine.lib.rst_copy(self.engine.handle, out.ptr, self.ptr, self.size))
        return out

    def __array__(self, dtype=None, copy=None):
        a = self.to_numpy()
        return a if dtype is None else a.astype(dtype)

    def __repr__(self):
        return "Array2(shape=%r, device=%d)" % (self.shape, self.engine.device)

    def __del__(self):
        try:
            if self._owns and self._ptr and self.engine.handle:
                self.engine.free(self._ptr)
            self._ptr = None
        except Exception:
            pass


_default_engine = None


def default_engine():
    """The process-wide engine on device ``RSTORCH_DEVICE`` (default 0)."""
    global _default_engine
    if _default_engine is None or not _default_engine.handle:
        _default_engine = Engine(int(os.environ.get("RSTORCH_DEVICE", "0")))
    return _default_engine


def as_array2(x, engine=None):
    """Accepts an ``Array2`` or anything numpy can view as a 2-D float64 array."""
    if isinstance(x, Array2):
        return x
    return (engine or default_engine()).from_numpy(x)
