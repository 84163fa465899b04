"""src/utils.rs:44-65 on the device."""
import ctypes

from . import _ffi
from .engine import as_array2


def accuracy(pred, truth):
    """Fraction of rows whose arg-max (first maximum wins) agrees; one scalar comes back."""
    p = as_array2(pred)
    t = as_array2(truth, p.engine)
    if p.shape != t.shape:
        raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "pred %r vs truth %r" % (p.shape, t.shape))
    acc = ctypes.c_double()
    _ffi.check(p.engine.lib.rst_accuracy(p.engine.handle, p.ptr, t.ptr, p.rows, p.cols,
                                         ctypes.byref(acc)))
    return acc.value
