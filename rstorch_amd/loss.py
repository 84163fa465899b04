"""src/loss/{mod,cross_entropy}.rs over the HIP backend."""
import ctypes

from . import _ffi
from .engine import as_array2


class Loss:
    """src/loss/mod.rs:6-11."""

    def forward(self, input, truth):
        raise NotImplementedError

    def backward(self):
        raise NotImplementedError


class CrossEntropyLoss(Loss):
    """src/loss/cross_entropy.rs:8-48.  ``forward`` returns the scalar loss (the one host
    round-trip of a training step); the softmax, the loss and ``pred - truth`` come out of one
    kernel, and ``backward`` hands that gradient over (not divided by the batch size)."""

    def __init__(self):
        self._grad = None

    @classmethod
    def new(cls):
        return cls()

    def forward(self, pred, truth):
        p = as_array2(pred)
        t = as_array2(truth, p.engine)
        if p.shape != t.shape:
            raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "pred %r vs truth %r" % (p.shape, t.shape))
        g = p.engine.empty(p.rows, p.cols)
        # the logits of a compiled Sequential: its compiled form takes the call (and, in a training
        # loop, launches the upper layers' input gradients behind the loss before the host waits)
        through = getattr(p, "_loss_through", None)
        through = through() if through is not None else None
        value = through(p, t, g) if through is not None else None
        if value is None:
            loss = ctypes.c_double()
            _ffi.check(p.engine.lib.rst_cross_entropy(p.engine.handle, p.ptr, t.ptr, g.ptr, None,
                                                      p.rows, p.cols, ctypes.byref(loss)))
            value = loss.value
        self._grad = g
        return value

    def backward(self):
        if self._grad is None:
            raise _ffi.StateError(_ffi.RST_ERR_STATE, "CrossEntropyLoss.backward without a forward")
        g, self._grad = self._grad, None  # take()
        return g
