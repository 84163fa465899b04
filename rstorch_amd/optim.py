"""src/optim/{mod,sgd}.rs over the HIP backend."""
import ctypes

from . import _ffi


class Optimizer:
    """src/optim/mod.rs:6-8."""

    def step(self, module):
        raise NotImplementedError


class SGD(Optimizer):
    """src/optim/sgd.rs:6-25: parm = parm - (lr * grad) over every parameter, one launch."""

    def __init__(self, lr):
        self.lr = float(lr)

    @classmethod
    def new(cls, lr):
        return cls(lr)

    def step(self, module):
        # a compiled Sequential that still owes its backward pass runs it with this update inside
        # the weight-gradient launches; the bits are those of the two passes apart
        plan = getattr(module, "_plan", None)
        if type(self) is SGD and plan is not None and plan.valid_for(module.layers) and plan.step_sgd(self.lr):
            return
        params = list(module.parameters())
        if not params:
            return
        n = len(params)
        parm_ptrs = (ctypes.c_void_p * n)(*[p.parm.ptr for p in params])
        grad_ptrs = (ctypes.c_void_p * n)(*[p.grad.ptr for p in params])
        counts = (ctypes.c_size_t * n)(*[p.parm.size for p in params])
        for p in params:
            if p.parm.shape != p.grad.shape:
                raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "parameter %r vs gradient %r"
                                      % (p.parm.shape, p.grad.shape))
        eng = params[0].parm.engine
        _ffi.check(eng.lib.rst_sgd_step(eng.handle, parm_ptrs, grad_ptrs, counts, n, self.lr))
