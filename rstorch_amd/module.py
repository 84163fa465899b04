"""Host-side mirror of the reference's ``module`` package over the HIP backend.

Same names, argument meaning and failure behaviour as
``src/module/{mod,linear,sequential}.rs`` and ``src/module/activation/{relu,identity}.rs``:
``forward`` / ``backward`` / ``parameters`` / ``train`` / ``eval``; caches are consumed by
``backward`` (a second ``backward`` raises, where the reference panics on ``unwrap``);
gradients are overwritten, never accumulated.  Arrays are device-resident ``Array2``.

A ``Sequential`` made only of ``Identity`` / ``Linear`` / ``ReLU`` layers is *compiled*: the first
``forward`` builds a device model (``rst_model``) over the layer list, moves the layers' weights
into its parameter arena (the layers keep views) and from then on

* ``forward`` runs the layers' launches from one call,
* ``backward`` launches nothing: it remembers its gradient, and the pass runs when somebody needs
  its results - ``SGD.step(model)`` runs it with the optimiser update inside the weight-gradient
  launches (the README loop's ``model.backward(loss.backward()); optim.step(model)`` reaches
  exactly the launches of ``rst_model_train_step``), while reading a
  gradient through ``parameters()`` or touching the input gradient that ``backward`` returned runs
  it on its own first, so every value a caller can observe is the value the reference computes at
  that point.  The input gradient itself is only computed if the returned array is kept.

Any other layer list (a ``Softmax`` module, a user-defined ``Module``) runs layer by layer.  Changing
the layer list (``push`` / ``insert`` / ``remove``) drops the compiled form; it is rebuilt on the next
``forward``.
"""
import ctypes
import weakref

from . import _ffi
from .engine import Array2, as_array2, default_engine
from .init import InitParameters, KaimingNormal


class Parameter:
    """src/module/mod.rs:16-19: a parameter and its gradient (device arrays)."""

    def __init__(self, parm, grad):
        self.parm = parm
        self.grad = grad


class Parameters:
    """src/module/mod.rs:21-40."""

    def __init__(self, parms=None):
        self.parms = list(parms or [])

    def add(self, parm, grad):
        self.parms.append(Parameter(parm, grad))
        return self

    def iter(self):
        return iter(self.parms)

    def __iter__(self):
        return iter(self.parms)

    def __len__(self):
        return len(self.parms)


class Module:
    """src/module/mod.rs:42-56."""

    def forward(self, input):
        raise NotImplementedError

    def backward(self, gradient):
        raise NotImplementedError

    def parameters(self):
        return Parameters()

    def train(self):
        pass

    def eval(self):
        pass


class Identity(Module):
    """src/module/activation/identity.rs:15-29."""

    @classmethod
    def new(cls):
        return cls()

    def forward(self, input):
        return input

    def backward(self, gradient):
        return gradient

    def __repr__(self):
        return "Identity"


class ReLU(Module):
    """src/module/activation/relu.rs:17-32."""

    def __init__(self):
        self.prev_input = None  # tensor whose sign gives the mask (pre-activation or output)

    @classmethod
    def new(cls):
        return cls()

    def forward(self, input):
        x = as_array2(input)
        out = x.engine.empty(x.rows, x.cols)
        _ffi.check(x.engine.lib.rst_relu_forward(x.engine.handle, x.ptr, out.ptr, x.size))
        self.prev_input = x
        return out

    def backward(self, gradient):
        if self.prev_input is None:
            raise _ffi.StateError(_ffi.RST_ERR_STATE, "ReLU.backward without a forward")
        g = as_array2(gradient, self.prev_input.engine)
        x, self.prev_input = self.prev_input, None  # take()
        if g.shape != x.shape:
            raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "gradient %r vs input %r" % (g.shape, x.shape))
        out = x.engine.empty(x.rows, x.cols)
        _ffi.check(x.engine.lib.rst_relu_backward(x.engine.handle, g.ptr, x.ptr, out.ptr, x.size))
        return out

    # used by Sequential when the neighbouring Linear kernels do this layer's work
    def _absorb_forward(self, activation):
        self.prev_input = activation

    def _absorb_backward(self):
        if self.prev_input is None:
            raise _ffi.StateError(_ffi.RST_ERR_STATE, "ReLU.backward without a forward")
        self.prev_input = None

    def __repr__(self):
        return "ReLU"


class Softmax(Module):
    """src/module/activation/softmax.rs:5-78: softmax along an axis; the backward pass builds the
    reference's single batch-summed Jacobian."""

    def __init__(self, axis=1):
        self.axis = int(axis)
        self.output = None

    @classmethod
    def new(cls):
        return cls(1)

    @classmethod
    def with_axis(cls, axis):
        return cls(axis)

    def forward(self, input):
        x = as_array2(input)
        out = x.engine.empty(x.rows, x.cols)
        _ffi.check(x.engine.lib.rst_softmax_forward(x.engine.handle, x.ptr, out.ptr, x.rows, x.cols,
                                                    self.axis))
        self.output = out
        return out.clone()  # the reference returns a clone and keeps the output (softmax.rs:58-59)

    def backward(self, gradient):
        if self.output is None:
            raise _ffi.StateError(_ffi.RST_ERR_STATE, "Softmax.backward without a forward")
        out, self.output = self.output, None  # take()
        g = as_array2(gradient, out.engine)
        if g.shape != out.shape:
            raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "gradient %r vs output %r" % (g.shape, out.shape))
        gin = out.engine.empty(out.rows, out.cols)
        _ffi.check(out.engine.lib.rst_softmax_backward(out.engine.handle, g.ptr, out.ptr, gin.ptr,
                                                       out.rows, out.cols))
        return gin

    def __repr__(self):
        return "Softmax(axis=%d)" % self.axis


class Linear(Module):
    """src/module/linear.rs:8-79.  weight (out, in), bias (1, out)."""

    def __init__(self, input_size, output_size, init=None, engine=None):
        init = init if init is not None else KaimingNormal()
        eng = engine or default_engine()
        self.engine = eng
        self.input_size, self.output_size = int(input_size), int(output_size)
        self.weight = as_array2(init.weight(self.input_size, self.output_size, eng), eng)
        self.bias = as_array2(init.bias(self.input_size, self.output_size, eng), eng)
        if self.weight.shape != (self.output_size, self.input_size):
            raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "init.weight returned %r" % (self.weight.shape,))
        if self.bias.shape != (1, self.output_size):
            raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "init.bias returned %r" % (self.bias.shape,))
        self.prev_input = None
        self.grad_weight = None
        self.grad_bias = None
        self._home = None       # the compiled Sequential (_Plan) whose arena holds the parameters
        self._has_grad = False  # a backward pass has been asked for since the layer was made

    @classmethod
    def new(cls, input_size, output_size):
        return cls(input_size, output_size)

    @classmethod
    def new_with_kernel(cls, input_size, output_size, init):
        return cls(input_size, output_size, init)

    def _forward(self, input, fuse_relu):
        x = as_array2(input, self.engine)
        if x.cols != self.input_size:
            raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "input has %d features, layer expects %d"
                                  % (x.cols, self.input_size))
        out = self.engine.empty(x.rows, self.output_size)
        _ffi.check(self.engine.lib.rst_linear_forward(
            self.engine.handle, x.ptr, self.weight.ptr, self.bias.ptr, out.ptr, x.rows,
            self.input_size, self.output_size, 1 if fuse_relu else 0))
        self.prev_input = x
        return out

    def forward(self, input):
        return self._forward(input, False)

    def _backward(self, gradient, mask_by_input, need_input_grad=True):
        if self.prev_input is None:
            raise _ffi.StateError(_ffi.RST_ERR_STATE, "Linear.backward without a forward")
        g = as_array2(gradient, self.engine)
        x, self.prev_input = self.prev_input, None  # take()
        if g.shape != (x.rows, self.output_size):
            raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "gradient %r vs expected %r"
                                  % (g.shape, (x.rows, self.output_size)))
        if self.grad_weight is None:
            self.grad_weight = self.engine.empty(self.output_size, self.input_size)
            self.grad_bias = self.engine.empty(1, self.output_size)
        self._has_grad = True
        gx = self.engine.empty(x.rows, self.input_size) if need_input_grad else None
        _ffi.check(self.engine.lib.rst_linear_backward(
            self.engine.handle, g.ptr, x.ptr, self.weight.ptr, self.grad_weight.ptr,
            self.grad_bias.ptr, gx.ptr if gx is not None else None,
            x.ptr if (mask_by_input and gx is not None) else None, x.rows, self.input_size,
            self.output_size))
        return gx

    def backward(self, gradient):
        return self._backward(gradient, False)

    def parameters(self):
        if not self._has_grad:
            raise _ffi.StateError(_ffi.RST_ERR_STATE,
                                  "Linear.parameters before any backward (no gradient yet)")
        return Parameters().add(self.weight, self.grad_weight).add(self.bias, self.grad_bias)

    def __repr__(self):
        return "Linear(%d, %d)" % (self.input_size, self.output_size)


class _Plan:
    """The compiled form of a Sequential of Identity / Linear / ReLU layers: an ``rst_model`` whose
    arena holds the layers' parameters and gradients, plus the backward pass that has been asked
    for but not launched yet."""

    def __init__(self, layers):
        from .model import DeviceModel
        self.key = tuple(id(l) for l in layers)
        self.linears = [l for l in layers if type(l) is Linear]
        spec = []
        for l in layers:
            if type(l) is Linear:
                spec.append(("linear", l.input_size, l.output_size))
            else:
                spec.append(("relu",) if type(l) is ReLU else ("identity",))
        self.engine = self.linears[0].engine
        for l in self.linears:  # whatever another compiled Sequential still owes these layers
            if l._home is not None:
                l._home.flush()
        self.device = DeviceModel(spec, self.engine)
        eng, params = self.engine, self.device.parameters()
        for i, l in enumerate(self.linears):
            (w, gw), (b, gb) = params[2 * i], params[2 * i + 1]
            _ffi.check(eng.lib.rst_copy(eng.handle, w._ptr, l.weight.ptr, w.size))
            _ffi.check(eng.lib.rst_copy(eng.handle, b._ptr, l.bias.ptr, b.size))
            if l._has_grad and l.grad_weight is not None:  # gradients computed before the move stay readable
                _ffi.check(eng.lib.rst_copy(eng.handle, gw._ptr, l.grad_weight.ptr, gw.size))
                _ffi.check(eng.lib.rst_copy(eng.handle, gb._ptr, l.grad_bias.ptr, gb.size))
            l.weight, l.bias = w, b
            # a look at (or a write into) a parameter between the loss and the backward pass: input
            # gradients launched ahead were computed with the weights of before
            w._before_access = b._before_access = self._parameters_touched
            # reading a gradient first runs the backward pass that is still owed
            gw._before_access = gb._before_access = self.flush
            l.grad_weight, l.grad_bias = gw, gb
            l._home = self
        self.in_width, self.out_width = self.device.in_width, self.device.out_width
        self.x = self.out = None      # the forward pass whose caches are live (kept alive until backward)
        self.pending = None           # (gradient, weak reference to the deferred input gradient)
        # a loss on the logits that a backward pass followed: the next step is taken for one of a training loop
        self._training = self._loss_seen = self._backward_followed = False
        self._inputs_from = None      # weak reference to the loss gradient that input gradients were launched from

    def valid_for(self, layers):
        return self.key == tuple(id(l) for l in layers) and all(l._home is self for l in self.linears)

    def forward(self, input):
        self.flush()  # a backward pass nobody looked at would otherwise read the new activations
        x = as_array2(input, self.engine)
        if x.cols != self.in_width:
            raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "input has %d features, layer expects %d"
                                  % (x.cols, self.in_width))
        out = self.engine.empty(x.rows, self.out_width)
        _ffi.check(self.engine.lib.rst_model_forward_to(self.device.handle, x.ptr, x.rows, out.ptr))
        self.x, self.out = x, out
        self._training = self._loss_seen and self._backward_followed
        self._loss_seen = self._backward_followed = False
        self._inputs_from = None
        out._loss_through = weakref.WeakMethod(self._loss_through)
        return out

    def _loss_through(self, pred, truth, grad):
        """CrossEntropyLoss.forward on the logits of the latest forward pass: the loss, or None when
        this is not the array forward() returned.  In a training loop the input gradients of the
        layers above the first are launched behind the loss before the host waits for it
        (rst_model_loss_accuracy_to), and the backward pass skips them if the gradient array reaches
        backward() without anybody having looked at it."""
        if self.x is None or self.pending is not None or pred is not self.out or pred.shape != truth.shape:
            return None
        loss = ctypes.c_double()
        _ffi.check(self.engine.lib.rst_model_loss_accuracy_to(
            self.device.handle, pred.ptr, truth.ptr, grad.ptr, 1 if self._training else 0, ctypes.byref(loss), None))
        self._loss_seen = True
        if self._training:
            self._inputs_from = weakref.ref(grad)
            grad._before_access = self._inputs_touched
        return loss.value

    def _parameters_touched(self):
        if self._inputs_from is not None:
            self._inputs_touched()

    def _inputs_touched(self):
        """Somebody looked at (and may have rewritten) the gradient the input gradients were launched from."""
        _ffi.check(self.engine.lib.rst_model_discard_inputs(self.device.handle))
        self._inputs_from = None

    def backward(self, gradient):
        if self.x is None or self.pending is not None:  # no forward yet, or its caches are taken
            raise _ffi.StateError(_ffi.RST_ERR_STATE, "Sequential.backward without a forward")
        g = as_array2(gradient, self.engine)
        if g.shape != (self.x.rows, self.out_width):
            raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "gradient %r vs expected %r"
                                  % (g.shape, (self.x.rows, self.out_width)))
        gin = Array2(self.engine, self.x.rows, self.in_width, resolver=self._resolve_input_grad)
        self.pending = (g, weakref.ref(gin))
        self._backward_followed = True
        for l in self.linears:
            l._has_grad = True
        return gin

    def _resolve_input_grad(self, gin):
        """Somebody looks at the array that backward() returned."""
        if self.pending is not None and self.pending[1]() is gin:
            self._run(False, 0.0)
        if gin._ptr is None:
            raise _ffi.StateError(_ffi.RST_ERR_STATE, "this input gradient was never computed")

    def _run(self, apply_sgd, lr):
        g, ref = self.pending
        self.pending = None
        gin = ref()  # still wanted by somebody?
        if gin is not None:
            gin._resolver = None
            gin._materialise()
        if self._inputs_from is not None:
            if self._inputs_from() is g:   # untouched since: our own access keeps the launched gradients
                g._before_access = None
            else:
                self._inputs_touched()
            self._inputs_from = None
        _ffi.check(self.engine.lib.rst_model_backward_to(
            self.device.handle, g.ptr, gin._ptr if gin is not None else None, 1 if apply_sgd else 0, float(lr)))
        self.x = self.out = None  # the caches are consumed

    def flush(self):
        """Runs the backward pass that is still owed, without an optimiser step."""
        if self.pending is not None:
            self._run(False, 0.0)

    def step_sgd(self, lr):
        """backward + SGD::step in one pass, if a backward is still owed; else False."""
        if self.pending is None:
            return False
        self._run(True, lr)
        return True


class Sequential(Module):
    """src/module/sequential.rs:11-110.  The layer list may change at any time; the
    Linear/ReLU fusion is decided afresh on every call."""

    # False (on the class or on one instance): always run layer by layer, one call per layer
    compile_enabled = True

    def __init__(self, layers=None):
        self.layers = list(layers or [])
        self._plan = None

    def _compiled(self):
        """The compiled form, built on demand; None when the layer list has a layer it cannot hold."""
        if not self.compile_enabled:
            self._drop_plan()
            return None
        if self._plan is not None and self._plan.valid_for(self.layers):
            return self._plan
        self._drop_plan()
        linears = [l for l in self.layers if type(l) is Linear]
        if not linears or any(type(l) not in (Linear, ReLU, Identity) for l in self.layers):
            return None
        if any(l.engine is not linears[0].engine for l in linears):
            return None
        if any(a.output_size != b.input_size for a, b in zip(linears, linears[1:])):
            return None  # the layer-by-layer pass raises the shape error where the reference panics
        self._plan = _Plan(self.layers)
        return self._plan

    def _drop_plan(self):
        if self._plan is not None:
            self._plan.flush()
            self._plan = None

    @classmethod
    def new(cls, layers):
        return cls(layers)

    def push(self, layer):
        self._drop_plan()
        self.layers.append(layer)

    push_box = push

    def insert(self, index, layer):
        self._drop_plan()
        self.layers.insert(index, layer)

    insert_box = insert

    def len(self):
        return len(self.layers)

    __len__ = len

    def is_empty(self):
        return not self.layers

    def remove(self, index):
        if index >= len(self.layers):
            return None
        self._drop_plan()
        return self.layers.pop(index)

    def _next_real(self, i):
        for j in range(i + 1, len(self.layers)):
            if not isinstance(self.layers[j], Identity):
                return j
        return -1

    def _prev_real(self, i):
        for j in range(i - 1, -1, -1):
            if not isinstance(self.layers[j], Identity):
                return j
        return -1

    def forward(self, input):
        plan = self._compiled()
        if plan is not None:
            return plan.forward(input)
        x = input
        skip = set()
        for i, layer in enumerate(self.layers):
            if i in skip:
                continue
            if type(layer) is Linear:
                j = self._next_real(i)
                if j >= 0 and type(self.layers[j]) is ReLU:
                    x = layer._forward(x, True)
                    self.layers[j]._absorb_forward(x)
                    skip.add(j)
                    continue
            x = layer.forward(x)
        return x

    def backward(self, gradient):
        if self._plan is not None and self._plan.valid_for(self.layers):
            return self._plan.backward(gradient)
        g = gradient
        skip = set()
        for i in range(len(self.layers) - 1, -1, -1):
            if i in skip:
                continue
            layer = self.layers[i]
            if type(layer) is Linear:
                j = self._prev_real(i)
                if j >= 0 and type(self.layers[j]) is ReLU and \
                        self.layers[j].prev_input is not None:
                    g = layer._backward(g, True)
                    self.layers[j]._absorb_backward()
                    skip.add(j)
                    continue
            g = layer.backward(g)
        return g

    def train(self):
        for layer in self.layers:
            layer.train()

    def eval(self):
        for layer in self.layers:
            layer.eval()

    def parameters(self):
        out = Parameters()
        for layer in self.layers:
            for p in layer.parameters():
                out.parms.append(p)
        return out

    def __repr__(self):
        return "Sequential(%s)" % ", ".join(repr(l) for l in self.layers)


def sequential(*layers):
    """The ``sequential!`` macro (src/module/sequential.rs:62-74): both spellings of the
    reference are accepted - layer instances, or ``(LayerClass, arg, ...)`` tuples."""
    built = []
    for l in layers:
        if isinstance(l, tuple):
            built.append(l[0].new(*l[1:]))
        elif isinstance(l, type):
            built.append(l.new())
        else:
            built.append(l)
    return Sequential.new(built)
