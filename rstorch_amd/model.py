"""``DeviceModel``: the whole Sequential + CrossEntropyLoss + SGD step behind one C-ABI call.

This is the shape of the reference's private ``BasicModel::step`` (src/model.rs:19-27):
forward, loss, backward, optimiser step, nothing handed back to the host but the scalar loss.
All parameters live in one arena so ``SGD::step`` is a single pass over it.
"""
import ctypes

import numpy as np

from . import _ffi
from .engine import Array2, as_array2, default_engine

_KINDS = {"identity": _ffi.LAYER_IDENTITY, "linear": _ffi.LAYER_LINEAR, "relu": _ffi.LAYER_RELU}


class DeviceModel:
    """layers: ("identity",) | ("linear", in, out) | ("relu",) tuples (or bare strings)."""

    def __init__(self, layers, engine=None):
        self.engine = engine or default_engine()
        self.spec = [(l,) if isinstance(l, str) else tuple(l) for l in layers]
        n = len(self.spec)
        kinds = (ctypes.c_int * max(n, 1))()
        ins = (ctypes.c_size_t * max(n, 1))()
        outs = (ctypes.c_size_t * max(n, 1))()
        for i, l in enumerate(self.spec):
            kinds[i] = _KINDS[l[0]]
            if l[0] == "linear":
                ins[i], outs[i] = int(l[1]), int(l[2])
        h = ctypes.c_void_p()
        _ffi.check(self.engine.lib.rst_model_create(self.engine.handle, kinds, ins, outs, n,
                                                    ctypes.byref(h)))
        self.handle = h
        linears = [l for l in self.spec if l[0] == "linear"]
        self.in_width = linears[0][1]
        self.out_width = linears[-1][2]
        self.batch = 0

    @classmethod
    def from_sequential(cls, model, engine=None):
        """Builds the device model from a ``rstorch_amd.Sequential`` and copies its weights."""
        from .module import Identity, Linear, ReLU
        spec, linears = [], []
        for layer in model.layers:
            if type(layer) is Linear:
                spec.append(("linear", layer.input_size, layer.output_size))
                linears.append(layer)
            elif type(layer) is ReLU:
                spec.append(("relu",))
            elif type(layer) is Identity:
                spec.append(("identity",))
            else:
                raise _ffi.RstorchError(_ffi.RST_ERR_UNSUPPORTED,
                                        "layer %r has no device-model form" % (layer,))
        dm = cls(spec, engine or (linears[0].engine if linears else None))
        params = dm.parameters()
        for i, layer in enumerate(linears):
            for dst, src in ((params[2 * i][0], layer.weight), (params[2 * i + 1][0], layer.bias)):
                _ffi.check(dm.engine.lib.rst_copy(dm.engine.handle, dst.ptr, src.ptr, src.size))
        return dm

    def close(self):
        if getattr(self, "handle", None) and self.engine.handle:
            self.engine.lib.rst_model_destroy(self.handle)
        self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- parameters ---------------------------------------------------------------------------
    def parameter_count(self):
        t, e = ctypes.c_size_t(), ctypes.c_size_t()
        _ffi.check(self.engine.lib.rst_model_parameter_count(self.handle, ctypes.byref(t),
                                                             ctypes.byref(e)))
        return t.value, e.value

    def parameters(self):
        """[(parm, grad)] as borrowed ``Array2`` views, reference order (weight, bias per Linear)."""
        out = []
        for i in range(self.parameter_count()[0]):
            p, g = ctypes.c_void_p(), ctypes.c_void_p()
            r, c = ctypes.c_size_t(), ctypes.c_size_t()
            _ffi.check(self.engine.lib.rst_model_parameter(self.handle, i, ctypes.byref(p),
                                                           ctypes.byref(g), ctypes.byref(r),
                                                           ctypes.byref(c)))
            out.append((Array2(self.engine, r.value, c.value, ptr=p.value, owner=self),
                        Array2(self.engine, r.value, c.value, ptr=g.value, owner=self)))
        return out

    def load_parameters(self, host_arrays):
        """host_arrays: one array per parameter tensor, reference order."""
        params = self.parameters()
        if len(host_arrays) != len(params):
            raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "expected %d tensors" % len(params))
        for (p, _), h in zip(params, host_arrays):
            p.assign(np.asarray(h, dtype=np.float64).reshape(p.shape))

    def state(self):
        """All parameters as one flat host array (reference order, no padding): a checkpoint."""
        n = self.parameter_count()[1]
        out = np.empty(n, dtype=np.float64)
        _ffi.check(self.engine.lib.rst_model_export_parameters(
            self.handle, out.ctypes.data_as(_ffi.c_double_p), n))
        return out

    def load_state(self, flat):
        flat = np.ascontiguousarray(flat, dtype=np.float64).ravel()
        _ffi.check(self.engine.lib.rst_model_import_parameters(
            self.handle, flat.ctypes.data_as(_ffi.c_double_p), flat.size))

    def save(self, path):
        """Writes the layer list and the parameters to an .npz file (no pickled objects)."""
        spec = np.array([[_KINDS[l[0]], l[1] if len(l) > 1 else 0, l[2] if len(l) > 2 else 0]
                         for l in self.spec], dtype=np.int64)
        np.savez(path, spec=spec, parameters=self.state())

    @classmethod
    def load(cls, path, engine=None):
        names = {v: k for k, v in _KINDS.items()}
        with np.load(path, allow_pickle=False) as f:
            spec = [(names[int(k)],) if int(k) != _ffi.LAYER_LINEAR else ("linear", int(i), int(o))
                    for k, i, o in f["spec"]]
            dm = cls(spec, engine)
            dm.load_state(f["parameters"])
        return dm

    def init_kaiming(self, seed, first_stream=0):
        _ffi.check(self.engine.lib.rst_model_init_kaiming(self.handle, seed, first_stream))

    # -- the step -------------------------------------------------------------------------------
    def forward(self, x):
        x = as_array2(x, self.engine)
        if x.cols != self.in_width:
            raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "input has %d features, model expects %d"
                                  % (x.cols, self.in_width))
        self._x = x  # the model references the input until backward
        self.batch = x.rows
        out = ctypes.c_void_p()
        _ffi.check(self.engine.lib.rst_model_forward(self.handle, x.ptr, x.rows, ctypes.byref(out)))
        return Array2(self.engine, x.rows, self.out_width, ptr=out.value, owner=self)

    def loss(self, truth, want_value=True):
        t = as_array2(truth, self.engine)
        if t.shape != (self.batch, self.out_width):
            raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "truth %r vs logits %r"
                                  % (t.shape, (self.batch, self.out_width)))
        v = ctypes.c_double()
        _ffi.check(self.engine.lib.rst_model_loss(self.handle, t.ptr,
                                                  ctypes.byref(v) if want_value else None))
        return v.value if want_value else None

    def backward(self, grad=None, need_input_grad=True):
        g = as_array2(grad, self.engine) if grad is not None else None
        if g is not None and g.shape != (self.batch, self.out_width):
            raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "gradient %r vs logits %r"
                                  % (g.shape, (self.batch, self.out_width)))
        out = ctypes.c_void_p()
        _ffi.check(self.engine.lib.rst_model_backward(self.handle, g.ptr if g is not None else None,
                                                      1 if need_input_grad else 0,
                                                      ctypes.byref(out)))
        if not need_input_grad or not out.value:
            return None
        return Array2(self.engine, self.batch, self.in_width, ptr=out.value, owner=self)

    def sgd_step(self, lr):
        _ffi.check(self.engine.lib.rst_model_sgd_step(self.handle, float(lr)))

    def train_step(self, x, truth, lr, want_loss=True):
        x = as_array2(x, self.engine)
        t = as_array2(truth, self.engine)
        if x.cols != self.in_width or t.shape != (x.rows, self.out_width):
            raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "x %r / truth %r do not fit the model"
                                  % (x.shape, t.shape))
        self._x, self.batch = x, x.rows
        v = ctypes.c_double()
        _ffi.check(self.engine.lib.rst_model_train_step(self.handle, x.ptr, t.ptr, x.rows, float(lr),
                                                        ctypes.byref(v) if want_loss else None))
        return v.value if want_loss else None

    def last_loss(self):
        v = ctypes.c_double()
        _ffi.check(self.engine.lib.rst_loss_value(self.engine.handle, ctypes.byref(v)))
        return v.value

    def fuse_sgd(self, on=True):
        """Apply SGD inside the weight-gradient launches of train_step (default) or as a pass."""
        _ffi.check(self.engine.lib.rst_model_fuse_sgd(self.handle, 1 if on else 0))

    def fuse_head(self, mode=True):
        """How much of a small classifier's tail train_step runs as one launch: False / 0 nothing (the
        separate launches), 1 the last Linear with the cross entropy and its input gradient, True / 2
        (default) also the Linear in front of it when both are small."""
        level = 2 if mode is True else 0 if mode is False else int(mode)
        _ffi.check(self.engine.lib.rst_model_fuse_head(self.handle, level))

    def pair_gradients(self, on=True):
        """Launch a layer's weight gradient in one grid with the next layer's input gradient
        when both are large (default), or one after the other."""
        _ffi.check(self.engine.lib.rst_model_pair_gradients(self.handle, 1 if on else 0))

    def graph_enable(self, on=True):
        """Replay the step as a HIP graph (True), launch its kernels one by one (False), or let the
        model's depth decide ("auto", the default: a graph from eight Linear layers on)."""
        mode = 2 if on == "auto" else 1 if on else 0
        _ffi.check(self.engine.lib.rst_model_graph_enable(self.handle, mode))

    def graph_active(self):
        v = ctypes.c_int()
        _ffi.check(self.engine.lib.rst_model_graph_active(self.handle, ctypes.byref(v)))
        return bool(v.value)

    # -- per-kernel timing -------------------------------------------------------------------
    def profile_enable(self, on=True):
        _ffi.check(self.engine.lib.rst_model_profile_enable(self.handle, 1 if on else 0))

    def profile_read(self, capacity=65536):
        cap = int(capacity)
        recs = (_ffi.KernelRecord * cap)()
        n = ctypes.c_size_t()
        _ffi.check(self.engine.lib.rst_model_profile_read(self.handle, recs, cap, ctypes.byref(n)))
        return [{"kernel": _ffi.KERNEL_NAMES.get(r.kind, str(r.kind)), "layer": r.layer, "ms": r.ms,
                 "flops": r.flops, "bytes": r.bytes} for r in recs[:min(n.value, cap)]]


class BasicModel:
    """src/model.rs:4-32: module + loss + optimiser with ``step`` and ``predict``, run as one
    device-resident step.  ``module`` is a ``Sequential`` of Identity / Linear / ReLU."""

    def __init__(self, module, loss, optim):
        self.module, self.loss, self.optim = module, loss, optim
        self.device = DeviceModel.from_sequential(module)

    @classmethod
    def new(cls, module, loss, optim):
        return cls(module, loss, optim)

    def step(self, input, truth, want_loss=False):
        return self.device.train_step(input, truth, self.optim.lr, want_loss=want_loss)

    def predict(self, input):
        return self.device.forward(input)


class BatchStager:
    """Pipelines host batches into HBM (pinned double buffering on a copy stream); labels travel
    as class indices and become dense one-hot rows on the device."""

    def __init__(self, max_rows, x_cols, classes, depth=2, engine=None):
        self.engine = engine or default_engine()
        self.x_cols, self.classes = int(x_cols), int(classes)
        self.max_rows = int(max_rows)
        h = ctypes.c_void_p()
        _ffi.check(self.engine.lib.rst_stager_create(self.engine.handle, self.max_rows, self.x_cols,
                                                     self.classes, int(depth), ctypes.byref(h)))
        self.handle = h

    def close(self):
        if getattr(self, "handle", None) and self.engine.handle:
            self.engine.lib.rst_stager_destroy(self.handle)
        self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def submit(self, x, labels=None, truth=None):
        x = np.ascontiguousarray(x, dtype=np.float64)
        if x.ndim != 2 or x.shape[1] != self.x_cols:
            raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "x %r does not have %d columns" % (x.shape, self.x_cols))
        if labels is not None:
            lab = np.ascontiguousarray(labels, dtype=np.uint32).ravel()
            if lab.size != x.shape[0]:
                raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "%d labels for %d rows" % (lab.size, x.shape[0]))
            _ffi.check(self.engine.lib.rst_stager_submit_labels(
                self.handle, x.ctypes.data_as(_ffi.c_double_p),
                lab.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32)), x.shape[0]))
        else:
            t = np.ascontiguousarray(truth, dtype=np.float64)
            if t.shape != (x.shape[0], self.classes):
                raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "truth %r" % (t.shape,))
            _ffi.check(self.engine.lib.rst_stager_submit_dense(
                self.handle, x.ctypes.data_as(_ffi.c_double_p), t.ctypes.data_as(_ffi.c_double_p),
                x.shape[0]))

    def host_slot(self, rows):
        """numpy views (x [rows, x_cols], labels [rows]) onto the pinned memory of the next free
        slot, to be filled in place and sent with ``commit(rows)``: no intermediate copy."""
        rows = int(rows)
        if rows < 1 or rows > self.max_rows:  # the views must stay inside the pinned slot
            raise _ffi.ShapeError(_ffi.RST_ERR_SHAPE, "%d rows requested from a slot of %d rows"
                                  % (rows, self.max_rows))
        px = _ffi.c_double_p()
        pl = ctypes.POINTER(ctypes.c_uint32)()
        _ffi.check(self.engine.lib.rst_stager_acquire_host(self.handle, ctypes.byref(px), ctypes.byref(pl)))
        return (np.ctypeslib.as_array(px, shape=(rows, self.x_cols)),
                np.ctypeslib.as_array(pl, shape=(rows,)))

    def commit(self, rows):
        _ffi.check(self.engine.lib.rst_stager_commit_labels(self.handle, int(rows)))

    def next(self):
        """(x, truth) device arrays of the oldest submitted batch (borrowed from the stager)."""
        xp, tp, rows = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_size_t()
        _ffi.check(self.engine.lib.rst_stager_next(self.handle, ctypes.byref(xp), ctypes.byref(tp),
                                                   ctypes.byref(rows)))
        return (Array2(self.engine, rows.value, self.x_cols, ptr=xp.value, owner=self),
                Array2(self.engine, rows.value, self.classes, ptr=tp.value, owner=self))
