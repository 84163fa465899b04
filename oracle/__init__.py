"""ctypes access to the CPU restatement of the rstorch training step (``liboracle.so``).

TEST INFRASTRUCTURE ONLY: this package is the checker the HIP path is compared with and
the CPU baseline that ``bench.py`` times.  Only ``tests/``, ``__graft_entry__.smoke()`` and
the ``cpu_baseline`` leg of ``bench.py`` may import it; the product package never does.

Every function here forwards to the C function of the same name in ``rstorch_oracle.c``,
which carries the reference citations.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

IDENTITY, LINEAR, RELU = 0, 1, 2

_c_double_p = ctypes.POINTER(ctypes.c_double)
_c_size_p = ctypes.POINTER(ctypes.c_size_t)


def build(force=False):
    """Compile ``liboracle.so`` with gcc (plain C, OpenMP only for the all-cores baseline)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "liboracle.so"])
    return _LIB_PATH


def _ptr(a):
    return a.ctypes.data_as(_c_double_p)


def _as2d(a):
    a = np.ascontiguousarray(a, dtype=np.float64)
    if a.ndim != 2:
        raise ValueError("expected a 2-D array, got shape %r" % (a.shape,))
    return a


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        build()
    L = ctypes.CDLL(_LIB_PATH)
    sz, dbl, dp, i32 = ctypes.c_size_t, ctypes.c_double, _c_double_p, ctypes.c_int
    u64 = ctypes.c_uint64
    sigs = {
        "rsto_set_threads": (None, [i32]),
        "rsto_get_threads": (i32, []),
        "rsto_linear_forward": (None, [dp, dp, dp, dp, sz, sz, sz]),
        "rsto_linear_backward": (None, [dp, dp, dp, dp, dp, dp, sz, sz, sz]),
        "rsto_relu_forward": (None, [dp, dp, sz]),
        "rsto_relu_backward": (None, [dp, dp, dp, sz]),
        "rsto_softmax": (i32, [dp, dp, sz, sz, i32]),
        "rsto_softmax_module_backward": (None, [dp, dp, dp, dp, sz, sz]),
        "rsto_cross_entropy_forward": (i32, [dp, dp, dp, sz, sz, dp]),
        "rsto_cross_entropy_backward": (None, [dp, dp, dp, sz]),
        "rsto_sgd_step": (None, [dp, dp, sz, dbl]),
        "rsto_accuracy": (dbl, [dp, dp, sz, sz]),
        "rsto_gemm_long_double": (None, [dp, dp, dp, sz, sz, sz, i32, i32]),
        "rsto_model_create": (ctypes.c_void_p, [ctypes.POINTER(i32), _c_size_p, _c_size_p, sz]),
        "rsto_model_destroy": (None, [ctypes.c_void_p]),
        "rsto_model_parameter_count": (sz, [ctypes.c_void_p]),
        "rsto_model_parameter": (i32, [ctypes.c_void_p, sz, ctypes.POINTER(dp), ctypes.POINTER(dp),
                                       _c_size_p, _c_size_p]),
        "rsto_model_forward": (dp, [ctypes.c_void_p, dp, sz]),
        "rsto_model_backward": (dp, [ctypes.c_void_p, dp]),
        "rsto_model_sgd_step": (None, [ctypes.c_void_p, dbl]),
        "rsto_model_train_step": (dbl, [ctypes.c_void_p, dp, dp, sz, dbl]),
        "rsto_model_last_loss_grad": (dp, [ctypes.c_void_p]),
        "rsto_rng_u64": (u64, [u64, u64, u64]),
        "rsto_fill_uniform": (None, [dp, sz, u64, u64, dbl, dbl]),
        "rsto_fill_normal": (None, [dp, sz, u64, u64, dbl, dbl]),
        "rsto_fill_one_hot": (None, [dp, sz, sz, u64, u64]),
    }
    for name, (res, args) in sigs.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


class NanLogits(Exception):
    """The reference panics (partial_cmp().unwrap()) when softmax meets a NaN."""


def set_threads(n):
    lib().rsto_set_threads(int(n))


def linear_forward(x, w, b=None):
    x, w = _as2d(x), _as2d(w)
    batch, k = x.shape
    n, k2 = w.shape
    assert k == k2, "shape mismatch"
    out = np.empty((batch, n), dtype=np.float64)
    if b is not None:
        b = _as2d(b)
        assert b.shape == (1, n)
    lib().rsto_linear_forward(_ptr(x), _ptr(w), _ptr(b) if b is not None else None, _ptr(out),
                              batch, k, n)
    return out


def linear_backward(g, x, w, need_gx=True):
    g, x, w = _as2d(g), _as2d(x), _as2d(w)
    batch, n = g.shape
    k = x.shape[1]
    assert x.shape[0] == batch and w.shape == (n, k)
    gw = np.empty((n, k), dtype=np.float64)
    gb = np.empty((1, n), dtype=np.float64)
    gx = np.empty((batch, k), dtype=np.float64) if need_gx else None
    lib().rsto_linear_backward(_ptr(g), _ptr(x), _ptr(w), _ptr(gw), _ptr(gb),
                               _ptr(gx) if need_gx else None, batch, k, n)
    return gw, gb, gx


def relu_forward(x):
    x = _as2d(x)
    out = np.empty_like(x)
    lib().rsto_relu_forward(_ptr(x), _ptr(out), x.size)
    return out


def relu_backward(g, x):
    g, x = _as2d(g), _as2d(x)
    out = np.empty_like(x)
    lib().rsto_relu_backward(_ptr(g), _ptr(x), _ptr(out), x.size)
    return out


def softmax(x, axis=1):
    x = _as2d(x)
    out = np.empty_like(x)
    if lib().rsto_softmax(_ptr(x), _ptr(out), x.shape[0], x.shape[1], axis) != 0:
        raise NanLogits()
    return out


def softmax_module_backward(grad, out):
    grad, out = _as2d(grad), _as2d(out)
    assert grad.shape == out.shape
    gin = np.empty_like(out)
    jac = np.empty((out.shape[1], out.shape[1]), dtype=np.float64)
    lib().rsto_softmax_module_backward(_ptr(grad), _ptr(out), _ptr(gin), _ptr(jac), out.shape[0],
                                       out.shape[1])
    return gin


def cross_entropy_forward(pred, truth):
    pred, truth = _as2d(pred), _as2d(truth)
    assert pred.shape == truth.shape
    prob = np.empty_like(pred)
    loss = ctypes.c_double()
    rc = lib().rsto_cross_entropy_forward(_ptr(pred), _ptr(truth), _ptr(prob), pred.shape[0],
                                          pred.shape[1], ctypes.byref(loss))
    if rc != 0:
        raise NanLogits()
    return loss.value, prob


def cross_entropy_backward(prob, truth):
    prob, truth = _as2d(prob), _as2d(truth)
    g = np.empty_like(prob)
    lib().rsto_cross_entropy_backward(_ptr(prob), _ptr(truth), _ptr(g), prob.size)
    return g


def sgd_step(parm, grad, lr):
    """Returns the updated copy of ``parm``."""
    p = np.array(parm, dtype=np.float64, order="C", copy=True)
    g = np.ascontiguousarray(grad, dtype=np.float64)
    assert p.shape == g.shape
    lib().rsto_sgd_step(_ptr(p), _ptr(g), p.size, float(lr))
    return p


def accuracy(pred, truth):
    pred, truth = _as2d(pred), _as2d(truth)
    return lib().rsto_accuracy(_ptr(pred), _ptr(truth), pred.shape[0], pred.shape[1])


def gemm_long_double(a, b, m, n, k, a_kc, b_kc):
    a = np.ascontiguousarray(a, dtype=np.float64)
    b = np.ascontiguousarray(b, dtype=np.float64)
    c = np.empty((m, n), dtype=np.float64)
    lib().rsto_gemm_long_double(_ptr(a), _ptr(b), _ptr(c), m, n, k, int(a_kc), int(b_kc))
    return c


def rng_u64(seed, stream, index):
    return lib().rsto_rng_u64(seed, stream, index)


def fill_uniform(shape, seed, stream, lo=0.0, hi=1.0):
    out = np.empty(shape, dtype=np.float64)
    lib().rsto_fill_uniform(_ptr(out), out.size, seed, stream, lo, hi)
    return out


def fill_normal(shape, seed, stream, mean=0.0, std=1.0):
    out = np.empty(shape, dtype=np.float64)
    lib().rsto_fill_normal(_ptr(out), out.size, seed, stream, mean, std)
    return out


def fill_one_hot(rows, cols, seed, stream):
    out = np.empty((rows, cols), dtype=np.float64)
    lib().rsto_fill_one_hot(_ptr(out), rows, cols, seed, stream)
    return out


class Model:
    """The Sequential restatement: a list of ("identity",) / ("linear", in, out) / ("relu",)."""

    def __init__(self, layers):
        self.spec = [tuple(l) if not isinstance(l, str) else (l,) for l in layers]
        kind_of = {"identity": IDENTITY, "linear": LINEAR, "relu": RELU}
        n = len(self.spec)
        kinds = (ctypes.c_int * max(n, 1))()
        ins = (ctypes.c_size_t * max(n, 1))()
        outs = (ctypes.c_size_t * max(n, 1))()
        for i, l in enumerate(self.spec):
            kinds[i] = kind_of[l[0]]
            if l[0] == "linear":
                ins[i], outs[i] = l[1], l[2]
        self._h = lib().rsto_model_create(kinds, ins, outs, n)
        self._batch = 0
        self._in_width = next((l[1] for l in self.spec if l[0] == "linear"), 0)
        self._out_width = next((l[2] for l in reversed(self.spec) if l[0] == "linear"),
                               self._in_width)

    def __del__(self):
        if getattr(self, "_h", None):
            lib().rsto_model_destroy(self._h)
            self._h = None

    def parameters(self):
        """[(parm_view, grad_view)] as numpy views onto the oracle's own memory, reference order."""
        out = []
        for i in range(lib().rsto_model_parameter_count(self._h)):
            p, g = _c_double_p(), _c_double_p()
            r, c = ctypes.c_size_t(), ctypes.c_size_t()
            lib().rsto_model_parameter(self._h, i, ctypes.byref(p), ctypes.byref(g),
                                       ctypes.byref(r), ctypes.byref(c))
            shape = (r.value, c.value)
            out.append((np.ctypeslib.as_array(p, shape=shape), np.ctypeslib.as_array(g, shape=shape)))
        return out

    def forward(self, x):
        x = _as2d(x)
        assert x.shape[1] == self._in_width
        self._batch = x.shape[0]
        p = lib().rsto_model_forward(self._h, _ptr(x), x.shape[0])
        return np.ctypeslib.as_array(p, shape=(x.shape[0], self._out_width)).copy()

    def backward(self, grad):
        grad = _as2d(grad)
        p = lib().rsto_model_backward(self._h, _ptr(grad))
        return np.ctypeslib.as_array(p, shape=(self._batch, self._in_width)).copy()

    def sgd_step(self, lr):
        lib().rsto_model_sgd_step(self._h, float(lr))

    def train_step(self, x, truth, lr):
        x, truth = _as2d(x), _as2d(truth)
        self._batch = x.shape[0]
        return lib().rsto_model_train_step(self._h, _ptr(x), _ptr(truth), x.shape[0], float(lr))

    def last_loss_grad(self):
        p = lib().rsto_model_last_loss_grad(self._h)
        return np.ctypeslib.as_array(p, shape=(self._batch, self._out_width)).copy()
