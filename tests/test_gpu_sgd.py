"""SGD::step on the GPU: bit-exact against the oracle and against numpy's `w - lr*g`
(both round the product, then the difference; src/optim/sgd.rs:23)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


class _Bag:
    """A module that only has parameters, to drive Optimizer::step."""

    def __init__(self, rs, engine, tensors):
        self.params = rs.Parameters()
        for w, g in tensors:
            self.params.add(engine.from_numpy(w), engine.from_numpy(g))

    def parameters(self):
        return self.params


@pytest.mark.parametrize("shapes", [
    [(1, 1)], [(2, 2), (1, 2)], [(100, 784), (1, 100), (100, 100), (1, 100), (10, 100), (1, 10)],
    [(3, 5), (1, 5), (7, 1), (1, 7), (513, 511)], [(2048, 2048), (1, 2048)] * 3,
])
def test_multi_tensor_step_bit_exact(engine, oracle, shapes):
    import rstorch_amd as rs
    rng = np.random.default_rng(len(shapes))
    tensors = [(rng.standard_normal(s) * 0.02, rng.standard_normal(s) * 1e-3) for s in shapes]
    bag = _Bag(rs, engine, tensors)
    lr = 0.01
    rs.SGD.new(lr).step(bag)
    for (w, g), p in zip(tensors, bag.parameters()):
        got = p.parm.to_numpy()
        np.testing.assert_array_equal(got, oracle.sgd_step(w, g, lr))
        np.testing.assert_array_equal(got, w - lr * g)
        np.testing.assert_array_equal(p.grad.to_numpy(), g)  # gradients untouched


def test_two_roundings_not_a_fused_multiply_add(engine):
    """Values chosen so that fma(-lr, g, w) differs from w - round(lr*g)."""
    import rstorch_amd as rs
    rng = np.random.default_rng(99)
    w = rng.standard_normal((64, 64))
    g = rng.standard_normal((64, 64))
    lr = 0.1
    import math
    fused = np.array([math.fma(-lr, gi, wi) if hasattr(math, "fma") else wi - lr * gi
                      for wi, gi in zip(w.ravel(), g.ravel())]).reshape(w.shape)
    bag = _Bag(rs, engine, [(w, g)])
    rs.SGD.new(lr).step(bag)
    got = next(iter(bag.parameters())).parm.to_numpy()
    np.testing.assert_array_equal(got, w - lr * g)
    if hasattr(math, "fma"):
        assert np.any(fused != got)


def test_reference_zero_gradient_case(engine):
    """src/optim/sgd.rs:34-43: zero input, zero gradient, step runs and leaves W unchanged."""
    import rstorch_amd as rs
    optim = rs.SGD.new(0.1)
    linear = rs.Linear.new(2, 2)
    w0 = linear.weight.to_numpy().copy()
    linear.forward(np.zeros((2, 2)))
    linear.backward(np.zeros((2, 2)))
    optim.step(linear)
    np.testing.assert_array_equal(linear.weight.to_numpy(), w0)
    np.testing.assert_array_equal(linear.bias.to_numpy(), np.zeros((1, 2)))


def test_flat_step_odd_count_and_repeat(engine, oracle):
    import ctypes
    from rstorch_amd import _ffi
    rng = np.random.default_rng(5)
    for n in (1, 2, 3, 511, 512, 513, 100001):
        w = rng.standard_normal((1, n)); g = rng.standard_normal((1, n))
        dw, dg = engine.from_numpy(w), engine.from_numpy(g)
        want = w
        for _ in range(3):
            _ffi.check(engine.lib.rst_sgd_step_flat(engine.handle, dw.ptr, dg.ptr, n, 0.01))
            want = oracle.sgd_step(want, g, 0.01)
        np.testing.assert_array_equal(dw.to_numpy(), want)
