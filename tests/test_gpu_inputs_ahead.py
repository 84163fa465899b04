"""rst_model_loss_accuracy_to: the loss and the accuracy of a model's logits, with the input gradients of
the upper layers launched behind the loss before the host waits for it (what the compiled Sequential
of the host mirrors does in a training loop).  Through the C ABI, against the same calls without that:
every gradient and every parameter to the bit, whatever happens to the gradient array in between."""
import ctypes

import numpy as np
import pytest

from test_gpu_sequential import README_MLP, batch_data, make_weights

pytestmark = pytest.mark.gpu

ODD_MLP = [("identity",), ("linear", 785, 101), ("relu",), ("linear", 101, 101), ("relu",), ("linear", 101, 11)]
WIDE = [("linear", 300, 2048), ("relu",), ("linear", 2048, 2048), ("relu",), ("linear", 2048, 10)]
TRAILING_RELU = [("linear", 30, 20), ("relu",), ("linear", 20, 8), ("relu",)]
CASES = [("readme_b32", README_MLP, 32), ("readme_b500", README_MLP, 500), ("readme_b8192", README_MLP, 8192),
         ("odd_b33", ODD_MLP, 33), ("wide_b256", WIDE, 256), ("trailing_relu_b16", TRAILING_RELU, 16)]


def _steps(rs, engine, oracle, spec, batch, how, steps=3):
    """how: 'plain' - rst_cross_entropy_accuracy; 'ahead' - rst_model_loss_accuracy_to with the input
    gradients ahead; 'discard' - the same, then rst_model_discard_inputs; 'other' - the same, but
    another gradient array goes into the backward pass; 'want_input' - ahead, and the backward pass
    also returns the gradient with respect to the model's input; 'loss_only' - ahead, no accuracy."""
    from rstorch_amd import _ffi
    lib = engine.lib
    dm = rs.DeviceModel(spec)
    dm.load_parameters(make_weights(oracle, spec, 123))
    out = []
    for step in range(steps):
        x, y = batch_data(oracle, batch, dm.in_width, dm.out_width, 7, step, False)
        xd, yd = engine.from_numpy(x), engine.from_numpy(y)
        logits = engine.empty(batch, dm.out_width)
        grad = engine.empty(batch, dm.out_width)
        gin = engine.empty(batch, dm.in_width) if how == "want_input" else None
        loss, acc = ctypes.c_double(), ctypes.c_double()
        _ffi.check(lib.rst_model_forward_to(dm.handle, xd.ptr, batch, logits.ptr))
        if how == "plain":
            _ffi.check(lib.rst_cross_entropy_accuracy(engine.handle, logits.ptr, yd.ptr, grad.ptr, batch, dm.out_width,
                                                      ctypes.byref(loss), ctypes.byref(acc)))
        elif how == "loss_only":  # (no accuracy asked for: what the Python mirror's loss does)
            _ffi.check(lib.rst_model_loss_accuracy_to(dm.handle, logits.ptr, yd.ptr, grad.ptr, 1, ctypes.byref(loss), None))
        else:
            _ffi.check(lib.rst_model_loss_accuracy_to(dm.handle, logits.ptr, yd.ptr, grad.ptr, 1,
                                                      ctypes.byref(loss), ctypes.byref(acc)))
        used = grad
        if how == "discard":
            _ffi.check(lib.rst_model_discard_inputs(dm.handle))
        if how == "other":  # (its own copy of the same numbers, at another address)
            used = engine.from_numpy(grad.to_numpy())
        _ffi.check(lib.rst_model_backward_to(dm.handle, used.ptr, gin.ptr if gin is not None else None, 1, 0.05))
        out.append((loss.value, acc.value, [(p.to_numpy(), g.to_numpy()) for p, g in dm.parameters()],
                    gin.to_numpy() if gin is not None else None))
    return out


@pytest.mark.parametrize("name,spec,batch", CASES, ids=[c[0] for c in CASES])
def test_input_gradients_ahead_change_no_bit(engine, oracle, name, spec, batch):
    import rstorch_amd as rs
    want = _steps(rs, engine, oracle, spec, batch, "plain")
    for how in ("ahead", "discard", "other", "want_input", "loss_only"):
        got = _steps(rs, engine, oracle, spec, batch, how)
        for step, ((l0, a0, p0, _), (l1, a1, p1, _)) in enumerate(zip(want, got)):
            assert l0 == l1 and (a0 == a1 or how == "loss_only"), (how, step)
            for (w0, g0), (w1, g1) in zip(p0, p1):
                assert np.array_equal(w0, w1) and np.array_equal(g0, g1), (how, step)
    # the gradient with respect to the input: the same with and without the upper layers ahead
    from rstorch_amd import _ffi
    a = _steps(rs, engine, oracle, spec, batch, "want_input", steps=1)[0][3]
    dm = rs.DeviceModel(spec)
    dm.load_parameters(make_weights(oracle, spec, 123))
    x, y = batch_data(oracle, batch, dm.in_width, dm.out_width, 7, 0, False)
    dm.forward(engine.from_numpy(x))
    dm.loss(engine.from_numpy(y))
    b = dm.backward(None, need_input_grad=True).to_numpy()
    assert np.array_equal(a, b)


def test_loss_accuracy_to_wants_the_models_own_logits(engine, oracle):
    import rstorch_amd as rs
    from rstorch_amd import _ffi
    dm = rs.DeviceModel(README_MLP)
    dm.load_parameters(make_weights(oracle, README_MLP, 5))
    x, y = batch_data(oracle, 16, 784, 10, 3, 0, False)
    xd, yd = engine.from_numpy(x), engine.from_numpy(y)
    logits, other, grad = engine.empty(16, 10), engine.zeros(16, 10), engine.empty(16, 10)
    loss, acc = ctypes.c_double(), ctypes.c_double()
    args = (yd.ptr, grad.ptr, 1, ctypes.byref(loss), ctypes.byref(acc))
    with pytest.raises(rs.StateError):  # no forward pass yet
        _ffi.check(engine.lib.rst_model_loss_accuracy_to(dm.handle, logits.ptr, *args))
    _ffi.check(engine.lib.rst_model_forward_to(dm.handle, xd.ptr, 16, logits.ptr))
    with pytest.raises(rs.StateError):  # somebody else's array
        _ffi.check(engine.lib.rst_model_loss_accuracy_to(dm.handle, other.ptr, *args))
    _ffi.check(engine.lib.rst_model_loss_accuracy_to(dm.handle, logits.ptr, *args))
    want_loss, _ = oracle.cross_entropy_forward(logits.to_numpy(), y)
    assert abs(loss.value - want_loss) <= 1e-12 * abs(want_loss)
    assert acc.value == oracle.accuracy(logits.to_numpy(), y)
