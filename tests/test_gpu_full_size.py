"""BASELINE.json's configurations at FULL size, checked through properties that do not need the
CPU oracle to redo the whole computation: row independence of the forward pass (the oracle runs
a sample of rows through the full-size weights), linearity of the backward pass, closed forms of
the loss, bit-exact SGD against numpy on all 268.6 M parameters."""
import numpy as np
import pytest

from conftest import rel_err

pytestmark = pytest.mark.gpu

C4_SPEC = [("linear", 4096, 4096), ("relu",)] * 8 + [("linear", 4096, 32768)]
C2_SPEC = [("linear", 1024, 4096), ("relu",), ("linear", 4096, 4096), ("relu",), ("linear", 4096, 1000)]


def _oracle_with_device_weights(oracle, dm, spec):
    ref = oracle.Model(spec)
    for (p, _), (q, _) in zip(ref.parameters(), dm.parameters()):
        p[...] = q.to_numpy()
    return ref


@pytest.mark.parametrize("name,spec,batch", [("C4", C4_SPEC, 1024), ("C2", C2_SPEC, 2048)])
def test_forward_and_loss_at_full_size(engine, oracle, name, spec, batch):
    import rstorch_amd as rs
    dm = rs.DeviceModel(spec)
    dm.init_kaiming(0x5EED, 0)
    n_in, n_out = dm.in_width, dm.out_width
    x = engine.normal(batch, n_in, 0x5EED, 1000)
    y = engine.one_hot(batch, n_out, 0x5EED, 1001)
    logits = dm.forward(x).to_numpy()
    # rows are independent: a sample of rows through the oracle with the same full-size weights
    rows = np.array([0, 1, batch // 3, batch // 2, batch - 2, batch - 1] + list(range(7, batch, batch // 10)))
    ref = _oracle_with_device_weights(oracle, dm, spec)
    oracle.set_threads(8)
    try:
        want = ref.forward(x.to_numpy()[rows])
    finally:
        oracle.set_threads(1)
    assert rel_err(logits[rows], want) <= 1e-10
    del ref
    # loss against the log-sum-exp closed form on the downloaded logits
    loss = dm.loss(y)
    target = y.to_numpy().argmax(axis=1)
    m = logits.max(axis=1)
    lse = np.log(np.exp(logits - m[:, None]).sum(axis=1)) + m
    want_loss = float(np.mean(lse - logits[np.arange(batch), target]))
    assert abs(loss - want_loss) <= 1e-10 * abs(want_loss)
    # the loss gradient is softmax - one_hot: rows sum to 0, entries in [-1, 1]
    gin = dm.backward(None, need_input_grad=True)
    assert gin.shape == (batch, n_in) and np.all(np.isfinite(gin.to_numpy()))
    dm.close()


def test_backward_is_linear_in_the_gradient_at_full_size(engine):
    """dW, db and dX are linear in the incoming gradient: backward(g1 + g2) = backward(g1) +
    backward(g2) on the C4 network at batch 1024 (each contraction sees its real shape)."""
    import rstorch_amd as rs
    dm = rs.DeviceModel(C4_SPEC)
    dm.init_kaiming(7, 0)
    x = engine.normal(1024, 4096, 7, 1000)
    g1 = engine.normal(1024, 32768, 7, 2000).to_numpy()
    g2 = engine.normal(1024, 32768, 7, 2001).to_numpy()
    watched = [0, 1, 8, 9, 16, 17]  # first, a middle and the head layer: weight and bias gradients

    def run(g):
        dm.forward(x)
        gin = dm.backward(g, need_input_grad=True).to_numpy()
        ps = dm.parameters()
        return gin, [ps[i][1].to_numpy() for i in watched]

    in1, gr1 = run(g1)
    in2, gr2 = run(g2)
    in12, gr12 = run(g1 + g2)
    assert rel_err(in12, in1 + in2) <= 1e-10
    for a, b, c in zip(gr12, gr1, gr2):
        assert rel_err(a, b + c) <= 1e-10
    # db is the column mean of the gradient that reaches the layer; for the head it is g itself
    head_db = gr1[-1]
    assert rel_err(head_db, g1.sum(axis=0, keepdims=True) / 1024.0) <= 1e-12
    dm.close()


def test_sgd_on_268m_parameters_is_bit_exact(engine):
    """configs[3]: 64 x (2048x2048 weight + 2048 bias), weights N(0, 0.02), gradients N(0, 1e-3),
    lr 0.01: one launch over the tensor list and one over the arena, both equal numpy's
    two-rounding w - lr*g on every element."""
    import ctypes
    from rstorch_amd import _ffi
    shapes = [(2048, 2048), (1, 2048)] * 64
    total = sum(r * c for r, c in shapes)
    assert total == 268566528
    parm = engine.normal(1, total, 3, 1, 0.0, 0.02)
    grad = engine.normal(1, total, 3, 2, 0.0, 1e-3)
    w0, g0 = parm.to_numpy(), grad.to_numpy()
    n = len(shapes)
    offs = np.concatenate([[0], np.cumsum([r * c for r, c in shapes])[:-1]])
    pp = (ctypes.c_void_p * n)(*[parm.ptr + 8 * int(o) for o in offs])
    gp = (ctypes.c_void_p * n)(*[grad.ptr + 8 * int(o) for o in offs])
    cnt = (ctypes.c_size_t * n)(*[r * c for r, c in shapes])
    _ffi.check(engine.lib.rst_sgd_step(engine.handle, pp, gp, cnt, n, 0.01))
    w1 = parm.to_numpy()
    want = w0 - 0.01 * g0
    assert np.array_equal(w1, want)
    _ffi.check(engine.lib.rst_sgd_step_flat(engine.handle, parm.ptr, grad.ptr, total, 0.01))
    assert np.array_equal(parm.to_numpy(), want - 0.01 * g0)
    assert np.array_equal(grad.to_numpy(), g0)
