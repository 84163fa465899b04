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
    # Backward from the loss.  The input gradient of a row depends on that row alone, so the same
    # sample of rows goes forward and backward through the oracle with the full-size weights.
    gin = dm.backward(None, need_input_grad=True).to_numpy()
    assert gin.shape == (batch, n_in)
    prob = np.exp(logits - lse[:, None])
    g_loss = prob - y.to_numpy()  # cross_entropy.rs:46
    ref = _oracle_with_device_weights(oracle, dm, spec)
    oracle.set_threads(8)
    try:
        ref.forward(x.to_numpy()[rows])
        want_gin = ref.backward(g_loss[rows])
    finally:
        oracle.set_threads(1)
    del ref
    assert rel_err(gin[rows], want_gin) <= 1e-10
    # the head's bias gradient is the column mean of the loss gradient (linear.rs:65-67)
    head_db = dm.parameters()[-1][1].to_numpy()
    assert rel_err(head_db, g_loss.sum(axis=0, keepdims=True) / batch) <= 1e-10
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


# The exact products of the headline configuration (hidden layer and head of C4, batch 1024) and of
# C2's widest layer, through Linear::forward / Linear::backward with the ReLU fused on both sides.
# The oracle side is numpy float64 on SAMPLED rows: 32 rows of the output (x[rows] . W^T + b), 32 rows
# of dW ((G[:, js]^T . x) / B), 32 rows of dX (G[rows] . W), db in full.
@pytest.mark.parametrize("batch,k,n", [(1024, 4096, 4096), (1024, 4096, 32768), (2048, 4096, 4096),
                                       (2048, 1024, 4096), (2048, 4096, 1000)])
def test_benchmark_products_sampled_values(engine, batch, k, n):
    import rstorch_amd as rs
    from rstorch_amd import _ffi
    seed = batch + k + n
    lib, h = engine.lib, engine.handle
    pre = engine.normal(batch, k, seed, 1)
    x = engine.empty(batch, k)
    _ffi.check(lib.rst_relu_forward(h, pre.ptr, x.ptr, x.size))  # the input came out of a ReLU
    w = engine.normal(n, k, seed, 2, 0.0, k ** -0.5)
    b = engine.normal(1, n, seed, 3)
    g = engine.normal(batch, n, seed, 4)
    out, gw, gb, gx = engine.empty(batch, n), engine.empty(n, k), engine.empty(1, n), engine.empty(batch, k)
    _ffi.check(lib.rst_linear_forward(h, x.ptr, w.ptr, b.ptr, out.ptr, batch, k, n, 1))
    _ffi.check(lib.rst_linear_backward(h, g.ptr, x.ptr, w.ptr, gw.ptr, gb.ptr, gx.ptr, x.ptr, batch, k, n))
    hx, hw, hb, hg = x.to_numpy(), w.to_numpy(), b.to_numpy(), g.to_numpy()
    rng = np.random.default_rng(seed)
    rows = np.unique(np.concatenate([[0, 1, 127, 128, batch - 1], rng.integers(0, batch, 27)]))
    js = np.unique(np.concatenate([[0, 1, 127, 128, n - 1], rng.integers(0, n, 27)]))
    got_out = out.to_numpy()
    want = np.maximum(hx[rows] @ hw.T + hb, 0.0)
    scale = np.max(np.abs(want))
    assert np.max(np.abs(got_out[rows] - want)) <= 1e-10 * scale
    got_gw = gw.to_numpy()
    want = hg[:, js].T @ hx / batch
    assert np.max(np.abs(got_gw[js] - want)) <= 1e-10 * np.max(np.abs(want))
    assert np.all(np.isfinite(got_gw)) and np.max(np.abs(got_gw)) <= 4 * np.max(np.abs(want))
    want = hg.sum(axis=0, keepdims=True) / batch
    assert np.max(np.abs(gb.to_numpy() - want)) <= 1e-10 * np.max(np.abs(want))
    got_gx = gx.to_numpy()
    want = (hg[rows] @ hw) * (hx[rows] > 0)
    assert np.max(np.abs(got_gx[rows] - want)) <= 1e-10 * np.max(np.abs(want))
    assert np.all(got_gx[hx <= 0] == 0.0)


# One fused step (SGD inside the weight-gradient launches, recorded and replayed as a graph) against
# the same step made of its parts (forward, loss, backward, SGD pass, plain launches) on a twin model,
# at the full size of the two large configurations: the loss, every gradient and every updated
# parameter must agree to the bit, on the recording call and on the first replay.
@pytest.mark.parametrize("name,spec,batch", [("C4", C4_SPEC, 1024), ("C2", C2_SPEC, 2048)])
def test_fused_graph_step_equals_piecewise_step_at_full_size(engine, name, spec, batch):
    import rstorch_amd as rs
    from rstorch_amd import _ffi
    fused, parts = rs.DeviceModel(spec), rs.DeviceModel(spec)
    fused.init_kaiming(0x5EED, 0)
    parts.init_kaiming(0x5EED, 0)
    x = engine.normal(batch, fused.in_width, 0x5EED, 1000)
    y = engine.one_hot(batch, fused.out_width, 0x5EED, 1001)
    w_before = fused.parameters()[0][0].to_numpy()
    for step in range(2):
        got = fused.train_step(x, y, 0.01)
        parts.forward(x)
        want = parts.loss(y)
        parts.backward(None, need_input_grad=False)
        parts.sgd_step(0.01)
        assert got == want, "step %d" % step
        for i, ((p, g), (q, h)) in enumerate(zip(fused.parameters(), parts.parameters())):
            assert np.array_equal(g.to_numpy(), h.to_numpy()), "gradient %d, step %d" % (i, step)
            assert np.array_equal(p.to_numpy(), q.to_numpy()), "parameter %d, step %d" % (i, step)
    # and the step did something: w1 = w0 - lr * dW with the gradient of the second step's predecessor
    assert abs(got - np.log(fused.out_width)) < 1.0
    assert not np.array_equal(fused.parameters()[0][0].to_numpy(), w_before)
    fused.close(); parts.close()


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
