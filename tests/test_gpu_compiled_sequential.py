"""The compiled Sequential (module interface over the device model): forward as one call,
backward deferred until the optimiser step or the first look at a gradient.  Whatever a caller can
observe must be what the layer-by-layer path computes - bit for bit where the two run the same tiles,
within rounding where a shared grid slices a long batch differently - and the reference's state
machine (src/module/sequential.rs:78-110, linear.rs:60-78) must hold in every order of calls."""
import gc

import numpy as np
import pytest

from conftest import rel_err
from test_gpu_sequential import README_MLP, batch_data, build_pair, make_weights

pytestmark = pytest.mark.gpu


def twins(rs, oracle, spec, seed):
    """The same network twice: compiled, and forced to run layer by layer; plus the oracle's."""
    weights = make_weights(oracle, spec, seed)
    fast, ref = build_pair(rs, oracle, spec, weights)
    slow, _ = build_pair(rs, oracle, spec, weights)
    slow.compile_enabled = False
    return fast, slow, ref


def params_np(model):
    return [(p.parm.to_numpy(), p.grad.to_numpy()) for p in model.parameters()]


SPECS = [
    ("readme_b32", README_MLP, 32, False, True),
    ("readme_b257", README_MLP, 257, False, True),
    ("ragged", [("linear", 13, 37), ("relu",), ("linear", 37, 5)], 19, True, True),
    ("relu_first_last", [("relu",), ("linear", 16, 32), ("identity",), ("relu",), ("relu",), ("linear", 32, 6),
                         ("relu",)], 10, True, True),
    ("wide", [("linear", 256, 512), ("relu",), ("linear", 512, 384), ("relu",), ("linear", 384, 250)], 192, True, True),
    # from a batch of about 4096 the shared weight-gradient grid cuts the batch into other slices
    ("readme_b8192", README_MLP, 8192, False, False),
]


@pytest.mark.parametrize("name,spec,batch,normal,exact", SPECS, ids=[s[0] for s in SPECS])
def test_readme_loop_compiled_equals_layer_by_layer(engine, oracle, name, spec, batch, normal, exact):
    import rstorch_amd as rs
    fast, slow, ref = twins(rs, oracle, spec, 0x5EED)
    n_in = [l for l in spec if l[0] == "linear"][0][1]
    n_out = [l for l in spec if l[0] == "linear"][-1][2]
    loss_f, loss_s = rs.CrossEntropyLoss.new(), rs.CrossEntropyLoss.new()
    opt_f, opt_s = rs.SGD.new(0.05), rs.SGD.new(0.05)
    same = np.array_equal if exact else (lambda a, b: rel_err(a, b) <= 1e-12)
    for step in range(4):
        x, y = batch_data(oracle, batch, n_in, n_out, 7, step % 2, normal)  # two batches in turn
        pf, ps = fast.forward(x), slow.forward(x)
        assert same(pf.to_numpy(), ps.to_numpy()), "logits, step %d" % step
        lf, ls = loss_f.forward(pf.clone(), y), loss_s.forward(ps.clone(), y)
        assert lf == ls if exact else abs(lf - ls) <= 1e-12 * abs(ls)
        assert rs.accuracy(pf, y) == rs.accuracy(ps, y)
        fast.backward(loss_f.backward())   # nothing is launched here ...
        slow.backward(loss_s.backward())
        if step == 2:                      # ... unless somebody looks: gradients before the step
            for (_, gf), (_, gs) in zip(params_np(fast), params_np(slow)):
                assert same(gf, gs), "gradient read between backward and step"
        opt_f.step(fast)                   # ... or here, with the update inside the launches
        opt_s.step(slow)
        for i, ((wf, gf), (ws, gs)) in enumerate(zip(params_np(fast), params_np(slow))):
            assert same(gf, gs), "gradient %d, step %d" % (i, step)
            assert same(wf, ws), "parameter %d, step %d" % (i, step)
        want = ref.train_step(x, y, 0.05)
        assert abs(lf - want) <= 1e-10 * abs(want)
    for (wf, _), (rp, _) in zip(params_np(fast), ref.parameters()):
        assert rel_err(wf, rp) <= 1e-10


@pytest.mark.parametrize("name,spec,batch", [("readme_b32", README_MLP, 32), ("readme_b257", README_MLP, 257),
                                             ("ragged", [("linear", 13, 37), ("relu",), ("linear", 37, 5)], 19)])
def test_training_loop_on_the_logits_themselves(engine, oracle, name, spec, batch):
    """loss.forward(pred, y) on the very array forward() returned: from the second step on the compiled
    form launches the upper layers' input gradients behind the loss, before the host has it.  Nothing
    observable changes - also when the gradient is looked at, replaced or rewritten on its way into
    backward(), or the loss is taken twice."""
    import rstorch_amd as rs
    fast, slow, _ = twins(rs, oracle, spec, 0xA11)
    n_in = [l for l in spec if l[0] == "linear"][0][1]
    n_out = [l for l in spec if l[0] == "linear"][-1][2]
    loss_f, loss_s = rs.CrossEntropyLoss.new(), rs.CrossEntropyLoss.new()
    opt_f, opt_s = rs.SGD.new(0.05), rs.SGD.new(0.05)
    for step in range(9):
        x, y = batch_data(oracle, batch, n_in, n_out, 9, step % 3, False)
        pf, ps = fast.forward(x), slow.forward(x)
        assert loss_f.forward(pf, y) == loss_s.forward(ps, y), step
        gf, gs = loss_f.backward(), loss_s.backward()
        if step == 8:    # a parameter is rewritten between the loss and the backward pass
            for m in (fast, slow):
                w = list(m.parameters())[-2].parm  # the last Linear's weight: its input gradient must see the new one
                w.assign(0.5 * w.to_numpy())
        if step == 3:    # somebody looks at the gradient
            assert np.array_equal(gf.to_numpy(), gs.to_numpy())
        if step == 4:    # somebody rewrites it in place
            half = 0.5 * gs.to_numpy()
            gf.assign(half)
            gs.assign(half)
        if step == 5:    # another array goes into backward
            gf = gs = engine.from_numpy(np.ones((batch, n_out)))
        if step == 6:    # the loss is taken a second time; its gradient is the one used
            assert loss_f.forward(pf, y) == loss_s.forward(ps, y)
            gf, gs = loss_f.backward(), loss_s.backward()
        kept_f, kept_s = fast.backward(gf), slow.backward(gs)
        if step == 7:    # the gradient with respect to the input is kept and read
            assert np.array_equal(kept_f.to_numpy(), kept_s.to_numpy())
        opt_f.step(fast)
        opt_s.step(slow)
        for i, ((wf, g1), (ws, g2)) in enumerate(zip(params_np(fast), params_np(slow))):
            assert np.array_equal(g1, g2), "gradient %d, step %d" % (i, step)
            assert np.array_equal(wf, ws), "parameter %d, step %d" % (i, step)


def test_the_input_gradient_is_computed_only_if_somebody_keeps_it(engine, oracle):
    import rstorch_amd as rs
    spec = [("linear", 24, 40), ("relu",), ("linear", 40, 6)]
    fast, slow, ref = twins(rs, oracle, spec, 3)
    x, y = batch_data(oracle, 48, 24, 6, 5, 0, True)
    g = oracle.fill_normal((48, 6), 5, 77)
    # kept and read before the step
    fast.forward(x); slow.forward(x)
    gin_f, gin_s = fast.backward(g), slow.backward(g)
    assert np.array_equal(gin_f.to_numpy(), gin_s.to_numpy())
    ref.forward(x)
    assert rel_err(gin_f.to_numpy(), ref.backward(g)) <= 1e-10
    # kept, but read only after the optimiser step has run: it was computed with the weights of before
    fast.forward(x); slow.forward(x)
    gin_f, gin_s = fast.backward(g), slow.backward(g)
    rs.SGD.new(0.1).step(fast); rs.SGD.new(0.1).step(slow)
    assert np.array_equal(gin_f.to_numpy(), gin_s.to_numpy())
    for (wf, gf), (ws, gs) in zip(params_np(fast), params_np(slow)):
        assert np.array_equal(wf, ws) and np.array_equal(gf, gs)
    # dropped: the pass still runs (the weights move), the first layer's input gradient is skipped
    fast.forward(x); slow.forward(x)
    fast.backward(g); slow.backward(g)
    gc.collect()
    rs.SGD.new(0.1).step(fast); rs.SGD.new(0.1).step(slow)
    for (wf, gf), (ws, gs) in zip(params_np(fast), params_np(slow)):
        assert np.array_equal(wf, ws) and np.array_equal(gf, gs)


def test_state_machine_of_the_compiled_form(engine, oracle):
    """Option::take() semantics (linear.rs:61, relu.rs:26): a consumed cache panics."""
    import rstorch_amd as rs
    spec = [("linear", 8, 16), ("relu",), ("linear", 16, 4)]
    model, _, _ = twins(rs, oracle, spec, 1)
    x, y = batch_data(oracle, 12, 8, 4, 2, 0, True)
    g = np.ones((12, 4))
    with pytest.raises(rs.StateError):
        model.backward(g)                 # before any forward (and before the model is compiled)
    with pytest.raises(rs.StateError):
        model.parameters()                # no gradient yet (linear.rs:73 unwraps None)
    model.forward(x)
    with pytest.raises(rs.StateError):
        model.parameters()
    with pytest.raises(rs.ShapeError):
        model.backward(np.ones((12, 5)))
    model.forward(x)                      # forward twice: the caches are simply overwritten
    model.backward(g)
    with pytest.raises(rs.StateError):
        model.backward(g)                 # consumed
    assert len(model.parameters()) == 4
    with pytest.raises(rs.ShapeError):
        model.forward(np.ones((3, 9)))
    # forward again without an optimiser step: the owed backward pass runs first, on the old caches
    model.forward(x)
    grads = [p.grad.to_numpy() for p in model.parameters()]
    model.forward(x)
    model.backward(2.0 * g)
    model.forward(x)                      # flushes the pass for 2g
    for p, before in zip(model.parameters(), grads):
        assert rel_err(p.grad.to_numpy(), 2.0 * before) <= 1e-12


def test_layer_list_mutation_drops_the_compiled_form(engine, oracle):
    """push / insert / remove at any time (sequential.rs:24-59): the weights move with the layers."""
    import rstorch_amd as rs
    spec = [("linear", 10, 20), ("relu",), ("linear", 20, 5)]
    fast, slow, _ = twins(rs, oracle, spec, 9)
    x, y = batch_data(oracle, 16, 10, 5, 4, 0, True)
    loss_f, loss_s = rs.CrossEntropyLoss.new(), rs.CrossEntropyLoss.new()

    def step(model, loss, opt):
        value = loss.forward(model.forward(x), y)
        model.backward(loss.backward())
        opt.step(model)
        return value

    opt_f, opt_s = rs.SGD.new(0.1), rs.SGD.new(0.1)
    assert step(fast, loss_f, opt_f) == step(slow, loss_s, opt_s)
    w_extra = oracle.fill_normal((5, 5), 1, 50, 0.0, 0.4)
    for m in (fast, slow):
        m.push(rs.ReLU.new())
        m.push(rs.Linear.new_with_kernel(5, 5, rs.FromArrays(w_extra, np.zeros((1, 5)))))
    for _ in range(2):
        assert step(fast, loss_f, opt_f) == step(slow, loss_s, opt_s)
    removed_f, removed_s = fast.remove(0), slow.remove(0)   # the first Linear leaves with its trained weights
    assert np.array_equal(removed_f.weight.to_numpy(), removed_s.weight.to_numpy())
    for m in (fast, slow):
        m.insert(0, rs.Linear.new_with_kernel(10, 20, rs.FromArrays(removed_s.weight.to_numpy(), removed_s.bias.to_numpy())))
        m.insert(1, rs.Identity.new())
    for _ in range(2):
        assert step(fast, loss_f, opt_f) == step(slow, loss_s, opt_s)
    for (wf, gf), (ws, gs) in zip(params_np(fast), params_np(slow)):
        assert np.array_equal(wf, ws) and np.array_equal(gf, gs)


class ClippedSGD:
    """A user-defined optimiser written against Parameter (src/module/mod.rs:16-19) and Optimizer
    (src/optim/mod.rs:6-8) only: element-wise gradient clipping on host copies."""

    def __init__(self, lr, clip):
        self.lr, self.clip = lr, clip

    def step(self, module):
        for p in module.parameters():
            g = np.clip(p.grad.to_numpy(), -self.clip, self.clip)
            p.parm.assign(p.parm.to_numpy() - self.lr * g)


def test_user_defined_optimizer_over_parameters(engine, oracle):
    """Parameter.parm / .grad are device arrays: to_numpy() is a copy taken after the work that
    produces it (never a live view), assign() writes through at once.  20 steps of a clipping
    optimiser written on those two calls match the same arithmetic on the oracle's parameters, and a
    recorded step graph sees parameters that were written this way."""
    import rstorch_amd as rs
    base = rs.Optimizer
    Clipped = type("Clipped", (base,), dict(ClippedSGD.__dict__))
    model, _, ref = twins(rs, oracle, README_MLP, 21)
    loss, opt = rs.CrossEntropyLoss.new(), Clipped(0.05, 0.01)
    for step in range(20):
        x, y = batch_data(oracle, 32, 784, 10, 8, step)
        got = loss.forward(model.forward(x), y)
        model.backward(loss.backward())
        opt.step(model)
        logits = ref.forward(x)
        want, prob = oracle.cross_entropy_forward(logits, y)
        ref.backward(oracle.cross_entropy_backward(prob, y))
        for p, g in ref.parameters():
            p[...] = p - 0.05 * np.clip(g, -0.01, 0.01)
        assert abs(got - want) <= 1e-9 * abs(want), "step %d" % step
    for p, (rp, _) in zip(model.parameters(), ref.parameters()):
        assert rel_err(p.parm.to_numpy(), rp) <= 1e-9
    # now the library's SGD on the same model: its graphs are recorded over the same arena ...
    sgd = rs.SGD.new(0.05)
    x, y = batch_data(oracle, 32, 784, 10, 8, 100)
    for _ in range(3):
        got = loss.forward(model.forward(x), y)
        model.backward(loss.backward())
        sgd.step(model)
        want = ref.train_step(x, y, 0.05)
        assert abs(got - want) <= 1e-9 * abs(want)
    # ... and a parameter written through assign() is what the next replay trains on
    for p, (rp, _) in zip(model.parameters(), ref.parameters()):
        rp[...] = 0.5 * rp
        p.parm.assign(rp)
    got = loss.forward(model.forward(x), y)
    model.backward(loss.backward())
    sgd.step(model)
    want = ref.train_step(x, y, 0.05)
    assert abs(got - want) <= 1e-9 * abs(want)
    for p, (rp, _) in zip(model.parameters(), ref.parameters()):
        assert rel_err(p.parm.to_numpy(), rp) <= 1e-9


def test_layers_that_cannot_be_compiled_run_layer_by_layer(engine, oracle):
    import rstorch_amd as rs
    w = make_weights(oracle, [("linear", 6, 6)], 2)
    model = rs.Sequential.new([rs.Linear.new_with_kernel(6, 6, rs.FromArrays(w[0], w[1])), rs.Softmax.new()])
    x = oracle.fill_normal((5, 6), 1, 1)
    out = model.forward(x).to_numpy()
    assert model._plan is None
    assert rel_err(out, oracle.softmax(oracle.linear_forward(x, w[0], w[1]))) <= 1e-10
    assert model.backward(np.ones((5, 6))).shape == (5, 6)
