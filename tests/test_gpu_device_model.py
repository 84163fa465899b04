"""The fused device-resident step (rst_model_*) against the oracle, including the shapes of
the benchmark configurations at sizes the oracle finishes in seconds."""
import numpy as np
import pytest

from conftest import rel_err
from test_gpu_sequential import README_MLP, batch_data, make_weights

pytestmark = pytest.mark.gpu
TOL = 1e-10


def pair(rs, oracle, spec, seed):
    weights = make_weights(oracle, spec, seed)
    dm = rs.DeviceModel(spec)
    dm.load_parameters(weights)
    ref = oracle.Model(spec)
    for (p, _), w in zip(ref.parameters(), weights):
        p[...] = w
    return dm, ref


CASES = [
    ("C0_readme_b32", README_MLP, 32, False, 0.01),
    ("C1_readme_b8192", README_MLP, 8192, False, 0.01),
    ("C2_wide_reduced", [("linear", 1024, 4096), ("relu",), ("linear", 4096, 4096), ("relu",),
                         ("linear", 4096, 1000)], 256, True, 0.01),
    ("C4_deep_reduced", [("linear", 512, 512), ("relu",)] * 8 + [("linear", 512, 4096)], 128, True, 0.01),
    ("ragged", [("identity",), ("linear", 33, 65), ("relu",), ("identity",), ("linear", 65, 129),
                ("relu",), ("linear", 129, 7)], 67, True, 0.05),
    # every extent odd: the shared grids with members that load singly (small batch), the K-sliced
    # 128x128 grid and the 64x64 tiles on 8-byte aligned pairs (long batch), and wide layers whose
    # gradients pair up on the tile DMA with the last row of the contraction kept back
    ("odd_readme_b33", [("identity",), ("linear", 785, 101), ("relu",), ("linear", 101, 101), ("relu",),
                        ("linear", 101, 11)], 33, False, 0.01),
    ("odd_readme_b8191", [("identity",), ("linear", 785, 101), ("relu",), ("linear", 101, 101), ("relu",),
                          ("linear", 101, 11)], 8191, False, 0.01),
    ("odd_wide_b1023", [("linear", 511, 2049), ("relu",), ("linear", 2049, 4095), ("relu",), ("linear", 4095, 2047),
                        ("relu",), ("linear", 2047, 999)], 1023, True, 0.01),
]


@pytest.mark.parametrize("name,spec,batch,normal,lr", CASES, ids=[c[0] for c in CASES])
def test_train_step_matches_oracle(engine, oracle, name, spec, batch, normal, lr):
    import rstorch_amd as rs
    dm, ref = pair(rs, oracle, spec, 0x5EED)
    oracle.set_threads(8)
    try:
        n_in, n_out = dm.in_width, dm.out_width
        x, y = batch_data(oracle, batch, n_in, n_out, 11, 0, normal)
        # piecewise first, to compare logits / gradients
        logits = dm.forward(x).to_numpy()
        want_logits = ref.forward(x)
        assert rel_err(logits, want_logits) <= TOL
        got_loss = dm.loss(y)
        want_loss, prob = oracle.cross_entropy_forward(want_logits, y)
        assert abs(got_loss - want_loss) <= TOL * abs(want_loss)
        gin = dm.backward(None, need_input_grad=True).to_numpy()
        want_gin = ref.backward(oracle.cross_entropy_backward(prob, y))
        assert rel_err(gin, want_gin) <= TOL
        for (_, g), (_, rg) in zip(dm.parameters(), ref.parameters()):
            assert g.shape == rg.shape and rel_err(g.to_numpy(), rg) <= TOL
        dm.sgd_step(lr)
        ref.sgd_step(lr)
        for (p, _), (rp, _) in zip(dm.parameters(), ref.parameters()):
            assert rel_err(p.to_numpy(), rp) <= TOL
        # then the single-call step, twice
        for step in (1, 2):
            x, y = batch_data(oracle, batch, n_in, n_out, 11, step, normal)
            got = dm.train_step(x, y, lr)
            want = ref.train_step(x, y, lr)
            assert abs(got - want) <= TOL * abs(want)
        for (p, _), (rp, _) in zip(dm.parameters(), ref.parameters()):
            assert rel_err(p.to_numpy(), rp) <= TOL
    finally:
        oracle.set_threads(1)


def test_hundred_fused_steps(engine, oracle):
    import rstorch_amd as rs
    dm, ref = pair(rs, oracle, README_MLP, 5)
    for step in range(100):
        x, y = batch_data(oracle, 32, 784, 10, 13, step)
        got = dm.train_step(x, y, 0.01)
        want = ref.train_step(x, y, 0.01)
        assert abs(got - want) <= 1e-8 * abs(want), "step %d" % step


def test_hundred_fused_steps_at_batch_8192(engine, oracle):
    """The 100-step criterion (loss within 1e-8 relative) on the README network at batch 8192, fresh
    inputs every step; the parameters after the run within 1e-8 as well."""
    import rstorch_amd as rs
    dm, ref = pair(rs, oracle, README_MLP, 6)
    oracle.set_threads(8)
    try:
        for step in range(100):
            x, y = batch_data(oracle, 8192, 784, 10, 17, step)
            got = dm.train_step(x, y, 0.01)
            want = ref.train_step(x, y, 0.01)
            assert abs(got - want) <= 1e-8 * abs(want), "step %d" % step
    finally:
        oracle.set_threads(1)
    for (p, _), (rp, _) in zip(dm.parameters(), ref.parameters()):
        assert rel_err(p.to_numpy(), rp) <= 1e-8


def test_basic_model_from_sequential(engine, oracle):
    """BasicModel::step (src/model.rs:19-27) == the layer-by-layer README loop."""
    import rstorch_amd as rs
    spec = [("linear", 20, 30), ("relu",), ("linear", 30, 4)]
    weights = make_weights(oracle, spec, 1)
    def seq():
        return rs.Sequential.new([rs.Linear.new_with_kernel(20, 30, rs.FromArrays(weights[0], weights[1])),
                                  rs.ReLU.new(),
                                  rs.Linear.new_with_kernel(30, 4, rs.FromArrays(weights[2], weights[3]))])
    loop_model, loss, optim = seq(), rs.CrossEntropyLoss.new(), rs.SGD.new(0.1)
    basic = rs.BasicModel.new(seq(), rs.CrossEntropyLoss.new(), rs.SGD.new(0.1))
    basic.device.fuse_head(False)
    fused = rs.BasicModel.new(seq(), rs.CrossEntropyLoss.new(), rs.SGD.new(0.1))  # the head as one launch
    for step in range(5):
        x, y = batch_data(oracle, 16, 20, 4, 3, step, True)
        l1 = loss.forward(loop_model.forward(x), y)
        loop_model.backward(loss.backward())
        optim.step(loop_model)
        l2 = basic.step(x, y, want_loss=True)
        assert l1 == l2  # same kernels, same order: bit-identical
        l3 = fused.step(x, y, want_loss=True)
        assert abs(l3 - l1) <= 1e-13 * abs(l1)  # the head's dot products add in another order
    for p, (q, _), (f, _) in zip(loop_model.parameters(), basic.device.parameters(), fused.device.parameters()):
        np.testing.assert_array_equal(p.parm.to_numpy(), q.to_numpy())
        assert rel_err(f.to_numpy(), q.to_numpy()) <= 1e-13
    np.testing.assert_array_equal(basic.predict(x).to_numpy(), loop_model.forward(x).to_numpy())


def test_state_machine_errors(engine):
    """Misuse that panics in the reference returns RST_ERR_STATE / RST_ERR_SHAPE, never UB."""
    import rstorch_amd as rs
    dm = rs.DeviceModel([("linear", 4, 3)])
    with pytest.raises(rs.StateError):
        dm.sgd_step(0.1)                      # step before backward (linear.rs:72 unwrap)
    with pytest.raises(rs.StateError):
        dm.backward(None)                     # backward before forward
    dm.forward(np.ones((2, 4)))
    with pytest.raises(rs.StateError):
        dm.backward(None)                     # loss gradient asked for before the loss
    dm.loss(np.eye(3)[:2])
    dm.backward(None)
    with pytest.raises(rs.StateError):
        dm.backward(None)                     # caches consumed
    dm.sgd_step(0.1)
    with pytest.raises(rs.ShapeError):
        dm.forward(np.ones((2, 5)))
    with pytest.raises(rs.ShapeError):
        rs.DeviceModel([("linear", 4, 3), ("linear", 5, 2)])
    z = np.zeros((2, 4)); z[0, 0] = np.nan
    with pytest.raises(rs.NanError):
        dm.train_step(z, np.eye(3)[:2], 0.1)


def test_profile_records_cover_every_launch(engine, oracle):
    import rstorch_amd as rs
    dm, _ = pair(rs, oracle, README_MLP, 2)
    dm.profile_enable(True)
    x, y = batch_data(oracle, 32, 784, 10, 1, 0)
    dm.train_step(x, y, 0.01)
    recs = dm.profile_read()
    kinds = [r["kernel"] for r in recs]
    # the last two Linears' forward and input gradients run inside the cross-entropy launch (the fused
    # tail of a small classifier); the first layer's input gradient is skipped
    assert kinds.count("linear_forward") == 1 and kinds.count("grad_weight") == 3
    assert kinds.count("grad_input") == 0
    # the optimiser rides in the weight-gradient launches unless asked to be a pass of its own
    assert kinds.count("cross_entropy") == 1 and kinds.count("sgd") == 0
    dm.fuse_head(1)   # the head alone
    dm.train_step(x, y, 0.01)
    kinds = [r["kernel"] for r in dm.profile_read()]
    assert kinds.count("linear_forward") == 2 and kinds.count("grad_input") == 1 and kinds.count("cross_entropy") == 1
    dm.fuse_head(False)
    dm.train_step(x, y, 0.01)
    kinds = [r["kernel"] for r in dm.profile_read()]
    assert kinds.count("linear_forward") == 3 and kinds.count("grad_input") == 2 and kinds.count("cross_entropy") == 1
    dm.fuse_head(True)
    assert "relu_forward" not in kinds and "relu_backward" not in kinds  # fused away
    assert all(r["ms"] > 0 for r in recs)
    dm.fuse_sgd(False)
    dm.train_step(x, y, 0.01)
    assert [r["kernel"] for r in dm.profile_read()].count("sgd") == 1
    dm.profile_enable(False)


GROUP_CASES = [
    ("readme_b32", README_MLP, 32, True),
    # Long batches: the weight gradients are cut into K slices, which share the reduction grid too.
    # From a batch of about 4096 the shared grid runs 128x128 tiles on slices of its own choice, so
    # the sums are taken in another order than in the per-layer launches: equal within rounding.
    ("readme_b8192", README_MLP, 8192, False),
    ("readme_b8200", README_MLP, 8200, False),  # batch not a multiple of the K step
    ("three_256_wide_b4096", [("linear", 256, 256), ("relu",), ("linear", 256, 256), ("relu",),
                              ("linear", 256, 10)], 4096, False),
    ("readme_b2048", README_MLP, 2048, True),
    ("readme_b500", README_MLP, 500, True),
    # more small layers than one shared grid holds (eight): two grids
    ("twelve_small_layers", [("linear", 20, 34), ("relu",)] + [("linear", 34, 34), ("relu",)] * 10 +
     [("linear", 34, 6)], 16, True),
    # a layer large enough for the 128x128 kernels between small ones, and an odd width (a member of
    # the shared grid that loads singly)
    ("mixed", [("linear", 64, 2048), ("relu",), ("linear", 2048, 2048), ("relu",), ("linear", 2048, 33),
               ("relu",), ("linear", 33, 10)], 64, True),
    # every extent odd: members that load singly (small batch) and the K-sliced 128x128 grid on
    # 8-byte aligned pairs (long batch)
    ("odd_readme_b33", [("identity",), ("linear", 785, 101), ("relu",), ("linear", 101, 101), ("relu",),
                        ("linear", 101, 11)], 33, True),
    ("odd_readme_b8191", [("identity",), ("linear", 785, 101), ("relu",), ("linear", 101, 101), ("relu",),
                          ("linear", 101, 11)], 8191, False),
]


@pytest.mark.parametrize("name,spec,batch,exact", GROUP_CASES, ids=[c[0] for c in GROUP_CASES])
@pytest.mark.parametrize("fused", [True, False])
def test_shared_grid_of_small_weight_gradients_equals_per_layer_launches(engine, oracle, name, spec, batch, exact, fused):
    """Small weight gradients share one grid at the end of backward; with profiling on every layer
    launches on its own.  Losses, parameters and gradients must agree: bit for bit where both paths
    slice the batch alike, to 1e-13 of the tensor's largest entry where the shared grid slices it
    differently (the first step's loss is bit-equal either way: it only depends on the forward pass)."""
    import rstorch_amd as rs
    models = [pair(rs, oracle, spec, 77)[0] for _ in range(2)]
    models[1].profile_enable(True)
    for dm in models:
        dm.fuse_sgd(fused)

    def same(a, b, what):
        if exact:
            assert np.array_equal(a, b), what
        else:
            assert np.max(np.abs(a - b)) <= 1e-13 * np.max(np.abs(b)), what

    for step in range(3):
        x, y = batch_data(oracle, batch, models[0].in_width, models[0].out_width, 5, step, True)
        losses = [dm.train_step(x, y, 0.05) for dm in models]
        if exact or step == 0:
            assert losses[0] == losses[1], "step %d" % step
        else:
            assert abs(losses[0] - losses[1]) <= 1e-13 * abs(losses[1]), "step %d" % step
        for (p, g), (q, h) in zip(models[0].parameters(), models[1].parameters()):
            same(p.to_numpy(), q.to_numpy(), "step %d" % step)
            same(g.to_numpy(), h.to_numpy(), "step %d" % step)
    kinds = [r["kernel"] for r in models[1].profile_read()]
    assert kinds.count("grad_weight") == 3 * sum(1 for l in spec if l[0] == "linear")
    models[1].profile_enable(False)


def test_graph_replay_equals_eager_launches(engine, oracle):
    """The captured step must give bit-identical results on every replay, with other eager work
    and synchronisations between replays, and must re-record when an argument changes."""
    import rstorch_amd as rs
    spec = README_MLP
    weights = make_weights(oracle, spec, 21)
    g = rs.DeviceModel(spec); g.load_parameters(weights); g.graph_enable(True)   # graph replay
    assert g.graph_active()
    e = rs.DeviceModel(spec); e.load_parameters(weights); e.graph_enable(False)
    other = rs.Linear.new(64, 64)
    x0, y0 = batch_data(oracle, 32, 784, 10, 5, 0)
    x1, y1 = batch_data(oracle, 32, 784, 10, 5, 1)
    dx0, dy0, dx1, dy1 = (engine.from_numpy(a) for a in (x0, y0, x1, y1))
    for step in range(12):
        x, y = (dx0, dy0) if step < 8 else (dx1, dy1)      # the change of batch re-records
        lr = 0.01 if step != 5 else 0.02                   # so does a change of lr
        lg = g.train_step(x, y, lr)
        other.forward(np.ones((8, 64)))                    # unrelated eager work on the stream
        engine.synchronize()
        le = e.train_step(x, y, lr)
        assert lg == le, "step %d" % step
    for (p, _), (q, _) in zip(g.parameters(), e.parameters()):
        np.testing.assert_array_equal(p.to_numpy(), q.to_numpy())
    # the graph path keeps the state machine of the eager path
    with pytest.raises(rs.StateError):
        g.backward(None)
    g.sgd_step(0.0)  # gradients exist


FUSE_CASES = [
    # tiny outputs (split-K with the ordered reduction), ragged tiles, a 128x128-tile problem that
    # takes the two-way split, and one that fills the chip without a split
    ("readme_b32", README_MLP, 32),
    ("readme_b4096", README_MLP, 4096),
    ("ragged", [("identity",), ("linear", 33, 65), ("relu",), ("identity",), ("linear", 65, 129),
                ("relu",), ("linear", 129, 7)], 67),
    ("two_way_split", [("linear", 24576, 2048), ("relu",), ("linear", 2048, 24576)], 2048),
    ("two_way_split_weight_gradient", [("linear", 2048, 2048), ("relu",), ("linear", 2048, 2560)], 24576),
    ("full_grid", [("linear", 1024, 4096), ("relu",), ("linear", 4096, 4096), ("relu",),
                   ("linear", 4096, 1000)], 512),
]


@pytest.mark.parametrize("name,spec,batch", FUSE_CASES, ids=[c[0] for c in FUSE_CASES])
@pytest.mark.parametrize("graph", [False, True], ids=["eager", "graph"])
def test_sgd_in_weight_gradient_epilogue_is_bit_identical(engine, oracle, name, spec, batch, graph):
    """train_step with the optimiser inside the weight-gradient launches against the same step
    with SGD as its own pass: losses, parameters and gradients must agree to the bit."""
    import rstorch_amd as rs
    weights = make_weights(oracle, spec, 77)
    models = []
    for fused in (True, False):
        dm = rs.DeviceModel(spec)
        dm.load_parameters(weights)
        dm.fuse_sgd(fused)
        dm.graph_enable(graph)
        models.append(dm)
    x, y = batch_data(oracle, batch, models[0].in_width, models[0].out_width, 3, 0, True)
    xd, yd = engine.from_numpy(x), engine.from_numpy(y)
    for step in range(3):
        losses = [dm.train_step(xd, yd, 0.05) for dm in models]
        assert losses[0] == losses[1], "step %d" % step
        for (p, g), (q, h) in zip(models[0].parameters(), models[1].parameters()):
            assert np.array_equal(p.to_numpy(), q.to_numpy()), "step %d" % step
            assert np.array_equal(g.to_numpy(), h.to_numpy()), "step %d" % step


PAIR_CASES = [
    # layer widths at which the hidden input gradients are 256..511 tiles of 128x128 and the weight
    # gradients at least 256: the two share a grid; the ragged net never pairs (tiles too few)
    ("paired", [("linear", 2048, 2048), ("relu",)] * 3 + [("linear", 2048, 4096)], 2048),
    ("paired_ragged_edges", [("linear", 2050, 2046), ("relu",), ("linear", 2046, 2064), ("relu",),
                             ("linear", 2064, 2304)], 2064),
    # every extent odd: both products of a pair on 8-byte aligned tile DMA, the last row of each
    # contraction with the tail
    ("paired_odd", [("linear", 2047, 2049), ("relu",), ("linear", 2049, 2047), ("relu",), ("linear", 2047, 4095)], 2047),
    ("never_paired", README_MLP, 64),
]


@pytest.mark.parametrize("name,spec,batch", PAIR_CASES, ids=[c[0] for c in PAIR_CASES])
@pytest.mark.parametrize("fused", [True, False], ids=["sgd_fused", "sgd_separate"])
def test_paired_gradient_launches_are_bit_identical(engine, oracle, name, spec, batch, fused):
    """The weight gradient of a layer launched in one grid with the next layer's input gradient
    against the same launches one after the other: loss, parameters and gradients to the bit."""
    import rstorch_amd as rs
    weights = make_weights(oracle, spec, 91)
    models = []
    for paired in (True, False):
        dm = rs.DeviceModel(spec)
        dm.load_parameters(weights)
        dm.fuse_sgd(fused)
        dm.pair_gradients(paired)
        dm.graph_enable(False)
        models.append(dm)
    x, y = batch_data(oracle, batch, models[0].in_width, models[0].out_width, 5, 0, True)
    xd, yd = engine.from_numpy(x), engine.from_numpy(y)
    models[0].profile_enable(True)
    for step in range(2):
        losses = [dm.train_step(xd, yd, 0.05) for dm in models]
        assert losses[0] == losses[1], "step %d" % step
        for (p, g), (q, h) in zip(models[0].parameters(), models[1].parameters()):
            assert np.array_equal(p.to_numpy(), q.to_numpy()), "step %d" % step
            assert np.array_equal(g.to_numpy(), h.to_numpy()), "step %d" % step
    kinds = [r["kernel"] for r in models[0].profile_read()]
    n_linear = sum(1 for l in spec if l[0] == "linear")
    if name == "never_paired":
        assert "grad_pair" not in kinds
    else:
        # per step: the last layer's input gradient goes alone (nothing is pending yet), every other
        # wanted one rides with the weight gradient of the layer above, and the two lowest weight
        # gradients go alone (the first layer's input gradient is not computed)
        assert kinds.count("grad_pair") == 2 * (n_linear - 2)
        assert kinds.count("grad_input") == 2 and kinds.count("grad_weight") == 4
    models[0].profile_enable(False)
    # the piecewise backward (rst_model_backward) takes the same path
    for dm in models:
        dm.forward(xd); dm.loss(yd, want_value=False)
    gins = [dm.backward(None, need_input_grad=True).to_numpy() for dm in models]
    assert np.array_equal(gins[0], gins[1])


def test_recorded_step_survives_other_users_of_the_engine(engine, oracle):
    """A recorded step graph must not name a buffer that another caller on the same engine can
    reallocate: model A replays its graph, a 4096-row cross entropy and a second model grow the
    engine-side scratch, model A replays again - and stays bit-identical to a twin that launches
    its kernels one by one."""
    import ctypes
    import rstorch_amd as rs
    from rstorch_amd import _ffi
    spec = [("linear", 64, 48), ("relu",), ("linear", 48, 24)]
    weights = [oracle.fill_normal((48, 64), 3, 0, 0.0, 0.125), np.zeros((1, 48)),
               oracle.fill_normal((24, 48), 3, 2, 0.0, 0.15), np.zeros((1, 24))]
    x = engine.from_numpy(oracle.fill_normal((256, 64), 3, 10))
    y = engine.from_numpy(oracle.fill_one_hot(256, 24, 3, 11))
    a, twin = rs.DeviceModel(spec, engine), rs.DeviceModel(spec, engine)
    a.load_parameters(weights); twin.load_parameters(weights)
    a.graph_enable(True)
    twin.graph_enable(False)

    def both():
        la, lt = a.train_step(x, y, 0.05), twin.train_step(x, y, 0.05)
        assert la == lt
        for (p, _), (q, _) in zip(a.parameters(), twin.parameters()):
            np.testing.assert_array_equal(p.to_numpy(), q.to_numpy())

    both(); both()  # record, replay
    big = engine.normal(4096, 50, 3, 12)
    t = engine.one_hot(4096, 50, 3, 13)
    g = engine.empty(4096, 50)
    loss = ctypes.c_double()
    _ffi.check(engine.lib.rst_cross_entropy(engine.handle, big.ptr, t.ptr, g.ptr, None, 4096, 50,
                                            ctypes.byref(loss)))
    other = rs.DeviceModel(spec, engine)
    other.load_parameters(weights)
    xb = engine.normal(8192, 64, 3, 14)
    yb = engine.one_hot(8192, 24, 3, 15)
    other.train_step(xb, yb, 0.05)
    both(); both()
    other.close(); a.close(); twin.close()


# Heads far wider than the 2048 logits that the loss kernel keeps in registers (the two-walk kernel,
# ragged widths), through the model: logits, loss, loss gradient, input and bias gradients.
@pytest.mark.parametrize("batch,k,n", [(512, 64, 16386), (640, 48, 13000)])
def test_wide_head_loss_through_the_model(engine, oracle, batch, k, n):
    import ctypes
    import rstorch_amd as rs
    from rstorch_amd import _ffi
    spec = [("linear", k, n)]
    dm = rs.DeviceModel(spec)
    w = oracle.fill_normal((n, k), 21, 0, 0.0, 1.5 * k ** -0.5)
    b = oracle.fill_normal((1, n), 21, 1)
    dm.load_parameters([w, b])
    x = oracle.fill_normal((batch, k), 21, 2)
    rng = np.random.default_rng(n)
    y = np.zeros((batch, n))
    y[np.arange(batch), rng.integers(0, n, batch)] = 1.0
    y[3] = rng.random(n); y[3] /= y[3].sum()  # a soft-label row
    logits = dm.forward(x).to_numpy()
    oracle.set_threads(8)
    try:
        assert rel_err(logits, oracle.linear_forward(x, w, b)) <= TOL
    finally:
        oracle.set_threads(1)
    got = dm.loss(y)
    want, prob = oracle.cross_entropy_forward(logits, y)
    assert abs(got - want) <= TOL * abs(want)
    # the gradient the model keeps, against the oracle and against the operator-level call on the same logits
    dl, dy = engine.from_numpy(logits), engine.from_numpy(y)
    g2 = engine.empty(batch, n)
    l2 = ctypes.c_double()
    _ffi.check(engine.lib.rst_cross_entropy(engine.handle, dl.ptr, dy.ptr, g2.ptr, None, batch, n, ctypes.byref(l2)))
    assert abs(got - l2.value) <= 1e-13 * abs(want)
    gin = dm.backward(None, need_input_grad=True).to_numpy()
    g = oracle.cross_entropy_backward(prob, y)
    assert rel_err(gin, g @ w) <= TOL
    assert rel_err(dm.parameters()[1][1].to_numpy(), g.sum(axis=0, keepdims=True) / batch) <= TOL
    assert rel_err(g2.to_numpy(), g) <= TOL
    dm.close()


def test_wide_head_special_values(engine):
    """-inf and +inf logits and NaN come out as in the reference's max-then-sum order
    (softmax.rs:37-53): an all -inf row and a row holding +inf give NaN, NaN logits are an error."""
    import rstorch_amd as rs
    batch, k, n = 512, 32, 16384
    dm = rs.DeviceModel([("linear", k, n)])
    rng = np.random.default_rng(5)
    w = rng.standard_normal((n, k)) * 0.1
    x = rng.standard_normal((batch, k))
    y = np.eye(n)[rng.integers(0, n, batch)]
    b = np.zeros((1, n)); b[0, 100:9000] = -np.inf  # whole 128-column tiles of -inf: harmless
    dm.load_parameters([w, b])
    dm.forward(x)
    # probabilities of exactly 0 under a zero truth are 0 * ln 0 = NaN in the reference's loss
    # (cross_entropy.rs:38), while the gradient p - t stays finite
    assert np.isnan(dm.loss(y))
    logits = x @ w.T + b
    e = np.exp(logits - logits.max(axis=1, keepdims=True))
    g = e / e.sum(axis=1, keepdims=True) - y
    gin = dm.backward(None, need_input_grad=True).to_numpy()
    assert rel_err(gin, g @ w) <= TOL
    b[0, 5] = np.inf
    dm.load_parameters([w, b])
    dm.forward(x)
    assert np.isnan(dm.loss(y))  # exp(inf - inf)
    b[...] = -np.inf
    dm.load_parameters([w, b])
    dm.forward(x)
    assert np.isnan(dm.loss(y))  # 0 / 0
    w[7, 3] = np.nan
    dm.load_parameters([w, np.zeros((1, n))])
    dm.forward(x)
    with pytest.raises(rs.NanError):
        dm.loss(y)
    dm.close()


def test_train_step_nan_logits(engine, oracle):
    """NaN logits are an error (softmax.rs:38 panics) in the one-call step too; a NaN in the input
    does not get there: max(NaN, 0) = 0 in the first ReLU, as with f64::max."""
    import rstorch_amd as rs
    dm, ref = pair(rs, oracle, README_MLP, 3)
    x, y = batch_data(oracle, 32, 784, 10, 23, 0)
    x[4, 7] = np.nan
    got, want = dm.train_step(x, y, 0.01), ref.train_step(x, y, 0.01)
    assert np.isfinite(got) and abs(got - want) <= TOL * abs(want)
    params = dm.parameters()
    bias = params[-1][0].to_numpy()
    bias[0, 3] = np.nan
    params[-1][0].assign(bias)
    x[4, 7] = 0.5
    with pytest.raises(rs.NanError):
        dm.train_step(x, y, 0.01)


def test_launch_mode_follows_the_depth(engine, oracle):
    """By default the step of a shallow model is launched plainly and that of a model with eight Linear
    layers or more is replayed from a recorded graph; either can be forced; both give the same bits."""
    import rstorch_amd as rs
    shallow = rs.DeviceModel(README_MLP)
    assert not shallow.graph_active()
    shallow.graph_enable(True)
    assert shallow.graph_active()
    shallow.graph_enable("auto")
    assert not shallow.graph_active()
    deep_spec = [("linear", 24, 24), ("relu",)] * 7 + [("linear", 24, 5)]
    weights = make_weights(oracle, deep_spec, 4)
    deep = rs.DeviceModel(deep_spec); deep.load_parameters(weights)
    plain = rs.DeviceModel(deep_spec); plain.load_parameters(weights); plain.graph_enable(False)
    assert deep.graph_active() and not plain.graph_active()
    deep.profile_enable(True)
    assert not deep.graph_active()       # per-launch events need plain launches
    deep.profile_enable(False)
    for step in range(4):
        x, y = batch_data(oracle, 48, 24, 5, 41, step % 2, True)
        assert deep.train_step(x, y, 0.05) == plain.train_step(x, y, 0.05)
    for (p, _), (q, _) in zip(deep.parameters(), plain.parameters()):
        np.testing.assert_array_equal(p.to_numpy(), q.to_numpy())
