"""The rows either side of the path: staged host batches (pinned double buffering, device one-hot)
and parameter export/import.  Data movement only: everything here is bit-exact."""
import os

import numpy as np
import pytest

from test_gpu_sequential import README_MLP, make_weights

pytestmark = pytest.mark.gpu


def test_staged_batches_arrive_intact_and_in_order(engine, oracle):
    import rstorch_amd as rs
    rows, cols, classes = 37, 19, 11
    st = rs.BatchStager(64, cols, classes, depth=3)
    rng = np.random.default_rng(0)
    sent = []
    for k in range(7):
        n = rows - k  # ragged batch sizes
        x = rng.standard_normal((n, cols)); lab = rng.integers(0, classes, n)
        if len(sent) - k + 3 <= 0:
            pass
        st.submit(x, labels=lab)
        sent.append((x, lab))
        if k >= 2:  # keep at most 3 in flight
            gx, gt = st.next()
            wx, wl = sent[k - 2]
            np.testing.assert_array_equal(gx.to_numpy(), wx)
            want = np.zeros((wx.shape[0], classes)); want[np.arange(wx.shape[0]), wl] = 1.0
            np.testing.assert_array_equal(gt.to_numpy(), want)
    with pytest.raises(rs.RstorchError):
        st.submit(np.zeros((3, cols)), labels=[0, 1, classes])  # label out of range
    with pytest.raises(rs.ShapeError):
        st.submit(np.zeros((65, cols)), labels=np.zeros(65))     # more rows than the slots hold


def test_dense_soft_labels_and_slot_exhaustion(engine):
    import rstorch_amd as rs
    st = rs.BatchStager(8, 4, 3, depth=2)
    x = np.arange(32.0).reshape(8, 4); t = np.full((8, 3), 1.0 / 3)
    st.submit(x, truth=t); st.submit(x + 1, truth=t)
    with pytest.raises(rs.StateError):
        st.submit(x, truth=t)  # both slots submitted, none taken
    a, b = st.next()
    np.testing.assert_array_equal(a.to_numpy(), x); np.testing.assert_array_equal(b.to_numpy(), t)
    a, _ = st.next()
    np.testing.assert_array_equal(a.to_numpy(), x + 1)
    with pytest.raises(rs.StateError):
        st.next()


def test_training_from_staged_inputs_equals_resident_inputs(engine, oracle):
    import rstorch_amd as rs
    weights = make_weights(oracle, README_MLP, 3)
    a = rs.DeviceModel(README_MLP); a.load_parameters(weights); a.graph_enable(True)   # one graph per slot
    b = rs.DeviceModel(README_MLP); b.load_parameters(weights)
    st = rs.BatchStager(32, 784, 10, depth=2)
    batches = []
    for k in range(10):
        x = oracle.fill_uniform((32, 784), 9, 2 * k)
        y = oracle.fill_one_hot(32, 10, 9, 2 * k + 1)
        batches.append((x, y, y.argmax(axis=1)))
    st.submit(batches[0][0], labels=batches[0][2])
    for k, (x, y, lab) in enumerate(batches):
        if k + 1 < len(batches):
            st.submit(batches[k + 1][0], labels=batches[k + 1][2])  # transfer overlaps this step
        dx, dy = st.next()
        la = a.train_step(dx, dy, 0.01)
        lb = b.train_step(x, y, 0.01)
        assert la == lb, "step %d" % k
    for (p, _), (q, _) in zip(a.parameters(), b.parameters()):
        np.testing.assert_array_equal(p.to_numpy(), q.to_numpy())


def test_fill_pinned_slot_in_place(engine):
    import rstorch_amd as rs
    st = rs.BatchStager(16, 5, 4, depth=2)
    for k in range(5):
        hx, hl = st.host_slot(12)
        hx[...] = np.arange(60.0).reshape(12, 5) + k
        hl[...] = np.arange(12) % 4
        st.commit(12)
        x, t = st.next()
        np.testing.assert_array_equal(x.to_numpy(), np.arange(60.0).reshape(12, 5) + k)
        np.testing.assert_array_equal(t.to_numpy(), np.eye(4)[np.arange(12) % 4])
    for rows in (0, 17, 1 << 40):  # views never reach beyond the 16-row pinned slot
        with pytest.raises(rs.ShapeError):
            st.host_slot(rows)
    st.close()


def test_checkpoint_round_trip(engine, oracle, tmp_path):
    import rstorch_amd as rs
    spec = [("identity",), ("linear", 13, 7), ("relu",), ("linear", 7, 5)]
    weights = make_weights(oracle, spec, 8)
    weights[1][...] = 0.25  # non-zero bias
    dm = rs.DeviceModel(spec); dm.load_parameters(weights)
    flat = dm.state()
    np.testing.assert_array_equal(flat, np.concatenate([w.ravel() for w in weights]))
    path = os.path.join(tmp_path, "ckpt.npz")
    dm.save(path)
    again = rs.DeviceModel.load(path)
    assert again.spec == dm.spec
    x = oracle.fill_normal((6, 13), 1, 1); y = oracle.fill_one_hot(6, 5, 1, 2)
    assert dm.train_step(x, y, 0.1) == again.train_step(x, y, 0.1)
    np.testing.assert_array_equal(dm.state(), again.state())
    with pytest.raises(rs.ShapeError):
        dm.load_state(np.zeros(3))
