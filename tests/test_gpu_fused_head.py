"""The classifier head as one launch inside the single-call step (rst_model_fuse_head): the last
Linear's forward (src/module/linear.rs:44-58), the cross entropy and its gradient
(src/loss/cross_entropy.rs:34-47), the Linear's input gradient under the preceding ReLU's mask
(linear.rs:68, relu.rs:25-28) and the final loss sum.  Checked against the oracle at 1e-10 and
against the same model run with the head as separate launches (equal within rounding)."""
import numpy as np
import pytest

from conftest import rel_err
from test_gpu_device_model import pair
from test_gpu_sequential import README_MLP, batch_data

pytestmark = pytest.mark.gpu
TOL = 1e-10

SPECS = {
    "readme": README_MLP,                                                # hidden 100 x 100 with the head, masks on both sides
    "head_only": [("linear", 20, 10)],                                   # the head is the first Linear: no input gradient
    "identity_then_head": [("identity",), ("linear", 7, 3), ("identity",)],
    "no_mask": [("linear", 12, 9), ("linear", 9, 16)],                   # a Linear feeds the head: gradient unmasked; it is the first Linear
    "relu_of_its_own": [("relu",), ("linear", 30, 21), ("identity",), ("relu",), ("linear", 21, 7)],
    "widest": [("linear", 64, 233), ("relu",), ("linear", 233, 16)],     # 16 classes on 233 inputs: the head alone
    "one_class": [("linear", 5, 8), ("relu",), ("linear", 8, 1)],
    "linear_in_front": [("linear", 20, 24), ("linear", 24, 18), ("relu",), ("linear", 18, 3)],   # hidden gradient unmasked
    "odd_extents": [("linear", 50, 111), ("relu",), ("linear", 111, 97), ("relu",), ("linear", 97, 13)],
    "limit": [("linear", 9, 112), ("relu",), ("linear", 112, 112), ("relu",), ("linear", 112, 16)],
    "hidden_too_wide": [("linear", 30, 200), ("relu",), ("linear", 200, 100), ("relu",), ("linear", 100, 10)],
}
CASES = [("readme", b) for b in (1, 5, 16, 17, 32, 100, 1000, 8192)] + \
        [(name, b) for name in SPECS if name != "readme" for b in (3, 48)]


@pytest.mark.parametrize("name,batch", CASES, ids=["%s_b%d" % c for c in CASES])
def test_fused_head_matches_oracle_and_separate_launches(engine, oracle, name, batch):
    import rstorch_amd as rs
    spec = SPECS[name]
    fused, ref = pair(rs, oracle, spec, 0xC1A55)
    apart, _ = pair(rs, oracle, spec, 0xC1A55)
    apart.fuse_head(False)
    head_alone, _ = pair(rs, oracle, spec, 0xC1A55)
    head_alone.fuse_head(1)
    oracle.set_threads(8)
    try:
        n_in, n_out = fused.in_width, fused.out_width
        for step in range(3):
            x, y = batch_data(oracle, batch, n_in, n_out, 23, step, True)
            got = fused.train_step(x, y, 0.05)
            other = apart.train_step(x, y, 0.05)
            middle = head_alone.train_step(x, y, 0.05)
            want = ref.train_step(x, y, 0.05)
            assert abs(got - want) <= TOL * abs(want), "step %d" % step
            assert abs(middle - want) <= TOL * abs(want), "step %d" % step
            assert abs(got - other) <= 1e-13 * abs(other), "step %d" % step
            for (p, g), (q, h), (u, v), (rp, rg) in zip(fused.parameters(), apart.parameters(),
                                                        head_alone.parameters(), ref.parameters()):
                assert rel_err(g.to_numpy(), rg) <= TOL
                assert rel_err(p.to_numpy(), rp) <= TOL
                assert rel_err(v.to_numpy(), rg) <= TOL
                assert rel_err(g.to_numpy(), h.to_numpy()) <= 1e-12
    finally:
        oracle.set_threads(1)


def test_fused_head_is_deterministic_and_replays(engine, oracle):
    """Two runs from the same state give the same bits (the loss is summed in a fixed order whichever
    workgroup arrives last), and the recorded graph gives what plain launches give, replay after replay."""
    import rstorch_amd as rs
    runs = []
    for graph in (True, False, True):
        dm, _ = pair(rs, oracle, README_MLP, 77)
        dm.graph_enable(graph)
        losses = []
        for step in range(6):
            x, y = batch_data(oracle, 1000, 784, 10, 29, step % 2)   # two batches in turn: two graphs, replayed
            losses.append(dm.train_step(x, y, 0.01))
        runs.append((losses, [p.to_numpy() for p, _ in dm.parameters()]))
    for losses, parms in runs[1:]:
        assert losses == runs[0][0]
        for a, b in zip(parms, runs[0][1]):
            np.testing.assert_array_equal(a, b)


def test_shapes_the_head_does_not_take_fall_back(engine, oracle):
    """17 classes, or a weight matrix that does not fit in LDS: the separate launches run, whatever
    the switch says, with the same bits as with the switch off."""
    import rstorch_amd as rs
    for spec in ([("linear", 10, 20), ("relu",), ("linear", 20, 17)],
                 [("linear", 10, 600), ("relu",), ("linear", 600, 10)]):
        a, _ = pair(rs, oracle, spec, 3)
        b, _ = pair(rs, oracle, spec, 3)
        b.fuse_head(False)
        x, y = batch_data(oracle, 40, 10, spec[-1][2], 31, 0, True)
        assert a.train_step(x, y, 0.1) == b.train_step(x, y, 0.1)
        for (p, _), (q, _) in zip(a.parameters(), b.parameters()):
            np.testing.assert_array_equal(p.to_numpy(), q.to_numpy())


def test_nan_logits_are_reported(engine, oracle):
    """NaN logits (here from a NaN input straight into the head; a ReLU would have turned it into 0, as
    f64::max does in relu.rs:21): RST_ERR_NAN as from the separate cross entropy (the reference panics in
    softmax.rs:38), and a clean step afterwards is clean."""
    import rstorch_amd as rs
    spec = [("linear", 20, 10)]
    dm, _ = pair(rs, oracle, spec, 9)
    x, y = batch_data(oracle, 64, 20, 10, 37, 0)
    bad = x.copy()
    bad[5, 3] = np.nan
    with pytest.raises(rs.NanError):
        dm.train_step(bad, y, 0.0)
    fresh, _ = pair(rs, oracle, spec, 9)
    assert np.isfinite(fresh.train_step(x, y, 0.01))
    with pytest.raises(rs.NanError):
        fresh.train_step(bad, y, 0.0)


def test_many_workgroups_and_many_launches(engine, oracle):
    """The loss hand-over at scale: a head alone on 40 000 rows (1250 workgroups of 32 rows, 18 inputs per
    lane) against the oracle, and 300 steps of the README network at batch 8192 on two models from the
    same state - every loss of the run the same bits on both (the arrival word is re-armed by each
    launch, whichever workgroup came last)."""
    import rstorch_amd as rs
    spec = [("linear", 64, 200), ("relu",), ("linear", 200, 10)]     # 200 inputs: too wide for the hidden variant
    dm, ref = pair(rs, oracle, spec, 12)
    oracle.set_threads(8)
    try:
        x, y = batch_data(oracle, 40000, 64, 10, 43, 0, True)
        got, want = dm.train_step(x, y, 0.05), ref.train_step(x, y, 0.05)
        assert abs(got - want) <= TOL * abs(want)
        for (p, g), (rp, rg) in zip(dm.parameters(), ref.parameters()):
            assert rel_err(g.to_numpy(), rg) <= TOL and rel_err(p.to_numpy(), rp) <= TOL
    finally:
        oracle.set_threads(1)
    a, _ = pair(rs, oracle, README_MLP, 13)
    b, _ = pair(rs, oracle, README_MLP, 13)
    x, y = batch_data(oracle, 8192, 784, 10, 47, 0)
    dx, dy = engine.from_numpy(x), engine.from_numpy(y)
    la = [a.train_step(dx, dy, 0.01) for _ in range(300)]
    lb = [b.train_step(dx, dy, 0.01) for _ in range(300)]
    assert la == lb
    assert la[-1] < la[0]
