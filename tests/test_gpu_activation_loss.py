"""ReLU, Identity, softmax and CrossEntropyLoss on the GPU against the oracle, the reference's
known answers and closed forms.  ReLU/Identity are selections: bit-exact.  softmax / loss:
max|got-want|/max|want| <= 1e-10 (exp/ln are the device library's, the oracle's are glibc's)."""
import json
import math
import os

import numpy as np
import pytest

from conftest import rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-10
KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))


def _softmax(engine, x):
    import ctypes
    from rstorch_amd import _ffi
    a = engine.from_numpy(x)
    out = engine.empty(a.rows, a.cols)
    _ffi.check(engine.lib.rst_softmax_rows(engine.handle, a.ptr, out.ptr, a.rows, a.cols))
    return out.to_numpy()


# ---- ReLU / Identity --------------------------------------------------------------------------
def test_relu_reference_known_answers(engine):
    import rstorch_amd as rs
    k = KATS["relu"]
    m = rs.ReLU.new()
    np.testing.assert_array_equal(m.forward(np.array(k["input"])).to_numpy(), np.array(k["forward"]))
    np.testing.assert_array_equal(m.backward(np.array(k["gradient"])).to_numpy(), np.array(k["backward"]))
    with pytest.raises(rs.StateError):
        m.backward(np.array(k["gradient"]))  # cache consumed (relu.rs:26)


@pytest.mark.parametrize("shape", [(1, 1), (3, 5), (32, 100), (257, 129), (1024, 4096)])
def test_relu_bit_exact(engine, oracle, shape):
    import rstorch_amd as rs
    rng = np.random.default_rng(shape[0] + shape[1])
    x = rng.standard_normal(shape)
    x[rng.random(shape) < 0.05] = 0.0
    x.flat[0] = -0.0
    g = rng.standard_normal(shape)
    m = rs.ReLU.new()
    np.testing.assert_array_equal(m.forward(x).to_numpy(), oracle.relu_forward(x))
    np.testing.assert_array_equal(m.backward(g).to_numpy(), oracle.relu_backward(g, x))


def test_relu_special_values(engine, oracle):
    """NaN -> 0 forward (f64::max), mask false for NaN; inf gradient * 0 mask = NaN (a multiply)."""
    import rstorch_amd as rs
    x = np.array([[np.nan, -np.inf, np.inf, 0.0, -0.0, 1e-320, -1e-320, 2.0]])
    g = np.array([[1.0, np.inf, np.inf, np.inf, 3.0, 4.0, 5.0, np.nan]])
    m = rs.ReLU.new()
    f = m.forward(x).to_numpy()
    np.testing.assert_array_equal(f, oracle.relu_forward(x))
    assert f[0, 0] == 0.0 and f[0, 2] == np.inf
    b = m.backward(g).to_numpy()
    np.testing.assert_array_equal(b, oracle.relu_backward(g, x))
    assert np.isnan(b[0, 1]) and np.isnan(b[0, 3]) and b[0, 2] == np.inf


def test_identity(engine):
    import rstorch_amd as rs
    x = np.array(KATS["identity"]["input"])
    m = rs.Identity.new()
    a = engine.from_numpy(x)
    assert m.forward(a) is a and m.backward(a) is a
    assert len(m.parameters()) == 0


# ---- softmax ------------------------------------------------------------------------------------
def test_softmax_reference_known_answer(engine):
    k = KATS["softmax_axis1"]
    p = _softmax(engine, np.array(k["input"]))
    assert np.all(np.abs(p.sum(axis=1) - np.array(k["row_sums"])) <= k["row_sum_tolerance"])
    assert p.sum() == k["total_exact"]  # the reference asserts exact equality (softmax.rs:92)


@pytest.mark.parametrize("rows,cols", [(1, 1), (3, 2), (32, 10), (33, 11), (8, 64), (5, 100),
                                       (17, 257), (64, 1000), (7, 1001), (9, 2048), (5, 2050), (6, 2051),
                                       (4, 4096), (3, 8190), (3, 12288), (2, 12301), (2, 32768),
                                       (2, 32770), (2, 40001), (1, 300000)])
def test_softmax_matches_oracle(engine, oracle, rows, cols):
    rng = np.random.default_rng(rows * 65537 + cols)
    x = rng.standard_normal((rows, cols)) * 3.0
    got = _softmax(engine, x)
    want = oracle.softmax(x)
    assert rel_err(got, want) <= TOL
    assert np.all(np.abs(got.sum(axis=1) - 1.0) <= 1e-12)


def test_softmax_uniform_power_of_two_is_exact(engine):
    for cols in (2, 16, 256, 4096, 32768):
        p = _softmax(engine, np.full((3, cols), 0.37))
        np.testing.assert_array_equal(p, np.full((3, cols), 1.0 / cols))


def test_softmax_shift_invariance(engine):
    rng = np.random.default_rng(11)
    x = rng.standard_normal((9, 50))
    np.testing.assert_array_equal(_softmax(engine, x + 64.0), _softmax(engine, (x + 64.0)))
    # shifting by a power of two keeps x - max exact, so the result is bit-identical
    np.testing.assert_array_equal(_softmax(engine, x), _softmax(engine, x + 0.0))
    big = _softmax(engine, x * 1e3)  # huge logits do not overflow
    assert np.all(np.isfinite(big)) and np.all(np.abs(big.sum(axis=1) - 1.0) <= 1e-12)


def test_softmax_nan_is_an_error(engine):
    import rstorch_amd as rs
    x = np.zeros((4, 12)); x[2, 7] = np.nan
    with pytest.raises(rs.NanError):
        _softmax(engine, x)
    # -inf is not NaN: partial_cmp succeeds and the maximum stays at the lowest finite double
    y = np.zeros((2, 6)); y[0, 1] = -np.inf
    p = _softmax(engine, y)
    assert p[0, 1] == 0.0 and abs(p[0].sum() - 1.0) < 1e-15


@pytest.mark.parametrize("cols", [2050, 4099, 16384, 33001])
def test_softmax_wide_rows_special_values(engine, oracle, cols):
    """Rows wider than 2048 logits are walked twice with a running maximum: the special values
    must come out as in the reference's max-then-sum order."""
    import rstorch_amd as rs
    rng = np.random.default_rng(cols)
    x = rng.standard_normal((6, cols))
    x[0, cols // 3] = -np.inf                      # contributes exp(-inf) = 0
    x[1, :] = -np.inf                              # all -inf: maximum stays at the lowest finite double, 0/0
    x[2, cols - 1] = 700.0                         # the maximum arrives last: every partial sum is rescaled
    x[3, 0] = 700.0                                # ... and first
    x[4, :] = np.sort(x[4, :])                     # ever growing maximum
    x[5, 5] = np.inf                               # inf - inf = NaN through the whole row (no NaN input)
    got = _softmax(engine, x)
    want = oracle.softmax(x)
    assert got[0, cols // 3] == 0.0
    assert np.all(np.isnan(got[1])) and np.all(np.isnan(want[1]))
    assert np.all(np.isnan(got[5])) and np.all(np.isnan(want[5]))
    ok = [0, 2, 3, 4]
    assert rel_err(got[ok], want[ok]) <= TOL
    assert np.all(np.abs(got[ok].sum(axis=1) - 1.0) <= 1e-12)
    y = x[:1].copy(); y[0, cols // 2] = np.nan
    with pytest.raises(rs.NanError):
        _softmax(engine, y)


# ---- the Softmax module (forward on both axes, batch-summed Jacobian backward) -----------------
def test_softmax_module_reference_known_answers(engine):
    import rstorch_amd as rs
    k1, k0 = KATS["softmax_axis1"], KATS["softmax_axis0"]
    out = rs.Softmax.new().forward(np.array(k1["input"])).to_numpy()
    assert np.all(np.abs(out.sum(axis=1) - 1.0) <= k1["row_sum_tolerance"]) and out.sum() == k1["total_exact"]
    out = rs.Softmax.with_axis(0).forward(np.array(k0["input"])).to_numpy()
    assert np.all(np.abs(out.sum(axis=0) - 1.0) <= k0["col_sum_tolerance"]) and out.sum() == k0["total_exact"]
    kb = KATS["softmax_module_backward"]
    m = rs.Softmax.new()
    m.forward(np.array(kb["input"]))
    got = m.backward(np.array(kb["gradient"])).to_numpy()
    assert np.all(np.abs(got - np.array(kb["expected"])) <= kb["tolerance"])
    with pytest.raises(rs.StateError):
        m.backward(np.array(kb["gradient"]))


@pytest.mark.parametrize("rows,cols,axis", [(3, 2, 1), (33, 11, 1), (64, 300, 1), (300, 64, 0), (7, 5, 0),
                                            (512, 1000, 1)])
def test_softmax_module_matches_oracle(engine, oracle, rows, cols, axis):
    import rstorch_amd as rs
    rng = np.random.default_rng(rows * 31 + cols + axis)
    x = rng.standard_normal((rows, cols)) * 2
    g = rng.standard_normal((rows, cols))
    m = rs.Softmax.with_axis(axis)
    out = m.forward(x).to_numpy()
    want = oracle.softmax(x, axis=axis)
    assert rel_err(out, want) <= TOL
    gin = m.backward(g).to_numpy()
    assert rel_err(gin, oracle.softmax_module_backward(g, want)) <= TOL


# ---- CrossEntropyLoss ---------------------------------------------------------------------------
@pytest.mark.parametrize("rows,cols", [(1, 2), (32, 10), (33, 11), (64, 100), (128, 1000),
                                       # either side of what one workgroup finishes on its own
                                       (64, 10), (65, 10), (16, 500), (17, 500), (4, 2000), (5, 2000),
                                       (9, 2048), (7, 2050), (5, 2051), (16, 4096), (6, 10000),
                                       (5, 12289), (4, 32768), (3, 33000), (2, 100001)])
def test_cross_entropy_matches_oracle(engine, oracle, rows, cols):
    import rstorch_amd as rs
    rng = np.random.default_rng(rows + 17 * cols)
    z = rng.standard_normal((rows, cols)) * 2.0
    t = np.zeros((rows, cols)); t[np.arange(rows), rng.integers(0, cols, rows)] = 1.0
    loss = rs.CrossEntropyLoss.new()
    got = loss.forward(z, t)
    want, prob = oracle.cross_entropy_forward(z, t)
    assert abs(got - want) <= TOL * abs(want)
    g = loss.backward().to_numpy()
    assert rel_err(g, oracle.cross_entropy_backward(prob, t)) <= TOL
    assert np.all(np.abs(g.sum(axis=1)) <= 1e-12)  # rows of prob - one_hot sum to 0
    with pytest.raises(rs.StateError):
        loss.backward()  # consumed (cross_entropy.rs:46)


def test_cross_entropy_soft_labels(engine, oracle):
    """truth need not be one-hot: every ln(prob) then contributes."""
    import rstorch_amd as rs
    rng = np.random.default_rng(21)
    z = rng.standard_normal((19, 37))
    t = rng.random((19, 37)); t /= t.sum(axis=1, keepdims=True)
    loss = rs.CrossEntropyLoss.new()
    got = loss.forward(z, t)
    want, prob = oracle.cross_entropy_forward(z, t)
    assert abs(got - want) <= TOL * abs(want)
    assert rel_err(loss.backward().to_numpy(), prob - t) <= TOL


@pytest.mark.parametrize("cols", [3000, 20000])
def test_cross_entropy_soft_labels_wide_rows(engine, oracle, cols):
    import rstorch_amd as rs
    rng = np.random.default_rng(cols)
    z = rng.standard_normal((5, cols)) * 3.0
    t = rng.random((5, cols)); t /= t.sum(axis=1, keepdims=True)
    loss = rs.CrossEntropyLoss.new()
    got = loss.forward(z, t)
    want, prob = oracle.cross_entropy_forward(z, t)
    assert abs(got - want) <= TOL * abs(want)
    assert rel_err(loss.backward().to_numpy(), prob - t) <= TOL


@pytest.mark.parametrize("cols", [4100, 16384])
def test_cross_entropy_wide_rows_underflow_and_nan(engine, oracle, cols):
    """The wide-row kernel keeps the reference's 0 * ln(0) = NaN and its NaN-logit error."""
    import rstorch_amd as rs
    rng = np.random.default_rng(cols)
    z = rng.standard_normal((3, cols))
    t = np.zeros((3, cols)); t[np.arange(3), [1, 2, 3]] = 1.0
    want, _ = oracle.cross_entropy_forward(z, t)
    got = rs.CrossEntropyLoss.new().forward(z, t)
    assert abs(got - want) <= TOL * abs(want)
    z[1, cols - 7] = -900.0  # probability underflows to 0 where truth is 0
    want, _ = oracle.cross_entropy_forward(z, t)
    got = rs.CrossEntropyLoss.new().forward(z, t)
    assert math.isnan(want) and math.isnan(got)
    z[1, cols - 7] = np.nan
    with pytest.raises(rs.NanError):
        rs.CrossEntropyLoss.new().forward(z, t)


def test_cross_entropy_closed_forms(engine):
    import rstorch_amd as rs
    rows, cols = 8, 64
    t = np.zeros((rows, cols)); t[np.arange(rows), np.arange(rows)] = 1.0
    # uniform logits: loss = ln C
    got = rs.CrossEntropyLoss.new().forward(np.full((rows, cols), 1.25), t)
    assert abs(got - math.log(cols)) <= 1e-14
    # one-hot truth: loss = mean(logsumexp(z) - z[target])
    rng = np.random.default_rng(2)
    z = rng.standard_normal((rows, cols))
    lse = np.log(np.exp(z - z.max(axis=1, keepdims=True)).sum(axis=1)) + z.max(axis=1)
    want = np.mean(lse - z[np.arange(rows), np.arange(rows)])
    got = rs.CrossEntropyLoss.new().forward(z, t)
    assert abs(got - want) <= 1e-13 * abs(want)


def test_cross_entropy_underflow_gives_nan_like_the_reference(engine, oracle):
    """A probability that underflows to 0 where truth is 0 makes 0 * ln(0) = NaN in the reference
    (cross_entropy.rs:38 takes ln of the probability); the kernel reproduces it."""
    import rstorch_amd as rs
    z = np.array([[0.0, -800.0, 1.0], [0.5, 0.25, 0.125]])
    t = np.array([[1.0, 0.0, 0.0], [0.0, 1.0, 0.0]])
    want, _ = oracle.cross_entropy_forward(z, t)
    got = rs.CrossEntropyLoss.new().forward(z, t)
    assert math.isnan(want) and math.isnan(got)


def test_cross_entropy_nan_logits_is_an_error(engine):
    import rstorch_amd as rs
    z = np.zeros((4, 10)); z[1, 3] = np.nan
    t = np.zeros((4, 10)); t[:, 0] = 1.0
    with pytest.raises(rs.NanError):
        rs.CrossEntropyLoss.new().forward(z, t)
    with pytest.raises(rs.ShapeError):
        rs.CrossEntropyLoss.new().forward(np.zeros((4, 10)), np.zeros((4, 9)))


def test_accuracy_first_maximum_wins(engine, oracle):
    import rstorch_amd as rs
    rng = np.random.default_rng(8)
    # (the three shapes from (9, 4096) on take the one-workgroup-per-row kernel for wide rows, the last three
    # the thread-per-row kernel for long batches of narrow rows)
    for rows, cols in [(32, 10), (100, 1000), (5, 70), (9, 4096), (40, 4100), (12, 32768), (3, 4097),
                       (9000, 10), (5000, 32), (4097, 17)]:
        pred = rng.integers(0, 4, size=(rows, cols)).astype(np.float64)  # many ties
        truth = np.zeros((rows, cols)); truth[np.arange(rows), rng.integers(0, cols, rows)] = 1.0
        truth[0, :] = 0.0
        truth[0, np.argmax(pred[0])] = 1.0
        if rows > 4:
            hit = rng.integers(0, cols, rows)          # rows whose single maximum sits on the label
            pred[np.arange(2, rows), hit[2:]] = 9.0
            truth[2:] = 0.0
            truth[np.arange(2, rows), hit[2:]] = 1.0
            pred[2, 0] = np.nan                         # a NaN in element 0 is never replaced (utils.rs:47-52)
            pred[3, cols // 2] = np.nan                 # anywhere else it never wins
        got, want = rs.accuracy(pred, truth), oracle.accuracy(pred, truth)
        assert got == want, (rows, cols, got, want)
        assert rows <= 4 or 0.0 < want < 1.0


# rst_cross_entropy_accuracy: the loss of rst_cross_entropy and the count of rst_accuracy after one
# wait.  One workgroup's worth of rows is counted inside the cross-entropy launch (first shapes), the
# others by the arg-max kernels that follow it on the stream.
@pytest.mark.parametrize("rows,cols", [(32, 10), (1, 2), (64, 64), (16, 512), (7, 33), (65, 10), (3000, 1000),
                                       (8192, 10), (40, 4100), (8, 32768),
                                       # several workgroups of rows of at most 64 threads: counted by the row
                                       # kernel, published by the reduction launch
                                       (300, 100), (5000, 64), (2000, 512), (1000, 33), (70, 257)])
def test_cross_entropy_with_accuracy_in_one_wait(engine, oracle, rows, cols):
    import ctypes
    from rstorch_amd import _ffi
    rng = np.random.default_rng(rows * 131 + cols)
    z = np.round(rng.standard_normal((rows, cols)) * 2.0, 1)      # coarse values: ties between columns happen
    labels = rng.integers(0, cols, rows)
    labels[: rows // 2] = z[: rows // 2].argmax(axis=1)           # half of the rows are hits
    t = np.zeros((rows, cols))
    t[np.arange(rows), labels] = 1.0
    if rows > 3 and cols > 3:
        t[1] = 0.0; t[1, [0, 2]] = 0.5                             # a soft-label row with a tie: column 0 wins
        z[2, :] = 0.25                                             # a row of equal logits: column 0 wins
    dz, dt = engine.from_numpy(z), engine.from_numpy(t)
    g1, g2 = engine.full(rows, cols, -3.0), engine.full(rows, cols, -4.0)
    loss1, loss2, acc1, acc2 = (ctypes.c_double(-1.0) for _ in range(4))
    _ffi.check(engine.lib.rst_cross_entropy(engine.handle, dz.ptr, dt.ptr, g1.ptr, None, rows, cols, ctypes.byref(loss1)))
    _ffi.check(engine.lib.rst_accuracy(engine.handle, dz.ptr, dt.ptr, rows, cols, ctypes.byref(acc1)))
    _ffi.check(engine.lib.rst_cross_entropy_accuracy(engine.handle, dz.ptr, dt.ptr, g2.ptr, rows, cols,
                                                     ctypes.byref(loss2), ctypes.byref(acc2)))
    assert loss2.value == loss1.value
    assert acc2.value == acc1.value == oracle.accuracy(z, t)
    np.testing.assert_array_equal(g2.to_numpy(), g1.to_numpy())
    want, _ = oracle.cross_entropy_forward(z, t)
    assert abs(loss2.value - want) <= 1e-10 * abs(want)
    # NaN logits: the status of rst_cross_entropy
    z[0, 0] = np.nan
    dz = engine.from_numpy(z)
    assert engine.lib.rst_cross_entropy_accuracy(engine.handle, dz.ptr, dt.ptr, g2.ptr, rows, cols, ctypes.byref(loss2),
                                                 ctypes.byref(acc2)) == _ffi.RST_ERR_NAN


def test_scalar_reads_keep_up_with_many_small_calls(engine, oracle):
    """The loss and the hit count are announced by a ticket that the host polls: 300 alternating
    calls on different data must each return their own result, never an earlier one."""
    import ctypes
    from rstorch_amd import _ffi
    rng = np.random.default_rng(5)
    cases = []
    for k in range(6):
        rows, cols = (32, 10) if k % 2 == 0 else (700, 12)
        z = rng.standard_normal((rows, cols)) * (1.0 + k)
        t = np.eye(cols)[rng.integers(0, cols, rows)]
        cases.append((rows, cols, engine.from_numpy(z), engine.from_numpy(t), oracle.cross_entropy_forward(z, t)[0],
                      oracle.accuracy(z, t)))
    g = engine.empty(700, 12)
    loss, acc = ctypes.c_double(), ctypes.c_double()
    for i in range(300):
        rows, cols, dz, dt, want_loss, want_acc = cases[i % 6]
        if i % 3 == 0:
            _ffi.check(engine.lib.rst_cross_entropy_accuracy(engine.handle, dz.ptr, dt.ptr, g.ptr, rows, cols,
                                                             ctypes.byref(loss), ctypes.byref(acc)))
        else:
            _ffi.check(engine.lib.rst_cross_entropy(engine.handle, dz.ptr, dt.ptr, g.ptr, None, rows, cols, ctypes.byref(loss)))
            _ffi.check(engine.lib.rst_accuracy(engine.handle, dz.ptr, dt.ptr, rows, cols, ctypes.byref(acc)))
        assert abs(loss.value - want_loss) <= 1e-10 * abs(want_loss), i
        assert acc.value == want_acc, i
