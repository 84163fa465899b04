"""Pins the CPU oracle (oracle/rstorch_oracle.c) without the GPU: the reference's own known
answers, exact rational arithmetic on tiny shapes, numpy as a second opinion, closed forms,
invariants and finite differences - chosen so that a dropped term, a wrong sign or index or a
transposed operand fails at least one of them."""
import json
import math
import os
from fractions import Fraction

import numpy as np
import pytest

import oracle

KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))
TOL = KATS["assert_array_eq_default_tolerance"]  # the reference's assert_array_eq! default


# ---- the reference's known answers ----------------------------------------------------------
def test_linear_forward_kat():
    k = KATS["linear_forward"]
    out = oracle.linear_forward(k["input"], k["weight"], k["bias"])
    np.testing.assert_array_equal(out, np.array(k["output"]))


def test_linear_backward_kat():
    k = KATS["linear_backward"]
    gw, gb, gx = oracle.linear_backward(k["gradient"], k["input"], k["weight"])
    np.testing.assert_array_equal(gw, np.array(k["grad_weight"]))
    np.testing.assert_array_equal(gb, np.array(k["grad_bias"]))
    np.testing.assert_array_equal(gx, np.array(k["grad_input"]))
    assert gw.shape == np.array(k["weight"]).shape and gb.shape == np.array(k["bias"]).shape


def test_relu_kat():
    k = KATS["relu"]
    np.testing.assert_array_equal(oracle.relu_forward(k["input"]), np.array(k["forward"]))
    np.testing.assert_array_equal(oracle.relu_backward(k["gradient"], k["input"]), np.array(k["backward"]))


def test_softmax_kats():
    k = KATS["softmax_axis1"]
    p = oracle.softmax(k["input"], axis=1)
    assert np.all(np.abs(p.sum(axis=1) - np.array(k["row_sums"])) <= k["row_sum_tolerance"])
    assert p.sum() == k["total_exact"]
    k = KATS["softmax_axis0"]
    p = oracle.softmax(k["input"], axis=0)
    assert np.all(np.abs(p.sum(axis=0) - np.array(k["col_sums"])) <= k["col_sum_tolerance"])
    assert p.sum() == k["total_exact"]


def test_sgd_zero_gradient_kat():
    k = KATS["sgd_zero_gradient"]
    rng = np.random.default_rng(0)
    w = rng.standard_normal(k["linear"])
    np.testing.assert_array_equal(oracle.sgd_step(w, np.zeros_like(w), k["lr"]), w)


def test_sequential_kat_shapes():
    k = KATS["sequential"]
    m = oracle.Model([tuple(l) for l in k["layers"] if l[0] != "softmax"])
    rng = np.random.default_rng(1)
    for p, _ in m.parameters():
        p[...] = rng.standard_normal(p.shape)
    out = oracle.softmax(m.forward(np.array(k["input"])))  # the reference's net ends in Softmax
    assert out.shape == (2, 2) and np.all(np.abs(out.sum(axis=1) - 1) < 1e-15)
    gin = m.backward(oracle.softmax_module_backward(np.array(k["backward_gradient"]), out))
    assert gin.shape == (2, 3)
    shapes = [p.shape for p, _ in m.parameters()]
    assert shapes == [(10, 3), (1, 10), (100, 10), (1, 100), (2, 100), (1, 2)]  # weight, bias per layer


# ---- Linear: exact arithmetic, numpy, structure ---------------------------------------------
def _exact(rows):
    return [[Fraction(v) for v in r] for r in rows]


def _close_to_exact(got, exact, scale):
    for g, e, s in zip(np.ravel(got), [v for r in exact for v in r], [v for r in scale for v in r]):
        assert abs(Fraction(float(g)) - e) <= Fraction(1, 2 ** 50) * s + Fraction(1, 10 ** 300)


@pytest.mark.parametrize("b,k,n", [(1, 1, 1), (2, 3, 4), (5, 7, 3), (8, 8, 8), (7, 13, 6)])
def test_linear_against_exact_rationals(b, k, n):
    rng = np.random.default_rng(b * 100 + k * 10 + n)
    x, w = rng.standard_normal((b, k)), rng.standard_normal((n, k))
    bias, g = rng.standard_normal((1, n)), rng.standard_normal((b, n))
    X, W, Bv, G = _exact(x), _exact(w), _exact(bias), _exact(g)
    z = [[sum(X[i][p] * W[j][p] for p in range(k)) + Bv[0][j] for j in range(n)] for i in range(b)]
    zs = [[sum(abs(X[i][p] * W[j][p]) for p in range(k)) + abs(Bv[0][j]) for j in range(n)] for i in range(b)]
    _close_to_exact(oracle.linear_forward(x, w, bias), z, zs)
    gw, gb, gx = oracle.linear_backward(g, x, w)
    dw = [[sum(G[r][j] * X[r][p] for r in range(b)) / b for p in range(k)] for j in range(n)]
    dws = [[sum(abs(G[r][j] * X[r][p]) for r in range(b)) for p in range(k)] for j in range(n)]
    _close_to_exact(gw, dw, dws)
    db = [[sum(G[r][j] for r in range(b)) / b for j in range(n)]]
    dbs = [[sum(abs(G[r][j]) for r in range(b)) for j in range(n)]]
    _close_to_exact(gb, db, dbs)
    dx = [[sum(G[i][j] * W[j][p] for j in range(n)) for p in range(k)] for i in range(b)]  # NOT / b
    dxs = [[sum(abs(G[i][j] * W[j][p]) for j in range(n)) for p in range(k)] for i in range(b)]
    _close_to_exact(gx, dx, dxs)


@pytest.mark.parametrize("b,k,n", [(32, 784, 100), (37, 101, 13), (300, 257, 190), (6, 1000, 7)])
def test_linear_against_numpy_and_long_double(b, k, n):
    rng = np.random.default_rng(k)
    x, w = rng.standard_normal((b, k)), rng.standard_normal((n, k))
    bias, g = rng.standard_normal((1, n)), rng.standard_normal((b, n))
    z = oracle.linear_forward(x, w, bias)
    np.testing.assert_allclose(z, x @ w.T + bias, rtol=0, atol=1e-12 * np.sqrt(k))
    np.testing.assert_allclose(z - bias, oracle.gemm_long_double(x, w, b, n, k, 1, 1), rtol=0, atol=1e-12 * np.sqrt(k))
    gw, gb, gx = oracle.linear_backward(g, x, w)
    np.testing.assert_allclose(gw, (g.T @ x) / b, rtol=0, atol=1e-12)
    np.testing.assert_allclose(gb, g.sum(axis=0, keepdims=True) / b, rtol=0, atol=1e-13)
    np.testing.assert_allclose(gx, g @ w, rtol=0, atol=1e-12 * np.sqrt(n))
    # invariants: dW * B = G^T X and db * B = column sums
    np.testing.assert_allclose(gw * b, oracle.gemm_long_double(g, x, n, k, b, 0, 0), rtol=0, atol=1e-11)


def test_linear_structure_cases():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((9, 6))
    np.testing.assert_array_equal(oracle.linear_forward(x, np.eye(6), np.zeros((1, 6))), x)  # W = I
    w = rng.standard_normal((4, 6)); b = rng.standard_normal((1, 4))
    onehot = np.eye(6)[[3, 0, 5]]
    np.testing.assert_array_equal(oracle.linear_forward(onehot, w, b), w[:, [3, 0, 5]].T + b)  # row select
    np.testing.assert_array_equal(oracle.linear_forward(np.zeros((2, 6)), w, b), np.repeat(b, 2, axis=0))


# ---- ReLU ---------------------------------------------------------------------------------------
def test_relu_selection_and_specials():
    x = np.array([[np.nan, -np.inf, np.inf, 0.0, -0.0, 5e-324, -5e-324, 2.0]])
    f = oracle.relu_forward(x)
    assert f[0, 0] == 0.0 and f[0, 1] == 0.0 and f[0, 2] == np.inf and f[0, 5] == 5e-324 and f[0, 6] == 0.0
    g = np.array([[1.0, np.inf, np.inf, np.inf, 3.0, 4.0, 5.0, 7.0]])
    b = oracle.relu_backward(g, x)
    assert b[0, 0] == 0.0 and np.isnan(b[0, 1]) and b[0, 2] == np.inf and np.isnan(b[0, 3])
    assert b[0, 4] == 0.0 and b[0, 5] == 4.0 and b[0, 6] == 0.0 and b[0, 7] == 7.0
    rng = np.random.default_rng(3)
    y = rng.standard_normal((50, 40))
    np.testing.assert_array_equal(oracle.relu_forward(y), np.where(y > 0, y, 0.0))
    np.testing.assert_array_equal(oracle.relu_backward(g[:, :1] * 0 + 2.5 + 0 * y, y), np.where(y > 0, 2.5, 0.0))


# ---- softmax --------------------------------------------------------------------------------------
def test_softmax_against_mpmath():
    mp = pytest.importorskip("mpmath")
    mp.mp.dps = 60
    rng = np.random.default_rng(4)
    x = rng.standard_normal((4, 7)) * 5
    p = oracle.softmax(x)
    for r in range(4):
        e = [mp.e ** mp.mpf(float(v)) for v in x[r]]
        s = sum(e)
        for c in range(7):
            # rounding x - max perturbs exp by |x - max| ulps: allow 2^-46 relative
            assert abs(mp.mpf(float(p[r, c])) - e[c] / s) <= mp.mpf(2) ** -46 * (e[c] / s)


def test_softmax_invariants():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((6, 33))
    p = oracle.softmax(x)
    assert np.all(np.abs(p.sum(axis=1) - 1) <= 1e-15 * 33)
    np.testing.assert_array_equal(oracle.softmax(x + 8.0), oracle.softmax(x + 8.0 + 0.0))
    np.testing.assert_allclose(oracle.softmax(x + 123.0), p, rtol=1e-13)  # shift invariance
    for c in (2, 8, 1024):  # uniform rows, power-of-two width: exactly 1/C
        np.testing.assert_array_equal(oracle.softmax(np.full((2, c), -3.7)), np.full((2, c), 1.0 / c))
    assert np.all(np.isfinite(oracle.softmax(x * 1e4)))  # max subtraction: no overflow
    with pytest.raises(oracle.NanLogits):
        oracle.softmax(np.array([[0.0, np.nan]]))
    y = np.array([[-np.inf, 0.0, 0.0]])
    np.testing.assert_array_equal(oracle.softmax(y), np.array([[0.0, 0.5, 0.5]]))


def test_softmax_module_backward_kat_and_independent_form():
    k = KATS["softmax_module_backward"]
    out = oracle.softmax(k["input"])
    got = oracle.softmax_module_backward(k["gradient"], out)
    assert np.all(np.abs(got - np.array(k["expected"])) <= k["tolerance"])
    # independent statement of softmax.rs:62-73: J = -(P^T P), J_ii = d (1 - d), result = G J
    rng = np.random.default_rng(12)
    p = oracle.softmax(rng.standard_normal((9, 5))); g = rng.standard_normal((9, 5))
    ptp = np.einsum("bi,bj->ij", p, p)
    jac = -ptp
    d = np.diag(ptp)
    jac[np.arange(5), np.arange(5)] = d * (1 - d)
    np.testing.assert_allclose(oracle.softmax_module_backward(g, p), g @ jac, rtol=0, atol=1e-14)


# ---- cross entropy (the reference has no test for it: closed forms only) ------------------------
def test_cross_entropy_closed_forms():
    rng = np.random.default_rng(6)
    rows, cols = 12, 10
    z = rng.standard_normal((rows, cols)) * 3
    t = np.zeros((rows, cols)); tgt = rng.integers(0, cols, rows); t[np.arange(rows), tgt] = 1.0
    loss, prob = oracle.cross_entropy_forward(z, t)
    m = z.max(axis=1)
    lse = np.log(np.exp(z - m[:, None]).sum(axis=1)) + m
    assert abs(loss - np.mean(lse - z[np.arange(rows), tgt])) <= 1e-14 * abs(loss)  # log-sum-exp form
    np.testing.assert_array_equal(prob, oracle.softmax(z))
    l2, _ = oracle.cross_entropy_forward(np.full((rows, 16), 0.3), np.eye(16)[:rows])
    assert abs(l2 - math.log(16)) <= 1e-15  # uniform logits: ln C
    g = oracle.cross_entropy_backward(prob, t)
    np.testing.assert_array_equal(g, prob - t)  # -(t - p) == p - t exactly
    assert np.all(np.abs(g.sum(axis=1)) <= 1e-15)


def test_cross_entropy_against_mpmath_soft_labels():
    mp = pytest.importorskip("mpmath")
    mp.mp.dps = 60
    rng = np.random.default_rng(7)
    z = rng.standard_normal((3, 5)); t = rng.random((3, 5)); t /= t.sum(axis=1, keepdims=True)
    loss, _ = oracle.cross_entropy_forward(z, t)
    acc = mp.mpf(0)
    for r in range(3):
        e = [mp.e ** mp.mpf(float(v)) for v in z[r]]
        s = sum(e)
        acc += sum(mp.mpf(float(t[r, c])) * mp.log(e[c] / s) for c in range(5))
    assert abs(mp.mpf(loss) - (-acc / 3)) <= mp.mpf(10) ** -14


def test_cross_entropy_underflow_nan_and_nan_logits():
    loss, _ = oracle.cross_entropy_forward(np.array([[0.0, -800.0]]), np.array([[1.0, 0.0]]))
    assert math.isnan(loss)  # 0 * ln(0): the reference takes ln of the probability
    with pytest.raises(oracle.NanLogits):
        oracle.cross_entropy_forward(np.array([[np.nan, 0.0]]), np.array([[1.0, 0.0]]))


def test_whole_network_finite_differences():
    """dW/db are d(mean CE)/dparam; the returned input gradient is batch * d(mean CE)/dx because
    the loss gradient is not divided by the batch (cross_entropy.rs:46) while dW, db are (linear.rs:63,66)."""
    spec = [("identity",), ("linear", 5, 7), ("relu",), ("linear", 7, 4)]
    rng = np.random.default_rng(8)
    m = oracle.Model(spec)
    for p, _ in m.parameters():
        p[...] = rng.standard_normal(p.shape) * 0.5
    x = rng.standard_normal((6, 5)); t = np.eye(4)[rng.integers(0, 4, 6)]

    def loss_at():
        return oracle.cross_entropy_forward(m.forward(x), t)[0]

    base, prob = oracle.cross_entropy_forward(m.forward(x), t)
    gin = m.backward(oracle.cross_entropy_backward(prob, t))
    grads = [g.copy() for _, g in m.parameters()]
    eps = 1e-6
    for (p, _), g in zip(m.parameters(), grads):
        for idx in [(0, 0), (p.shape[0] - 1, p.shape[1] - 1), (0, p.shape[1] // 2)]:
            old = p[idx]
            p[idx] = old + eps; up = loss_at()
            p[idx] = old - eps; dn = loss_at()
            p[idx] = old
            assert abs((up - dn) / (2 * eps) - g[idx]) <= 1e-7
    for idx in [(0, 0), (5, 4), (2, 3)]:
        old = x[idx]
        x[idx] = old + eps; up = loss_at()
        x[idx] = old - eps; dn = loss_at()
        x[idx] = old
        assert abs((up - dn) / (2 * eps) * 6 - gin[idx]) <= 1e-6


# ---- SGD ------------------------------------------------------------------------------------------
def test_sgd_two_roundings_bit_exact():
    rng = np.random.default_rng(9)
    w = rng.standard_normal((257, 129)) * 0.02; g = rng.standard_normal((257, 129)) * 1e-3
    for lr in (0.01, 0.1, 1.0):
        np.testing.assert_array_equal(oracle.sgd_step(w, g, lr), w - lr * g)


def test_sgd_is_not_a_fused_multiply_add():
    """Find operands where round(w - lr*g exactly) differs from round(w - round(lr*g)) and check
    that the oracle returns the latter (src/optim/sgd.rs:23 builds the product array first)."""
    rng = np.random.default_rng(10)
    lr = 0.1
    found = 0
    for _ in range(2000):
        w, g = float(rng.standard_normal()), float(rng.standard_normal())
        exact = Fraction(w) - Fraction(lr) * Fraction(g)
        fused = float(exact)  # correctly rounded: what one FMA would give
        two = w - lr * g
        if fused != two:
            found += 1
            assert oracle.sgd_step(np.array([[w]]), np.array([[g]]), lr)[0, 0] == two
    assert found > 0


# ---- Sequential order, accuracy, generator ----------------------------------------------------
def test_model_step_equals_layer_functions():
    spec = [("linear", 6, 5), ("relu",), ("linear", 5, 3)]
    rng = np.random.default_rng(11)
    m = oracle.Model(spec)
    ws = [rng.standard_normal(p.shape) for p, _ in m.parameters()]
    for (p, _), w in zip(m.parameters(), ws):
        p[...] = w
    x = rng.standard_normal((4, 6)); t = np.eye(3)[[0, 2, 1, 1]]
    loss = m.train_step(x, t, 0.1)
    z1 = oracle.linear_forward(x, ws[0], ws[1]); a1 = oracle.relu_forward(z1)
    z2 = oracle.linear_forward(a1, ws[2], ws[3])
    l, prob = oracle.cross_entropy_forward(z2, t)
    assert l == loss
    g2 = oracle.cross_entropy_backward(prob, t)
    gw2, gb2, gx2 = oracle.linear_backward(g2, a1, ws[2])
    gw1, gb1, _ = oracle.linear_backward(oracle.relu_backward(gx2, z1), x, ws[0])
    want = [oracle.sgd_step(w, g, 0.1) for w, g in zip(ws, [gw1, gb1, gw2, gb2])]
    for (p, _), wv in zip(m.parameters(), want):
        np.testing.assert_array_equal(p, wv)


def test_accuracy_first_maximum_wins():
    pred = np.array([[1.0, 3.0, 3.0], [2.0, 2.0, 1.0], [0.0, 0.0, 0.0], [5.0, 1.0, 9.0]])
    truth = np.array([[0.0, 1.0, 0.0], [0.0, 1.0, 0.0], [1.0, 0.0, 0.0], [0.0, 0.0, 1.0]])
    assert oracle.accuracy(pred, truth) == 0.75  # row 1: first max is column 0, truth says 1


def _mix64(z):
    with np.errstate(over="ignore"):
        z = z + np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def test_generator_definition_and_distributions():
    seed, stream = 0x5EED, 7
    with np.errstate(over="ignore"):
        key = _mix64(_mix64(np.uint64(seed)) ^ (np.uint64(stream) * np.uint64(0xD1342543DE82EF95)))
        idx = np.arange(1000, dtype=np.uint64)
        r = _mix64(key + idx * np.uint64(0x9E3779B97F4A7C15))
    assert [oracle.rng_u64(seed, stream, int(i)) for i in (0, 1, 999)] == [int(r[0]), int(r[1]), int(r[999])]
    u = oracle.fill_uniform((1, 1000), seed, stream)
    np.testing.assert_array_equal(u.ravel(), (r >> np.uint64(11)).astype(np.float64) * 2.0 ** -53)
    big = oracle.fill_uniform((1, 200000), 1, 2)
    assert 0.0 <= big.min() and big.max() < 1.0 and abs(big.mean() - 0.5) < 5e-3
    nrm = oracle.fill_normal((1, 200000), 1, 3, 1.0, 2.0)
    assert abs(nrm.mean() - 1.0) < 2e-2 and abs(nrm.std() - 2.0) < 2e-2
    oh = oracle.fill_one_hot(500, 10, 1, 4)
    assert np.all(oh.sum(axis=1) == 1.0) and set(np.unique(oh)) == {0.0, 1.0}
    assert np.all(np.bincount(oh.argmax(axis=1), minlength=10) > 20)
